// stack_model.h — a decoder described by a LIST OF LAYERS instead of one fixed block.  Every layer names its mixer and its feed-forward
// with all sizes and constants; the record of the whole stack names the block form, the norm and how positions enter.
//
//   block   parallel:    x <- x + m * (mixer(h) + ff(h)),  h = norm(x)                      (Ditilix)
//           sequential:  x <- x + mixer(norm1(x)),  x <- x + ff(norm2(x))                   (Gaperax)
//           sandwich:    x <- x + norm1b(mixer(norm1(x))),  x <- x + norm2b(ff(norm2(x)))   (Zifetar: RMS norms, norm_offset added to the weights;
//                        Sudosun: Dynamic Tanh norms, the head is the embedding table)
//   norm    rms: RMS norm over `groups` equal parts of the width;  dyt: Dynamic Tanh  tanh(alpha x) w + b  (no statistics)
//   pos     sinusoid: a position vector added to the embedding;  none: positions enter inside the mixers
//   embedding (sandwich stacks): embed * embed_scale + a row of a hashed (previous token, token) table (pair_buckets, pair_mul_prev,
//           pair_mul_cur; the table's last row for a sequence's first token), then an RMS norm of its own
//   mixer   attention: causal softmax, query temperature, soft cap, grouped key/value heads, optionally another layer's keys / values
//           latent:    queries and keys / values through low-rank latents, a rotated key part shared by the heads (rotary with optional
//                      YaRN scaling), a softmax sink per head; the cache holds one row [latent | rotated part] per token and the
//                      up-projections are absorbed: q' = [W_uk_h^T q_h | rot(q_h)], values = the latent, W_uv_h after the sum over keys
//           sigmoid:   biased q / k / v, one RMS norm over all of q and all of k, weights sigmoid(score - slope_h * distance + bias_h)
//                      without normalisation, a window that keeps the first tokens, heads mixed by a matrix, a sigmoid output gate
//   delta:     gated delta rule: short causal convolutions + silu on q / k / v, unit-vector q and k, a write strength per head, a decay per
//                      head and key channel from a low-rank projection, per-head output norm and a low-rank sigmoid gate
//           retention: linear attention with a constant decay per head, rotary (rotate-half layout) on q and k, per-head output norm, silu gate
//           parallel:  two branches on the same input, summed with constant scales: softmax attention (biases, per-head q / k norm, rotary
//                      with wavelength-dependent scaling, visibility inside blocks of `chunk` positions) and a gated linear attention
//                      (decay per key channel sigmoid(z)^(1 / tau) from a low-rank projection)
//           delta, retention and the right branch keep a matrix state [dim, vdim] per head and sequence (f32, one slot per live sequence)
//           lightning: linear attention with a constant decay per head, q / k / v through silu, no rotation, ONE norm over the concatenated
//                      heads, sigmoid gate
//           delta with lowrank=0: one decay per head and token, decay and silu gate projected at full rank (no low-rank stages)
//           parallel with right=rglru: the left branch's softmax attention sees a sliding window, has a sink per head, a temperature per
//                      head, a sigmoid output gate per head and rotary on neighbouring pairs (YaRN-scaled); the right branch is a gelu branch
//                      times a real-gated diagonal recurrence behind a short convolution (block-diagonal gates); each branch's output has an
//                      RMS norm of its own over the width (branch_norm=1) before the scaled sum
//   mlp     none | dense (PolyNorm activation) | moe (sigmoid router, clamped gated experts, gated shared expert) | gated (gelu_tanh(gate) * up)
//           | clamped (dense, the clamped gated form of the experts above);  moe with router=softmax_all: scores are a softmax over all
//           router outputs, a correction is added for the choice only, the choice is restricted to the best `keep` of `groups` groups of
//           neighbouring experts, the weights are the plain scores, and the last `identity` outputs are experts that return their input
//   sandwich blocks with norm=dyt use Dynamic Tanh for all four norms of a layer; tie_head=1: the head is the embedding table
//   weights_of=j: the layer runs with layer j's tensors and a cache of its own
// vllm_rs_amd/checkpoint.py turns a design's config.json into the spec text below.
//
// Precision: the residual stream, norms, router, rotary angles, attention scores and weights are f32; projections, the cache and
// activations are bf16 (f32 accumulation) or, for a VRA_F32 model, f32 throughout.
//
// Spec text, one record per line, `key=value` fields:
//   stack width=.. vocab=.. eps=.. groups=.. residual_mult=.. logit_scale=.. pos_base=.. block=.. norm=.. pos=..
//   layer mixer=.. heads=.. kv_heads=.. dim=.. vdim=.. scale=.. softcap=.. temp_coef=.. temp_every=.. kv_from=.. weights_of=..
//         rot_dim=.. kv_rank=.. q_rank=.. rot_dims=.. rot_base=.. yarn_factor=.. yarn_original=.. yarn_fast=.. yarn_slow=.. sink=0|1
//         window=.. keep_first=.. slope_exp=..
//         conv=.. rank_a=.. rank_g=.. decay=d0,d1,.. chunk=.. qk_norm=0|1 bias=0|1 rs_factor=.. rs_low=.. rs_high=.. rs_original=..
//         r_heads=.. r_dim=.. r_vdim=.. tau=.. left_scale=.. right_scale=..
//         lowrank=0|1 right=gla|rglru r_width=.. r_blocks=.. r_conv=.. head_temp=0|1 head_gate=0|1 rot_layout=half|pairs branch_norm=0|1
//         mlp=none|dense|moe|gated|clamped ff=.. experts=.. top=.. limit=.. shared_ff=.. shared_limit=.. router=sigmoid|softmax|softmax_all
//         act=clamped|silu identity=.. groups=.. keep=..
#pragma once
#include <map>
#include <string>
#include <vector>

#include "model_base.h"

namespace vra {

struct StackLayer {
  // mixer: 0 softmax attention, 1 latent attention, 2 sigmoid attention, 3 gated delta rule, 4 retention, 5 parallel (softmax attention
  // beside a gated linear attention or a real-gated diagonal recurrence), 6 lightning
  int mixer = 0;
  int heads = 0, kv_heads = 0, dim = 0, vdim = 0, temp_every = 0, kv_from = -1, weights_of = -1;
  float scale = 1.f, softcap = 0.f, temp_coef = 0.f;
  // latent attention
  int rot_dim = 0, kv_rank = 0, q_rank = 0, rot_dims = 0, sink = 0;
  double rot_base = 10000.0, yarn_factor = 0.0, yarn_original = 0.0, yarn_fast = 32.0, yarn_slow = 1.0;
  // sigmoid attention: window <= 0 = every earlier token; slope_h = 2^(-slope_exp (h + 1) / heads), 0 = no distance penalty
  int window = 0, keep_first = 0;
  double slope_exp = 0.0;
  // recurrent mixers.  delta: taps of the short convolutions, ranks of the decay / gate projections (a loaded checkpoint's tensor shapes
  // override the ranks); retention: one decay per head; softmax branch of a parallel mixer: block mask, per-head q / k norm, biases,
  // rotary scaling by wavelength (rs_factor 0: none); its right branch: r_* sizes, tau, and the two branches' scales
  int conv = 0, rank_a = 0, rank_g = 0, chunk = 0, qk_norm = 0, has_bias = 0;
  std::vector<float> decay;
  double rs_factor = 0.0, rs_low = 1.0, rs_high = 4.0, rs_original = 0.0;
  int r_heads = 0, r_dim = 0, r_vdim = 0;
  float tau = 1.f, left_scale = 1.f, right_scale = 1.f;
  // delta: lowrank 0 = decay (one per head) and gate come from the joint projection.  parallel: right_kind 1 = real-gated diagonal recurrence
  // of r_width channels with r_blocks gate blocks behind a convolution of `conv` taps; the left branch's per-head temperature and output
  // gate, rotary layout (1 = neighbouring pairs), a norm per branch before the sum
  int lowrank = 1, right_kind = 0, r_width = 0, r_blocks = 1, head_temp = 0, head_gate = 0, rot_layout = 0, branch_norm = 0;
  // router_kind 2: identity experts and expert groups
  int n_identity = 0, n_groups = 0, keep = 0;
  // feed-forward: 0 none, 1 dense (PolyNorm), 2 mixture of experts, 3 gated dense (gelu_tanh(gate) * up), 4 clamped gated dense
  int mlp = 0, ff = 0, experts = 0, top = 0, shared_ff = 0;
  float limit = 0.f, shared_limit = 0.f;
  // mixture of experts: router 0 = sigmoid scores as weights on the experts' inputs, 1 = biased logits, softmax over the chosen ones, weights
  // on the experts' outputs; act 0 = clamped gated form, 2 = silu(gate) * up
  int router_kind = 0, act_kind = 0;
  // derived
  int cache = -1;          // index of the paged cache this layer reads (its own, or the one of layer kv_from)
  bool owns_cache = false;
  int ffp = 0, sffp = 0;   // expert / shared (or gated dense) widths rounded up to 16 (zero rows and columns)
  int nq() const { return heads * (mixer == 1 ? dim + rot_dim : dim); }
  int nk() const { return kv_heads * dim; }
  int nv() const { return kv_heads * vdim; }
  // columns of the joint input projection: q (| k | v) of softmax attention, q | k | v | gate of sigmoid attention, the three latents
  int nqkv() const {
    if (mixer == 1) return q_rank + kv_rank + rot_dim;
    if (mixer == 2) return nq() + nk() + nv() + heads * vdim;
    if (mixer == 3) return 2 * nk() + heads * vdim + heads + (lowrank ? 0 : heads + heads * vdim);  // q | k (kv_heads each) | v | write strengths (| decays | gate)
    if (mixer == 4 || mixer == 6) return 2 * heads * dim + 2 * heads * vdim;       // q | k | v | gate
    if (mixer == 5 && right_kind == 1) return nq() + nk() + nv() + (head_gate ? heads : 0) + 2 * r_width;  // left q | k | v | gates, right gelu branch | recurrent branch
    if (mixer == 5) return nq() + nk() + nv() + r_heads * (2 * r_dim + 2 * r_vdim);  // left q | k | v, right q | k | v | gate
    return nq() + (owns_cache ? nk() + nv() : 0);
  }
  bool has_cache() const { return mixer != 3 && mixer != 4 && mixer != 6; }
  // the recurrent part: heads, key and value sizes of the matrix state (0 heads: none)
  int s_heads() const { return mixer == 5 ? (right_kind == 1 ? 0 : r_heads) : (mixer == 3 || mixer == 4 || mixer == 6 ? heads : 0); }
  int vec_state() const { return mixer == 5 && right_kind == 1 ? r_width : 0; }  // a diagonal recurrence: one state value per channel
  int s_dim() const { return mixer == 5 ? r_dim : dim; }
  int s_vdim() const { return mixer == 5 ? r_vdim : vdim; }
  int conv_channels() const { return mixer == 3 ? 2 * nk() + heads * vdim : vec_state(); }
  // elements of one token's cache rows
  int k_row() const { return mixer == 1 ? kv_rank + rot_dim : nk(); }
  int v_row() const { return mixer == 1 ? 0 : nv(); }
  // device weights
  float* norm_w = nullptr;
  float *norm_b = nullptr, *norm2_w = nullptr, *norm2_b = nullptr;  // Dynamic Tanh: offsets, and the second norm of a sequential block
  float norm_alpha = 1.f, norm2_alpha = 1.f;
  void* qkv = nullptr;     // [nqkv(), width]
  float* qkv_bias = nullptr;  // sigmoid attention: f32 [nqkv()] (zeros for the gate rows)
  void* o = nullptr;       // [width, heads * vdim]
  void* uq = nullptr;      // latent: [heads * (dim + rot_dim), q_rank]
  void* ukt = nullptr;     // latent: [heads][kv_rank][dim] — W_uk of a head, transposed
  void* uv = nullptr;      // latent: [heads * vdim, kv_rank]
  float *qn_w = nullptr, *kn_w = nullptr;  // latent: norms of the two latents; sigmoid: norms over all of q / all of k
  float *sink_w = nullptr, *freq_hi = nullptr, *freq_lo = nullptr;
  int rot_pairs = 0;
  float rot_mag = 1.f;
  float *talk = nullptr, *head_bias = nullptr, *slopes = nullptr;
  void* up = nullptr;      // dense [ff, width]
  void* down = nullptr;    // dense [width, ff]
  float* act = nullptr;    // PolyNorm a, b, c, e
  void* router = nullptr;  // [experts (+ 1: the shared expert's gate), width]
  void* e_gu = nullptr;    // [experts][2 * ffp][width], gate / up rows interleaved in blocks of 16
  void* e_down = nullptr;  // [experts][width][ffp]
  void* s_gu = nullptr;    // [2 * sffp][width]  (shared expert, or the gated dense feed-forward)
  void* s_down = nullptr;  // [width][sffp]
  // sandwich blocks and recurrent mixers
  float *post1_w = nullptr, *post2_w = nullptr;  // norms of the mixer's / the feed-forward's output
  float* router_bias = nullptr;
  void* lr1 = nullptr;          // first stage of the low-rank projections [rank_a (+ rank_g), width]
  void* lr2 = nullptr;          // second stage [heads * dim (+ heads * vdim), rank_a (+ rank_g)], block diagonal
  float* lr2_bias = nullptr;
  float *conv_w = nullptr, *rate = nullptr, *dt_bias = nullptr, *out_norm_w = nullptr, *head_decay = nullptr;
  void* r_o = nullptr;          // right branch: [width, r_heads * r_vdim]
  float *post1_b = nullptr, *post2_b = nullptr;  // Dynamic Tanh in sandwich blocks: offsets and slopes of the output norms
  float post1_alpha = 1.f, post2_alpha = 1.f;
  float *temp_w = nullptr, *left_out_w = nullptr, *right_out_w = nullptr;
  float *conv_b = nullptr, *gates_w = nullptr, *gates_b = nullptr, *lam = nullptr;  // gates_w f32 [r_blocks][2 * bw][bw]: recurrence gate rows, then input gate rows
  float* state = nullptr;       // [slots, heads, vdim, dim];  a diagonal recurrence: [slots, r_width]
  float* conv_state = nullptr;  // [slots, conv - 1, conv_channels()]
};

class StackModel : public ModelBase {
 public:
  StackModel(const vra_model_config& mc, const vra_engine_config& ec, const char* spec);
  ~StackModel() override;
  bool init_synthetic(uint64_t seed) override;
  bool load_tensor(const std::string& name, const void* host, const int64_t* shape, int ndim, int elem_bytes) override;
  bool finalize_weights() override;
  bool init_kv_cache(int num_blocks) override;
  int64_t state_bytes_per_slot() const override;
  bool init_state(int slots) override;
  int num_blocks() const override { return num_blocks_; }
  int kv_layers() const override { return (int)kc_.size(); }
  size_t k_block_bytes(int c) const override;
  size_t v_block_bytes(int c) const override;
  void* k_cache(int c) const override { return kc_[c]; }
  void* v_cache(int c) const override { return vc_[c]; }
  int64_t kv_bytes_per_block() const override;
  bool init_buffers(int max_tokens, int max_seqs) override;
  int max_logit_rows() const override { return logit_rows_cap_; }
  void set_comm(void*) override {}
  bool has_comm() const override { return false; }
  int world() const override { return 1; }
  bool forward(const InputMetadata& md, int64_t stream, uint32_t* tokens = nullptr) override;
  float* logits() const override { return logits_; }
  size_t weight_bytes() const override { return weight_bytes_; }
  void set_layer_trace(bool on) override { trace_on_ = on; }
  int64_t read_layer_trace(void* host, int64_t max_bytes, int64_t stream) override;
  const std::vector<StackLayer>& layers() const { return layers_; }

 private:
  struct HostTensor {
    std::vector<uint8_t> data;
    std::vector<int64_t> shape;
    int elem_bytes = 0;
  };
  void* dalloc(size_t bytes);
  void* upload(const void* host, size_t bytes);
  bool need(const std::string& name, int64_t d0, int64_t d1, const HostTensor** out);
  float* upload_f32(const HostTensor& t);
  bool parse_spec(const char* spec);
  bool feed_forward(const StackLayer& L, int T, int64_t stream);
  bool mixer_softmax(const StackLayer& L, const InputMetadata& md, int64_t stream);
  bool mixer_latent(const StackLayer& L, const InputMetadata& md, int64_t stream);
  bool mixer_sigmoid(const StackLayer& L, const InputMetadata& md, int64_t stream);
  bool mixer_delta(const StackLayer& L, const InputMetadata& md, int64_t stream);
  bool mixer_retention(const StackLayer& L, const InputMetadata& md, int64_t stream);
  bool mixer_parallel(const StackLayer& L, const InputMetadata& md, int64_t stream);
  bool mixer_lightning(const StackLayer& L, const InputMetadata& md, int64_t stream);
  bool mixer_hybrid(const StackLayer& L, const InputMetadata& md, int64_t stream);
  bool recurrent_tail(const StackLayer& L, const InputMetadata& md, const float* gate, int gate_ld, int gate_act, const void* w_o, float* out, int64_t stream);
  bool forward_sandwich(const InputMetadata& md, int64_t stream);
  void rotary_table(StackLayer& L);
  float* upload_floats(const std::vector<float>& v);
  bool norm_into_h(const float* w, const float* b, float alpha, const float* add, float* x, void* h, int T, int64_t stream);
  bool expert_pair(const void* a, int lda, const void* w_gu, int64_t gu_stride, const void* w_down, int64_t down_stride, int rows, int fp, int f,
                   float limit, const int* tile_group, int granule, const int* a_row, const float* a_scale, const int* out_row, float* out,
                   int64_t stream, int act = 0);
  vra_model_config mc_;
  vra_engine_config ec_;
  std::string spec_error_;
  int dt_ = 0;
  size_t es_ = 2;
  int width_ = 0, vocab_ = 0, groups_ = 1;
  int block_ = 0, norm_kind_ = 0, pos_kind_ = 0;  // 0 parallel / rms / sinusoid, 1 sequential / dyt / none, block 2 sandwich
  float norm_offset_ = 0.f, embed_scale_ = 1.f;    // added to every norm weight at load; multiplies the embedding row
  int embed_norm_ = 0, pair_buckets_ = 0, tie_head_ = 0;
  float *h32_ = nullptr, *id_weight_ = nullptr;  // identity experts: the unrounded feed-forward input and the summed weight of a token's identity picks
  int64_t pair_mul_prev_ = 0, pair_mul_cur_ = 0;
  void* pair_table_ = nullptr;
  float* embed_norm_w_ = nullptr;
  int state_slots_ = 0;
  float *z2_ = nullptr, *rec_ = nullptr, *ro_ = nullptr;
  float eps_ = 1e-6f, residual_mult_ = 1.f, logit_scale_ = 1.f;
  double pos_base_ = 10000.0;
  std::vector<StackLayer> layers_;
  std::map<std::string, HostTensor> staged_;
  bool finalized_ = false;
  std::vector<void*> allocs_;
  size_t weight_bytes_ = 0;
  void* embed_ = nullptr;
  void* head_ = nullptr;
  float* final_norm_ = nullptr;
  float* final_b_ = nullptr;
  float final_alpha_ = 1.f;
  float* inv_freq_ = nullptr;
  // paged caches of the layers that own one: K [blocks * BS, kv_heads * dim], V [blocks * BS, kv_heads * vdim]
  std::vector<void*> kc_, vc_;
  std::vector<int> cache_layer_;
  int num_blocks_ = 0;
  // activations
  int max_tokens_ = 0, max_seqs_ = 0, logit_rows_cap_ = 0, max_rows_ = 0;
  float *x_ = nullptr, *o_ = nullptr, *z_ = nullptr, *pair_out_ = nullptr, *sh_ = nullptr, *xl_ = nullptr, *logits_ = nullptr;
  void *h_ = nullptr, *qkv_ = nullptr, *attn_ = nullptr, *act_ = nullptr, *hl_ = nullptr, *qa_ = nullptr;
  int *pair_expert_ = nullptr, *row_token_ = nullptr, *row_pair_ = nullptr, *tile_group_ = nullptr;
  float *pair_weight_ = nullptr, *row_scale_ = nullptr, *gate_ = nullptr;
  float* sig_scratch_ = nullptr;
  size_t sig_scratch_bytes_ = 0;
  bool trace_on_ = false;
  float* trace_ = nullptr;
  size_t trace_cap_ = 0, trace_bytes_ = 0;
};

}  // namespace vra
