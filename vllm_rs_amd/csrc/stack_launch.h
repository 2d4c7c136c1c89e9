// stack_launch.h — internal entry points of stack_ops.hip: the operators of config-driven layer stacks (host/stack_model.cpp).
// Element type `dtype`: VRA_BF16 (16-bit storage, f32 accumulation; norms, routers, attention scores and weights and the residual stay f32) or
// VRA_F32 (everything in 32-bit, no reduced-precision matrix mode).  All pointers are device pointers; launches are asynchronous
// on `stream` and graph-capturable (no allocation, no synchronisation, no memset nodes).
#pragma once
#include <stdint.h>

// out[r', n] = alpha * sum_k A[row(r), k] * scale(r) * W_g[n, k]  for logical rows r < M ("NT" GEMM, weights stored [N, K]).
// Grouped form: the logical rows are cut into granules of `granule` rows, granule t uses the weights of group tile_group[t]
// (w + group * w_group_stride elements; -1 = an empty granule).  a_row gathers (logical row -> row of A, -1 = no row),
// a_scale multiplies the gathered row (bf16: the product is rounded to bf16 before the matrix product), out_row scatters
// (logical row -> row of out, -1 = not written).  Null pointers = identity / one group.
// epi 0: plain.  epi 1: gated pair — W holds gate and up rows interleaved in blocks of 16 (block 2b = gate rows 16b.., block 2b+1 =
// up rows 16b..), N counts both; out gets N/2 columns of  g' * sigmoid(act_alpha * g') * (u' + 1),  g' = min(g, limit),
// u' = clamp(u, -limit, limit)  (limit <= 0: no clamp).
struct StkGemmArgs {
  const void* a = nullptr;
  int lda = 0;
  const void* w = nullptr;
  int64_t w_group_stride = 0;
  void* out = nullptr;
  int ldo = 0;
  int out_f32 = 0;
  int M = 0, N = 0, K = 0;
  float alpha = 1.f;
  const int* tile_group = nullptr;
  int granule = 0;
  const int* a_row = nullptr;
  const float* a_scale = nullptr;
  const int* out_row = nullptr;
  int epi = 0;
  float limit = 0.f, act_alpha = 1.702f;
  int act = 0;                  // the gated pair of epi 1: 0 the clamped form above, 1  gelu_tanh(g) * u, 2  silu(g) * u
  const float* bias = nullptr;  // f32 [N], added after alpha (plain epilogue)
  // batched form (no row groups): product z of `batch` reads a + z * a_batch_stride, w + z * w_batch_stride and writes out + z * out_batch_stride
  // (element counts; a column offset per head turns one launch into a product per head)
  int batch = 1;
  int64_t a_batch_stride = 0, w_batch_stride = 0, out_batch_stride = 0;
  int64_t bias_batch_stride = 0;  // elements between the bias rows of two products of a batch
};
void vra_stack_gemm(const StkGemmArgs& g, int dtype, int64_t stream);
// rows per granule the grouped launches of an M-row problem over `groups` groups want (16 or 64)
int vra_stack_gemm_granule(int rows, int groups);

// x[t, c] = embed[ids[t], c] + pe(positions[t], c),  pe(p, 2i) = sin(p * inv_freq[i]),  pe(p, 2i+1) = cos(p * inv_freq[i])  (f32);
// inv_freq null: no position vector
void vra_stack_embed_sinpos(const uint32_t* ids, const int64_t* positions, const void* embed, const float* inv_freq, float* x, int T, int W, int V,
                            int dtype, int64_t stream);

// RMS norm in `groups` equal consecutive parts: h = x / sqrt(mean_part(x^2) + eps) * w   (x, w f32; h in dtype).
// Router (router_w != null, [n_router (+1 when gate_row), W] in dtype): z = router_w . h in f32 on the unrounded h; the `top` largest of the
// first n_router give pair_expert / pair_weight [T, top] (weight = sigmoid(z), not renormalised; ties: the lower index); with
// gate_row the last row gives gate_out[t] = sigmoid(z_last).
struct StkNormArgs {
  const float* x = nullptr;
  const float* w = nullptr;
  void* h = nullptr;
  int T = 0, W = 0, groups = 1;
  float eps = 1e-6f;
  const void* router_w = nullptr;
  int n_router = 0, top = 0, gate_row = 0;
  int* pair_expert = nullptr;
  float* pair_weight = nullptr;
  float* gate_out = nullptr;
};
void vra_stack_group_norm(const StkNormArgs& a, int dtype, int64_t stream);

// Token-expert pairs -> granule-padded rows sorted by expert: row_token / row_scale / row_pair [max_rows] (-1 / 0 in padding rows),
// tile_group [max_rows / granule].  max_rows >= P + n_groups * granule rounded up to the granule.
void vra_stack_moe_sort(const int* pair_expert, const float* pair_weight, int P, int top, int n_groups, int granule, int max_rows, int* row_token,
                        float* row_scale, int* row_pair, int* tile_group, int64_t stream);

// the gated pair of epi 1 on an f32 [M, 2 * F] matrix whose column blocks of 16 alternate gate / up -> out [M, F] in dtype
void vra_stack_gated_act(const float* gu, void* out, int M, int F, float limit, float act_alpha, int dtype, int64_t stream, int act = 0);

// PolyNorm: out = a N(z) + b N(z^2) + c N(z^3) + e,  N(v) = v / sqrt(mean(v^2) + eps) over a token's F values; coef = {a, b, c, e} (device, f32)
void vra_stack_polynorm(const float* z, void* out, const float* coef, int M, int F, float eps, int dtype, int64_t stream);

// x[t] += mult * (o[t] + sum_{j < n1} p1[t * n1 + j] + gate[t] * p2[t])     (all f32 [*, W]; null pointers drop their term; gate null = 1)
void vra_stack_residual_combine(float* x, const float* o, const float* p1, int n1, const float* p2, const float* gate, float mult, int T, int W,
                                int64_t stream);

// k / v rows of a step -> the paged cache of their layer: K [slots, G * dim], V [slots, G * vdim]; slot < 0: nothing written
void vra_stack_kv_store(const void* k, const void* v, int ld, void* kc, void* vc, const int64_t* slots, int T, int kdim, int vdim, int dtype,
                        int64_t stream);

// Causal softmax attention over the paged cache, scores and weights in f32:
//   s(i, j) = (q_i . k_j) * temp(p_i) * scale,  temp(p) = 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)  (temp_every <= 0: 1),
//   s <- softcap * tanh(s / softcap) (softcap > 0),  key j visible iff j <= p_i.
// q [T, ldq] (head h at column h * dim), out [T, H * vdim]; query head h reads kv head h / (H / G).
struct StkAttnArgs {
  const void* q = nullptr;
  int ldq = 0;
  void* out = nullptr;
  const void* kc = nullptr;
  const void* vc = nullptr;
  const int64_t* positions = nullptr;
  const uint32_t* block_tables = nullptr;
  const uint32_t* context_lens = nullptr;
  const uint32_t* cu_q = nullptr;  // prefill form: [B + 1]; null: decode form, one token per sequence
  int B = 0, T = 0, max_q = 1, H = 0, G = 0, dim = 0, vdim = 0, BS = 64, max_blocks = 0;
  float scale = 1.f, softcap = 0.f, temp_coef = 0.f;
  int temp_every = 0;
  const float* sink = nullptr;  // f32 [H]: the softmax denominator also holds exp(sink[h]) — a term without key or value, counted once
  int k_ld = 0, v_ld = 0;       // elements between the rows of kc / vc (0: G * dim / G * vdim).  A latent cache keeps one row [c | rotated
                                // part] per token: keys are the whole row, values its first columns (vc = kc, v_ld = k_ld)
  int chunk = 0;                // > 0: key j is visible only if it lies in the query's own block of `chunk` positions,
                                // floor(j / chunk) = floor(p_i / chunk); blocks count from position 0 of the sequence
  int window = 0;               // > 0: key j is visible only if p_i - j < window (the query's own position and the window - 1 before it)
  const float* head_scale = nullptr;  // f32 [H]: head h's scores are also multiplied by head_scale[h] (the sink is not)
  const float* gate = nullptr;  // f32 [T, gate_ld], column h: head h's output row is multiplied by sigmoid(gate[t, h])
  int gate_ld = 0;
};
void vra_stack_attention(const StkAttnArgs& a, int dtype, int64_t stream);

// rows of a [*, W] f32 matrix picked by index -> dst (f32)
void vra_stack_gather_rows_f32(const float* src, const uint32_t* rows, float* dst, int n, int W, int64_t stream);

// ---------------------------------------------------------------------------------------------------------------------------------------
// Operators of sequential pre-norm blocks with other mixers (stack_mixers.hip)

// Dynamic Tanh "norm" with the residual sum folded in:  x += add (add null: x as it is);  h = tanh(alpha * x) * w + b   (x, add, w, b f32;
// h in dtype).  No statistics of the row.
void vra_stack_dyt(float* x, const float* add, const float* w, const float* b, float alpha, void* h, int T, int W, int dtype, int64_t stream);

// Rotary angles: pair i of a vector at position p turns by p * (freq_hi[i] + freq_lo[i]) (the frequency as an unevaluated sum of two f32,
// so that the f32 angle carries no rounding of the frequency); (u, v) -> mag * (u cos - v sin, v cos + u sin); the pair is (2i, 2i + 1).
struct StkRotary {
  const float* freq_hi = nullptr;
  const float* freq_lo = nullptr;
  int pairs = 0;      // rotated dimensions / 2; the dimensions behind them pass unchanged
  float mag = 1.f;    // multiplies cos and sin
};

// Latent projections of one token, from the f32 row  raw = [a | b | r]  of the joint down-projection:
//   cq = rmsnorm(a) * qn_w                      -> cq [T, q_rank] in dtype
//   c  = rmsnorm(b) * kvn_w, rot(r) at position -> cache row [c | rot(r)] at the token's slot (cache_ld elements per row; slot < 0: skipped)
// rmsnorm(v) = v / sqrt(mean(v^2) + eps).
struct StkLatentPrepArgs {
  const float* raw = nullptr;
  int ld = 0, q_rank = 0, kv_rank = 0, rot_dim = 0;
  const float* qn_w = nullptr;
  const float* kvn_w = nullptr;
  float eps = 1e-6f;
  void* cq = nullptr;
  void* cache = nullptr;
  int cache_ld = 0;
  const int64_t* slots = nullptr;
  const int64_t* positions = nullptr;
  StkRotary rot;
  int T = 0;
};
void vra_stack_latent_prep(const StkLatentPrepArgs& a, int dtype, int64_t stream);

// Rotary on the rows of a head-by-head matrix: for every token t and head h the `n` values at in[t, h * in_hs + in_off ..] are rotated at
// positions[t] and written to out[t, h * out_hs + out_off ..] (both in dtype; in == out allowed when the ranges are the same).
void vra_stack_rope_heads(const void* in, int in_ld, int in_hs, int in_off, void* out, int out_ld, int out_hs, int out_off, int n, int H,
                          const int64_t* positions, const StkRotary& rot, int T, int dtype, int64_t stream);

// One RMS norm over ALL of q and one over ALL of k (before the split into heads), from the f32 row  raw = [q | k | v | ...]:
//   q_out = rmsnorm(q) * q_w (dtype) ; cache K row = rmsnorm(k) * k_w ; cache V row = v   (q_w / k_w null: that norm is skipped)
void vra_stack_qk_norm_store(const float* raw, int ld, int nq, int nk, int nv, const float* q_w, const float* k_w, float eps, void* q_out, void* kc,
                             void* vc, const int64_t* slots, int T, int dtype, int64_t stream);

// Attention without softmax over the paged cache: every visible key j of query i (positions p_i, j) weighs
//   w_h(i, j) = sigmoid((q_h . k_g) * scale - slopes[h] * (p_i - j) + head_bias[h]),   visible: j <= p_i and (p_i - j < window or j < keep_first)
// (window <= 0: every j <= p_i), not normalised over keys; the heads' weights are mixed, w'_h = sum_g talk[h, g] w_g; head h applies w'_h to
// the values of its own key/value head; the output row is multiplied by sigmoid(gate) element by element.  slopes, head_bias, talk, gate
// null: that term is absent.  Scores, weights and sums f32; keys are summed in ascending order in tiles aligned to absolute positions.
struct StkSigAttnArgs {
  const void* q = nullptr;
  int ldq = 0;
  void* out = nullptr;  // [T, H * vdim] in dtype
  const void* kc = nullptr;
  const void* vc = nullptr;
  const int64_t* positions = nullptr;
  const uint32_t* block_tables = nullptr;
  const uint32_t* context_lens = nullptr;
  const uint32_t* cu_q = nullptr;  // prefill form [B + 1]; null: one token per sequence
  int B = 0, T = 0, max_q = 1, H = 0, G = 0, dim = 0, vdim = 0, BS = 64, max_blocks = 0;
  float scale = 1.f;
  int window = 0, keep_first = 0;
  const float* slopes = nullptr;     // [H]
  const float* head_bias = nullptr;  // [H]
  const float* talk = nullptr;       // [H, H]
  const float* gate = nullptr;       // f32 [T, gate_ld], H * vdim columns used
  int gate_ld = 0;
  // f32 scratch for the forms that sum in two launches (null: the one-launch kernel, any shape).  Prompt portions of bf16 models on the
  // matrix cores need T * H * G * vdim floats, one token per sequence needs B * S * H * vdim with S <= 64 key tiles; max_len bounds the
  // context of an unwindowed layer (it fixes S, and with it the order of the sums).
  float* scratch = nullptr;
  size_t scratch_bytes = 0;
  int max_len = 0;
};
void vra_stack_sigmoid_attention(const StkSigAttnArgs& a, int dtype, int64_t stream);

// ---------------------------------------------------------------------------------------------------------------------------------------
// Operators of sandwich-norm blocks with recurrent mixers (stack_recurrent.hip).  A sequence's recurrent state lives in the slot
// state_slots[b] names (-1: a padded lane, nothing is read or written); a sequence whose first token of the step stands at position 0
// starts from zeros, whatever the slot holds.  cu_q null: one token per sequence.

// x[t] = N(embed[id_t] * scale + table[row_t]; norm_w),  row_t = (prev_t * mul_prev + id_t * mul_cur) mod buckets, and row `buckets` (the
// table's last) for a sequence's first token; prev_t is the token before t: the row before it in the step, or prev_tokens[b] for the first
// row of sequence b (the engine keeps every sequence's tokens).  N(v; w) = v / sqrt(mean(v^2) + eps) * w; norm_w null: no norm.
struct StkEmbedPairArgs {
  const uint32_t* ids = nullptr;
  const int64_t* positions = nullptr;
  const uint32_t* cu_q = nullptr;
  const uint32_t* prev_tokens = nullptr;  // [B]
  const void* embed = nullptr;            // [V, W]
  const void* table = nullptr;            // [buckets + 1, W]; null: no pair term
  int buckets = 0;
  int64_t mul_prev = 0, mul_cur = 0;
  float scale = 1.f;
  const float* norm_w = nullptr;
  float eps = 1e-6f;
  float* x = nullptr;
  int T = 0, B = 0, W = 0, V = 0;
};
void vra_stack_embed_pair(const StkEmbedPairArgs& a, int dtype, int64_t stream);

// The seam between two sub-blocks of a sandwich-norm stack, one launch:
//   s = c1 * sum_{j < n1} pw[t * n1 + j] * p1[(t * n1 + j), :]  +  c2 * p2w[t] * p2[t, :]   (pw, p2w null: weights 1; p2 null: no second part;
//                                                                                       pe: pairs with pe[t * n1 + j] < 0 have no row and are left out)
//   with p1_norm_w / p2_norm_w (n1 = 1): each part is first divided by its root mean square over the row and multiplied by that weight
//   x[t] += N(s; post_w)                                                              (post_w null: nothing is added)
//   h[t]  = N(x[t]; pre_w)  in dtype                                                  (pre_w null: no h);  h32: also the unrounded h (f32)
// N is an RMS norm with a weight, or (dyt) Dynamic Tanh  tanh(alpha v) w + b  with the slopes post_alpha / pre_alpha and offsets post_b / pre_b.
// With router_w ([n_router, W] in dtype): z = router_w . h + router_bias on the unrounded h, the `top` largest (ties: the lower
// index) -> pair_expert / pair_weight [T, top].  router_kind 0: weights = softmax over the chosen logits.  router_kind 1: scores =
// softmax over all n_router logits; the choice goes by score + router_bias (a correction that the weights do not carry) among the experts of
// the `keep` groups (of n_groups equal groups of neighbours) whose largest corrected score is largest; weights = the chosen scores as they
// are; the last n_identity router outputs are experts without tensors that hand their input back: their pairs get expert -1 and their
// weights are summed into id_weight[t].  All f32.
struct StkSandwichArgs {
  float* x = nullptr;
  const float* p1 = nullptr;
  int n1 = 1;
  const float* pw = nullptr;
  float c1 = 1.f;
  const float* p2 = nullptr;
  float c2 = 1.f;
  const float* post_w = nullptr;
  const float* pre_w = nullptr;
  void* h = nullptr;
  float eps = 1e-6f;
  int T = 0, W = 0;
  const void* router_w = nullptr;
  const float* router_bias = nullptr;
  int n_router = 0, top = 0;
  int* pair_expert = nullptr;
  float* pair_weight = nullptr;
  int dyt = 0;
  const float* post_b = nullptr;
  const float* pre_b = nullptr;
  float post_alpha = 1.f, pre_alpha = 1.f;
  const float* p1_norm_w = nullptr;
  const float* p2_norm_w = nullptr;
  const int* pe = nullptr;
  const float* p2w = nullptr;
  float* h32 = nullptr;
  int router_kind = 0, n_groups = 0, keep = 0, n_identity = 0;
  float* id_weight = nullptr;
};
void vra_stack_sandwich_norm(const StkSandwichArgs& a, int dtype, int64_t stream);

// Heads of one token from the f32 row of a joint projection: per head an optional RMS norm over `dim` (weight [dim] shared by the heads),
// rotary on the first 2 * rot.pairs dimensions in the rotate-half layout (dimension i pairs with i + rot.pairs), a scale.
// q heads -> q_out [T, q_ld]; k heads -> k_out: rows by token (slots null) or the paged cache's rows by slot; v -> v_out likewise (null:
// not written).  out_f32: outputs are f32 instead of dtype.
struct StkHeadPrepArgs {
  const float* raw = nullptr;
  int ld = 0, q_off = 0, k_off = 0, v_off = 0;
  int Hq = 0, Hk = 0, dim = 0, nv = 0;
  const float* qn_w = nullptr;
  const float* kn_w = nullptr;
  float eps = 1e-6f;
  StkRotary rot;
  float q_scale = 1.f, k_scale = 1.f;
  const int64_t* positions = nullptr;
  void* q_out = nullptr;
  int q_ld = 0;
  void* k_out = nullptr;
  int k_ld = 0;
  void* v_out = nullptr;
  int v_ld = 0;
  const int64_t* slots = nullptr;
  int out_f32 = 0;
  int T = 0;
  int rot_pairs_layout = 0;  // 1: dimension 2i pairs with 2i + 1 (neighbours) instead of i with i + rot.pairs
};
void vra_stack_head_prep(const StkHeadPrepArgs& a, int dtype, int64_t stream);

// Inputs of a gated delta rule from the f32 rows  raw = [q (G * dim) | k (G * dim) | v (H * vdim) | b (H)]  and  raw2 = [a (H * dim) | ..]:
// q, k, v pass a causal convolution over time per channel (conv_w [C, taps], last column = the current token; the taps - 1 inputs before a
// step's first row come from conv_state [slots, taps - 1, C], zeros for a sequence that starts) and silu; q and k heads become unit
// vectors (x / sqrt(sum x^2 + 1e-6)), q times q_scale  -> qkv_out [T, C] f32;  beta = sigmoid(b) -> beta_out [T, H];
// decay = exp(-rate[h] * softplus(a + dt_bias)) -> decay_out [T, H * dim].  vra_stack_conv_state_update then moves the state on.
struct StkDeltaPrepArgs {
  const float* raw = nullptr;
  int ld = 0;
  const float* raw2 = nullptr;
  int ld2 = 0;
  const float* conv_w = nullptr;
  int taps = 1;
  float* conv_state = nullptr;
  const float* rate = nullptr;     // [H]
  const float* dt_bias = nullptr;  // [H * dim]
  float q_scale = 1.f;
  int decay_dim = 0;               // decays a head: 0 = one per key channel (raw2 / dt_bias / decay_out carry H * dim), 1 = one per head (H)
  float* qkv_out = nullptr;
  float* beta_out = nullptr;
  float* decay_out = nullptr;
  const int64_t* positions = nullptr;
  const uint32_t* cu_q = nullptr;
  const int32_t* state_slots = nullptr;
  int T = 0, B = 0, H = 0, G = 0, dim = 0, vdim = 0;
};
void vra_stack_delta_prep(const StkDeltaPrepArgs& a, int64_t stream);
void vra_stack_conv_state_update(const StkDeltaPrepArgs& a, int64_t stream);

// out = exp(-softplus(-z) * inv_tau) = sigmoid(z)^(1 / tau), element by element (f32 [T, n] with row strides)
void vra_stack_sigmoid_pow(const float* z, int ldz, float* out, int ldo, int T, int n, float inv_tau, int64_t stream);

// Linear recurrence over a sequence's tokens with a matrix state S [dim, vdim] per head (f32, kept as its transpose [slots, H, vdim, dim]):
//   S <- diag(d_t) S   (d_t: decay [T, ldd], head h at column h * dim; or head_decay[h] for every row)
//   u = v_t (beta null)   or   u = beta_t (v_t - S^T k_t)  (delta rule)
//   S <- S + k_t u^T ;  o_t = S^T (q_scale q_t)
// q / k head of value head h = h / qk_rep.  Tokens run one after the other in one fixed order of operations, so a step's cut leaves no trace.
struct StkScanArgs {
  const float* q = nullptr;
  int ldq = 0;
  const float* k = nullptr;
  int ldk = 0;
  const float* v = nullptr;
  int ldv = 0;
  const float* decay = nullptr;
  int ldd = 0;
  int decay_per_head = 0;  // 1: decay [T, ldd] holds ONE decay per head and token (column h) instead of one per key channel
  int act_silu = 0;        // 1: q, k and v pass silu on their way in (constant decays per head only)
  const float* head_decay = nullptr;
  const float* beta = nullptr;
  int ldb = 0;
  float q_scale = 1.f;
  float* state = nullptr;
  const int32_t* state_slots = nullptr;
  const int64_t* positions = nullptr;
  const uint32_t* cu_q = nullptr;
  float* out = nullptr;
  int ldo = 0;
  int B = 0, H = 0, qk_rep = 1, dim = 0, vdim = 0;
};
void vra_stack_linear_scan(const StkScanArgs& a, int64_t stream);

// out[t, h * vdim + c] = o[t, h, c] / sqrt(mean_c(o^2) + eps) * w[c] * act(gate[t, h * vdim + c])   (w null: 1; gate null: no gate;
// gate_act 1: silu, 2: sigmoid);  o f32 [T, H * vdim], out in dtype
void vra_stack_head_norm_gate(const float* o, const float* w, const float* gate, int gate_ld, int gate_act, float eps, void* out, int T, int H, int vdim,
                              int dtype, int64_t stream);

// ---------------------------------------------------------------------------------------------------------------------------------------
// A short causal convolution over time per channel with its state, and a gated diagonal linear recurrence (stack_recurrent.hip)

// y[t, c] = act(bias[c] + sum_j w[c, j] x[t - (taps - 1 - j), c])   (x f32 [T, ld]; w f32 [C, taps], last column = the current token; the inputs
// before a step's first row come from conv_state [slots, taps - 1, C], zeros for a sequence that starts; act 0 none, 1 silu; bias may be null).
// vra_stack_conv_rows_update then moves the state on (the last taps - 1 inputs of every sequence).
struct StkConvArgs {
  const float* x = nullptr;
  int ld = 0, C = 0, taps = 1;
  const float* w = nullptr;
  const float* bias = nullptr;
  float* conv_state = nullptr;
  int act = 0;
  float* y = nullptr;
  int ldy = 0;
  const int64_t* positions = nullptr;
  const uint32_t* cu_q = nullptr;
  const int32_t* state_slots = nullptr;
  int T = 0, B = 0;
};
void vra_stack_conv_rows(const StkConvArgs& a, int64_t stream);
void vra_stack_conv_rows_update(const StkConvArgs& a, int64_t stream);

// Real-gated diagonal recurrence over a sequence's tokens, one state value per channel (f32 [slots, C]):
//   r = sigmoid(gr[t, c]), i = sigmoid(gi[t, c]), a = exp(-rate * r * softplus(lam[c])),  S <- a S + sqrt(1 - a^2) (i u[t, c]),
//   out[t, c] = S * gelu_tanh(y[t, c])  in dtype.
// Tokens run in order; a sequence whose first row stands at position 0 starts from S = 0.  T = rows of the step.  A prompt step (cu_q)
// OVERWRITES gr, gi and y with the decay, the weighted input and the activated branch.
struct StkGatedScanArgs {
  const float* u = nullptr;
  int ldu = 0;
  const float* gr = nullptr;
  const float* gi = nullptr;
  int ldg = 0;
  int block = 0;  // > 0: the gates come in blocks — channel c's logits stand at column (c / block) * 2 * block + c % block of gr and gi
  const float* y = nullptr;
  int ldy = 0;
  const float* lam = nullptr;
  float rate = 8.f;
  float* state = nullptr;
  const int32_t* state_slots = nullptr;
  const int64_t* positions = nullptr;
  const uint32_t* cu_q = nullptr;
  void* out = nullptr;
  int ldo = 0;
  int B = 0, C = 0;
};
void vra_stack_gated_scan(const StkGatedScanArgs& a, int T, int dtype, int64_t stream);
