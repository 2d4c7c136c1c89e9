// stack_model.cpp — see stack_model.h.
#include "stack_model.h"

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <sstream>

#include "../csrc/stack_launch.h"
#include "host_utils.h"
#include "model.h"

namespace vra {

std::unique_ptr<ModelBase> make_model(const vra_model_config& mc, const vra_engine_config& ec, const char* spec, std::string* error) {
  if (mc.arch == VRA_ARCH_STACK) {
    if (!spec || !spec[0]) {
      if (error) *error = "a layer-stack model needs its layer list (vra_engine_create_spec)";
      return nullptr;
    }
    return std::unique_ptr<ModelBase>(new StackModel(mc, ec, spec));
  }
  return std::unique_ptr<ModelBase>(new Model(mc, ec));
}

static int round_up(int v, int m) { return (v + m - 1) / m * m; }

StackModel::StackModel(const vra_model_config& mc, const vra_engine_config& ec, const char* spec) : mc_(mc), ec_(ec) {
  dt_ = mc.dtype == VRA_F32 ? VRA_F32 : VRA_BF16;
  es_ = dt_ == VRA_F32 ? 4 : 2;
  if (mc.dtype != VRA_F32 && mc.dtype != VRA_BF16) spec_error_ = "layer stack: dtype must be bfloat16 or float32";
  else if (ec.tp_world_size > 1) spec_error_ = "layer stack: tensor parallelism is not wired for this model class";
  else if (ec.fp8_kvcache) spec_error_ = "layer stack: the cache keeps the model's element type (no fp8 cache)";
  else parse_spec(spec);
}
StackModel::~StackModel() {
  for (void* p : allocs_) (void)hipFree(p);
}

bool StackModel::parse_spec(const char* spec) {
  std::istringstream in(spec);
  std::string line;
  bool have_stack = false;
  while (std::getline(in, line)) {
    std::istringstream ls(line);
    std::string kind, kv;
    if (!(ls >> kind)) continue;
    std::map<std::string, std::string> f;
    while (ls >> kv) {
      const size_t eq = kv.find('=');
      if (eq == std::string::npos) return spec_error_ = "layer stack spec: field without '=': " + kv, false;
      f[kv.substr(0, eq)] = kv.substr(eq + 1);
    }
    auto num = [&](const char* k, double dflt) { return f.count(k) ? strtod(f[k].c_str(), nullptr) : dflt; };
    if (kind == "stack") {
      have_stack = true;
      width_ = (int)num("width", 0), vocab_ = (int)num("vocab", 0), groups_ = (int)num("groups", 1);
      eps_ = (float)num("eps", 1e-6), residual_mult_ = (float)num("residual_mult", 1.0), logit_scale_ = (float)num("logit_scale", 1.0);
      pos_base_ = num("pos_base", 10000.0);
      auto pick = [&](const char* k, const char* a, const char* b, int* out, const char* c = nullptr) {
        const std::string v = f.count(k) ? f[k] : a;
        if (v != a && v != b && !(c && v == c)) return spec_error_ = std::string("layer stack spec: ") + k + " must be " + a + " or " + b + (c ? std::string(" or ") + c : ""), false;
        *out = v == b ? 1 : (c && v == c ? 2 : 0);
        return true;
      };
      if (!pick("block", "parallel", "sequential", &block_, "sandwich") || !pick("norm", "rms", "dyt", &norm_kind_) || !pick("pos", "sinusoid", "none", &pos_kind_))
        return false;
      norm_offset_ = (float)num("norm_offset", 0.0), embed_scale_ = (float)num("embed_scale", 1.0), embed_norm_ = (int)num("embed_norm", 0);
      pair_buckets_ = (int)num("pair_buckets", 0), pair_mul_prev_ = (int64_t)num("pair_mul_prev", 0), pair_mul_cur_ = (int64_t)num("pair_mul_cur", 0);
      tie_head_ = (int)num("tie_head", 0);
    } else if (kind == "layer") {
      StackLayer L;
      L.heads = (int)num("heads", 0), L.kv_heads = (int)num("kv_heads", L.heads), L.dim = (int)num("dim", 0), L.vdim = (int)num("vdim", L.dim);
      L.scale = (float)num("scale", L.dim > 0 ? 1.0 / sqrt((double)L.dim) : 1.0), L.softcap = (float)num("softcap", 0.0);
      L.temp_coef = (float)num("temp_coef", 0.0), L.temp_every = (int)num("temp_every", 0), L.kv_from = (int)num("kv_from", -1);
      const std::string mix = f.count("mixer") ? f["mixer"] : "attention";
      L.mixer = mix == "latent" ? 1 : (mix == "sigmoid" ? 2 : (mix == "delta" ? 3 : (mix == "retention" ? 4 : (mix == "parallel" ? 5 : (mix == "lightning" ? 6 : 0)))));
      if (mix != "attention" && L.mixer == 0) return spec_error_ = "layer stack spec: unknown mixer " + mix, false;
      L.conv = (int)num("conv", 0), L.rank_a = (int)num("rank_a", 0), L.rank_g = (int)num("rank_g", 0), L.chunk = (int)num("chunk", 0);
      L.qk_norm = (int)num("qk_norm", 0), L.has_bias = (int)num("bias", 0);
      L.rs_factor = num("rs_factor", 0.0), L.rs_low = num("rs_low", 1.0), L.rs_high = num("rs_high", 4.0), L.rs_original = num("rs_original", 0.0);
      L.r_heads = (int)num("r_heads", 0), L.r_dim = (int)num("r_dim", 0), L.r_vdim = (int)num("r_vdim", L.r_dim), L.tau = (float)num("tau", 1.0);
      L.left_scale = (float)num("left_scale", 1.0), L.right_scale = (float)num("right_scale", 1.0);
      if (f.count("decay")) {
        std::istringstream ds(f["decay"]);
        std::string item;
        while (std::getline(ds, item, ',')) L.decay.push_back((float)strtod(item.c_str(), nullptr));
      }
      {
        const std::string rk = f.count("router") ? f["router"] : "sigmoid", ak = f.count("act") ? f["act"] : "clamped";
        if ((rk != "sigmoid" && rk != "softmax" && rk != "softmax_all") || (ak != "clamped" && ak != "silu"))
          return spec_error_ = "layer stack spec: router is sigmoid or softmax or softmax_all, act clamped or silu", false;
        L.router_kind = rk == "softmax" ? 1 : (rk == "softmax_all" ? 2 : 0), L.act_kind = ak == "silu" ? 2 : 0;
        L.n_identity = (int)num("identity", 0), L.n_groups = (int)num("groups", 0), L.keep = (int)num("keep", 0);
      }
      {
        const std::string rt = f.count("right") ? f["right"] : "gla", rl = f.count("rot_layout") ? f["rot_layout"] : "half";
        if ((rt != "gla" && rt != "rglru") || (rl != "half" && rl != "pairs")) return spec_error_ = "layer stack spec: right is gla or rglru, rot_layout half or pairs", false;
        L.right_kind = rt == "rglru", L.rot_layout = rl == "pairs";
        L.lowrank = (int)num("lowrank", 1), L.r_width = (int)num("r_width", 0), L.r_blocks = (int)num("r_blocks", 1);
        L.head_temp = (int)num("head_temp", 0), L.head_gate = (int)num("head_gate", 0), L.branch_norm = (int)num("branch_norm", 0);
        if (L.right_kind == 1) L.conv = (int)num("r_conv", 1);
      }
      L.weights_of = (int)num("weights_of", -1);
      L.rot_dim = (int)num("rot_dim", 0), L.kv_rank = (int)num("kv_rank", 0), L.q_rank = (int)num("q_rank", 0), L.rot_dims = (int)num("rot_dims", L.rot_dim);
      L.sink = (int)num("sink", 0), L.rot_base = num("rot_base", 10000.0), L.yarn_factor = num("yarn_factor", 0.0);
      L.yarn_original = num("yarn_original", 0.0), L.yarn_fast = num("yarn_fast", 32.0), L.yarn_slow = num("yarn_slow", 1.0);
      L.window = (int)num("window", 0), L.keep_first = (int)num("keep_first", 0), L.slope_exp = num("slope_exp", 0.0);
      const std::string mlp = f.count("mlp") ? f["mlp"] : "none";
      L.mlp = mlp == "dense" ? 1 : (mlp == "moe" ? 2 : (mlp == "gated" ? 3 : (mlp == "clamped" ? 4 : 0)));
      if (mlp != "dense" && mlp != "moe" && mlp != "none" && mlp != "gated" && mlp != "clamped") return spec_error_ = "layer stack spec: unknown feed-forward kind " + mlp, false;
      L.ff = (int)num("ff", 0), L.experts = (int)num("experts", 0), L.top = (int)num("top", 1), L.limit = (float)num("limit", 0.0);
      L.shared_ff = (int)num("shared_ff", 0), L.shared_limit = (float)num("shared_limit", 0.0);
      layers_.push_back(L);
    } else {
      return spec_error_ = "layer stack spec: unknown record " + kind, false;
    }
  }
  if (!have_stack || width_ <= 0 || vocab_ <= 0 || layers_.empty()) return spec_error_ = "layer stack spec: width, vocab and at least one layer are needed", false;
  if (groups_ < 1 || width_ % groups_) return spec_error_ = "layer stack spec: the width must split into equal norm groups", false;
  if (width_ != mc_.hidden_size || vocab_ != mc_.vocab_size || (int)layers_.size() != mc_.num_layers)
    return spec_error_ = "layer stack spec: width / vocab / layers differ from the model config", false;
  for (size_t i = 0; i < layers_.size(); i++) {
    StackLayer& L = layers_[i];
    const std::string at = " (layer " + std::to_string(i) + ")";
    if (L.heads <= 0 || L.kv_heads <= 0 || L.heads % L.kv_heads || L.dim <= 0 || L.vdim <= 0 || (L.mixer == 0 && L.vdim > 256))
      return spec_error_ = "layer stack spec: heads must be a multiple of kv_heads, sizes positive, value size at most 256" + at, false;
    if ((L.mixer == 1 || L.mixer == 2) && block_ != 1) return spec_error_ = "layer stack spec: latent and sigmoid mixers run in sequential blocks" + at, false;
    if (L.mixer == 0 && block_ != 0) return spec_error_ = "layer stack spec: the softmax mixer with temperature and cap runs in parallel blocks" + at, false;
    if (L.mixer >= 3 && block_ != 2) return spec_error_ = "layer stack spec: delta, retention and parallel mixers run in sandwich blocks" + at, false;
    if (block_ == 2 && (L.mixer < 3 || (L.mlp != 0 && L.mlp != 2 && L.mlp != 4) || L.weights_of >= 0))
      return spec_error_ = "layer stack spec: sandwich blocks hold delta, retention, lightning or parallel mixers and a mixture of experts, a clamped dense feed-forward or none" + at, false;
    if (L.mlp == 4 && block_ != 2) return spec_error_ = "layer stack spec: the clamped dense feed-forward belongs to sandwich blocks" + at, false;
    if (L.mixer == 3 && (L.conv < 1 || (L.lowrank && (L.rank_a < 1 || L.rank_g < 1)) || L.dim > 256)) return spec_error_ = "layer stack spec: the delta mixer needs conv >= 1, rank_a, rank_g, dim <= 256" + at, false;
    if (L.mixer == 6 && ((int)L.decay.size() != L.heads || L.kv_heads != L.heads || L.dim > 256))
      return spec_error_ = "layer stack spec: lightning needs one decay per head, kv_heads = heads, dim <= 256" + at, false;
    if (L.mixer == 5 && L.right_kind == 1 &&
        (L.r_width <= 0 || L.r_blocks < 1 || L.r_width % L.r_blocks || L.conv < 1 || L.rot_dims < 0 || L.rot_dims > L.dim || L.rot_dims % 2 || L.chunk < 0 ||
         L.window < 0 || L.vdim > 256 || (L.yarn_factor > 0.0 && (L.yarn_original <= 0.0 || L.yarn_fast <= 0.0 || L.yarn_slow <= 0.0))))
      return spec_error_ = "layer stack spec: the parallel mixer with a gated recurrence needs r_width in r_blocks equal blocks, r_conv >= 1, an even rot_dims <= dim, vdim <= 256" + at, false;
    if ((L.window > 0 || L.head_temp || L.head_gate || L.rot_layout || L.branch_norm) && L.mixer != 5 && L.mixer != 2)
      return spec_error_ = "layer stack spec: window, head_temp, head_gate, rot_layout and branch_norm belong to the parallel mixer" + at, false;
    if (L.router_kind == 2 && (L.n_identity < 0 ||
                               (L.n_groups > 1 && ((L.experts + L.n_identity) % L.n_groups || L.keep < 1 || L.keep > L.n_groups))))
      return spec_error_ = "layer stack spec: router groups must divide experts + identity, 1 <= keep <= groups" + at, false;
    if (L.mixer == 4 && ((int)L.decay.size() != L.heads || L.kv_heads != L.heads || L.rot_dims < 0 || L.rot_dims > L.dim || L.rot_dims % 2 || L.dim > 256))
      return spec_error_ = "layer stack spec: retention needs one decay per head, kv_heads = heads, an even rot_dims <= dim <= 256" + at, false;
    if (L.mixer == 5 && L.right_kind == 0 && (L.r_heads <= 0 || L.r_dim <= 0 || L.r_dim > 256 || L.r_vdim <= 0 || L.rank_a < 1 || !(L.tau > 0.f) || L.rot_dims < 0 || L.rot_dims > L.dim || L.rot_dims % 2 ||
                         L.chunk < 0 || L.vdim > 256 || (L.rs_factor > 0.0 && (L.rs_original <= 0.0 || L.rs_high <= L.rs_low))))
      return spec_error_ = "layer stack spec: the parallel mixer needs r_heads, r_dim <= 256, r_vdim, rank_a, tau > 0, an even rot_dims <= dim, vdim <= 256" + at, false;
    if (L.router_kind >= 1 && (block_ != 2 || L.shared_ff > 0)) return spec_error_ = "layer stack spec: the softmax router belongs to sandwich blocks and has no shared expert" + at, false;
    if (L.mixer != 0 && L.kv_from >= 0) return spec_error_ = "layer stack spec: kv_from belongs to the softmax mixer" + at, false;
    if (L.mixer == 1 && (L.kv_rank <= 0 || L.q_rank <= 0 || L.rot_dim < 0 || L.kv_rank > 256 || L.rot_dims < 0 || L.rot_dims > L.rot_dim || L.rot_dims % 2 ||
                         (L.yarn_factor > 0.0 && (L.yarn_original <= 0.0 || L.yarn_fast <= 0.0 || L.yarn_slow <= 0.0))))
      return spec_error_ = "layer stack spec: latent attention needs q_rank, 0 < kv_rank <= 256, an even rot_dims <= rot_dim" + at, false;
    if ((L.mlp == 3) != (block_ == 1) && L.mlp != 0) return spec_error_ = "layer stack spec: the gated feed-forward belongs to sequential blocks, the others to parallel ones" + at, false;
    if (L.weights_of >= 0) {
      int root = L.weights_of;  // (a chain of references ends at a layer with tensors of its own)
      for (size_t hop = 0; hop < layers_.size() && root >= 0 && root < (int)layers_.size() && layers_[root].weights_of >= 0; hop++) root = layers_[root].weights_of;
      if (root < 0 || root >= (int)layers_.size() || root == (int)i || layers_[root].weights_of >= 0)
        return spec_error_ = "layer stack spec: weights_of must name another layer with tensors of its own" + at, false;
      L.weights_of = root;
      const StackLayer& S = layers_[root];
      if (S.mixer != L.mixer || S.heads != L.heads || S.kv_heads != L.kv_heads || S.dim != L.dim || S.vdim != L.vdim || S.rot_dim != L.rot_dim ||
          S.kv_rank != L.kv_rank || S.q_rank != L.q_rank || S.mlp != L.mlp || S.ff != L.ff || S.kv_from >= 0 || L.kv_from >= 0)
        return spec_error_ = "layer stack spec: a layer that shares weights has the shapes of the layer it names" + at, false;
    }
    if (!L.has_cache()) {
      if (L.kv_from >= 0) return spec_error_ = "layer stack spec: kv_from belongs to the softmax mixer" + at, false;
    } else if (L.kv_from >= 0) {
      if (L.kv_from >= (int)i) return spec_error_ = "layer stack spec: kv_from must name an earlier layer" + at, false;
      const StackLayer& S = layers_[L.kv_from];
      if (!S.owns_cache || S.kv_heads != L.kv_heads || S.dim != L.dim || S.vdim != L.vdim)
        return spec_error_ = "layer stack spec: kv_from must name a layer with projections of its own and equal key / value shapes" + at, false;
      L.cache = S.cache;
    } else {
      L.owns_cache = true;
      L.cache = (int)cache_layer_.size();
      cache_layer_.push_back((int)i);
    }
    if (!L.has_cache()) L.owns_cache = false;  // (their past lives in the state slot; the cache entry keeps the tables uniform and holds no bytes)
    if (L.mlp == 1 && L.ff <= 0) return spec_error_ = "layer stack spec: dense feed-forward without ff" + at, false;
    if (L.mlp == 2 && (L.ff <= 0 || L.experts <= 0 || L.top < 1 || L.top > L.experts + L.n_identity))
      return spec_error_ = "layer stack spec: mixture of experts needs ff, experts and 1 <= top <= experts" + at, false;
    if (L.mlp == 4 && L.ff <= 0) return spec_error_ = "layer stack spec: clamped feed-forward without ff" + at, false;
    if (L.mlp == 3 || L.mlp == 4) {
      if (L.ff <= 0) return spec_error_ = "layer stack spec: gated feed-forward without ff" + at, false;
      L.shared_ff = L.ff;  // (laid out like a shared expert: gate / up rows interleaved, one weight set for all rows)
    }
    L.ffp = round_up(L.ff, 16), L.sffp = round_up(L.shared_ff, 16);
  }
  return true;
}

void* StackModel::dalloc(size_t bytes) {
  void* p = nullptr;
  if (hipMalloc(&p, bytes ? bytes : 16) != hipSuccess) {
    error = "hipMalloc failed for " + std::to_string(bytes) + " bytes";
    return nullptr;
  }
  allocs_.push_back(p);
  return p;
}
void* StackModel::upload(const void* host, size_t bytes) {
  void* p = dalloc(bytes);
  if (p && hipMemcpy(p, host, bytes, hipMemcpyHostToDevice) != hipSuccess) {
    error = "hipMemcpy failed";
    return nullptr;
  }
  return p;
}

// ---------------------------------------------------------------------------------------------
// weights: tensors are staged on the host under their checkpoint names and laid out for the kernels in finalize_weights()
// ---------------------------------------------------------------------------------------------
bool StackModel::load_tensor(const std::string& name, const void* host, const int64_t* shape, int ndim, int elem_bytes) {
  if (!spec_error_.empty()) return error = spec_error_, false;
  if (finalized_) return error = "load_tensor after finalize", false;
  if (elem_bytes != 2 && elem_bytes != 4) return error = "tensor " + name + ": 2- or 4-byte elements expected", false;
  HostTensor t;
  size_t n = 1;
  for (int i = 0; i < ndim; i++) t.shape.push_back(shape[i]), n *= (size_t)shape[i];
  t.elem_bytes = elem_bytes;
  t.data.assign((const uint8_t*)host, (const uint8_t*)host + n * elem_bytes);
  staged_[name] = std::move(t);
  return true;
}

bool StackModel::need(const std::string& name, int64_t d0, int64_t d1, const HostTensor** out) {
  auto it = staged_.find(name);
  if (it == staged_.end()) return error = "missing tensor: " + name, false;
  const HostTensor& t = it->second;
  int64_t n = 1;
  for (int64_t d : t.shape) n *= d;
  const bool ok = d1 < 0 ? n == d0 : (t.shape.size() == 2 && t.shape[0] == d0 && t.shape[1] == d1);
  if (!ok) return error = "tensor " + name + ": shape differs from the config", false;
  *out = &t;
  return true;
}
// small f32 tensors (norm weights, activation coefficients) whatever the checkpoint's element type
float* StackModel::upload_f32(const HostTensor& t) {
  const size_t n = t.data.size() / t.elem_bytes;
  std::vector<float> f(n);
  for (size_t i = 0; i < n; i++) {
    if (t.elem_bytes == 4) memcpy(&f[i], t.data.data() + i * 4, 4);
    else {
      uint16_t b;
      memcpy(&b, t.data.data() + i * 2, 2);
      const uint32_t u = (uint32_t)b << 16;
      memcpy(&f[i], &u, 4);
    }
  }
  weight_bytes_ += n * 4;
  return (float*)upload(f.data(), n * 4);
}

float* StackModel::upload_floats(const std::vector<float>& v) {
  weight_bytes_ += v.size() * 4;
  return (float*)upload(v.data(), std::max<size_t>(v.size(), 1) * 4);
}

bool StackModel::finalize_weights() {
  if (finalized_) return true;
  if (!spec_error_.empty()) return error = spec_error_, false;
  const int W = width_;
  const size_t es = es_;
  auto matrix = [&](const HostTensor* t) -> bool {
    if ((size_t)t->elem_bytes != es) return error = "matrix tensors must come in the model's element type", false;
    return true;
  };
  auto up_mat = [&](const std::string& name, int64_t r, int64_t c, void** dst) {
    const HostTensor* t;
    if (!need(name, r, c, &t) || !matrix(t)) return false;
    weight_bytes_ += t->data.size();
    return (*dst = upload(t->data.data(), t->data.size())) != nullptr;
  };
  auto up_vec = [&](const std::string& name, int64_t n, float** dst) {
    const HostTensor* t;
    if (!need(name, n, -1, &t)) return false;
    return (*dst = upload_f32(*t)) != nullptr;
  };
  // gate / up rows of one expert -> [2 * fp][W], blocks of 16 rows alternating gate / up, zero rows beyond f
  auto interleave = [&](const HostTensor* g, const HostTensor* u, int f, int fp, uint8_t* dst) {
    memset(dst, 0, (size_t)2 * fp * W * es);
    for (int r = 0; r < f; r++) {
      const size_t blk = r / 16, i = r % 16;
      memcpy(dst + ((2 * blk) * 16 + i) * W * es, g->data.data() + (size_t)r * W * es, W * es);
      memcpy(dst + ((2 * blk + 1) * 16 + i) * W * es, u->data.data() + (size_t)r * W * es, W * es);
    }
  };
  // down [W][f] -> [W][fp], zero columns beyond f
  auto pad_cols = [&](const HostTensor* d, int f, int fp, uint8_t* dst) {
    memset(dst, 0, (size_t)W * fp * es);
    for (int r = 0; r < W; r++) memcpy(dst + (size_t)r * fp * es, d->data.data() + (size_t)r * f * es, (size_t)f * es);
  };
  auto up_scalar = [&](const std::string& name, float* dst) {
    const HostTensor* t;
    if (!need(name, 1, -1, &t)) return false;
    float* d = upload_f32(*t);  // (kept on the device too: synthetic and loaded weights take one path)
    if (!d) return false;
    return hipMemcpy(dst, d, 4, hipMemcpyDeviceToHost) == hipSuccess;
  };
  auto up_norm = [&](const std::string& name, float** w, float** b, float* alpha) {
    if (!up_vec(name, W, w)) return false;
    if (norm_kind_ == 1 && (!up_vec(name + ".b", W, b) || !up_scalar(name + ".alpha", alpha))) return false;
    return true;
  };
  // rows of several matrices of equal width under one another -> one device matrix
  auto up_rows = [&](const std::vector<const HostTensor*>& parts, void** dst) {
    std::vector<uint8_t> cat;
    for (const HostTensor* t : parts) cat.insert(cat.end(), t->data.begin(), t->data.end());
    weight_bytes_ += cat.size();
    return (*dst = upload(cat.data(), cat.size())) != nullptr;
  };
  auto f32_of = [&](const HostTensor& t, std::vector<float>* out) {
    const size_t n = t.data.size() / t.elem_bytes;
    for (size_t i = 0; i < n; i++) {
      float v;
      if (t.elem_bytes == 4) memcpy(&v, t.data.data() + i * 4, 4);
      else {
        uint16_t b16;
        memcpy(&b16, t.data.data() + i * 2, 2);
        const uint32_t u = (uint32_t)b16 << 16;
        memcpy(&v, &u, 4);
      }
      out->push_back(v);
    }
  };
  // a norm weight stored around zero: the offset is added once, here
  auto up_norm_off = [&](const std::string& name, int64_t n, float** w) {
    const HostTensor* t;
    if (!need(name, n, -1, &t)) return false;
    std::vector<float> v;
    f32_of(*t, &v);
    for (float& e : v) e += norm_offset_;
    return (*w = upload_floats(v)) != nullptr;
  };
  // the shape a staged tensor came with (sizes the config does not carry: the ranks of low-rank projections)
  auto rows_of = [&](const std::string& name, int64_t cols) -> int64_t {
    auto it = staged_.find(name);
    if (it == staged_.end() || it->second.shape.size() != 2 || it->second.shape[1] != cols) return -1;
    return it->second.shape[0];
  };
  if (!up_mat("embed", vocab_, W, &embed_)) return false;
  if (tie_head_) head_ = embed_;
  else if (!up_mat("head", vocab_, W, &head_)) return false;
  if (block_ == 2 && norm_kind_ == 1) {
    if (!up_norm("final.norm", &final_norm_, &final_b_, &final_alpha_)) return false;
  } else if (block_ == 2) {
    if (!up_norm_off("final.norm", W, &final_norm_)) return false;
    if (embed_norm_ && !up_norm_off("embed.norm", W, &embed_norm_w_)) return false;
    if (pair_buckets_ > 0 && !up_mat("bigram", (int64_t)pair_buckets_ + 1, W, &pair_table_)) return false;
  } else if (!up_norm("final.norm", &final_norm_, &final_b_, &final_alpha_)) {
    return false;
  }
  for (size_t li = 0; li < layers_.size(); li++) {
    StackLayer& L = layers_[li];
    if (L.weights_of >= 0) continue;
    const std::string p = "l" + std::to_string(li) + ".";
    if (block_ == 2 && norm_kind_ == 1) {
      if (!up_norm(p + "norm1", &L.norm_w, &L.norm_b, &L.norm_alpha) || !up_norm(p + "norm1b", &L.post1_w, &L.post1_b, &L.post1_alpha)) return false;
      if (L.mlp != 0 && (!up_norm(p + "norm2", &L.norm2_w, &L.norm2_b, &L.norm2_alpha) || !up_norm(p + "norm2b", &L.post2_w, &L.post2_b, &L.post2_alpha))) return false;
    } else if (block_ == 2) {
      if (!up_norm_off(p + "norm1", W, &L.norm_w) || !up_norm_off(p + "norm1b", W, &L.post1_w)) return false;
      if (L.mlp != 0 && (!up_norm_off(p + "norm2", W, &L.norm2_w) || !up_norm_off(p + "norm2b", W, &L.post2_w))) return false;
    } else {
      if (!up_norm(p + "norm1", &L.norm_w, &L.norm_b, &L.norm_alpha)) return false;
      if (block_ == 1 && L.mlp != 0 && !up_norm(p + "norm2", &L.norm2_w, &L.norm2_b, &L.norm2_alpha)) return false;
    }
    // two low-rank second stages side by side: [na + nb, ra + rb] with zeros off the diagonal blocks, so that one product serves both
    auto block_diag = [&](const HostTensor* a2, int na, int ra, const HostTensor* b2, int nb, int rb, void** dst) {
      const int R = ra + rb;
      std::vector<uint8_t> m((size_t)(na + nb) * R * es, 0);
      for (int r = 0; r < na; r++) memcpy(m.data() + (size_t)r * R * es, a2->data.data() + (size_t)r * ra * es, (size_t)ra * es);
      for (int r = 0; r < nb; r++) memcpy(m.data() + ((size_t)(na + r) * R + ra) * es, b2->data.data() + (size_t)r * rb * es, (size_t)rb * es);
      weight_bytes_ += m.size();
      return (*dst = upload(m.data(), m.size())) != nullptr;
    };
    auto conv_taps = [&](const std::string& name) {  // the taps of a short convolution are the columns of its tensor
      auto it = staged_.find(name);
      if (it != staged_.end() && it->second.shape.size() == 2 && it->second.shape[1] >= 1) L.conv = (int)it->second.shape[1];
    };
    if (L.mixer == 3 && !L.lowrank) {
      // gated delta rule with full-rank side projections: q | k | v | write strengths | decays | gate in one matrix
      const int H = L.heads, nk = L.nk(), nv = H * L.vdim, C = L.conv_channels();
      conv_taps(p + "mix.q.conv");
      const HostTensor *q, *k, *v, *bw, *aw, *gw, *cq, *ck, *cv, *al;
      if (!need(p + "mix.q", nk, W, &q) || !need(p + "mix.k", nk, W, &k) || !need(p + "mix.v", nv, W, &v) || !need(p + "mix.b", H, W, &bw) ||
          !need(p + "mix.a", H, W, &aw) || !need(p + "mix.g", nv, W, &gw) || !matrix(q) || !matrix(k) || !matrix(v) || !matrix(bw) || !matrix(aw) || !matrix(gw))
        return false;
      if (!up_rows({q, k, v, bw, aw, gw}, &L.qkv)) return false;
      if (!need(p + "mix.q.conv", nk, L.conv, &cq) || !need(p + "mix.k.conv", nk, L.conv, &ck) || !need(p + "mix.v.conv", nv, L.conv, &cv)) return false;
      std::vector<float> cw;
      f32_of(*cq, &cw), f32_of(*ck, &cw), f32_of(*cv, &cw);
      if ((int)cw.size() != C * L.conv || !(L.conv_w = upload_floats(cw))) return false;
      if (!need(p + "mix.A_log", H, -1, &al)) return false;
      std::vector<float> rate;
      f32_of(*al, &rate);
      for (float& r : rate) r = expf(r);
      if (!(L.rate = upload_floats(rate)) || !up_vec(p + "mix.dt_bias", H, &L.dt_bias) || !up_vec(p + "mix.norm", L.vdim, &L.out_norm_w)) return false;
      if (!up_mat(p + "mix.o", W, nv, &L.o)) return false;
    } else if (L.mixer == 6) {
      const int H = L.heads;
      const HostTensor *q, *k, *v, *g;
      if (!need(p + "mix.q", (int64_t)H * L.dim, W, &q) || !need(p + "mix.k", (int64_t)H * L.dim, W, &k) || !need(p + "mix.v", (int64_t)H * L.vdim, W, &v) ||
          !need(p + "mix.g", (int64_t)H * L.vdim, W, &g) || !matrix(q) || !matrix(k) || !matrix(v) || !matrix(g))
        return false;
      if (!up_rows({q, k, v, g}, &L.qkv) || !(L.head_decay = upload_floats(L.decay)) || !up_mat(p + "mix.o", W, H * L.vdim, &L.o) ||
          !up_vec(p + "mix.norm", (int64_t)H * L.vdim, &L.out_norm_w))
        return false;
    } else if (L.mixer == 5 && L.right_kind == 1) {
      const std::string pl = p + "mix.left.", pr = p + "mix.right.";
      const int H = L.heads, Wr = L.r_width, nb = L.r_blocks, bw = Wr / nb;
      conv_taps(pr + "conv");
      const HostTensor *q, *k, *v, *g = nullptr, *y, *xr, *cw, *ra, *ri, *rab, *rib;
      if (!need(pl + "q", L.nq(), W, &q) || !need(pl + "k", L.nk(), W, &k) || !need(pl + "v", L.nv(), W, &v) || !need(pr + "y", Wr, W, &y) ||
          !need(pr + "x", Wr, W, &xr) || !matrix(q) || !matrix(k) || !matrix(v) || !matrix(y) || !matrix(xr))
        return false;
      if (L.head_gate && (!need(pl + "g", H, W, &g) || !matrix(g))) return false;
      std::vector<const HostTensor*> parts{q, k, v};
      if (g) parts.push_back(g);
      parts.push_back(y), parts.push_back(xr);
      if (!up_rows(parts, &L.qkv)) return false;
      std::vector<float> bias;
      if (L.has_bias) {
        const HostTensor *qb, *kb, *vb;
        if (!need(pl + "q.b", L.nq(), -1, &qb) || !need(pl + "k.b", L.nk(), -1, &kb) || !need(pl + "v.b", L.nv(), -1, &vb)) return false;
        f32_of(*qb, &bias), f32_of(*kb, &bias), f32_of(*vb, &bias);
      }
      bias.resize(L.nq() + L.nk() + L.nv() + (g ? H : 0), 0.f);
      {
        const HostTensor *yb, *xb;
        if (!need(pr + "y.b", Wr, -1, &yb) || !need(pr + "x.b", Wr, -1, &xb)) return false;
        f32_of(*yb, &bias), f32_of(*xb, &bias);
      }
      if ((int)bias.size() != L.nqkv() || !(L.qkv_bias = upload_floats(bias))) return false;
      if (L.qk_norm && (!up_vec(pl + "q.norm", L.dim, &L.qn_w) || !up_vec(pl + "k.norm", L.dim, &L.kn_w))) return false;
      if (L.head_temp && !up_vec(pl + "temp", H, &L.temp_w)) return false;
      if (L.sink && !up_vec(pl + "sink", H, &L.sink_w)) return false;
      if (L.branch_norm && (!up_vec(pl + "out", W, &L.left_out_w) || !up_vec(pr + "out", W, &L.right_out_w))) return false;
      if (!up_mat(pl + "o", W, H * L.vdim, &L.o) || !up_mat(pr + "o", W, Wr, &L.r_o)) return false;
      if (!need(pr + "conv", Wr, L.conv, &cw) || !(L.conv_w = upload_f32(*cw)) || !up_vec(pr + "conv.b", Wr, &L.conv_b) || !up_vec(pr + "lam", Wr, &L.lam)) return false;
      // the gates of the recurrence are computed in f32: per block the rows of the recurrence gate, then those of the input gate
      if (!need(pr + "ra", (int64_t)nb * bw * bw, -1, &ra) || !need(pr + "ri", (int64_t)nb * bw * bw, -1, &ri) || !need(pr + "ra.b", Wr, -1, &rab) ||
          !need(pr + "ri.b", Wr, -1, &rib))
        return false;
      std::vector<float> fa, fi, ba, bi, gw, gb;
      f32_of(*ra, &fa), f32_of(*ri, &fi), f32_of(*rab, &ba), f32_of(*rib, &bi);
      for (int b = 0; b < nb; b++) {
        gw.insert(gw.end(), fa.begin() + (size_t)b * bw * bw, fa.begin() + (size_t)(b + 1) * bw * bw);
        gw.insert(gw.end(), fi.begin() + (size_t)b * bw * bw, fi.begin() + (size_t)(b + 1) * bw * bw);
        gb.insert(gb.end(), ba.begin() + (size_t)b * bw, ba.begin() + (size_t)(b + 1) * bw);
        gb.insert(gb.end(), bi.begin() + (size_t)b * bw, bi.begin() + (size_t)(b + 1) * bw);
      }
      if (!(L.gates_w = upload_floats(gw)) || !(L.gates_b = upload_floats(gb))) return false;
      rotary_table(L);
      if (!L.freq_hi || !L.freq_lo) return false;
    } else if (L.mixer == 3) {
      // gated delta rule: q | k | v | write strengths in one matrix; the first stages of the decay and gate projections in a second one,
      // their second stages block-diagonal in a third
      const int H = L.heads, nk = L.nk(), nv = H * L.vdim, C = L.conv_channels();
      const int64_t ra = rows_of(p + "mix.a1", W), rg = rows_of(p + "mix.g1", W);
      if (ra < 1 || rg < 1) return error = "tensor " + p + "mix.a1 / g1: missing or of another width", false;
      L.rank_a = (int)ra, L.rank_g = (int)rg;
      {  // the taps of the short convolutions are the columns of their tensors
        auto it = staged_.find(p + "mix.q.conv");
        if (it != staged_.end() && it->second.shape.size() == 2 && it->second.shape[1] >= 1) L.conv = (int)it->second.shape[1];
      }
      const HostTensor *q, *k, *v, *bw, *a1, *g1, *a2, *g2, *cq, *ck, *cv, *al;
      if (!need(p + "mix.q", nk, W, &q) || !need(p + "mix.k", nk, W, &k) || !need(p + "mix.v", nv, W, &v) || !need(p + "mix.b", H, W, &bw) ||
          !need(p + "mix.a1", ra, W, &a1) || !need(p + "mix.g1", rg, W, &g1) || !need(p + "mix.a2", (int64_t)H * L.dim, ra, &a2) ||
          !need(p + "mix.g2", nv, rg, &g2) || !matrix(q) || !matrix(k) || !matrix(v) || !matrix(bw) || !matrix(a1) || !matrix(g1) || !matrix(a2) || !matrix(g2))
        return false;
      if (!up_rows({q, k, v, bw}, &L.qkv) || !up_rows({a1, g1}, &L.lr1) || !block_diag(a2, H * L.dim, (int)ra, g2, nv, (int)rg, &L.lr2)) return false;
      if (!need(p + "mix.q.conv", nk, L.conv, &cq) || !need(p + "mix.k.conv", nk, L.conv, &ck) || !need(p + "mix.v.conv", nv, L.conv, &cv)) return false;
      std::vector<float> cw;
      f32_of(*cq, &cw), f32_of(*ck, &cw), f32_of(*cv, &cw);
      if ((int)cw.size() != C * L.conv || !(L.conv_w = upload_floats(cw))) return false;
      if (!need(p + "mix.A_log", H, -1, &al)) return false;
      std::vector<float> rate;
      f32_of(*al, &rate);
      for (float& r : rate) r = expf(r);
      if (!(L.rate = upload_floats(rate)) || !up_vec(p + "mix.dt_bias", (int64_t)H * L.dim, &L.dt_bias) || !up_vec(p + "mix.norm", L.vdim, &L.out_norm_w)) return false;
      if (!up_mat(p + "mix.o", W, nv, &L.o)) return false;
    } else if (L.mixer == 4) {
      const int H = L.heads;
      const HostTensor *q, *k, *v, *g;
      if (!need(p + "mix.q", (int64_t)H * L.dim, W, &q) || !need(p + "mix.k", (int64_t)H * L.dim, W, &k) || !need(p + "mix.v", (int64_t)H * L.vdim, W, &v) ||
          !need(p + "mix.g", (int64_t)H * L.vdim, W, &g) || !matrix(q) || !matrix(k) || !matrix(v) || !matrix(g))
        return false;
      if (!up_rows({q, k, v, g}, &L.qkv) || !(L.head_decay = upload_floats(L.decay)) || !up_mat(p + "mix.o", W, H * L.vdim, &L.o)) return false;
      rotary_table(L);
      if (!L.freq_hi || !L.freq_lo) return false;
    } else if (L.mixer == 5) {
      const std::string pl = p + "mix.left.", pr = p + "mix.right.";
      const int rq = L.r_heads * L.r_dim, rv = L.r_heads * L.r_vdim;
      const int64_t ra = rows_of(pr + "a1", W);
      if (ra < 1) return error = "tensor " + pr + "a1: missing or of another width", false;
      L.rank_a = (int)ra;
      const HostTensor *q, *k, *v, *q2, *k2, *v2, *g2, *a1;
      if (!need(pl + "q", L.nq(), W, &q) || !need(pl + "k", L.nk(), W, &k) || !need(pl + "v", L.nv(), W, &v) || !need(pr + "q", rq, W, &q2) ||
          !need(pr + "k", rq, W, &k2) || !need(pr + "v", rv, W, &v2) || !need(pr + "g", rv, W, &g2) || !need(pr + "a1", ra, W, &a1) || !matrix(q) || !matrix(k) ||
          !matrix(v) || !matrix(q2) || !matrix(k2) || !matrix(v2) || !matrix(g2) || !matrix(a1))
        return false;
      if (!up_rows({q, k, v, q2, k2, v2, g2}, &L.qkv) || !up_rows({a1}, &L.lr1)) return false;
      std::vector<float> bias;
      if (L.has_bias) {
        const HostTensor *qb, *kb, *vb;
        if (!need(pl + "q.b", L.nq(), -1, &qb) || !need(pl + "k.b", L.nk(), -1, &kb) || !need(pl + "v.b", L.nv(), -1, &vb)) return false;
        f32_of(*qb, &bias), f32_of(*kb, &bias), f32_of(*vb, &bias);
        bias.resize(L.nqkv(), 0.f);
        if (!(L.qkv_bias = upload_floats(bias))) return false;
      }
      if (L.qk_norm && (!up_vec(pl + "q.norm", L.dim, &L.qn_w) || !up_vec(pl + "k.norm", L.dim, &L.kn_w))) return false;
      if (!up_mat(pl + "o", W, L.heads * L.vdim, &L.o) || !up_mat(pr + "o", W, rv, &L.r_o) || !up_mat(pr + "a2", rq, ra, &L.lr2) ||
          !up_vec(pr + "a2.b", rq, &L.lr2_bias) || !up_vec(pr + "norm", L.r_vdim, &L.out_norm_w))
        return false;
      rotary_table(L);
      if (!L.freq_hi || !L.freq_lo) return false;
    } else if (L.mixer == 0) {  // q (| k | v) in one matrix: one launch projects them all
      const HostTensor *q, *k = nullptr, *v = nullptr;
      if (!need(p + "mix.q", L.nq(), W, &q) || !matrix(q)) return false;
      if (L.owns_cache && (!need(p + "mix.k", L.nk(), W, &k) || !need(p + "mix.v", L.nv(), W, &v) || !matrix(k) || !matrix(v))) return false;
      std::vector<const HostTensor*> parts{q};
      if (k) parts.push_back(k), parts.push_back(v);
      if (!up_rows(parts, &L.qkv)) return false;
    } else if (L.mixer == 1) {
      // the two down-projections in one matrix [q latent | kv latent | rotated key part]; W_uk per head transposed, so that a query is
      // carried into the latent's space (q_h . (W_uk_h c) = (W_uk_h^T q_h) . c) and the cache needs the latent alone
      const HostTensor *dq, *dkv, *uk;
      const int H = L.heads, qd = L.dim + L.rot_dim;
      if (!need(p + "mix.dq", L.q_rank, W, &dq) || !need(p + "mix.dkv", L.kv_rank + L.rot_dim, W, &dkv) || !matrix(dq) || !matrix(dkv)) return false;
      if (!up_rows({dq, dkv}, &L.qkv)) return false;
      if (!up_vec(p + "mix.dq.norm", L.q_rank, &L.qn_w) || !up_vec(p + "mix.dkv.norm", L.kv_rank, &L.kn_w)) return false;
      if (!up_mat(p + "mix.uq", (int64_t)H * qd, L.q_rank, &L.uq) || !up_mat(p + "mix.uv", (int64_t)H * L.vdim, L.kv_rank, &L.uv)) return false;
      if (!need(p + "mix.uk", (int64_t)H * L.dim, L.kv_rank, &uk) || !matrix(uk)) return false;
      std::vector<uint8_t> tr(uk->data.size());
      for (int h = 0; h < H; h++)
        for (int d = 0; d < L.dim; d++)
          for (int r = 0; r < L.kv_rank; r++)
            memcpy(tr.data() + (((size_t)h * L.kv_rank + r) * L.dim + d) * es, uk->data.data() + (((size_t)h * L.dim + d) * L.kv_rank + r) * es, es);
      weight_bytes_ += tr.size();
      if (!(L.ukt = upload(tr.data(), tr.size()))) return false;
      if (L.sink && !up_vec(p + "mix.sink", H, &L.sink_w)) return false;
      // rotary frequencies in f64, kept as hi + lo f32 pairs
      L.rot_pairs = L.rot_dims / 2;
      std::vector<float> fh(std::max(L.rot_pairs, 1)), fl(std::max(L.rot_pairs, 1));
      const double dims = (double)L.rot_dims, lnb = log(L.rot_base);
      double lo = 0.0, hi = 0.0;
      L.rot_mag = 1.f;
      if (L.yarn_factor > 0.0) {
        auto turn_dim = [&](double turns) { return dims * log(L.yarn_original / (2.0 * M_PI * turns)) / (2.0 * lnb); };
        lo = std::max(floor(turn_dim(L.yarn_fast)), 0.0), hi = std::min(ceil(turn_dim(L.yarn_slow)), dims - 1.0);
        L.rot_mag = (float)(0.1 * log(L.yarn_factor) + 1.0);
      }
      for (int i = 0; i < L.rot_pairs; i++) {
        double fr = pow(L.rot_base, -2.0 * (double)i / dims);
        if (L.yarn_factor > 0.0) {
          const double ramp = std::min(std::max(((double)i - lo) / std::max(hi - lo, 0.001), 0.0), 1.0);
          fr = fr / L.yarn_factor * ramp + fr * (1.0 - ramp);
        }
        fh[i] = (float)fr, fl[i] = (float)(fr - (double)fh[i]);
      }
      if (!(L.freq_hi = upload_floats(fh)) || !(L.freq_lo = upload_floats(fl))) return false;
    } else {
      // q | k | v | output gate in one matrix, the biases of q, k, v as one f32 row (zeros under the gate)
      const HostTensor *q, *k, *v, *g, *qb, *kb, *vb, *tk;
      const int H = L.heads, ng = H * L.vdim;
      if (!need(p + "mix.q", L.nq(), W, &q) || !need(p + "mix.k", L.nk(), W, &k) || !need(p + "mix.v", L.nv(), W, &v) || !need(p + "mix.g", ng, W, &g) ||
          !matrix(q) || !matrix(k) || !matrix(v) || !matrix(g))
        return false;
      if (!up_rows({q, k, v, g}, &L.qkv)) return false;
      if (!need(p + "mix.q.b", L.nq(), -1, &qb) || !need(p + "mix.k.b", L.nk(), -1, &kb) || !need(p + "mix.v.b", L.nv(), -1, &vb)) return false;
      std::vector<float> bias;
      f32_of(*qb, &bias), f32_of(*kb, &bias), f32_of(*vb, &bias);
      bias.resize(bias.size() + ng, 0.f);
      if (!(L.qkv_bias = upload_floats(bias))) return false;
      if (!up_vec(p + "mix.q.norm", L.nq(), &L.qn_w) || !up_vec(p + "mix.k.norm", L.nk(), &L.kn_w) || !up_vec(p + "mix.pb", H, &L.head_bias)) return false;
      if (!need(p + "mix.talk", H, H, &tk) || !(L.talk = upload_f32(*tk))) return false;
      if (L.slope_exp != 0.0) {
        std::vector<float> sl(H);
        for (int h = 0; h < H; h++) sl[h] = (float)pow(2.0, -L.slope_exp * (double)(h + 1) / (double)H);
        if (!(L.slopes = upload_floats(sl))) return false;
      }
    }
    if (L.mixer < 3 && !up_mat(p + "mix.o", W, L.heads * L.vdim, &L.o)) return false;
    if (L.mlp == 1) {
      if (!up_mat(p + "mlp.up", L.ff, W, &L.up) || !up_mat(p + "mlp.down", W, L.ff, &L.down) || !up_vec(p + "mlp.act", 4, &L.act)) return false;
    } else if (L.mlp == 3 || L.mlp == 4) {
      const HostTensor *g, *u, *d;
      if (!need(p + "mlp.gate", L.ff, W, &g) || !need(p + "mlp.up", L.ff, W, &u) || !need(p + "mlp.down", W, L.ff, &d) || !matrix(g) || !matrix(u) || !matrix(d))
        return false;
      std::vector<uint8_t> sgu((size_t)2 * L.sffp * W * es), sdn((size_t)W * L.sffp * es);
      interleave(g, u, L.ff, L.sffp, sgu.data());
      pad_cols(d, L.ff, L.sffp, sdn.data());
      weight_bytes_ += sgu.size() + sdn.size();
      if (!(L.s_gu = upload(sgu.data(), sgu.size())) || !(L.s_down = upload(sdn.data(), sdn.size()))) return false;
    } else if (L.mlp == 2) {
      const HostTensor *r, *sg = nullptr;
      if (!need(p + "mlp.router", L.experts + L.n_identity, W, &r) || !matrix(r)) return false;
      if (L.shared_ff > 0 && (!need(p + "mlp.shared.sg", W, -1, &sg) || !matrix(sg))) return false;
      std::vector<uint8_t> rt(r->data);
      if (sg) rt.insert(rt.end(), sg->data.begin(), sg->data.end());
      weight_bytes_ += rt.size();
      if (!(L.router = upload(rt.data(), rt.size()))) return false;
      if (L.router_kind == 1 && !up_vec(p + "mlp.router.b", L.experts, &L.router_bias)) return false;
      if (L.router_kind == 2 && !up_vec(p + "mlp.correction", L.experts + L.n_identity, &L.router_bias)) return false;
      std::vector<uint8_t> gu((size_t)L.experts * 2 * L.ffp * W * es), dn((size_t)L.experts * W * L.ffp * es);
      for (int e = 0; e < L.experts; e++) {
        const std::string pe = p + "mlp.e" + std::to_string(e) + ".";
        const HostTensor *g, *u, *d;
        if (!need(pe + "gate", L.ff, W, &g) || !need(pe + "up", L.ff, W, &u) || !need(pe + "down", W, L.ff, &d) || !matrix(g) || !matrix(u) || !matrix(d))
          return false;
        interleave(g, u, L.ff, L.ffp, gu.data() + (size_t)e * 2 * L.ffp * W * es);
        pad_cols(d, L.ff, L.ffp, dn.data() + (size_t)e * W * L.ffp * es);
      }
      weight_bytes_ += gu.size() + dn.size();
      if (!(L.e_gu = upload(gu.data(), gu.size())) || !(L.e_down = upload(dn.data(), dn.size()))) return false;
      if (L.shared_ff > 0) {
        const HostTensor *g, *u, *d;
        if (!need(p + "mlp.shared.gate", L.shared_ff, W, &g) || !need(p + "mlp.shared.up", L.shared_ff, W, &u) ||
            !need(p + "mlp.shared.down", W, L.shared_ff, &d) || !matrix(g) || !matrix(u) || !matrix(d))
          return false;
        std::vector<uint8_t> sgu((size_t)2 * L.sffp * W * es), sdn((size_t)W * L.sffp * es);
        interleave(g, u, L.shared_ff, L.sffp, sgu.data());
        pad_cols(d, L.shared_ff, L.sffp, sdn.data());
        weight_bytes_ += sgu.size() + sdn.size();
        if (!(L.s_gu = upload(sgu.data(), sgu.size())) || !(L.s_down = upload(sdn.data(), sdn.size()))) return false;
      }
    }
  }
  // a layer that shares weights runs with the tensors of the layer it names and keeps a cache of its own
  for (StackLayer& L : layers_) {
    if (L.weights_of < 0) continue;
    const int cache = L.cache, wo = L.weights_of;
    const bool owns = L.owns_cache;
    L = layers_[wo];
    L.cache = cache, L.owns_cache = owns, L.weights_of = wo;
  }
  // the angle of channel pair i is p * base^(-2i / width): the factor is formed in f64 and rounded once, the product is f32
  std::vector<float> inv((W + 1) / 2);
  for (size_t i = 0; i < inv.size(); i++) inv[i] = (float)pow(pos_base_, -2.0 * (double)i / (double)W);
  if (pos_kind_ == 0 && !(inv_freq_ = (float*)upload(inv.data(), inv.size() * 4))) return false;
  staged_.clear();
  finalized_ = hipDeviceSynchronize() == hipSuccess;
  if (!finalized_) error = "layer stack: device error while loading weights";
  return finalized_;
}

// random weights of the configured shapes (benchmarks, tests of the engine path): N(0, 1 / sqrt(fan in)) matrices, norm weights near 1
bool StackModel::init_synthetic(uint64_t seed) {
  if (!spec_error_.empty()) return error = spec_error_, false;
  uint64_t s = seed * 0x9E3779B97F4A7C15ull + 0x1234567ull;
  auto rnd = [&]() {  // xorshift64*; the sum of four uniforms is close enough to a normal for synthetic weights
    s ^= s >> 12, s ^= s << 25, s ^= s >> 27;
    return (double)((s * 0x2545F4914F6CDD1Dull) >> 11) / (double)(1ull << 53);
  };
  auto normal = [&]() { return (rnd() + rnd() + rnd() + rnd() - 2.0) * 1.7320508; };
  auto put = [&](const std::string& name, int64_t r, int64_t c, double mean, double sd) {
    const size_t n = (size_t)r * (c > 0 ? c : 1);
    HostTensor t;
    t.elem_bytes = (int)es_;
    t.shape.push_back(r);
    if (c > 0) t.shape.push_back(c);
    t.data.resize(n * es_);
    for (size_t i = 0; i < n; i++) {
      const float v = (float)(mean + sd * normal());
      if (es_ == 4) memcpy(t.data.data() + i * 4, &v, 4);
      else {
        const uint16_t b = host_f32_to_bf16(v);
        memcpy(t.data.data() + i * 2, &b, 2);
      }
    }
    staged_[name] = std::move(t);
  };
  const int W = width_;
  put("embed", vocab_, W, 0, 1.0);
  if (!tie_head_) put("head", vocab_, W, 0, 1.0 / sqrt((double)W));
  auto put_norm = [&](const std::string& name) {
    put(name, W, 0, 1, 0.05);
    if (norm_kind_ == 1) put(name + ".b", W, 0, 0, 0.02), put(name + ".alpha", 1, 0, 0.5, 0.0);
  };
  if (block_ == 2 && norm_kind_ == 1) {
    put_norm("final.norm");
  } else if (block_ == 2) {  // norm weights are stored around zero; the embedding's own norm and the token-pair table
    put("final.norm", W, 0, 0, 0.05);
    if (embed_norm_) put("embed.norm", W, 0, 0, 0.05);
    if (pair_buckets_ > 0) put("bigram", (int64_t)pair_buckets_ + 1, W, 0, 1.0);
  } else {
    put_norm("final.norm");
  }
  for (size_t li = 0; li < layers_.size(); li++) {
    const StackLayer& L = layers_[li];
    if (L.weights_of >= 0) continue;
    const std::string p = "l" + std::to_string(li) + ".";
    const double sw = 1.0 / sqrt((double)W);
    if (block_ == 2 && norm_kind_ == 1) {
      put_norm(p + "norm1"), put_norm(p + "norm1b");
      if (L.mlp != 0) put_norm(p + "norm2"), put_norm(p + "norm2b");
    } else if (block_ == 2) {
      put(p + "norm1", W, 0, 0, 0.05), put(p + "norm1b", W, 0, 0, 0.05);
      if (L.mlp != 0) put(p + "norm2", W, 0, 0, 0.05), put(p + "norm2b", W, 0, 0, 0.05);
    } else {
      put_norm(p + "norm1");
      if (block_ == 1 && L.mlp != 0) put_norm(p + "norm2");
    }
    if (L.mixer == 3 && !L.lowrank) {
      const int H = L.heads, nk = L.nk(), nv = H * L.vdim;
      put(p + "mix.q", nk, W, 0, sw), put(p + "mix.k", nk, W, 0, sw), put(p + "mix.v", nv, W, 0, sw), put(p + "mix.b", H, W, 0, sw);
      put(p + "mix.q.conv", nk, L.conv, 0.3, 0.3), put(p + "mix.k.conv", nk, L.conv, 0.3, 0.3), put(p + "mix.v.conv", nv, L.conv, 0.3, 0.3);
      put(p + "mix.a", H, W, 0, sw), put(p + "mix.g", nv, W, 0, sw);
      put(p + "mix.A_log", H, 0, -1.0, 0.5), put(p + "mix.dt_bias", H, 0, -2.0, 1.0), put(p + "mix.norm", L.vdim, 0, 1, 0.05);
      put(p + "mix.o", W, nv, 0, 1.0 / sqrt((double)nv));
    } else if (L.mixer == 6) {
      const int H = L.heads;
      put(p + "mix.q", (int64_t)H * L.dim, W, 0, sw), put(p + "mix.k", (int64_t)H * L.dim, W, 0, sw), put(p + "mix.v", (int64_t)H * L.vdim, W, 0, sw);
      put(p + "mix.g", (int64_t)H * L.vdim, W, 0, sw), put(p + "mix.o", W, H * L.vdim, 0, 1.0 / sqrt((double)H * L.vdim));
      put(p + "mix.norm", (int64_t)H * L.vdim, 0, 1, 0.05);
    } else if (L.mixer == 5 && L.right_kind == 1) {
      const std::string pl = p + "mix.left.", pr = p + "mix.right.";
      const int H = L.heads, Wr = L.r_width, nb = L.r_blocks, bw = Wr / nb;
      put(pl + "q", L.nq(), W, 0, sw), put(pl + "k", L.nk(), W, 0, sw), put(pl + "v", L.nv(), W, 0, sw);
      if (L.has_bias) put(pl + "q.b", L.nq(), 0, 0, 0.02), put(pl + "k.b", L.nk(), 0, 0, 0.02), put(pl + "v.b", L.nv(), 0, 0, 0.02);
      if (L.qk_norm) put(pl + "q.norm", L.dim, 0, 1, 0.05), put(pl + "k.norm", L.dim, 0, 1, 0.05);
      if (L.head_temp) put(pl + "temp", H, 0, 1, 0.1);
      if (L.sink) put(pl + "sink", H, 0, 0, 1.0);
      if (L.head_gate) put(pl + "g", H, W, 0, sw);
      put(pl + "o", W, H * L.vdim, 0, 1.0 / sqrt((double)H * L.vdim));
      put(pr + "y", Wr, W, 0, sw), put(pr + "y.b", Wr, 0, 0, 0.02), put(pr + "x", Wr, W, 0, sw), put(pr + "x.b", Wr, 0, 0, 0.02);
      put(pr + "conv", Wr, L.conv, 0.3, 0.3), put(pr + "conv.b", Wr, 0, 0, 0.02);
      put(pr + "ra", (int64_t)nb * bw, bw, 0, 1.0 / sqrt((double)bw)), put(pr + "ri", (int64_t)nb * bw, bw, 0, 1.0 / sqrt((double)bw));
      put(pr + "ra.b", Wr, 0, 0, 0.1), put(pr + "ri.b", Wr, 0, 0, 0.1), put(pr + "lam", Wr, 0, -2.0, 1.0);
      put(pr + "o", W, Wr, 0, 1.0 / sqrt((double)Wr));
      if (L.branch_norm) put(pl + "out", W, 0, 1, 0.05), put(pr + "out", W, 0, 1, 0.05);
    } else if (L.mixer == 3) {
      const int H = L.heads, nk = L.nk(), nv = H * L.vdim;
      put(p + "mix.q", nk, W, 0, sw), put(p + "mix.k", nk, W, 0, sw), put(p + "mix.v", nv, W, 0, sw), put(p + "mix.b", H, W, 0, sw);
      put(p + "mix.q.conv", nk, L.conv, 0.3, 0.3), put(p + "mix.k.conv", nk, L.conv, 0.3, 0.3), put(p + "mix.v.conv", nv, L.conv, 0.3, 0.3);
      put(p + "mix.a1", L.rank_a, W, 0, sw), put(p + "mix.a2", (int64_t)H * L.dim, L.rank_a, 0, 1.0 / sqrt((double)L.rank_a));
      put(p + "mix.g1", L.rank_g, W, 0, sw), put(p + "mix.g2", nv, L.rank_g, 0, 1.0 / sqrt((double)L.rank_g));
      put(p + "mix.A_log", H, 0, -1.0, 0.5), put(p + "mix.dt_bias", (int64_t)H * L.dim, 0, -2.0, 1.0), put(p + "mix.norm", L.vdim, 0, 1, 0.05);
      put(p + "mix.o", W, nv, 0, 1.0 / sqrt((double)nv));
    } else if (L.mixer == 4) {
      const int H = L.heads;
      put(p + "mix.q", (int64_t)H * L.dim, W, 0, sw), put(p + "mix.k", (int64_t)H * L.dim, W, 0, sw), put(p + "mix.v", (int64_t)H * L.vdim, W, 0, sw);
      put(p + "mix.g", (int64_t)H * L.vdim, W, 0, sw), put(p + "mix.o", W, H * L.vdim, 0, 1.0 / sqrt((double)H * L.vdim));
    } else if (L.mixer == 5) {
      const std::string pl = p + "mix.left.", pr = p + "mix.right.";
      const int rq = L.r_heads * L.r_dim, rv = L.r_heads * L.r_vdim;
      put(pl + "q", L.nq(), W, 0, sw), put(pl + "k", L.nk(), W, 0, sw), put(pl + "v", L.nv(), W, 0, sw);
      if (L.has_bias) put(pl + "q.b", L.nq(), 0, 0, 0.02), put(pl + "k.b", L.nk(), 0, 0, 0.02), put(pl + "v.b", L.nv(), 0, 0, 0.02);
      if (L.qk_norm) put(pl + "q.norm", L.dim, 0, 1, 0.05), put(pl + "k.norm", L.dim, 0, 1, 0.05);
      put(pl + "o", W, L.heads * L.vdim, 0, 1.0 / sqrt((double)L.heads * L.vdim));
      put(pr + "q", rq, W, 0, sw), put(pr + "k", rq, W, 0, sw), put(pr + "v", rv, W, 0, sw), put(pr + "g", rv, W, 0, sw);
      put(pr + "a1", L.rank_a, W, 0, sw), put(pr + "a2", rq, L.rank_a, 0, 1.0 / sqrt((double)L.rank_a)), put(pr + "a2.b", rq, 0, 2.0, 1.0);
      put(pr + "norm", L.r_vdim, 0, 1, 0.05), put(pr + "o", W, rv, 0, 1.0 / sqrt((double)rv));
    } else if (L.mixer == 0) {
      put(p + "mix.q", L.nq(), W, 0, sw);
      if (L.owns_cache) put(p + "mix.k", L.nk(), W, 0, sw), put(p + "mix.v", L.nv(), W, 0, sw);
    } else if (L.mixer == 1) {
      put(p + "mix.dq", L.q_rank, W, 0, sw), put(p + "mix.dq.norm", L.q_rank, 0, 1, 0.05);
      put(p + "mix.uq", (int64_t)L.heads * (L.dim + L.rot_dim), L.q_rank, 0, 1.0 / sqrt((double)L.q_rank));
      put(p + "mix.dkv", L.kv_rank + L.rot_dim, W, 0, sw), put(p + "mix.dkv.norm", L.kv_rank, 0, 1, 0.05);
      put(p + "mix.uk", (int64_t)L.heads * L.dim, L.kv_rank, 0, 1.0 / sqrt((double)L.kv_rank));
      put(p + "mix.uv", (int64_t)L.heads * L.vdim, L.kv_rank, 0, 1.0 / sqrt((double)L.kv_rank));
      if (L.sink) put(p + "mix.sink", L.heads, 0, 0, 1.0);
    } else {
      put(p + "mix.q", L.nq(), W, 0, sw), put(p + "mix.k", L.nk(), W, 0, sw), put(p + "mix.v", L.nv(), W, 0, sw);
      put(p + "mix.g", (int64_t)L.heads * L.vdim, W, 0, sw);
      put(p + "mix.q.b", L.nq(), 0, 0, 0.02), put(p + "mix.k.b", L.nk(), 0, 0, 0.02), put(p + "mix.v.b", L.nv(), 0, 0, 0.02);
      put(p + "mix.q.norm", L.nq(), 0, 1, 0.05), put(p + "mix.k.norm", L.nk(), 0, 1, 0.05);
      put(p + "mix.pb", L.heads, 0, -3.0, 0.5), put(p + "mix.talk", L.heads, L.heads, 1.0 / L.heads, 0.1 / L.heads);
    }
    if (L.mixer < 3) put(p + "mix.o", W, L.heads * L.vdim, 0, 1.0 / sqrt((double)L.heads * L.vdim));
    if (L.mlp == 3 || L.mlp == 4) {
      put(p + "mlp.gate", L.ff, W, 0, sw), put(p + "mlp.up", L.ff, W, 0, sw), put(p + "mlp.down", W, L.ff, 0, 1.0 / sqrt((double)L.ff));
    } else if (L.mlp == 1) {
      put(p + "mlp.up", L.ff, W, 0, sw), put(p + "mlp.down", W, L.ff, 0, 1.0 / sqrt((double)L.ff));
      HostTensor a;
      a.elem_bytes = 4, a.shape = {4};
      const float c[4] = {0.6f, 0.3f, 0.1f, 0.02f};
      a.data.assign((const uint8_t*)c, (const uint8_t*)c + 16);
      staged_[p + "mlp.act"] = a;
    } else if (L.mlp == 2) {
      put(p + "mlp.router", L.experts + L.n_identity, W, 0, sw);
      if (L.router_kind == 1) put(p + "mlp.router.b", L.experts, 0, 0, 0.1);
      if (L.router_kind == 2) put(p + "mlp.correction", L.experts + L.n_identity, 0, 0, 0.02);
      for (int e = 0; e < L.experts; e++) {
        const std::string pe = p + "mlp.e" + std::to_string(e) + ".";
        put(pe + "gate", L.ff, W, 0, sw), put(pe + "up", L.ff, W, 0, sw), put(pe + "down", W, L.ff, 0, 1.0 / sqrt((double)L.ff));
      }
      if (L.shared_ff > 0) {
        put(p + "mlp.shared.gate", L.shared_ff, W, 0, sw), put(p + "mlp.shared.up", L.shared_ff, W, 0, sw);
        put(p + "mlp.shared.down", W, L.shared_ff, 0, 1.0 / sqrt((double)L.shared_ff)), put(p + "mlp.shared.sg", 1, W, 0, sw);
      }
    }
  }
  return finalize_weights();
}

// ---------------------------------------------------------------------------------------------
// cache and buffers
// ---------------------------------------------------------------------------------------------
size_t StackModel::k_block_bytes(int c) const {
  const StackLayer& L = layers_[cache_layer_[c]];
  return (size_t)ec_.block_size * L.k_row() * es_;
}
size_t StackModel::v_block_bytes(int c) const {
  const StackLayer& L = layers_[cache_layer_[c]];
  return (size_t)ec_.block_size * L.v_row() * es_;
}
int64_t StackModel::kv_bytes_per_block() const {
  int64_t b = 0;
  for (size_t c = 0; c < cache_layer_.size(); c++) b += (int64_t)k_block_bytes((int)c) + (int64_t)v_block_bytes((int)c);
  return std::max<int64_t>(b, 16);  // (a stack without any cached layer still plans a block count)
}
bool StackModel::init_kv_cache(int num_blocks) {
  if (!spec_error_.empty()) return error = spec_error_, false;
  num_blocks_ = num_blocks;
  kc_.assign(cache_layer_.size(), nullptr);
  vc_.assign(cache_layer_.size(), nullptr);
  for (size_t c = 0; c < cache_layer_.size(); c++) {
    const size_t kb = (size_t)num_blocks * k_block_bytes((int)c), vb = (size_t)num_blocks * v_block_bytes((int)c);
    if (!(kc_[c] = dalloc(kb)) || !(vc_[c] = dalloc(vb))) return false;
    if (hipMemset(kc_[c], 0, kb) != hipSuccess || hipMemset(vc_[c], 0, vb) != hipSuccess) return error = "kv cache clear failed", false;
  }
  return hipDeviceSynchronize() == hipSuccess;
}

// what one sequence carries between steps: per recurrent layer the matrix state of every head (f32) and the last inputs of its short
// convolutions
int64_t StackModel::state_bytes_per_slot() const {
  int64_t b = 0;
  for (const StackLayer& L : layers_) {
    if (L.s_heads() <= 0 && L.vec_state() <= 0) continue;
    b += (int64_t)L.s_heads() * L.s_dim() * L.s_vdim() * 4 + (int64_t)L.vec_state() * 4;
    if (L.conv > 1) b += (int64_t)(L.conv - 1) * L.conv_channels() * 4;
  }
  return b;
}
bool StackModel::init_state(int slots) {
  if (!spec_error_.empty()) return error = spec_error_, false;
  state_slots_ = slots;
  for (StackLayer& L : layers_) {
    if (L.s_heads() <= 0 && L.vec_state() <= 0) continue;
    const size_t sb = (size_t)slots * ((size_t)L.s_heads() * L.s_dim() * L.s_vdim() + (size_t)L.vec_state()) * 4;
    if (!(L.state = (float*)dalloc(sb)) || hipMemset(L.state, 0, sb) != hipSuccess) return error = "state slots: allocation failed", false;
    if (L.conv > 1) {
      const size_t cb = (size_t)slots * (L.conv - 1) * L.conv_channels() * 4;
      if (!(L.conv_state = (float*)dalloc(cb)) || hipMemset(L.conv_state, 0, cb) != hipSuccess) return error = "state slots: allocation failed", false;
    }
  }
  return hipDeviceSynchronize() == hipSuccess;
}

// rotary frequencies base^(-2i / dims) in f64, optionally slowed down by wavelength (waves longer than original / low are divided by
// `factor`, shorter than original / high kept, those between blended linearly in original / wavelength), kept as hi + lo f32 pairs
void StackModel::rotary_table(StackLayer& L) {
  L.rot_pairs = L.rot_dims / 2;
  L.rot_mag = 1.f;
  std::vector<float> fh(std::max(L.rot_pairs, 1), 0.f), fl(std::max(L.rot_pairs, 1), 0.f);
  // YaRN: pairs that turn fewer than yarn_slow times over the original length are slowed down by the factor, those that turn more than
  // yarn_fast times are kept, a linear ramp over the pair index between; cos and sin grow by 0.1 ln(factor) + 1
  double ylo = 0.0, yhi = 0.0;
  if (L.yarn_factor > 0.0) {
    const double dims = (double)L.rot_dims, lnb = log(L.rot_base);
    auto turn_dim = [&](double turns) { return dims * log(L.yarn_original / (2.0 * M_PI * turns)) / (2.0 * lnb); };
    ylo = std::max(floor(turn_dim(L.yarn_fast)), 0.0), yhi = std::min(ceil(turn_dim(L.yarn_slow)), dims - 1.0);
    L.rot_mag = (float)(0.1 * log(L.yarn_factor) + 1.0);
  }
  for (int i = 0; i < L.rot_pairs; i++) {
    double fr = pow(L.rot_base, -2.0 * (double)i / (double)L.rot_dims);
    if (L.yarn_factor > 0.0) {
      const double ramp = std::min(std::max(((double)i - ylo) / std::max(yhi - ylo, 0.001), 0.0), 1.0);
      fr = fr / L.yarn_factor * ramp + fr * (1.0 - ramp);
    }
    if (L.rs_factor > 0.0) {
      const double wl = 2.0 * M_PI / fr;
      if (wl > L.rs_original / L.rs_low) fr = fr / L.rs_factor;
      else if (!(wl < L.rs_original / L.rs_high)) {
        const double sm = (L.rs_original / wl - L.rs_low) / (L.rs_high - L.rs_low);
        fr = (1.0 - sm) * fr / L.rs_factor + sm * fr;
      }
    }
    fh[i] = (float)fr, fl[i] = (float)(fr - (double)fh[i]);
  }
  L.freq_hi = upload_floats(fh), L.freq_lo = upload_floats(fl);
}

bool StackModel::init_buffers(int max_tokens, int max_seqs) {
  if (!spec_error_.empty()) return error = spec_error_, false;
  max_tokens_ = max_tokens, max_seqs_ = max_seqs;
  const size_t T = max_tokens, W = width_;
  size_t nqkv = 0, nattn = 0, zc = 0, actc = 0, top = 0, experts = 0;
  size_t nqa = 0, z2c = 0, recc = 0, roc = 0;
  bool want_h32 = false;
  for (const StackLayer& L : layers_) {
    // softmax / sigmoid: the joint projection in the model's type; latent: q, later the heads' values (the joint projection is f32 in z_)
    nqkv = std::max(nqkv, L.mixer == 0 ? (size_t)L.nqkv() : std::max((size_t)L.nq(), (size_t)L.heads * L.vdim));
    if (L.mixer >= 3) zc = std::max(zc, T * L.nqkv());
    nattn = std::max(nattn, (size_t)L.heads * (L.mixer == 1 ? L.kv_rank : L.vdim));
    if (L.mixer == 1) nqa = std::max(nqa, (size_t)L.heads * (L.kv_rank + L.rot_dim)), actc = std::max(actc, T * L.q_rank);
    if (L.mixer != 0) zc = std::max(zc, T * L.nqkv());
    if (L.mlp == 2) top = std::max(top, (size_t)L.top), experts = std::max(experts, (size_t)L.experts);
    if (L.mlp == 3 || L.mlp == 4) zc = std::max(zc, T * 2 * L.sffp), actc = std::max(actc, T * L.sffp);
    if (L.mlp == 2 && L.n_identity > 0) want_h32 = true;
    if (L.mixer == 5 && L.right_kind == 1) {  // the convolved branch in rec_, both gates' logits in z2_, the recurrence's output in attn_
      nattn = std::max(nattn, (size_t)L.r_width), z2c = std::max(z2c, (size_t)2 * L.r_width), recc = std::max(recc, (size_t)L.r_width), roc = std::max<size_t>(roc, 1);
    } else if (L.mixer >= 3) {  // the joint projection is f32 in z_, the low-rank first stages in act_, their second stages in z2_
      const size_t sh = L.s_heads(), sd = L.s_dim(), sv = L.s_vdim();
      nattn = std::max(nattn, sh * sv);
      actc = std::max(actc, T * (size_t)(L.rank_a + L.rank_g));
      z2c = std::max(z2c, sh * sd + (L.mixer == 3 ? sh * sv : 0));
      recc = std::max(recc, L.mixer == 3 ? (size_t)L.conv_channels() + sh + sh * sd : (L.mixer == 4 ? 2 * sh * sd : sh * sd));
      if (L.mixer == 6) z2c = std::max<size_t>(z2c, 1);
      roc = std::max(roc, sh * sv);
    }
  }
  max_rows_ = (int)round_up((int)(T * std::max<size_t>(top, 1) + experts * 63), 64);
  for (const StackLayer& L : layers_) {
    if (L.mlp == 1) zc = std::max(zc, T * L.ff), actc = std::max(actc, T * L.ff);
    if (L.mlp == 2 && L.n_identity > 0) experts = std::max(experts, (size_t)L.experts);
    if (L.mlp == 2) {
      zc = std::max(zc, std::max((size_t)max_rows_ * 2 * L.ffp, T * 2 * L.sffp));
      actc = std::max(actc, std::max((size_t)max_rows_ * L.ffp, T * L.sffp));
    }
  }
  // logits rows: at least one per sequence; replayed traces ask for many rows of one step, so take what 256 MiB hold
  logit_rows_cap_ = (int)std::max<size_t>(max_seqs, std::min<size_t>(T, ((size_t)256 << 20) / ((size_t)vocab_ * 4)));
  const size_t R = logit_rows_cap_;
  if (!(x_ = (float*)dalloc(T * W * 4)) || !(o_ = (float*)dalloc(T * W * 4)) || !(h_ = dalloc(T * W * es_)) || !(qkv_ = dalloc(T * nqkv * es_)) ||
      !(attn_ = dalloc(T * nattn * es_)) || !(z_ = (float*)dalloc(std::max<size_t>(zc, 4) * 4)) || !(act_ = dalloc(std::max<size_t>(actc, 4) * es_)) ||
      !(pair_out_ = (float*)dalloc(T * std::max<size_t>(top, 1) * W * 4)) || !(sh_ = (float*)dalloc(T * W * 4)) || !(xl_ = (float*)dalloc(R * W * 4)) ||
      !(hl_ = dalloc(R * W * es_)) || !(logits_ = (float*)dalloc(R * (size_t)vocab_ * 4)) || !(qa_ = dalloc(std::max<size_t>(T * nqa, 4) * es_)))
    return false;
  if (z2c && (!(z2_ = (float*)dalloc(T * z2c * 4)) || !(rec_ = (float*)dalloc(T * recc * 4)) || !(ro_ = (float*)dalloc(T * roc * 4)))) return false;
  // sigmoid attention sums in two launches: per-head-pair sums of a prompt portion (bf16, at most 1 GiB: longer steps take the one-launch
  // kernel), per-tile partial sums of decoded tokens
  for (const StackLayer& L : layers_) {
    if (L.mixer != 2) continue;
    const size_t hv = (size_t)L.heads * L.vdim;
    if (dt_ == VRA_BF16) sig_scratch_bytes_ = std::max(sig_scratch_bytes_, std::min<size_t>(T * hv * L.kv_heads * 4, (size_t)1 << 30));
    sig_scratch_bytes_ = std::max(sig_scratch_bytes_, (size_t)max_seqs * 64 * hv * 4);
  }
  if (sig_scratch_bytes_ && !(sig_scratch_ = (float*)dalloc(sig_scratch_bytes_))) return false;
  if (want_h32 && (!(h32_ = (float*)dalloc(T * W * 4)) || !(id_weight_ = (float*)dalloc(T * 4)))) return false;
  const size_t P = T * std::max<size_t>(top, 1);
  if (!(pair_expert_ = (int*)dalloc(P * 4)) || !(pair_weight_ = (float*)dalloc(P * 4)) || !(gate_ = (float*)dalloc(T * 4)) ||
      !(row_token_ = (int*)dalloc((size_t)max_rows_ * 4)) || !(row_pair_ = (int*)dalloc((size_t)max_rows_ * 4)) ||
      !(row_scale_ = (float*)dalloc((size_t)max_rows_ * 4)) || !(tile_group_ = (int*)dalloc((size_t)max_rows_ / 16 * 4)))
    return false;
  return hipDeviceSynchronize() == hipSuccess;
}

// ---------------------------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------------------------
static bool take_stack_err(std::string& error, const char* where) {
  const char* e = vra_last_error();
  if (e && e[0]) {
    error = std::string(where) + ": " + e;
    vra_clear_error();
    return true;
  }
  return false;
}

// gate / up -> clamped gated activation -> down for `rows` logical rows (one expert per granule, or one weight set for all):
// bf16: the activation is the epilogue of the gate / up launch; f32: product, activation and product as three launches
bool StackModel::expert_pair(const void* a, int lda, const void* w_gu, int64_t gu_stride, const void* w_down, int64_t down_stride, int rows, int fp,
                             int f, float limit, const int* tile_group, int granule, const int* a_row, const float* a_scale, const int* out_row,
                             float* out, int64_t stream, int act) {
  const int W = width_;
  StkGemmArgs g;
  g.a = a, g.lda = lda, g.w = w_gu, g.w_group_stride = gu_stride, g.M = rows, g.N = 2 * fp, g.K = W;
  g.tile_group = tile_group, g.granule = granule, g.a_row = a_row, g.a_scale = a_scale;
  g.limit = limit, g.act = act;
  const bool fused = dt_ == VRA_BF16 && W % 8 == 0 && lda % 8 == 0;
  if (fused) {
    g.epi = 1, g.out = act_, g.ldo = fp;
    vra_stack_gemm(g, dt_, stream);
  } else {
    g.out = z_, g.ldo = 2 * fp, g.out_f32 = 1;
    vra_stack_gemm(g, dt_, stream);
    vra_stack_gated_act(z_, act_, rows, f, limit, 1.702f, dt_, stream, act);
  }
  StkGemmArgs d;
  d.a = act_, d.lda = fp, d.w = w_down, d.w_group_stride = down_stride, d.M = rows, d.N = W, d.K = fp;
  d.out = out, d.ldo = W, d.out_f32 = 1;
  d.tile_group = tile_group, d.granule = granule, d.out_row = out_row;
  // rows of a granule that hold no pair are neither read nor written: a_row of the first launch marks them, the second sees them through out_row
  vra_stack_gemm(d, dt_, stream);
  return !take_stack_err(error, "expert feed-forward");
}

bool StackModel::feed_forward(const StackLayer& L, int T, int64_t stream) {
  const int W = width_;
  if (L.mlp == 1) {
    StkGemmArgs u;
    u.a = h_, u.lda = W, u.w = L.up, u.M = T, u.N = L.ff, u.K = W, u.out = z_, u.ldo = L.ff, u.out_f32 = 1;
    vra_stack_gemm(u, dt_, stream);
    vra_stack_polynorm(z_, act_, L.act, T, L.ff, eps_, dt_, stream);
    StkGemmArgs d;
    d.a = act_, d.lda = L.ff, d.w = L.down, d.M = T, d.N = W, d.K = L.ff, d.out = pair_out_, d.ldo = W, d.out_f32 = 1;
    vra_stack_gemm(d, dt_, stream);
    vra_stack_residual_combine(x_, o_, pair_out_, 1, nullptr, nullptr, residual_mult_, T, W, stream);
    return !take_stack_err(error, "dense feed-forward");
  }
  if (L.mlp == 2) {
    const int P = T * L.top;
    const int granule = vra_stack_gemm_granule(P, L.experts);
    const int rows = round_up(P + L.experts * (granule - 1), granule);
    if (rows > max_rows_) return error = "feed-forward: more expert rows than the buffers hold", false;
    vra_stack_moe_sort(pair_expert_, pair_weight_, P, L.top, L.experts, granule, rows, row_token_, row_scale_, row_pair_, tile_group_, stream);
    if (take_stack_err(error, "expert rows")) return false;
    if (!expert_pair(h_, W, L.e_gu, (int64_t)2 * L.ffp * W, L.e_down, (int64_t)W * L.ffp, rows, L.ffp, L.ff, L.limit, tile_group_, granule, row_token_,
                     row_scale_, row_pair_, pair_out_, stream))
      return false;
    if (L.shared_ff > 0 &&
        !expert_pair(h_, W, L.s_gu, 0, L.s_down, 0, T, L.sffp, L.shared_ff, L.shared_limit, nullptr, 0, nullptr, nullptr, nullptr, sh_, stream))
      return false;
    vra_stack_residual_combine(x_, o_, pair_out_, L.top, L.shared_ff > 0 ? sh_ : nullptr, L.shared_ff > 0 ? gate_ : nullptr, residual_mult_, T, W, stream);
    return !take_stack_err(error, "mixture of experts");
  }
  vra_stack_residual_combine(x_, o_, nullptr, 0, nullptr, nullptr, residual_mult_, T, W, stream);
  return !take_stack_err(error, "residual");
}

// h = norm(x + add) with x updated in place (add null: x as it is); sequential blocks norm every sub-block's input
bool StackModel::norm_into_h(const float* w, const float* b, float alpha, const float* add, float* x, void* h, int T, int64_t stream) {
  if (norm_kind_ == 1) {
    vra_stack_dyt(x, add, w, b, alpha, h, T, width_, dt_, stream);
  } else {
    if (add) vra_stack_residual_combine(x, add, nullptr, 0, nullptr, nullptr, 1.f, T, width_, stream);
    StkNormArgs n;
    n.x = x, n.w = w, n.h = h, n.T = T, n.W = width_, n.groups = groups_, n.eps = eps_;
    vra_stack_group_norm(n, dt_, stream);
  }
  return !take_stack_err(error, "norm");
}

// causal softmax attention with its own (or a borrowed) key / value cache: h_ -> o_ (f32 [T, width])
bool StackModel::mixer_softmax(const StackLayer& L, const InputMetadata& md, int64_t stream) {
  const int T = md.n_tokens, B = md.n_seqs, W = width_;
  // q (| k | v) in one launch
  const int nqkv = L.nqkv();
  StkGemmArgs p;
  p.a = h_, p.lda = W, p.w = L.qkv, p.M = T, p.N = nqkv, p.K = W, p.out = qkv_, p.ldo = nqkv;
  vra_stack_gemm(p, dt_, stream);
  if (L.owns_cache)
    vra_stack_kv_store((const char*)qkv_ + (size_t)L.nq() * es_, (const char*)qkv_ + (size_t)(L.nq() + L.nk()) * es_, nqkv, kc_[L.cache], vc_[L.cache],
                       md.slot_mapping, T, L.nk(), L.nv(), dt_, stream);
  StkAttnArgs a;
  a.q = qkv_, a.ldq = nqkv, a.out = attn_, a.kc = kc_[L.cache], a.vc = vc_[L.cache];
  a.positions = md.positions, a.block_tables = md.block_tables, a.context_lens = md.context_lens;
  a.cu_q = md.is_prefill ? md.cu_seqlens_q : nullptr;
  a.B = B, a.T = T, a.max_q = md.is_prefill ? md.max_seqlen_q : 1, a.H = L.heads, a.G = L.kv_heads, a.dim = L.dim, a.vdim = L.vdim;
  a.BS = ec_.block_size, a.max_blocks = md.max_blocks;
  a.scale = L.scale, a.softcap = L.softcap, a.temp_coef = L.temp_coef, a.temp_every = L.temp_every;
  vra_stack_attention(a, dt_, stream);
  StkGemmArgs o;
  o.a = attn_, o.lda = L.heads * L.vdim, o.w = L.o, o.M = T, o.N = W, o.K = L.heads * L.vdim, o.out = o_, o.ldo = W, o.out_f32 = 1;
  vra_stack_gemm(o, dt_, stream);
  return !take_stack_err(error, "mixer");
}

// Latent attention in its absorbed form: the cache row of a token is [normed kv latent | rotated key part]; a head's query becomes
// [W_uk_h^T q_h | rot(q_h's rotated part)], so the scores are plain dot products with the cache rows of ONE shared key/value head, the
// values are the latents themselves, and W_uv_h is applied to the weighted sum.
bool StackModel::mixer_latent(const StackLayer& L, const InputMetadata& md, int64_t stream) {
  const int T = md.n_tokens, B = md.n_seqs, W = width_, H = L.heads, qd = L.dim + L.rot_dim, kd = L.kv_rank + L.rot_dim;
  StkGemmArgs d;  // both down-projections, f32 out: the norms read unrounded values
  d.a = h_, d.lda = W, d.w = L.qkv, d.M = T, d.N = L.nqkv(), d.K = W, d.out = z_, d.ldo = L.nqkv(), d.out_f32 = 1;
  vra_stack_gemm(d, dt_, stream);
  StkLatentPrepArgs lp;
  lp.raw = z_, lp.ld = L.nqkv(), lp.q_rank = L.q_rank, lp.kv_rank = L.kv_rank, lp.rot_dim = L.rot_dim, lp.qn_w = L.qn_w, lp.kvn_w = L.kn_w, lp.eps = eps_;
  lp.cq = act_, lp.cache = kc_[L.cache], lp.cache_ld = kd, lp.slots = md.slot_mapping, lp.positions = md.positions, lp.T = T;
  lp.rot.freq_hi = L.freq_hi, lp.rot.freq_lo = L.freq_lo, lp.rot.pairs = L.rot_pairs, lp.rot.mag = L.rot_mag;
  vra_stack_latent_prep(lp, dt_, stream);
  StkGemmArgs uq;
  uq.a = act_, uq.lda = L.q_rank, uq.w = L.uq, uq.M = T, uq.N = H * qd, uq.K = L.q_rank, uq.out = qkv_, uq.ldo = H * qd;
  vra_stack_gemm(uq, dt_, stream);
  if (L.rot_dim > 0) vra_stack_rope_heads(qkv_, H * qd, qd, L.dim, qa_, H * kd, kd, L.kv_rank, L.rot_dim, H, md.positions, lp.rot, T, dt_, stream);
  StkGemmArgs ab;  // per head: [T, dim] x W_uk_h -> [T, kv_rank]
  ab.a = qkv_, ab.lda = H * qd, ab.a_batch_stride = qd, ab.w = L.ukt, ab.w_batch_stride = (int64_t)L.kv_rank * L.dim, ab.batch = H;
  ab.M = T, ab.N = L.kv_rank, ab.K = L.dim, ab.out = qa_, ab.ldo = H * kd, ab.out_batch_stride = kd;
  vra_stack_gemm(ab, dt_, stream);
  StkAttnArgs a;
  a.q = qa_, a.ldq = H * kd, a.out = attn_, a.kc = kc_[L.cache], a.vc = kc_[L.cache], a.k_ld = kd, a.v_ld = kd, a.sink = L.sink ? L.sink_w : nullptr;
  a.positions = md.positions, a.block_tables = md.block_tables, a.context_lens = md.context_lens;
  a.cu_q = md.is_prefill ? md.cu_seqlens_q : nullptr;
  a.B = B, a.T = T, a.max_q = md.is_prefill ? md.max_seqlen_q : 1, a.H = H, a.G = 1, a.dim = kd, a.vdim = L.kv_rank;
  a.BS = ec_.block_size, a.max_blocks = md.max_blocks, a.scale = L.scale;
  vra_stack_attention(a, dt_, stream);
  StkGemmArgs uv;  // per head: [T, kv_rank] x W_uv_h^T -> [T, vdim]
  uv.a = attn_, uv.lda = H * L.kv_rank, uv.a_batch_stride = L.kv_rank, uv.w = L.uv, uv.w_batch_stride = (int64_t)L.vdim * L.kv_rank, uv.batch = H;
  uv.M = T, uv.N = L.vdim, uv.K = L.kv_rank, uv.out = qkv_, uv.ldo = H * L.vdim, uv.out_batch_stride = L.vdim;
  vra_stack_gemm(uv, dt_, stream);
  StkGemmArgs o;
  o.a = qkv_, o.lda = H * L.vdim, o.w = L.o, o.M = T, o.N = W, o.K = H * L.vdim, o.out = o_, o.ldo = W, o.out_f32 = 1;
  vra_stack_gemm(o, dt_, stream);
  return !take_stack_err(error, "latent attention");
}

// sigmoid attention: q | k | v | gate in one launch (biases in its epilogue, f32 out), the two whole-projection norms and the cache rows
// in one launch, then the attention with the gate in its epilogue
bool StackModel::mixer_sigmoid(const StackLayer& L, const InputMetadata& md, int64_t stream) {
  const int T = md.n_tokens, B = md.n_seqs, W = width_, n4 = L.nqkv();
  StkGemmArgs p;
  p.a = h_, p.lda = W, p.w = L.qkv, p.bias = L.qkv_bias, p.M = T, p.N = n4, p.K = W, p.out = z_, p.ldo = n4, p.out_f32 = 1;
  vra_stack_gemm(p, dt_, stream);
  vra_stack_qk_norm_store(z_, n4, L.nq(), L.nk(), L.nv(), L.qn_w, L.kn_w, eps_, qkv_, kc_[L.cache], vc_[L.cache], md.slot_mapping, T, dt_, stream);
  StkSigAttnArgs a;
  a.q = qkv_, a.ldq = L.nq(), a.out = attn_, a.kc = kc_[L.cache], a.vc = vc_[L.cache];
  a.positions = md.positions, a.block_tables = md.block_tables, a.context_lens = md.context_lens;
  a.cu_q = md.is_prefill ? md.cu_seqlens_q : nullptr;
  a.B = B, a.T = T, a.max_q = md.is_prefill ? md.max_seqlen_q : 1, a.H = L.heads, a.G = L.kv_heads, a.dim = L.dim, a.vdim = L.vdim;
  a.BS = ec_.block_size, a.max_blocks = md.max_blocks, a.scale = L.scale, a.window = L.window, a.keep_first = L.keep_first;
  a.slopes = L.slopes, a.head_bias = L.head_bias, a.talk = L.talk, a.gate = z_ + L.nq() + L.nk() + L.nv(), a.gate_ld = n4;
  a.scratch = sig_scratch_, a.scratch_bytes = sig_scratch_bytes_, a.max_len = mc_.max_position_embeddings;
  vra_stack_sigmoid_attention(a, dt_, stream);
  StkGemmArgs o;
  o.a = attn_, o.lda = L.heads * L.vdim, o.w = L.o, o.M = T, o.N = W, o.K = L.heads * L.vdim, o.out = o_, o.ldo = W, o.out_f32 = 1;
  vra_stack_gemm(o, dt_, stream);
  return !take_stack_err(error, "sigmoid attention");
}

bool StackModel::forward(const InputMetadata& md, int64_t stream, uint32_t* tokens) {
  if (!finalized_) return error = "forward before the weights are complete", false;
  const int T = md.n_tokens, B = md.n_seqs, W = width_;
  if (T <= 0 || T > max_tokens_ || B <= 0 || B > max_seqs_) return error = "forward: batch out of range", false;
  if (!md.is_prefill && T != B) return error = "forward: a decode step carries one token per sequence", false;
  error.clear();
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (trace_on_) {
    const size_t need_b = layers_.size() * (size_t)T * W * 4;
    if (trace_cap_ < need_b) {
      if (!(trace_ = (float*)dalloc(need_b))) return false;
      trace_cap_ = need_b;
    }
    trace_bytes_ = need_b;
  }
  if (block_ == 2) {
    if (!forward_sandwich(md, stream)) return false;
  } else {
    vra_stack_embed_sinpos(md.input_ids, md.positions, embed_, pos_kind_ == 0 ? inv_freq_ : nullptr, x_, T, W, vocab_, dt_, stream);
    if (take_stack_err(error, "embedding")) return false;
  }
  // sequential blocks: the output of a sub-block is added to the residual inside the launch of the next norm (`pending`)
  const float* pending = nullptr;
  for (size_t li = 0; li < layers_.size() && block_ != 2; li++) {
    const StackLayer& L = layers_[li];
    if (block_ == 0) {
      // h = norm(x); a mixture-of-experts layer's router (and its shared expert's gate) reads h inside the same launch
      StkNormArgs n;
      n.x = x_, n.w = L.norm_w, n.h = h_, n.T = T, n.W = W, n.groups = groups_, n.eps = eps_;
      if (L.mlp == 2) {
        n.router_w = L.router, n.n_router = L.experts, n.top = L.top, n.gate_row = L.shared_ff > 0;
        n.pair_expert = pair_expert_, n.pair_weight = pair_weight_, n.gate_out = gate_;
      }
      vra_stack_group_norm(n, dt_, stream);
      if (!mixer_softmax(L, md, stream)) return false;
      if (!feed_forward(L, T, stream)) return false;
    } else {
      if (!norm_into_h(L.norm_w, L.norm_b, L.norm_alpha, pending, x_, h_, T, stream)) return false;
      if (!(L.mixer == 1 ? mixer_latent(L, md, stream) : (L.mixer == 2 ? mixer_sigmoid(L, md, stream) : mixer_softmax(L, md, stream)))) return false;
      pending = o_;
      if (L.mlp == 3) {
        if (!norm_into_h(L.norm2_w, L.norm2_b, L.norm2_alpha, pending, x_, h_, T, stream)) return false;
        if (!expert_pair(h_, W, L.s_gu, 0, L.s_down, 0, T, L.sffp, L.ff, 0.f, nullptr, 0, nullptr, nullptr, nullptr, pair_out_, stream, 1)) return false;
        pending = pair_out_;
      }
      if (trace_on_ || li + 1 == layers_.size()) {
        vra_stack_residual_combine(x_, pending, nullptr, 0, nullptr, nullptr, 1.f, T, W, stream);
        pending = nullptr;
        if (take_stack_err(error, "residual")) return false;
      }
    }
    if (trace_on_ && hipMemcpyAsync(trace_ + li * (size_t)T * W, x_, (size_t)T * W * 4, hipMemcpyDeviceToDevice, st) != hipSuccess)
      return error = "layer trace copy failed", false;
  }
  // the rows whose logits are wanted -> final norm -> head
  const float* xin = x_;
  int rows = T;
  const uint32_t* sel = md.n_logit_rows > 0 ? md.logit_rows : (md.is_prefill ? md.last_token_rows : nullptr);
  if (sel) {
    rows = md.n_logit_rows > 0 ? md.n_logit_rows : B;
    if (rows > logit_rows_cap_) return error = "forward: more logit rows than the logits buffer holds", false;
    vra_stack_gather_rows_f32(x_, sel, xl_, rows, W, stream);
    xin = xl_;
  } else if (rows > logit_rows_cap_) {
    return error = "forward: more logit rows than the logits buffer holds", false;
  }
  if (norm_kind_ == 1) {
    // (the gathered rows are a copy: the kernel may read them through a non-const pointer, it adds nothing)
    vra_stack_dyt(const_cast<float*>(xin), nullptr, final_norm_, final_b_, final_alpha_, hl_, rows, W, dt_, stream);
  } else {
    StkNormArgs fn;
    fn.x = xin, fn.w = final_norm_, fn.h = hl_, fn.T = rows, fn.W = W, fn.groups = groups_, fn.eps = eps_;
    vra_stack_group_norm(fn, dt_, stream);
  }
  StkGemmArgs hd;
  hd.a = hl_, hd.lda = W, hd.w = head_, hd.M = rows, hd.N = vocab_, hd.K = W, hd.out = logits_, hd.ldo = vocab_, hd.out_f32 = 1, hd.alpha = logit_scale_;
  vra_stack_gemm(hd, dt_, stream);
  if (tokens) vra_argmax_f32(logits_, tokens, rows, vocab_, stream);
  return !take_stack_err(error, "head");
}

// ---------------------------------------------------------------------------------------------
// sandwich blocks with recurrent mixers
// ---------------------------------------------------------------------------------------------
// the recurrence has left o (f32 [T, heads * vdim]) in ro_: per-head norm, gate, output projection -> out (f32 [T, width])
bool StackModel::recurrent_tail(const StackLayer& L, const InputMetadata& md, const float* gate, int gate_ld, int gate_act, const void* w_o, float* out,
                                int64_t stream) {
  const int T = md.n_tokens, H = L.s_heads(), V = L.s_vdim();
  vra_stack_head_norm_gate(ro_, L.out_norm_w, gate, gate_ld, gate_act, eps_, attn_, T, H, V, dt_, stream);
  StkGemmArgs o;
  o.a = attn_, o.lda = H * V, o.w = w_o, o.M = T, o.N = width_, o.K = H * V, o.out = out, o.ldo = width_, o.out_f32 = 1;
  vra_stack_gemm(o, dt_, stream);
  return !take_stack_err(error, "recurrent mixer");
}

static void scan_common(StkScanArgs& sc, const StackLayer& L, const InputMetadata& md, float* out) {
  sc.state = L.state, sc.state_slots = md.state_slots, sc.positions = md.positions, sc.cu_q = md.is_prefill ? md.cu_seqlens_q : nullptr;
  sc.out = out, sc.ldo = L.s_heads() * L.s_vdim(), sc.B = md.n_seqs, sc.H = L.s_heads(), sc.dim = L.s_dim(), sc.vdim = L.s_vdim();
}

// gated delta rule: joint projection (f32), the low-rank first stages (model type) and their second stages (f32), then one launch for
// the convolutions, unit vectors, write strengths and decays, one that moves the convolution state on, the recurrence, norm + gate, o
bool StackModel::mixer_delta(const StackLayer& L, const InputMetadata& md, int64_t stream) {
  const int T = md.n_tokens, W = width_, H = L.heads, G = L.kv_heads, D = L.dim, V = L.vdim, n1 = L.nqkv(), C = L.conv_channels(), R = L.rank_a + L.rank_g;
  StkGemmArgs p;
  p.a = h_, p.lda = W, p.w = L.qkv, p.M = T, p.N = n1, p.K = W, p.out = z_, p.ldo = n1, p.out_f32 = 1;
  vra_stack_gemm(p, dt_, stream);
  if (!L.lowrank) {  // decays (one per head) and gate are columns of the joint projection
    StkDeltaPrepArgs d;
    d.raw = z_, d.ld = n1, d.raw2 = z_ + C + H, d.ld2 = n1, d.conv_w = L.conv_w, d.taps = L.conv, d.conv_state = L.conv_state ? L.conv_state : rec_;
    d.rate = L.rate, d.dt_bias = L.dt_bias, d.q_scale = 1.f / sqrtf((float)D), d.decay_dim = 1;
    d.qkv_out = rec_, d.beta_out = rec_ + (size_t)T * C, d.decay_out = rec_ + (size_t)T * (C + H);
    d.positions = md.positions, d.cu_q = md.is_prefill ? md.cu_seqlens_q : nullptr, d.state_slots = md.state_slots;
    d.T = T, d.B = md.n_seqs, d.H = H, d.G = G, d.dim = D, d.vdim = V;
    vra_stack_delta_prep(d, stream);
    vra_stack_conv_state_update(d, stream);
    StkScanArgs sc;
    sc.q = rec_, sc.ldq = C, sc.k = rec_ + G * D, sc.ldk = C, sc.v = rec_ + 2 * G * D, sc.ldv = C, sc.qk_rep = H / G;
    sc.decay = d.decay_out, sc.ldd = H, sc.decay_per_head = 1, sc.beta = d.beta_out, sc.ldb = H;
    scan_common(sc, L, md, ro_);
    vra_stack_linear_scan(sc, stream);
    if (take_stack_err(error, "delta rule")) return false;
    return recurrent_tail(L, md, z_ + C + 2 * H, n1, 1, L.o, o_, stream);
  }
  StkGemmArgs l1;
  l1.a = h_, l1.lda = W, l1.w = L.lr1, l1.M = T, l1.N = R, l1.K = W, l1.out = act_, l1.ldo = R;
  vra_stack_gemm(l1, dt_, stream);
  const int n2 = H * D + H * V;
  StkGemmArgs l2;
  l2.a = act_, l2.lda = R, l2.w = L.lr2, l2.M = T, l2.N = n2, l2.K = R, l2.out = z2_, l2.ldo = n2, l2.out_f32 = 1;
  vra_stack_gemm(l2, dt_, stream);
  StkDeltaPrepArgs d;
  d.raw = z_, d.ld = n1, d.raw2 = z2_, d.ld2 = n2, d.conv_w = L.conv_w, d.taps = L.conv, d.conv_state = L.conv_state ? L.conv_state : z2_;
  d.rate = L.rate, d.dt_bias = L.dt_bias, d.q_scale = 1.f / sqrtf((float)D);
  d.qkv_out = rec_, d.beta_out = rec_ + (size_t)T * C, d.decay_out = rec_ + (size_t)T * (C + H);
  d.positions = md.positions, d.cu_q = md.is_prefill ? md.cu_seqlens_q : nullptr, d.state_slots = md.state_slots;
  d.T = T, d.B = md.n_seqs, d.H = H, d.G = G, d.dim = D, d.vdim = V;
  vra_stack_delta_prep(d, stream);
  vra_stack_conv_state_update(d, stream);
  StkScanArgs sc;
  sc.q = rec_, sc.ldq = C, sc.k = rec_ + G * D, sc.ldk = C, sc.v = rec_ + 2 * G * D, sc.ldv = C, sc.qk_rep = H / G;
  sc.decay = d.decay_out, sc.ldd = H * D, sc.beta = d.beta_out, sc.ldb = H;
  scan_common(sc, L, md, ro_);
  vra_stack_linear_scan(sc, stream);
  if (take_stack_err(error, "delta rule")) return false;
  return recurrent_tail(L, md, z2_ + H * D, n2, 2, L.o, o_, stream);
}

// retention: q | k | v | gate in one launch (f32), rotary on q and k with the key's scale, the recurrence with one decay per head
bool StackModel::mixer_retention(const StackLayer& L, const InputMetadata& md, int64_t stream) {
  const int T = md.n_tokens, W = width_, H = L.heads, D = L.dim, V = L.vdim, n1 = L.nqkv();
  StkGemmArgs p;
  p.a = h_, p.lda = W, p.w = L.qkv, p.M = T, p.N = n1, p.K = W, p.out = z_, p.ldo = n1, p.out_f32 = 1;
  vra_stack_gemm(p, dt_, stream);
  StkHeadPrepArgs hp;
  hp.raw = z_, hp.ld = n1, hp.q_off = 0, hp.k_off = H * D, hp.Hq = H, hp.Hk = H, hp.dim = D, hp.eps = eps_;
  hp.rot.freq_hi = L.freq_hi, hp.rot.freq_lo = L.freq_lo, hp.rot.pairs = L.rot_pairs, hp.rot.mag = 1.f;
  hp.k_scale = 1.f / sqrtf((float)D), hp.positions = md.positions;
  hp.q_out = rec_, hp.q_ld = 2 * H * D, hp.k_out = rec_ + H * D, hp.k_ld = 2 * H * D, hp.out_f32 = 1, hp.T = T;
  vra_stack_head_prep(hp, dt_, stream);
  StkScanArgs sc;
  sc.q = rec_, sc.ldq = 2 * H * D, sc.k = rec_ + H * D, sc.ldk = 2 * H * D, sc.v = z_ + 2 * H * D, sc.ldv = n1, sc.head_decay = L.head_decay;
  scan_common(sc, L, md, ro_);
  vra_stack_linear_scan(sc, stream);
  if (take_stack_err(error, "retention")) return false;
  return recurrent_tail(L, md, z_ + 2 * H * D + H * V, n1, 1, L.o, o_, stream);
}

// two branches on one input.  Left: softmax attention over the paged cache (biases in the projection's epilogue, per-head q / k norm and
// rotary in the launch that writes the cache rows, visibility inside blocks of `chunk` positions) -> o_.  Right: gated linear attention
// (decay per key channel sigmoid(z)^(1 / tau), z from a low-rank projection with a bias) -> sh_.  The caller sums them with their scales.
bool StackModel::mixer_parallel(const StackLayer& L, const InputMetadata& md, int64_t stream) {
  const int T = md.n_tokens, B = md.n_seqs, W = width_, n1 = L.nqkv(), H = L.heads, RH = L.r_heads, RD = L.r_dim, RV = L.r_vdim;
  const int lq = L.nq(), lk = L.nk(), lv = L.nv(), r0 = lq + lk + lv;
  StkGemmArgs p;
  p.a = h_, p.lda = W, p.w = L.qkv, p.bias = L.qkv_bias, p.M = T, p.N = n1, p.K = W, p.out = z_, p.ldo = n1, p.out_f32 = 1;
  vra_stack_gemm(p, dt_, stream);
  StkGemmArgs l1;
  l1.a = h_, l1.lda = W, l1.w = L.lr1, l1.M = T, l1.N = L.rank_a, l1.K = W, l1.out = act_, l1.ldo = L.rank_a;
  vra_stack_gemm(l1, dt_, stream);
  StkGemmArgs l2;
  l2.a = act_, l2.lda = L.rank_a, l2.w = L.lr2, l2.bias = L.lr2_bias, l2.M = T, l2.N = RH * RD, l2.K = L.rank_a, l2.out = z2_, l2.ldo = RH * RD, l2.out_f32 = 1;
  vra_stack_gemm(l2, dt_, stream);
  // left
  StkHeadPrepArgs hp;
  hp.raw = z_, hp.ld = n1, hp.q_off = 0, hp.k_off = lq, hp.v_off = lq + lk, hp.Hq = H, hp.Hk = L.kv_heads, hp.dim = L.dim, hp.nv = lv;
  hp.qn_w = L.qn_w, hp.kn_w = L.kn_w, hp.eps = eps_;
  hp.rot.freq_hi = L.freq_hi, hp.rot.freq_lo = L.freq_lo, hp.rot.pairs = L.rot_pairs, hp.rot.mag = 1.f;
  hp.positions = md.positions, hp.q_out = qkv_, hp.q_ld = lq, hp.k_out = kc_[L.cache], hp.k_ld = lk, hp.v_out = vc_[L.cache], hp.v_ld = lv;
  hp.slots = md.slot_mapping, hp.T = T;
  vra_stack_head_prep(hp, dt_, stream);
  StkAttnArgs a;
  a.q = qkv_, a.ldq = lq, a.out = attn_, a.kc = kc_[L.cache], a.vc = vc_[L.cache];
  a.positions = md.positions, a.block_tables = md.block_tables, a.context_lens = md.context_lens;
  a.cu_q = md.is_prefill ? md.cu_seqlens_q : nullptr;
  a.B = B, a.T = T, a.max_q = md.is_prefill ? md.max_seqlen_q : 1, a.H = H, a.G = L.kv_heads, a.dim = L.dim, a.vdim = L.vdim;
  a.BS = ec_.block_size, a.max_blocks = md.max_blocks, a.scale = L.scale, a.chunk = L.chunk;
  vra_stack_attention(a, dt_, stream);
  StkGemmArgs o;
  o.a = attn_, o.lda = H * L.vdim, o.w = L.o, o.M = T, o.N = W, o.K = H * L.vdim, o.out = o_, o.ldo = W, o.out_f32 = 1;
  vra_stack_gemm(o, dt_, stream);
  if (take_stack_err(error, "parallel mixer (attention)")) return false;
  // right
  vra_stack_sigmoid_pow(z2_, RH * RD, rec_, RH * RD, T, RH * RD, 1.f / L.tau, stream);
  StkScanArgs sc;
  sc.q = z_ + r0, sc.ldq = n1, sc.k = z_ + r0 + RH * RD, sc.ldk = n1, sc.v = z_ + r0 + 2 * RH * RD, sc.ldv = n1, sc.q_scale = 1.f / sqrtf((float)RD);
  sc.decay = rec_, sc.ldd = RH * RD;
  scan_common(sc, L, md, ro_);
  vra_stack_linear_scan(sc, stream);
  if (take_stack_err(error, "parallel mixer (linear attention)")) return false;
  return recurrent_tail(L, md, z_ + r0 + 2 * RH * RD + RH * RV, n1, 1, L.r_o, sh_, stream);
}

// embedding (+ token-pair table, + its norm), then per layer  x += N(mixer(N(x))),  x += N(ff(N(x))).  A sub-block's output is normed and
// added inside the launch that norms the next sub-block's input (and, before a mixture of experts, runs its router).
bool StackModel::forward_sandwich(const InputMetadata& md, int64_t stream) {
  const int T = md.n_tokens, W = width_;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (!md.state_slots || !md.prev_tokens) return error = "forward: this model needs the sequences' state slots and previous tokens", false;
  StkEmbedPairArgs e;
  e.ids = md.input_ids, e.positions = md.positions, e.cu_q = md.is_prefill ? md.cu_seqlens_q : nullptr, e.prev_tokens = md.prev_tokens;
  e.embed = embed_, e.table = pair_table_, e.buckets = pair_buckets_, e.mul_prev = pair_mul_prev_, e.mul_cur = pair_mul_cur_, e.scale = embed_scale_;
  e.norm_w = embed_norm_w_, e.eps = eps_, e.x = x_, e.T = T, e.B = md.n_seqs, e.W = W, e.V = vocab_;
  vra_stack_embed_pair(e, dt_, stream);
  if (take_stack_err(error, "embedding")) return false;
  StkSandwichArgs pend;  // the parts of the last sub-block's output, not yet normed and added (post_w null: none)
  auto seam = [&](const float* pre_w, const float* pre_b, float pre_alpha, const StackLayer* router) {
    StkSandwichArgs s = pend;
    s.x = x_, s.pre_w = pre_w, s.pre_b = pre_b, s.pre_alpha = pre_alpha, s.dyt = norm_kind_ == 1, s.h = h_, s.eps = eps_, s.T = T, s.W = W;
    if (router) {
      s.router_w = router->router, s.router_bias = router->router_bias, s.n_router = router->experts + router->n_identity, s.top = router->top;
      s.pair_expert = pair_expert_, s.pair_weight = pair_weight_;
      if (router->router_kind == 2) {
        s.router_kind = 1, s.n_groups = router->n_groups, s.keep = router->keep, s.n_identity = router->n_identity;
        if (router->n_identity > 0) s.h32 = h32_, s.id_weight = id_weight_;
      }
    }
    if (s.post_w || s.pre_w) vra_stack_sandwich_norm(s, dt_, stream);
    pend = StkSandwichArgs();
    return !take_stack_err(error, "norm");
  };
  for (size_t li = 0; li < layers_.size(); li++) {
    const StackLayer& L = layers_[li];
    if (!seam(L.norm_w, L.norm_b, L.norm_alpha, nullptr)) return false;
    bool ok = false;
    switch (L.mixer) {
      case 3: ok = mixer_delta(L, md, stream); break;
      case 4: ok = mixer_retention(L, md, stream); break;
      case 6: ok = mixer_lightning(L, md, stream); break;
      default: ok = L.right_kind == 1 ? mixer_hybrid(L, md, stream) : mixer_parallel(L, md, stream); break;
    }
    if (!ok) return false;
    pend.p1 = o_, pend.n1 = 1, pend.post_w = L.post1_w, pend.post_b = L.post1_b, pend.post_alpha = L.post1_alpha;
    if (L.mixer == 5) {
      pend.c1 = L.left_scale, pend.p2 = sh_, pend.c2 = L.right_scale;
      if (L.branch_norm) pend.p1_norm_w = L.left_out_w, pend.p2_norm_w = L.right_out_w;
    }
    if (L.mlp == 2) {
      if (!seam(L.norm2_w, L.norm2_b, L.norm2_alpha, &L)) return false;
      const int P = T * L.top;
      const int granule = vra_stack_gemm_granule(P, L.experts);
      const int rows = round_up(P + L.experts * (granule - 1), granule);
      if (rows > max_rows_) return error = "feed-forward: more expert rows than the buffers hold", false;
      vra_stack_moe_sort(pair_expert_, pair_weight_, P, L.top, L.experts, granule, rows, row_token_, row_scale_, row_pair_, tile_group_, stream);
      if (take_stack_err(error, "expert rows")) return false;
      // (the weights of a softmax router multiply the experts' OUTPUTS: the rows go in unscaled, the sum over a token's pairs carries them)
      if (!expert_pair(h_, W, L.e_gu, (int64_t)2 * L.ffp * W, L.e_down, (int64_t)W * L.ffp, rows, L.ffp, L.ff, L.limit, tile_group_, granule, row_token_,
                       L.router_kind >= 1 ? nullptr : row_scale_, row_pair_, pair_out_, stream, L.act_kind))
        return false;
      pend.p1 = pair_out_, pend.n1 = L.top, pend.pw = L.router_kind >= 1 ? pair_weight_ : nullptr;
      pend.post_w = L.post2_w, pend.post_b = L.post2_b, pend.post_alpha = L.post2_alpha;
      if (L.router_kind == 2 && L.n_identity > 0) {  // an identity expert's pair has no row: its weight times the feed-forward's own input
        pend.pe = pair_expert_, pend.p2 = h32_, pend.p2w = id_weight_, pend.c2 = 1.f;
      }
    } else if (L.mlp == 4) {
      if (!seam(L.norm2_w, L.norm2_b, L.norm2_alpha, nullptr)) return false;
      if (!expert_pair(h_, W, L.s_gu, 0, L.s_down, 0, T, L.sffp, L.ff, L.limit, nullptr, 0, nullptr, nullptr, nullptr, pair_out_, stream, 0)) return false;
      pend.p1 = pair_out_, pend.n1 = 1, pend.post_w = L.post2_w, pend.post_b = L.post2_b, pend.post_alpha = L.post2_alpha;
    }
    if (trace_on_ || li + 1 == layers_.size()) {
      if (!seam(nullptr, nullptr, 1.f, nullptr)) return false;
      if (trace_on_ && hipMemcpyAsync(trace_ + li * (size_t)T * W, x_, (size_t)T * W * 4, hipMemcpyDeviceToDevice, st) != hipSuccess)
        return error = "layer trace copy failed", false;
    }
  }
  return true;
}

// lightning: q | k | v | gate in one launch (f32); q, k, v pass silu on their way into the recurrence (one constant decay per head);
// one norm over the concatenated heads, sigmoid gate, output projection
bool StackModel::mixer_lightning(const StackLayer& L, const InputMetadata& md, int64_t stream) {
  const int T = md.n_tokens, W = width_, H = L.heads, D = L.dim, V = L.vdim, n1 = L.nqkv();
  StkGemmArgs p;
  p.a = h_, p.lda = W, p.w = L.qkv, p.M = T, p.N = n1, p.K = W, p.out = z_, p.ldo = n1, p.out_f32 = 1;
  vra_stack_gemm(p, dt_, stream);
  StkScanArgs sc;
  sc.q = z_, sc.ldq = n1, sc.k = z_ + H * D, sc.ldk = n1, sc.v = z_ + 2 * H * D, sc.ldv = n1, sc.head_decay = L.head_decay, sc.act_silu = 1;
  scan_common(sc, L, md, ro_);
  vra_stack_linear_scan(sc, stream);
  if (take_stack_err(error, "lightning")) return false;
  vra_stack_head_norm_gate(ro_, L.out_norm_w, z_ + 2 * H * D + H * V, n1, 2, eps_, attn_, T, 1, H * V, dt_, stream);
  StkGemmArgs o;
  o.a = attn_, o.lda = H * V, o.w = L.o, o.M = T, o.N = W, o.K = H * V, o.out = o_, o.ldo = W, o.out_f32 = 1;
  vra_stack_gemm(o, dt_, stream);
  return !take_stack_err(error, "lightning");
}

// two branches on one input, each with a norm of its own in the seam that follows.  Left: softmax attention over the paged cache (biases
// in the projection's epilogue; per-head q / k norm and rotary on neighbouring pairs in the launch that writes the cache rows; sliding
// window, sink, per-head temperature and the per-head sigmoid output gate inside the attention) -> o_.  Right: gelu branch times a
// real-gated diagonal recurrence behind a short convolution; its gates are block-diagonal products in f32 -> sh_.
bool StackModel::mixer_hybrid(const StackLayer& L, const InputMetadata& md, int64_t stream) {
  const int T = md.n_tokens, B = md.n_seqs, W = width_, n1 = L.nqkv(), H = L.heads, Wr = L.r_width, nb = L.r_blocks, bw = Wr / nb;
  const int lq = L.nq(), lk = L.nk(), lv = L.nv(), g0 = lq + lk + lv, y0 = g0 + (L.head_gate ? H : 0), x0 = y0 + Wr;
  StkGemmArgs p;
  p.a = h_, p.lda = W, p.w = L.qkv, p.bias = L.qkv_bias, p.M = T, p.N = n1, p.K = W, p.out = z_, p.ldo = n1, p.out_f32 = 1;
  vra_stack_gemm(p, dt_, stream);
  // left
  StkHeadPrepArgs hp;
  hp.raw = z_, hp.ld = n1, hp.q_off = 0, hp.k_off = lq, hp.v_off = lq + lk, hp.Hq = H, hp.Hk = L.kv_heads, hp.dim = L.dim, hp.nv = lv;
  hp.qn_w = L.qn_w, hp.kn_w = L.kn_w, hp.eps = eps_;
  hp.rot.freq_hi = L.freq_hi, hp.rot.freq_lo = L.freq_lo, hp.rot.pairs = L.rot_pairs, hp.rot.mag = L.rot_mag, hp.rot_pairs_layout = L.rot_layout;
  hp.positions = md.positions, hp.q_out = qkv_, hp.q_ld = lq, hp.k_out = kc_[L.cache], hp.k_ld = lk, hp.v_out = vc_[L.cache], hp.v_ld = lv;
  hp.slots = md.slot_mapping, hp.T = T;
  vra_stack_head_prep(hp, dt_, stream);
  StkAttnArgs a;
  a.q = qkv_, a.ldq = lq, a.out = attn_, a.kc = kc_[L.cache], a.vc = vc_[L.cache];
  a.positions = md.positions, a.block_tables = md.block_tables, a.context_lens = md.context_lens;
  a.cu_q = md.is_prefill ? md.cu_seqlens_q : nullptr;
  a.B = B, a.T = T, a.max_q = md.is_prefill ? md.max_seqlen_q : 1, a.H = H, a.G = L.kv_heads, a.dim = L.dim, a.vdim = L.vdim;
  a.BS = ec_.block_size, a.max_blocks = md.max_blocks, a.scale = L.scale, a.chunk = L.chunk, a.window = L.window;
  a.sink = L.sink ? L.sink_w : nullptr, a.head_scale = L.head_temp ? L.temp_w : nullptr;
  if (L.head_gate) a.gate = z_ + g0, a.gate_ld = n1;
  vra_stack_attention(a, dt_, stream);
  StkGemmArgs o;
  o.a = attn_, o.lda = H * L.vdim, o.w = L.o, o.M = T, o.N = W, o.K = H * L.vdim, o.out = o_, o.ldo = W, o.out_f32 = 1;
  vra_stack_gemm(o, dt_, stream);
  if (take_stack_err(error, "parallel mixer (attention)")) return false;
  // right
  StkConvArgs cv;
  cv.x = z_ + x0, cv.ld = n1, cv.C = Wr, cv.taps = L.conv, cv.w = L.conv_w, cv.bias = L.conv_b, cv.conv_state = L.conv_state, cv.y = rec_, cv.ldy = Wr;
  cv.positions = md.positions, cv.cu_q = md.is_prefill ? md.cu_seqlens_q : nullptr, cv.state_slots = md.state_slots, cv.T = T, cv.B = B;
  vra_stack_conv_rows(cv, stream);
  vra_stack_conv_rows_update(cv, stream);
  StkGemmArgs g;  // per block: [T, bw] x [2 bw, bw]^T -> both gates' logits, f32 whatever the model's type
  g.a = rec_, g.lda = Wr, g.a_batch_stride = bw, g.w = L.gates_w, g.w_batch_stride = (int64_t)2 * bw * bw, g.batch = nb;
  g.bias = L.gates_b, g.bias_batch_stride = 2 * bw, g.M = T, g.N = 2 * bw, g.K = bw, g.out = z2_, g.ldo = 2 * Wr, g.out_batch_stride = 2 * bw, g.out_f32 = 1;
  vra_stack_gemm(g, VRA_F32, stream);
  StkGatedScanArgs gs;
  gs.u = rec_, gs.ldu = Wr, gs.gr = z2_, gs.gi = z2_ + bw, gs.ldg = 2 * Wr, gs.y = z_ + y0, gs.ldy = n1, gs.lam = L.lam, gs.rate = 8.f;
  gs.state = L.state, gs.state_slots = md.state_slots, gs.positions = md.positions, gs.cu_q = cv.cu_q, gs.out = attn_, gs.ldo = Wr, gs.B = B, gs.C = Wr;
  gs.block = bw;
  vra_stack_gated_scan(gs, T, dt_, stream);
  StkGemmArgs ro;
  ro.a = attn_, ro.lda = Wr, ro.w = L.r_o, ro.M = T, ro.N = W, ro.K = Wr, ro.out = sh_, ro.ldo = W, ro.out_f32 = 1;
  vra_stack_gemm(ro, dt_, stream);
  return !take_stack_err(error, "parallel mixer (gated recurrence)");
}

int64_t StackModel::read_layer_trace(void* host, int64_t max_bytes, int64_t stream) {
  if (!trace_ || !host || (int64_t)trace_bytes_ > max_bytes) return -1;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (hipMemcpyAsync(host, trace_, trace_bytes_, hipMemcpyDeviceToHost, st) != hipSuccess || hipStreamSynchronize(st) != hipSuccess) return -1;
  return (int64_t)trace_bytes_;
}

}  // namespace vra
