// stack_recurrent.hip — operators of sandwich-norm layer stacks whose mixers carry a state from token to token (host/stack_model.cpp; each is
// specified in stack_launch.h), gfx950: the embedding with a hashed token-pair table, the seam between two sub-blocks (norm of a sub-block's
// output, residual sum, norm of the next one's input, router), per-head norm / rotary / cache rows, the inputs of a gated delta rule
// (short convolutions with their state, unit vectors, step sizes and decays), the linear recurrence itself and its output norm and gate.
//
// Everything here is f32 except what is stored for a matrix product (h, q, cache rows, the gated output): norms, routers, angles, decays and
// their logarithms, the recurrent state and all that enters it.  Tokens of a sequence pass the recurrence one after the other in one fixed
// order of operations, and a sequence's state sits in its slot between steps, so a token's result does not depend on how its prompt was cut,
// on the rest of the batch or on the slot.
#include <algorithm>

#include "stack_common.cuh"
#include "stack_launch.h"

namespace {

__device__ __forceinline__ float softplusf_(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }
__device__ __forceinline__ float siluf_(float z) { return z / (1.f + expf(-z)); }

// sequence of row t in a step whose rows are cut by cu_q [B + 1] (cu_q null: one row per sequence)
__device__ __forceinline__ int seq_of_row(const uint32_t* cu_q, int B, int t) {
  if (!cu_q) return t;
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if ((int)cu_q[mid] <= t) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

// ------------------------------------------------------------------------------------------------ embedding + token-pair table + norm
template <typename T>
__global__ __launch_bounds__(256) void stk_embed_pair_kernel(StkEmbedPairArgs a) {
  extern __shared__ float lds[];
  __shared__ float red[4];
  float* xs = lds;
  const int t = blockIdx.x, W = a.W, tid = threadIdx.x;
  uint32_t id = a.ids[t];
  if (id >= (uint32_t)a.V) id = 0;
  const T* e = (const T*)a.embed + (size_t)id * W;
  const T* pr = nullptr;
  if (a.table) {
    const int b = seq_of_row(a.cu_q, a.B, t);
    const int t0 = a.cu_q ? (int)a.cu_q[b] : t;
    int64_t row = a.buckets;
    if (a.positions[t] > 0) {
      const uint32_t prev = t > t0 ? a.ids[t - 1] : a.prev_tokens[b];
      row = ((int64_t)prev * a.mul_prev + (int64_t)id * a.mul_cur) % (int64_t)a.buckets;
      if (row < 0) row += a.buckets;
    }
    pr = (const T*)a.table + (size_t)row * W;
  }
  float s = 0.f;
  for (int c = tid; c < W; c += 256) {
    float v = El<T>::ld(e + c) * a.scale;
    if (pr) v += El<T>::ld(pr + c);
    xs[c] = v;
    s = fmaf(v, v, s);
  }
  float* x = a.x + (size_t)t * W;
  if (!a.norm_w) {
    for (int c = tid; c < W; c += 256) x[c] = xs[c];
    return;
  }
  const float r = 1.f / sqrtf(block_sum_256(s, red) / (float)W + a.eps);
  for (int c = tid; c < W; c += 256) x[c] = xs[c] * r * a.norm_w[c];
}

// ------------------------------------------------------------------------------------------------ seam of two sub-blocks (+ router)
template <typename T>
__global__ __launch_bounds__(256) void stk_sandwich_kernel(StkSandwichArgs a) {
  extern __shared__ float lds[];
  __shared__ float red[4];
  float* xs = lds;             // [W]
  float* zs = lds + a.W;       // [n_router] logits / corrected scores, [n_router] scores, [n_groups] group scores
  const int t = blockIdx.x, W = a.W, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float* x = a.x + (size_t)t * W;
  if (a.post_w) {
    // a branch with a norm of its own: its row's root mean square first (f32, the same order of sums as every norm here)
    float r1 = 1.f, r2 = 1.f;
    if (a.p1_norm_w) {
      float q = 0.f;
      for (int c = tid; c < W; c += 256) {
        const float v = a.p1[(size_t)t * W + c];
        q = fmaf(v, v, q);
      }
      r1 = 1.f / sqrtf(block_sum_256(q, red) / (float)W + a.eps);
    }
    if (a.p2 && a.p2_norm_w) {
      float q = 0.f;
      for (int c = tid; c < W; c += 256) {
        const float v = a.p2[(size_t)t * W + c];
        q = fmaf(v, v, q);
      }
      r2 = 1.f / sqrtf(block_sum_256(q, red) / (float)W + a.eps);
    }
    const float w2 = a.p2w ? a.p2w[t] : 1.f;
    float s = 0.f;
    for (int c = tid; c < W; c += 256) {
      float v = 0.f;
      if (a.p1_norm_w) {
        v = a.p1[(size_t)t * W + c] * r1 * a.p1_norm_w[c];
      } else {
        for (int j = 0; j < a.n1; j++) {
          const size_t r = (size_t)t * a.n1 + j;
          if (a.pe && a.pe[r] < 0) continue;
          const float pv = a.p1[r * W + c];
          v = a.pw ? fmaf(a.pw[r], pv, v) : v + pv;
        }
      }
      v *= a.c1;
      if (a.p2) {
        float v2 = a.p2[(size_t)t * W + c];
        if (a.p2_norm_w) v2 = v2 * r2 * a.p2_norm_w[c];
        v = fmaf(a.c2 * w2, v2, v);
      }
      xs[c] = v;
      s = fmaf(v, v, s);
    }
    if (a.dyt) {
      for (int c = tid; c < W; c += 256) {
        const float v = x[c] + (tanhf(a.post_alpha * xs[c]) * a.post_w[c] + a.post_b[c]);
        x[c] = v;
        xs[c] = v;
      }
    } else {
      const float r = 1.f / sqrtf(block_sum_256(s, red) / (float)W + a.eps);
      for (int c = tid; c < W; c += 256) {
        const float v = x[c] + xs[c] * r * a.post_w[c];
        x[c] = v;
        xs[c] = v;
      }
    }
  } else {
    for (int c = tid; c < W; c += 256) xs[c] = x[c];
  }
  if (!a.pre_w) return;
  float r = 1.f;
  if (!a.dyt) {
    float s = 0.f;
    for (int c = tid; c < W; c += 256) s = fmaf(xs[c], xs[c], s);
    r = 1.f / sqrtf(block_sum_256(s, red) / (float)W + a.eps);
  }
  T* h = (T*)a.h + (size_t)t * W;
  for (int c = tid; c < W; c += 256) {
    const float v = a.dyt ? tanhf(a.pre_alpha * xs[c]) * a.pre_w[c] + a.pre_b[c] : xs[c] * r * a.pre_w[c];
    xs[c] = v;
    El<T>::st(h + c, v);
    if (a.h32) a.h32[(size_t)t * W + c] = v;
  }
  if (!a.router_w) return;
  __syncthreads();
  const T* rw = (const T*)a.router_w;
  // a wave takes EB outputs at a time and requests their weights together: the rows of one output after the other would each wait for
  // their own trip to memory.  An output's sum keeps its order (a lane's columns ascending, then the lanes).
  constexpr int EB = 8;
  const bool vec8 = sizeof(T) == 2 && W % 8 == 0 && ((uintptr_t)rw % 16) == 0;  // 8 weights a load
  for (int e0 = wave * EB; e0 < a.n_router; e0 += 4 * EB) {
    float z[EB];
#pragma unroll
    for (int u = 0; u < EB; u++) z[u] = 0.f;
    if (vec8) {
      for (int c = lane * 8; c < W; c += 64 * 8) {
        u32x4 v[EB];
#pragma unroll
        for (int u = 0; u < EB; u++) v[u] = *(const u32x4*)((const uint16_t*)rw + (size_t)min(e0 + u, a.n_router - 1) * W + c);
#pragma unroll
        for (int u = 0; u < EB; u++)
          for (int i = 0; i < 4; i++) {
            z[u] = fmaf(xs[c + 2 * i], __uint_as_float(v[u][i] << 16), z[u]);
            z[u] = fmaf(xs[c + 2 * i + 1], __uint_as_float(v[u][i] & 0xffff0000u), z[u]);
          }
      }
    } else {
      for (int c = lane; c < W; c += 64) {
        float wv[EB];
#pragma unroll
        for (int u = 0; u < EB; u++) wv[u] = El<T>::ld(rw + (size_t)min(e0 + u, a.n_router - 1) * W + c);
#pragma unroll
        for (int u = 0; u < EB; u++) z[u] = fmaf(xs[c], wv[u], z[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < EB; u++) {
      const float zu = wave_sum(z[u]);
      const int e = e0 + u;
      if (lane == 0 && e < a.n_router) zs[e] = zu + (a.router_kind == 0 && a.router_bias ? a.router_bias[e] : 0.f);
    }
  }
  __syncthreads();
  const int n = a.n_router;
  if (a.router_kind == 0) {  // the `top` largest in turn (ties: the lower index); a picked logit leaves the list
    if (tid != 0) return;
    float zmax = 0.f, sum = 0.f;
    for (int j = 0; j < a.top; j++) {
      int best = 0;
      float bz = zs[0];
      for (int e = 1; e < n; e++)
        if (zs[e] > bz) best = e, bz = zs[e];
      zs[best] = -INFINITY;
      if (j == 0) zmax = bz;  // (the first pick is the largest logit)
      const float w = expf(bz - zmax);
      a.pair_expert[(size_t)t * a.top + j] = best;
      a.pair_weight[(size_t)t * a.top + j] = w;
      sum += w;
    }
    const float inv = 1.f / sum;
    for (int j = 0; j < a.top; j++) a.pair_weight[(size_t)t * a.top + j] *= inv;
    return;
  }
  // Scores over all outputs; corrected scores choose, restricted to the best groups; the plain scores weigh.  The outputs are spread
  // over the lanes of wave 0 (their corrections are fetched side by side, not one after the other), the groups over the threads.
  float* sc = zs + n;        // [n] scores
  float* gs = zs + 2 * n;    // [n_groups]
  if (wave == 0) {
    float m = -INFINITY, sum = 0.f;
    for (int e = lane; e < n; e += 64) m = fmaxf(m, zs[e]);
    m = wave_max(m);
    for (int e = lane; e < n; e += 64) {
      const float ex = expf(zs[e] - m);
      sc[e] = ex;
      sum += ex;
    }
    const float inv = 1.f / wave_sum(sum);
    for (int e = lane; e < n; e += 64) {
      const float sv = sc[e] * inv;
      sc[e] = sv;
      zs[e] = sv + (a.router_bias ? a.router_bias[e] : 0.f);
    }
  }
  __syncthreads();
  if (a.n_groups > 1 && a.keep < a.n_groups) {  // (uniform over the workgroup)
    const int per = n / a.n_groups;
    for (int g = tid; g < a.n_groups; g += 256) {
      float b = zs[g * per];
      for (int e = 1; e < per; e++) b = fmaxf(b, zs[g * per + e]);
      gs[g] = b;
    }
    __syncthreads();
    for (int g = tid; g < a.n_groups; g += 256) {  // a group stays if fewer than `keep` groups come before it (larger score, or equal and lower index)
      int before = 0;
      for (int o = 0; o < a.n_groups; o++) before += (gs[o] > gs[g] || (gs[o] == gs[g] && o < g)) ? 1 : 0;
      if (before >= a.keep)
        for (int e = 0; e < per; e++) zs[g * per + e] = -INFINITY;
    }
    __syncthreads();
  }
  const int n_real = n - a.n_identity;
  if (n <= 64) {  // one output a lane: a pick is a wave maximum and the lowest lane that holds it
    if (wave != 0) return;
    const bool have = lane < n;
    const float val = have ? zs[lane] : 0.f, sv = have ? sc[lane] : 0.f;
    bool avail = have;
    float idw = 0.f;
    for (int j = 0; j < a.top; j++) {
      const float v = avail ? val : -INFINITY;
      const float m = wave_max(v);
      const unsigned long long holders = __ballot(avail && v == m);  // (left-out groups hold -inf: still chosen, in index order, once nothing else is left)
      const int best = __ffsll((long long)holders) - 1;
      const float w = __shfl(sv, best, 64);
      if (lane == best) avail = false;
      const bool ident = best >= n_real;
      if (lane == 0) {
        a.pair_expert[(size_t)t * a.top + j] = ident ? -1 : best;
        a.pair_weight[(size_t)t * a.top + j] = w;
      }
      if (ident) idw += w;
    }
    if (lane == 0 && a.id_weight) a.id_weight[t] = idw;
    return;
  }
  if (tid != 0) return;
  float idw = 0.f;
  for (int j = 0; j < a.top; j++) {
    int best = -1;
    float bz = -INFINITY;
    for (int e = 0; e < n; e++)
      if (sc[e] >= 0.f && (best < 0 || zs[e] > bz)) best = e, bz = zs[e];
    const float w = sc[best];
    sc[best] = -1.f;  // (picked: out of the list)
    const bool ident = best >= n_real;
    a.pair_expert[(size_t)t * a.top + j] = ident ? -1 : best;
    a.pair_weight[(size_t)t * a.top + j] = w;
    if (ident) idw += w;
  }
  if (a.id_weight) a.id_weight[t] = idw;
}

// ------------------------------------------------------------------------------------------------ per-head norm, rotary, cache rows
template <typename TO>
__global__ __launch_bounds__(256) void stk_head_prep_kernel(StkHeadPrepArgs a) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, dim = a.dim;
  const float* raw = a.raw + (size_t)t * a.ld;
  const float p = (float)a.positions[t];
  const int64_t slot = a.slots ? a.slots[t] : (int64_t)t;
  const int rp = a.rot.pairs;
  for (int hh = blockIdx.y * 4 + wave; hh < a.Hq + a.Hk; hh += 4 * gridDim.y) {
    const bool is_q = hh < a.Hq;
    const int h = is_q ? hh : hh - a.Hq;
    if (!is_q && slot < 0) continue;
    const float* src = raw + (is_q ? a.q_off : a.k_off) + h * dim;
    const float* nw = is_q ? a.qn_w : a.kn_w;
    float r = 1.f;
    if (nw) {
      float s = 0.f;
      for (int c = lane; c < dim; c += 64) s = fmaf(src[c], src[c], s);
      r = 1.f / sqrtf(wave_sum(s) / (float)dim + a.eps);
    }
    const float sc = is_q ? a.q_scale : a.k_scale;
    TO* dst = is_q ? (TO*)a.q_out + (size_t)t * a.q_ld + h * dim : (TO*)a.k_out + (size_t)slot * a.k_ld + h * dim;
    for (int c = lane; c < dim; c += 64) {
      float v = nw ? src[c] * r * nw[c] : src[c];
      if (c < 2 * rp) {
        const bool first = a.rot_pairs_layout ? (c & 1) == 0 : c < rp;
        const int i = a.rot_pairs_layout ? c >> 1 : (c < rp ? c : c - rp);
        const int oc = a.rot_pairs_layout ? c ^ 1 : (c < rp ? c + rp : c - rp);
        const float o = nw ? src[oc] * r * nw[oc] : src[oc];
        float cs, sn;
        rot_cos_sin(a.rot, i, p, &cs, &sn);
        v = first ? v * cs - o * sn : v * cs + o * sn;
      }
      El<TO>::st(dst + c, v * sc);
    }
  }
  if (a.v_out && slot >= 0) {
    TO* dst = (TO*)a.v_out + (size_t)slot * a.v_ld;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < a.nv; c += 256 * gridDim.y) El<TO>::st(dst + c, raw[a.v_off + c]);
  }
}

// ------------------------------------------------------------------------------------------------ inputs of the gated delta rule
__global__ __launch_bounds__(256) void stk_delta_prep_kernel(StkDeltaPrepArgs a) {
  extern __shared__ float lds[];
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int H = a.H, G = a.G, dim = a.dim, vdim = a.vdim, nqk = G * dim, C = 2 * nqk + H * vdim, taps = a.taps;
  float* ys = lds;  // [C] the convolved, activated row
  const int b = seq_of_row(a.cu_q, a.B, t);
  const int slot = a.state_slots[b];
  if (slot < 0) return;
  const int t0 = a.cu_q ? (int)a.cu_q[b] : t;
  const int i = t - t0;                                   // place of the row in its sequence's part of the step
  const bool fresh = a.positions[t0] == 0;                // the sequence starts in this step: nothing before its first row
  const float* cs = a.conv_state + (size_t)slot * (taps - 1) * C;
  // tap j of a row reads the input taps - 1 - j places back: a row of this step, the slot's kept inputs, or nothing (a sequence's start).
  // Every address is valid whatever the case (the weight of a load that does not count is 0), so no load waits for a branch; four
  // channels go side by side.
  for (int c0 = tid; c0 < C; c0 += 4 * 256) {
    float y[4] = {0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < taps; j++) {
      const int e = i - (taps - 1) + j;
      const bool from_step = e >= 0, counts = from_step || (!fresh && taps > 1);
      const float* src = from_step ? a.raw + (size_t)(t0 + e) * a.ld : (counts ? cs + (size_t)(taps - 1 + e) * C : a.raw + (size_t)t * a.ld);
#pragma unroll
      for (int u = 0; u < 4; u++) {
        const int c = min(c0 + u * 256, C - 1);
        const float wv = counts ? a.conv_w[(size_t)c * taps + j] : 0.f;
        y[u] = fmaf(wv, src[c], y[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < 4; u++)
      if (c0 + u * 256 < C) ys[c0 + u * 256] = siluf_(y[u]);
  }
  __syncthreads();
  float* out = a.qkv_out + (size_t)t * C;
  for (int hh = wave; hh < 2 * G; hh += 4) {  // q heads, then k heads: unit vectors
    const float* src = ys + hh * dim;
    float s = 0.f;
    for (int c = lane; c < dim; c += 64) s = fmaf(src[c], src[c], s);
    const float r = (hh < G ? a.q_scale : 1.f) / sqrtf(wave_sum(s) + 1e-6f);
    for (int c = lane; c < dim; c += 64) out[hh * dim + c] = src[c] * r;
  }
  for (int c = tid; c < H * vdim; c += 256) out[2 * nqk + c] = ys[2 * nqk + c];
  for (int h = tid; h < H; h += 256) a.beta_out[(size_t)t * H + h] = sigmoidf_(a.raw[(size_t)t * a.ld + C + h]);
  const int dd = a.decay_dim == 1 ? 1 : dim;
  for (int c = tid; c < H * dd; c += 256)
    a.decay_out[(size_t)t * H * dd + c] = expf(-a.rate[c / dd] * softplusf_(a.raw2[(size_t)t * a.ld2 + c] + a.dt_bias[c]));
}

// the last taps - 1 inputs of every sequence of the step -> its slot (after the step's rows have read what the slot held)
__global__ __launch_bounds__(256) void stk_conv_state_update_kernel(StkDeltaPrepArgs a) {
  const int b = blockIdx.x;
  const int slot = a.state_slots[b];
  if (slot < 0) return;
  const int C = 2 * a.G * a.dim + a.H * a.vdim, taps = a.taps;
  const int t0 = a.cu_q ? (int)a.cu_q[b] : b, n = a.cu_q ? (int)a.cu_q[b + 1] - t0 : 1;
  const bool fresh = a.positions[t0] == 0;
  float* cs = a.conv_state + (size_t)slot * (taps - 1) * C;
  for (int c = threadIdx.x; c < C; c += 256)
    for (int r = 0; r < taps - 1; r++) {  // row r: the input taps - 1 - r places before the next token (rows are read above where they are written)
      const int e = n - (taps - 1) + r;
      float v = 0.f;
      if (e >= 0) v = a.raw[(size_t)(t0 + e) * a.ld + c];
      else if (!fresh) v = cs[(size_t)(taps - 1 + e) * C + c];
      cs[(size_t)r * C + c] = v;
    }
}

__global__ __launch_bounds__(256) void stk_sigmoid_pow_kernel(const float* z, int ldz, float* out, int ldo, int n, int64_t total, float inv_tau) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t t = i / n;
    const int c = (int)(i % n);
    out[t * ldo + c] = expf(-softplusf_(-z[t * ldz + c]) * inv_tau);
  }
}

// ------------------------------------------------------------------------------------------------ the linear recurrence
// A workgroup owns 256 / P columns of one head's state (a column = one value channel); a column's `dim` rows are spread over P
// neighbouring lanes, R rows each, in registers for the whole step.  Sums over the rows (S^T k, S^T q) add a lane's R products in order,
// then the P lanes by xor shuffles: an order fixed by `dim` alone.  q, k and the decays of TT tokens are staged in LDS once for all
// columns.
// sum over the P neighbouring lanes that share a column (P a power of two, lanes aligned to P), left in all of them.  Inside a row of 16
// lanes the partner comes by DPP (quad permutes, then mirrors of half a row and of a row: after each step the lanes of a group hold one
// value, so a mirror is as good as an xor); beyond 16 lanes by a cross-lane read.  One fixed order for a given P.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int P>
__device__ __forceinline__ float group_sum(float v) {
  if (P >= 2) v += dpp_f32<0xB1>(v);    // quad_perm [1, 0, 3, 2]
  if (P >= 4) v += dpp_f32<0x4E>(v);    // quad_perm [2, 3, 0, 1]
  if (P >= 8) v += dpp_f32<0x141>(v);   // row_half_mirror
  if (P >= 16) v += dpp_f32<0x140>(v);  // row_mirror
  if (P >= 32) v += __shfl_xor(v, 16, 64);
  return v;
}

// P, the presence of per-row decays and of the delta rule are template parameters: the 16 tokens of a tile are one straight line of code, so
// the LDS reads of the tokens ahead are in flight while a token's sums run.
// DECAY 0: one constant per head; 1: one per row and key channel; 2: one per row and head.  ACT: q, k, v pass silu on their way into LDS.
template <int R, int P, int DECAY, bool BETA, bool ACT>
__global__ __launch_bounds__(256) void stk_linear_scan_kernel(StkScanArgs a) {
  constexpr int TT = 16, NL = 4;     // tokens a tile; 16-byte loads a thread and array for one tile (TT * dimP / 4 / 256, dimP <= 256)
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int dimP = P * R, CPB = 256 / P, d4n = dimP / 4;
  const int dim = a.dim, vdim = a.vdim;
  float* ks = lds;                   // [TT][dimP]
  float* qs = ks + TT * dimP;        // [TT][dimP]
  float* ds = qs + TT * dimP;        // [TT][dimP]
  float* vs = ds + TT * dimP;        // [TT][CPB]
  float* bs = vs + TT * CPB;         // [TT]
  float* gs = bs + TT;               // [TT] one decay per token (DECAY 2)
  const int b = blockIdx.z, h = blockIdx.y, hq = h / a.qk_rep, tid = threadIdx.x;
  const int slot = a.state_slots[b];
  if (slot < 0) return;
  const int r = tid % P, cl = tid / P, c = blockIdx.x * CPB + cl;
  const bool col = c < vdim;
  const int t0 = a.cu_q ? (int)a.cu_q[b] : b, n = a.cu_q ? (int)a.cu_q[b + 1] - t0 : 1;
  const bool fresh = a.positions[t0] == 0;
  float* sp = a.state + (((size_t)slot * a.H + h) * vdim + (col ? c : 0)) * dim + r * R;
  float S[R];
#pragma unroll
  for (int j = 0; j < R; j++) S[j] = (!fresh && col && r * R + j < dim) ? sp[j] : 0.f;
  const float hd = a.head_decay ? a.head_decay[h] : 1.f;
  // rows of dim floats that start on 16 bytes are fetched four floats a load
  const bool vec = dim % 4 == 0 && a.ldk % 4 == 0 && a.ldq % 4 == 0 && (DECAY != 1 || a.ldd % 4 == 0) && ((uintptr_t)a.k % 16) == 0 && ((uintptr_t)a.q % 16) == 0 &&
                   (DECAY != 1 || ((uintptr_t)a.decay % 16) == 0);
  // A tile's q, k, decays, values and write strengths travel global memory -> registers -> LDS; the registers of the NEXT tile are requested
  // before the current tile's tokens run, so their way from memory lies beside the arithmetic.
  float4 kn[NL], qn[NL], dn[NL];
  float vbuf[16], bn = 0.f, gn = 1.f;
  constexpr int vcount = TT * CPB;     // values of a tile: a thread takes elements tid, tid + 256, ... (at most 16)
  auto row4 = [&](const float* base, int ld, int hh, size_t t, int d, float fill) {
    const float* p = base + t * ld + hh * dim + d;
    if (vec && d + 3 < dim) return *(const float4*)p;
    float4 o;
    o.x = d < dim ? p[0] : fill, o.y = d + 1 < dim ? p[1] : fill, o.z = d + 2 < dim ? p[2] : fill, o.w = d + 3 < dim ? p[3] : fill;
    return o;
  };
  auto request = [&](int i0) {
    const int nt = min(TT, n - i0);
#pragma unroll
    for (int u = 0; u < NL; u++) {
      const int e = tid + u * 256, i = e / d4n, d = (e % d4n) * 4;
      kn[u] = qn[u] = make_float4(0.f, 0.f, 0.f, 0.f), dn[u] = make_float4(1.f, 1.f, 1.f, 1.f);
      if (e < TT * d4n && i < nt) {
        const size_t t = (size_t)(t0 + i0 + i);
        kn[u] = row4(a.k, a.ldk, hq, t, d, 0.f);
        qn[u] = row4(a.q, a.ldq, hq, t, d, 0.f);
        if (DECAY == 1) dn[u] = row4(a.decay, a.ldd, h, t, d, 1.f);
      }
    }
#pragma unroll
    for (int u = 0; u < 16; u++) {
      const int e = tid + u * 256;
      if (e < vcount) {
        const int i = e / CPB, cc = blockIdx.x * CPB + e % CPB;
        vbuf[u] = (i < nt && cc < vdim) ? a.v[(size_t)(t0 + i0 + i) * a.ldv + h * vdim + cc] : 0.f;
      }
    }
    if (BETA && tid < nt) bn = a.beta[(size_t)(t0 + i0 + tid) * a.ldb + h];
    if (DECAY == 2 && tid < nt) gn = a.decay[(size_t)(t0 + i0 + tid) * a.ldd + h];
  };
  auto deposit = [&]() {
#pragma unroll
    for (int u = 0; u < NL; u++) {
      const int e = tid + u * 256;
      if (e < TT * d4n) {
        float4 kk = kn[u], qv = qn[u];
        if (ACT) {
          kk.x = siluf_(kk.x), kk.y = siluf_(kk.y), kk.z = siluf_(kk.z), kk.w = siluf_(kk.w);
          qv.x = siluf_(qv.x), qv.y = siluf_(qv.y), qv.z = siluf_(qv.z), qv.w = siluf_(qv.w);
        }
        *(float4*)(ks + e * 4) = kk;
        qv.x *= a.q_scale, qv.y *= a.q_scale, qv.z *= a.q_scale, qv.w *= a.q_scale;
        *(float4*)(qs + e * 4) = qv;
        if (DECAY == 1) *(float4*)(ds + e * 4) = dn[u];
      }
    }
#pragma unroll
    for (int u = 0; u < 16; u++) {
      const int e = tid + u * 256;
      if (e < vcount) vs[e] = ACT ? siluf_(vbuf[u]) : vbuf[u];
    }
    if (BETA && tid < TT) bs[tid] = bn;
    if (DECAY == 2 && tid < TT) gs[tid] = gn;
  };
  request(0);
  for (int i0 = 0; i0 < n; i0 += TT) {
    const int nt = min(TT, n - i0);
    __syncthreads();
    deposit();
    __syncthreads();
    if (i0 + TT < n) request(i0 + TT);
    // a token's operands come from LDS one token ahead of its arithmetic (two register sets, 16-byte reads)
    float kv[2][R], qv[2][R], dv[2][R], uv[2], bv[2], gv[2];
    auto fetch = [&](int i, int w) {
#pragma unroll
      for (int j = 0; j < R; j += 4) {
        const float4 k4 = *(const float4*)(ks + i * dimP + r * R + j), q4 = *(const float4*)(qs + i * dimP + r * R + j);
        kv[w][j] = k4.x, kv[w][j + 1] = k4.y, kv[w][j + 2] = k4.z, kv[w][j + 3] = k4.w;
        qv[w][j] = q4.x, qv[w][j + 1] = q4.y, qv[w][j + 2] = q4.z, qv[w][j + 3] = q4.w;
        if (DECAY == 1) {
          const float4 d4 = *(const float4*)(ds + i * dimP + r * R + j);
          dv[w][j] = d4.x, dv[w][j + 1] = d4.y, dv[w][j + 2] = d4.z, dv[w][j + 3] = d4.w;
        }
      }
      uv[w] = vs[i * CPB + cl];
      if (BETA) bv[w] = bs[i];
      if (DECAY == 2) gv[w] = gs[i];
    };
    auto token = [&](int i, int w) {
#pragma unroll
      for (int j = 0; j < R; j++) S[j] *= DECAY == 1 ? dv[w][j] : (DECAY == 2 ? gv[w] : hd);
      float u = uv[w];
      if (BETA) {
        float d0 = 0.f, d1 = 0.f;  // (two chains; their sum order is fixed)
#pragma unroll
        for (int j = 0; j < R; j += 2) d0 = fmaf(S[j], kv[w][j], d0), d1 = fmaf(S[j + 1], kv[w][j + 1], d1);
        u = bv[w] * (u - group_sum<P>(d0 + d1));
      }
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int j = 0; j < R; j += 2) {
        S[j] = fmaf(kv[w][j], u, S[j]), S[j + 1] = fmaf(kv[w][j + 1], u, S[j + 1]);
        o0 = fmaf(S[j], qv[w][j], o0), o1 = fmaf(S[j + 1], qv[w][j + 1], o1);
      }
      const float o_ = group_sum<P>(o0 + o1);
      if (r == 0 && col) a.out[(size_t)(t0 + i0 + i) * a.ldo + h * vdim + c] = o_;
    };
    fetch(0, 0);
    if (nt == TT) {
#pragma unroll
      for (int i = 0; i < TT; i++) {
        if (i + 1 < TT) fetch(i + 1, (i + 1) & 1);
        token(i, i & 1);
      }
    } else {
      for (int i = 0; i < nt; i++) {
        fetch(i, 0);
        token(i, 0);
      }
    }
  }
  if (col)
#pragma unroll
    for (int j = 0; j < R; j++)
      if (r * R + j < dim) sp[j] = S[j];
}

// ------------------------------------------------------------------------------------------------ per-head output norm and gate
template <typename T>
__global__ __launch_bounds__(256) void stk_head_norm_gate_kernel(const float* o, const float* w, const float* gate, int gate_ld, int gate_act, float eps,
                                                                 T* out, int H, int vdim) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (H == 1) {  // one norm over the whole row: the four waves share it
    __shared__ float red[4];
    const float* src = o + (size_t)t * vdim;
    float s = 0.f;
    for (int c = threadIdx.x; c < vdim; c += 256) s = fmaf(src[c], src[c], s);
    const float r = 1.f / sqrtf(block_sum_256(s, red) / (float)vdim + eps);
    for (int c = threadIdx.x; c < vdim; c += 256) {
      float v = src[c] * r;
      if (w) v *= w[c];
      if (gate) {
        const float g = gate[(size_t)t * gate_ld + c];
        v *= gate_act == 1 ? siluf_(g) : sigmoidf_(g);
      }
      El<T>::st(out + (size_t)t * vdim + c, v);
    }
    return;
  }
  for (int h = wave; h < H; h += 4) {
    const float* src = o + ((size_t)t * H + h) * vdim;
    float s = 0.f;
    for (int c = lane; c < vdim; c += 64) s = fmaf(src[c], src[c], s);
    const float r = 1.f / sqrtf(wave_sum(s) / (float)vdim + eps);
    for (int c = lane; c < vdim; c += 64) {
      float v = src[c] * r;
      if (w) v *= w[c];
      if (gate) {
        const float g = gate[(size_t)t * gate_ld + h * vdim + c];
        v *= gate_act == 1 ? siluf_(g) : sigmoidf_(g);
      }
      El<T>::st(out + ((size_t)t * H + h) * vdim + c, v);
    }
  }
}

// ------------------------------------------------------------------------------------------------ short causal convolution with its state
__global__ __launch_bounds__(256) void stk_conv_rows_kernel(StkConvArgs a) {
  const int t = blockIdx.x, C = a.C, taps = a.taps;
  const int b = seq_of_row(a.cu_q, a.B, t);
  const int slot = a.state_slots[b];
  if (slot < 0) return;
  const int t0 = a.cu_q ? (int)a.cu_q[b] : t;
  const int i = t - t0;
  const bool fresh = a.positions[t0] == 0;
  const float* cs = a.conv_state + (size_t)slot * (taps - 1) * C;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += 256 * gridDim.y) {
    float y = a.bias ? a.bias[c] : 0.f;
    for (int j = 0; j < taps; j++) {
      const int e = i - (taps - 1) + j;
      const bool from_step = e >= 0, counts = from_step || (!fresh && taps > 1);
      const float* src = from_step ? a.x + (size_t)(t0 + e) * a.ld : (counts ? cs + (size_t)(taps - 1 + e) * C : a.x + (size_t)t * a.ld);
      const float wv = counts ? a.w[(size_t)c * taps + j] : 0.f;
      y = fmaf(wv, src[c], y);
    }
    a.y[(size_t)t * a.ldy + c] = a.act == 1 ? siluf_(y) : y;
  }
}
__global__ __launch_bounds__(256) void stk_conv_rows_update_kernel(StkConvArgs a) {
  const int b = blockIdx.x;
  const int slot = a.state_slots[b];
  if (slot < 0) return;
  const int C = a.C, taps = a.taps;
  const int t0 = a.cu_q ? (int)a.cu_q[b] : b, n = a.cu_q ? (int)a.cu_q[b + 1] - t0 : 1;
  const bool fresh = a.positions[t0] == 0;
  float* cs = a.conv_state + (size_t)slot * (taps - 1) * C;
  for (int c = blockIdx.y * 256 + threadIdx.x; c < C; c += 256 * gridDim.y)
    for (int r = 0; r < taps - 1; r++) {  // (rows are read above where they are written)
      const int e = n - (taps - 1) + r;
      float v = 0.f;
      if (e >= 0) v = a.x[(size_t)(t0 + e) * a.ld + c];
      else if (!fresh) v = cs[(size_t)(taps - 1 + e) * C + c];
      cs[(size_t)r * C + c] = v;
    }
}

// ------------------------------------------------------------------------------------------------ real-gated diagonal recurrence
// Two forms.  One token per sequence: one launch forms gates, decay and input weight and moves the state on.  Prompt portions: an
// element-wise launch over all tokens and channels first turns the gate logits into the decay a and the weighted input b IN PLACE (and the
// gelu branch into its activation), so that the launch that walks a sequence's tokens in order has one multiply-add per token and three
// operands to fetch — requested two tiles ahead, since nothing in them depends on the state.
__device__ __forceinline__ float gelu_tanhf_(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
// (a, b) of one token and channel: a = exp(-sl r), b = sqrt(1 - a^2) i u with 1 - a^2 = -expm1(2 ln a) (no cancellation near a = 1)
__device__ __forceinline__ void gated_coef(float sl, float gr, float gi, float u, float* a, float* b) {
  const float la = -sl * sigmoidf_(gr);
  *a = expf(la);
  *b = sqrtf(-expm1f(2.f * la)) * (sigmoidf_(gi) * u);
}
__global__ __launch_bounds__(256) void stk_gated_prep_kernel(StkGatedScanArgs a, int T) {
  const int64_t total = (int64_t)T * a.C;
  for (int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x; e < total; e += (int64_t)gridDim.x * 256) {
    const int64_t t = e / a.C;
    const int c = (int)(e % a.C);
    const int gc = a.block > 0 ? c / a.block * 2 * a.block + c % a.block : c;
    float* gr = const_cast<float*>(a.gr) + t * a.ldg + gc;
    float* gi = const_cast<float*>(a.gi) + t * a.ldg + gc;
    float* y = const_cast<float*>(a.y) + t * a.ldy + c;
    float av, bv;
    gated_coef(a.rate * softplusf_(a.lam[c]), *gr, *gi, a.u[t * a.ldu + c], &av, &bv);
    *gr = av, *gi = bv, *y = gelu_tanhf_(*y);
  }
}
template <typename T, bool PREPARED>
__global__ __launch_bounds__(64) void stk_gated_scan_kernel(StkGatedScanArgs a) {
  constexpr int GT = 8;
  const int b = blockIdx.y, c = blockIdx.x * 64 + threadIdx.x;
  const int slot = a.state_slots[b];
  if (slot < 0 || c >= a.C) return;
  const int t0 = a.cu_q ? (int)a.cu_q[b] : b, n = a.cu_q ? (int)a.cu_q[b + 1] - t0 : 1;
  const bool fresh = a.positions[t0] == 0;
  float* sp = a.state + (size_t)slot * a.C + c;
  float S = fresh ? 0.f : *sp;
  const int gc = a.block > 0 ? c / a.block * 2 * a.block + c % a.block : c;
  T* out = (T*)a.out;
  if (!PREPARED) {
    const float sl = a.rate * softplusf_(a.lam[c]);
    for (int i = 0; i < n; i++) {
      const size_t t = (size_t)(t0 + i);
      float av, bv;
      gated_coef(sl, a.gr[t * a.ldg + gc], a.gi[t * a.ldg + gc], a.u[t * a.ldu + c], &av, &bv);
      S = fmaf(av, S, bv);
      El<T>::st(out + t * a.ldo + c, S * gelu_tanhf_(a.y[t * a.ldy + c]));
    }
    *sp = S;
    return;
  }
  float av[3][GT], bv[3][GT], yv[3][GT];  // three tiles of operands: one in use, two on their way
  auto request = [&](int i0, int w) {
#pragma unroll
    for (int j = 0; j < GT; j++) {
      const size_t t = (size_t)(t0 + min(i0 + j, n - 1));
      av[w][j] = a.gr[t * a.ldg + gc], bv[w][j] = a.gi[t * a.ldg + gc], yv[w][j] = a.y[t * a.ldy + c];
    }
  };
  auto run = [&](int i0, int w) {
#pragma unroll
    for (int j = 0; j < GT; j++)
      if (i0 + j < n) {
        S = fmaf(av[w][j], S, bv[w][j]);
        El<T>::st(out + (size_t)(t0 + i0 + j) * a.ldo + c, S * yv[w][j]);
      }
  };
  request(0, 0);
  if (GT < n) request(GT, 1);
  for (int i0 = 0; i0 < n; i0 += 3 * GT) {  // (the tile index is a compile-time constant in every call: the operands stay in registers)
    if (i0 + 2 * GT < n) request(i0 + 2 * GT, 2);
    run(i0, 0);
    if (i0 + GT >= n) break;
    if (i0 + 3 * GT < n) request(i0 + 3 * GT, 0);
    run(i0 + GT, 1);
    if (i0 + 2 * GT >= n) break;
    if (i0 + 4 * GT < n) request(i0 + 4 * GT, 1);
    run(i0 + 2 * GT, 2);
  }
  *sp = S;
}

}  // namespace

// ================================================================================================ launchers
void vra_stack_embed_pair(const StkEmbedPairArgs& a, int dtype, int64_t stream) {
  VRA_CHECK_ARG(a.ids && a.positions && a.embed && a.x && a.T > 0 && a.W > 0 && a.V > 0, "stack embedding: null pointer or empty shape");
  VRA_CHECK_ARG(!a.table || (a.buckets > 0 && a.prev_tokens && a.B > 0), "stack embedding: the pair table needs its bucket count and the previous tokens");
  const size_t lds = (size_t)a.W * sizeof(float);
  VRA_CHECK_ARG(lds <= 64 * 1024, "stack embedding: row does not fit LDS");
  if (dtype == VRA_F32) launch_checked("stack embedding", [&] { stk_embed_pair_kernel<float><<<a.T, 256, lds, as_stream(stream)>>>(a); });
  else launch_checked("stack embedding", [&] { stk_embed_pair_kernel<uint16_t><<<a.T, 256, lds, as_stream(stream)>>>(a); });
}

void vra_stack_sandwich_norm(const StkSandwichArgs& a, int dtype, int64_t stream) {
  VRA_CHECK_ARG(a.x && a.T > 0 && a.W > 0 && (!a.post_w || (a.p1 && a.n1 >= 1)) && (!a.pre_w || a.h), "stack seam norm: null pointer or empty shape");
  VRA_CHECK_ARG(!a.router_w || (a.pre_w && a.pair_expert && a.pair_weight && a.top >= 1 && a.top <= a.n_router), "stack seam norm: router outputs");
  VRA_CHECK_ARG(!a.dyt || ((!a.post_w || a.post_b) && (!a.pre_w || a.pre_b)), "stack seam norm: Dynamic Tanh needs its offsets");
  VRA_CHECK_ARG((!a.p1_norm_w && !a.p2_norm_w) || a.n1 == 1, "stack seam norm: a part with a norm of its own is one row a token");
  VRA_CHECK_ARG(a.router_kind == 0 || !a.router_w ||
                    (a.n_identity >= 0 && a.n_identity < a.n_router && (a.n_groups <= 1 || (a.n_router % a.n_groups == 0 && a.keep >= 1)) &&
                     (a.n_identity == 0 || a.id_weight)),
                "stack seam norm: router groups / identity experts");
  const size_t lds = ((size_t)a.W + 2 * (size_t)a.n_router + (size_t)std::max(a.n_groups, 0) + 1) * sizeof(float);
  VRA_CHECK_ARG(lds <= 64 * 1024, "stack seam norm: row does not fit LDS");
  if (dtype == VRA_F32) launch_checked("stack seam norm", [&] { stk_sandwich_kernel<float><<<a.T, 256, lds, as_stream(stream)>>>(a); });
  else launch_checked("stack seam norm", [&] { stk_sandwich_kernel<uint16_t><<<a.T, 256, lds, as_stream(stream)>>>(a); });
}

void vra_stack_head_prep(const StkHeadPrepArgs& a, int dtype, int64_t stream) {
  VRA_CHECK_ARG(a.raw && a.positions && a.T > 0 && a.dim > 0 && a.Hq >= 0 && a.Hk >= 0 && (a.Hq == 0 || a.q_out) && (a.Hk == 0 || a.k_out),
                "stack head prep: null pointer or empty shape");
  VRA_CHECK_ARG(2 * a.rot.pairs <= a.dim && (a.rot.pairs == 0 || a.rot.freq_hi), "stack head prep: more rotated dimensions than the head has");
  const dim3 grid(a.T, std::min((a.Hq + a.Hk + 3) / 4, 64));  // a head per wave
  if (a.out_f32 || dtype == VRA_F32) launch_checked("stack head prep", [&] { stk_head_prep_kernel<float><<<grid, 256, 0, as_stream(stream)>>>(a); });
  else launch_checked("stack head prep", [&] { stk_head_prep_kernel<uint16_t><<<grid, 256, 0, as_stream(stream)>>>(a); });
}

void vra_stack_delta_prep(const StkDeltaPrepArgs& a, int64_t stream) {
  VRA_CHECK_ARG(a.raw && a.raw2 && a.conv_w && a.conv_state && a.rate && a.dt_bias && a.qkv_out && a.beta_out && a.decay_out && a.positions && a.state_slots,
                "stack delta prep: null pointer");
  VRA_CHECK_ARG(a.T > 0 && a.B > 0 && a.H > 0 && a.G > 0 && a.H % a.G == 0 && a.dim > 0 && a.vdim > 0 && a.taps >= 1, "stack delta prep: shapes");
  const size_t lds = ((size_t)2 * a.G * a.dim + (size_t)a.H * a.vdim) * sizeof(float);
  VRA_CHECK_ARG(lds <= 64 * 1024, "stack delta prep: row does not fit LDS");
  launch_checked("stack delta prep", [&] { stk_delta_prep_kernel<<<a.T, 256, lds, as_stream(stream)>>>(a); });
}

void vra_stack_conv_state_update(const StkDeltaPrepArgs& a, int64_t stream) {
  VRA_CHECK_ARG(a.raw && a.conv_state && a.positions && a.state_slots && a.B > 0 && a.taps >= 1, "stack conv state: null pointer or empty shape");
  if (a.taps < 2) return;
  launch_checked("stack conv state", [&] { stk_conv_state_update_kernel<<<a.B, 256, 0, as_stream(stream)>>>(a); });
}

void vra_stack_sigmoid_pow(const float* z, int ldz, float* out, int ldo, int T, int n, float inv_tau, int64_t stream) {
  VRA_CHECK_ARG(z && out && T > 0 && n > 0, "stack decay: null pointer or empty shape");
  const int64_t total = (int64_t)T * n;
  const int grid = (int)std::min<int64_t>((total + 255) / 256, 4096);
  launch_checked("stack decay", [&] { stk_sigmoid_pow_kernel<<<grid, 256, 0, as_stream(stream)>>>(z, ldz, out, ldo, n, total, inv_tau); });
}

void vra_stack_linear_scan(const StkScanArgs& a, int64_t stream) {
  VRA_CHECK_ARG(a.q && a.k && a.v && a.state && a.state_slots && a.positions && a.out && (a.decay || a.head_decay), "stack linear scan: null pointer");
  VRA_CHECK_ARG(a.B > 0 && a.H > 0 && a.qk_rep >= 1 && a.H % a.qk_rep == 0 && a.dim > 0 && a.dim <= 256 && a.vdim > 0, "stack linear scan: key size at most 256");
  constexpr int R = 8;
  int P = 1;
  while (P * R < a.dim) P <<= 1;
  const int CPB = 256 / P, dimP = P * R;
  const size_t lds = ((size_t)16 * dimP * 3 + (size_t)16 * CPB + 32) * sizeof(float);
  dim3 grid((a.vdim + CPB - 1) / CPB, a.H, a.B);
  hipStream_t st = as_stream(stream);
  const bool decay = a.decay != nullptr, beta = a.beta != nullptr, per_head = decay && a.decay_per_head;
  VRA_CHECK_ARG(decay || !beta, "stack linear scan: the delta rule comes with per-row decays");
  VRA_CHECK_ARG(!a.act_silu || (!decay && !beta), "stack linear scan: the activation on the way in goes with constant decays");
  VRA_CHECK_ARG(!per_head || beta, "stack linear scan: one decay per head and token goes with the delta rule");
#define STK_SCAN(PV)                                                                                                            \
  launch_checked("stack linear scan", [&] {                                                                                     \
    if (per_head) stk_linear_scan_kernel<R, PV, 2, true, false><<<grid, 256, lds, st>>>(a);                                     \
    else if (beta) stk_linear_scan_kernel<R, PV, 1, true, false><<<grid, 256, lds, st>>>(a);                                    \
    else if (decay) stk_linear_scan_kernel<R, PV, 1, false, false><<<grid, 256, lds, st>>>(a);                                  \
    else if (a.act_silu) stk_linear_scan_kernel<R, PV, 0, false, true><<<grid, 256, lds, st>>>(a);                              \
    else stk_linear_scan_kernel<R, PV, 0, false, false><<<grid, 256, lds, st>>>(a);                                             \
  })
  switch (P) {
    case 1: STK_SCAN(1); break;
    case 2: STK_SCAN(2); break;
    case 4: STK_SCAN(4); break;
    case 8: STK_SCAN(8); break;
    case 16: STK_SCAN(16); break;
    default: STK_SCAN(32); break;
  }
#undef STK_SCAN
}

void vra_stack_head_norm_gate(const float* o, const float* w, const float* gate, int gate_ld, int gate_act, float eps, void* out, int T, int H, int vdim,
                              int dtype, int64_t stream) {
  VRA_CHECK_ARG(o && out && T > 0 && H > 0 && vdim > 0, "stack head norm: null pointer or empty shape");
  if (dtype == VRA_F32)
    launch_checked("stack head norm", [&] { stk_head_norm_gate_kernel<float><<<T, 256, 0, as_stream(stream)>>>(o, w, gate, gate_ld, gate_act, eps, (float*)out, H, vdim); });
  else
    launch_checked("stack head norm", [&] {
      stk_head_norm_gate_kernel<uint16_t><<<T, 256, 0, as_stream(stream)>>>(o, w, gate, gate_ld, gate_act, eps, (uint16_t*)out, H, vdim);
    });
}

void vra_stack_conv_rows(const StkConvArgs& a, int64_t stream) {
  VRA_CHECK_ARG(a.x && a.w && a.y && a.positions && a.state_slots && (a.taps < 2 || a.conv_state), "stack convolution: null pointer");
  VRA_CHECK_ARG(a.T > 0 && a.B > 0 && a.C > 0 && a.taps >= 1 && a.ld >= a.C && a.ldy >= a.C, "stack convolution: shapes");
  StkConvArgs k = a;
  if (!k.conv_state) k.conv_state = k.y;  // (one tap: never read)
  const dim3 grid(a.T, std::min((a.C + 255) / 256, 64));
  launch_checked("stack convolution", [&] { stk_conv_rows_kernel<<<grid, 256, 0, as_stream(stream)>>>(k); });
}
void vra_stack_conv_rows_update(const StkConvArgs& a, int64_t stream) {
  VRA_CHECK_ARG(a.x && a.positions && a.state_slots && a.B > 0 && a.taps >= 1 && a.C > 0, "stack convolution state: null pointer or empty shape");
  if (a.taps < 2) return;
  VRA_CHECK_ARG(a.conv_state, "stack convolution state: null pointer");
  const dim3 grid(a.B, std::min((a.C + 255) / 256, 64));
  launch_checked("stack convolution state", [&] { stk_conv_rows_update_kernel<<<grid, 256, 0, as_stream(stream)>>>(a); });
}
void vra_stack_gated_scan(const StkGatedScanArgs& a, int T, int dtype, int64_t stream) {
  VRA_CHECK_ARG(a.u && a.gr && a.gi && a.y && a.lam && a.state && a.state_slots && a.positions && a.out, "stack gated scan: null pointer");
  VRA_CHECK_ARG(a.B > 0 && a.C > 0 && a.ldu >= a.C && a.ldy >= a.C && a.ldo >= a.C, "stack gated scan: shapes");
  const dim3 grid((a.C + 63) / 64, a.B);
  hipStream_t st = as_stream(stream);
  if (!a.cu_q) {
    if (dtype == VRA_F32) launch_checked("stack gated scan", [&] { stk_gated_scan_kernel<float, false><<<grid, 64, 0, st>>>(a); });
    else launch_checked("stack gated scan", [&] { stk_gated_scan_kernel<uint16_t, false><<<grid, 64, 0, st>>>(a); });
    return;
  }
  VRA_CHECK_ARG(T > 0, "stack gated scan: a prompt step names its rows");
  const int pg = (int)std::min<int64_t>(((int64_t)T * a.C + 255) / 256, 8192);
  launch_checked("stack gated scan (gates)", [&] { stk_gated_prep_kernel<<<pg, 256, 0, st>>>(a, T); });
  if (dtype == VRA_F32) launch_checked("stack gated scan", [&] { stk_gated_scan_kernel<float, true><<<grid, 64, 0, st>>>(a); });
  else launch_checked("stack gated scan", [&] { stk_gated_scan_kernel<uint16_t, true><<<grid, 64, 0, st>>>(a); });
}

// ================================================================================================ C entry points (operator tests)
extern "C" void vra_stack_op_attention_chunk(const void* q, int32_t ldq, void* out, const void* kc, const void* vc, const int64_t* positions,
                                             const uint32_t* block_tables, const uint32_t* context_lens, const uint32_t* cu_q, int32_t B, int32_t T,
                                             int32_t max_q, int32_t H, int32_t G, int32_t dim, int32_t vdim, int32_t BS, int32_t max_blocks, float scale,
                                             int32_t chunk, int32_t dtype, int64_t stream) {
  StkAttnArgs a;
  a.q = q, a.ldq = ldq, a.out = out, a.kc = kc, a.vc = vc, a.positions = positions, a.block_tables = block_tables, a.context_lens = context_lens;
  a.cu_q = cu_q, a.B = B, a.T = T, a.max_q = max_q, a.H = H, a.G = G, a.dim = dim, a.vdim = vdim, a.BS = BS, a.max_blocks = max_blocks;
  a.scale = scale, a.chunk = chunk;
  vra_stack_attention(a, dtype, stream);
}
extern "C" void vra_stack_op_linear_scan(const float* q, int32_t ldq, const float* k, int32_t ldk, const float* v, int32_t ldv, const float* decay, int32_t ldd,
                                         const float* head_decay, const float* beta, int32_t ldb, float q_scale, float* state, const int32_t* state_slots,
                                         const int64_t* positions, const uint32_t* cu_q, float* out, int32_t ldo, int32_t B, int32_t H, int32_t qk_rep,
                                         int32_t dim, int32_t vdim, int64_t stream) {
  StkScanArgs a;
  a.q = q, a.ldq = ldq, a.k = k, a.ldk = ldk, a.v = v, a.ldv = ldv, a.decay = decay, a.ldd = ldd, a.head_decay = head_decay, a.beta = beta, a.ldb = ldb;
  a.q_scale = q_scale, a.state = state, a.state_slots = state_slots, a.positions = positions, a.cu_q = cu_q, a.out = out, a.ldo = ldo;
  a.B = B, a.H = H, a.qk_rep = qk_rep, a.dim = dim, a.vdim = vdim;
  vra_stack_linear_scan(a, stream);
}
extern "C" void vra_stack_op_sandwich_norm(float* x, const float* p1, int32_t n1, const float* pw, float c1, const float* p2, float c2, const float* post_w,
                                           const float* pre_w, void* h, float eps, int32_t T, int32_t W, const void* router_w, const float* router_bias,
                                           int32_t n_router, int32_t top, int32_t* pair_expert, float* pair_weight, int32_t dtype, int64_t stream) {
  StkSandwichArgs a;
  a.x = x, a.p1 = p1, a.n1 = n1, a.pw = pw, a.c1 = c1, a.p2 = p2, a.c2 = c2, a.post_w = post_w, a.pre_w = pre_w, a.h = h, a.eps = eps, a.T = T, a.W = W;
  a.router_w = router_w, a.router_bias = router_bias, a.n_router = n_router, a.top = top, a.pair_expert = pair_expert, a.pair_weight = pair_weight;
  vra_stack_sandwich_norm(a, dtype, stream);
}

// the softmax attention with a sliding window, a sink, a scale per head and a sigmoid output gate per head
extern "C" void vra_stack_op_attention_window(const void* q, int32_t ldq, void* out, const void* kc, const void* vc, const int64_t* positions,
                                              const uint32_t* block_tables, const uint32_t* context_lens, const uint32_t* cu_q, int32_t B, int32_t T,
                                              int32_t max_q, int32_t H, int32_t G, int32_t dim, int32_t vdim, int32_t BS, int32_t max_blocks, float scale,
                                              int32_t window, const float* sink, const float* head_scale, const float* gate, int32_t gate_ld,
                                              int32_t dtype, int64_t stream) {
  StkAttnArgs a;
  a.q = q, a.ldq = ldq, a.out = out, a.kc = kc, a.vc = vc, a.positions = positions, a.block_tables = block_tables, a.context_lens = context_lens;
  a.cu_q = cu_q, a.B = B, a.T = T, a.max_q = max_q, a.H = H, a.G = G, a.dim = dim, a.vdim = vdim, a.BS = BS, a.max_blocks = max_blocks;
  a.scale = scale, a.window = window, a.sink = sink, a.head_scale = head_scale, a.gate = gate, a.gate_ld = gate_ld;
  vra_stack_attention(a, dtype, stream);
}
// the seam with Dynamic Tanh norms, per-branch norms, pairs without a row, a weighted second part and the router over all outputs
extern "C" void vra_stack_op_seam(float* x, const float* p1, int32_t n1, const float* pw, const int32_t* pe, float c1, const float* p2, const float* p2w,
                                  float c2, const float* p1_norm_w, const float* p2_norm_w, int32_t dyt, const float* post_w, const float* post_b,
                                  float post_alpha, const float* pre_w, const float* pre_b, float pre_alpha, void* h, float* h32, float eps, int32_t T,
                                  int32_t W, const void* router_w, const float* router_bias, int32_t router_kind, int32_t n_router, int32_t top,
                                  int32_t n_groups, int32_t keep, int32_t n_identity, int32_t* pair_expert, float* pair_weight, float* id_weight,
                                  int32_t dtype, int64_t stream) {
  StkSandwichArgs a;
  a.x = x, a.p1 = p1, a.n1 = n1, a.pw = pw, a.pe = pe, a.c1 = c1, a.p2 = p2, a.p2w = p2w, a.c2 = c2, a.p1_norm_w = p1_norm_w, a.p2_norm_w = p2_norm_w;
  a.dyt = dyt, a.post_w = post_w, a.post_b = post_b, a.post_alpha = post_alpha, a.pre_w = pre_w, a.pre_b = pre_b, a.pre_alpha = pre_alpha;
  a.h = h, a.h32 = h32, a.eps = eps, a.T = T, a.W = W, a.router_w = router_w, a.router_bias = router_bias, a.router_kind = router_kind;
  a.n_router = n_router, a.top = top, a.n_groups = n_groups, a.keep = keep, a.n_identity = n_identity;
  a.pair_expert = pair_expert, a.pair_weight = pair_weight, a.id_weight = id_weight;
  vra_stack_sandwich_norm(a, dtype, stream);
}
// short causal convolution with its state (rows, then the state's update) and the real-gated diagonal recurrence
extern "C" void vra_stack_op_conv_rows(const float* x, int32_t ld, int32_t C, int32_t taps, const float* w, const float* bias, float* conv_state,
                                       int32_t act, float* y, int32_t ldy, const int64_t* positions, const uint32_t* cu_q, const int32_t* state_slots,
                                       int32_t T, int32_t B, int64_t stream) {
  StkConvArgs a;
  a.x = x, a.ld = ld, a.C = C, a.taps = taps, a.w = w, a.bias = bias, a.conv_state = conv_state, a.act = act, a.y = y, a.ldy = ldy;
  a.positions = positions, a.cu_q = cu_q, a.state_slots = state_slots, a.T = T, a.B = B;
  vra_stack_conv_rows(a, stream);
  vra_stack_conv_rows_update(a, stream);
}
extern "C" void vra_stack_op_gated_scan(const float* u, int32_t ldu, float* gr, float* gi, int32_t ldg, int32_t block, float* y, int32_t ldy,
                                        const float* lam, float rate, float* state, const int32_t* state_slots, const int64_t* positions,
                                        const uint32_t* cu_q, void* out, int32_t ldo, int32_t B, int32_t C, int32_t T, int32_t dtype, int64_t stream) {
  StkGatedScanArgs a;
  a.u = u, a.ldu = ldu, a.gr = gr, a.gi = gi, a.ldg = ldg, a.block = block, a.y = y, a.ldy = ldy, a.lam = lam, a.rate = rate, a.state = state;
  a.state_slots = state_slots, a.positions = positions, a.cu_q = cu_q, a.out = out, a.ldo = ldo, a.B = B, a.C = C;
  vra_stack_gated_scan(a, T, dtype, stream);
}
// the linear recurrence with one decay per head and token (delta rule) or silu on q, k, v (constant decays)
extern "C" void vra_stack_op_linear_scan_ex(const float* q, int32_t ldq, const float* k, int32_t ldk, const float* v, int32_t ldv, const float* decay,
                                            int32_t ldd, int32_t decay_per_head, int32_t act_silu, const float* head_decay, const float* beta, int32_t ldb,
                                            float q_scale, float* state, const int32_t* state_slots, const int64_t* positions, const uint32_t* cu_q,
                                            float* out, int32_t ldo, int32_t B, int32_t H, int32_t qk_rep, int32_t dim, int32_t vdim, int64_t stream) {
  StkScanArgs a;
  a.q = q, a.ldq = ldq, a.k = k, a.ldk = ldk, a.v = v, a.ldv = ldv, a.decay = decay, a.ldd = ldd, a.decay_per_head = decay_per_head, a.act_silu = act_silu;
  a.head_decay = head_decay, a.beta = beta, a.ldb = ldb, a.q_scale = q_scale, a.state = state, a.state_slots = state_slots, a.positions = positions;
  a.cu_q = cu_q, a.out = out, a.ldo = ldo, a.B = B, a.H = H, a.qk_rep = qk_rep, a.dim = dim, a.vdim = vdim;
  vra_stack_linear_scan(a, stream);
}
