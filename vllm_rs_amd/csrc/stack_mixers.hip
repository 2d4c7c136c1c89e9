// stack_mixers.hip — operators of sequential pre-norm layer stacks (host/stack_model.cpp; each is specified in stack_launch.h), gfx950:
// Dynamic Tanh with the residual sum, the latent (low-rank) attention's norms / rotary / cache rows, the whole-projection query / key norm,
// and the attention without softmax (sigmoid weights, distance penalty, window with kept first tokens, mixed heads, output gate).
//
// f32 whatever the storage type: positions and angles, norms, scores and weights, every sum over keys.  The order of every sum depends
// on the model's shapes and on absolute positions alone, never on the step's rows, so a token's result does not depend on how its
// prompt was cut or on its batch.
#include <algorithm>

#include "stack_common.cuh"
#include "stack_launch.h"

namespace {

// ------------------------------------------------------------------------------------------------ Dynamic Tanh (+ residual sum)
template <typename T>
__global__ __launch_bounds__(256) void stk_dyt_kernel(float* x, const float* add, const float* w, const float* b, float alpha, T* h, int W, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const int c = (int)(i % W);
    float v = x[i];
    if (add) {
      v += add[i];
      x[i] = v;
    }
    El<T>::st(h + i, tanhf(alpha * v) * w[c] + b[c]);
  }
}

// ------------------------------------------------------------------------------------------------ latent attention: norms, rotary, cache row
template <typename T>
__global__ __launch_bounds__(256) void stk_latent_prep_kernel(StkLatentPrepArgs a) {
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float* raw = a.raw + (size_t)t * a.ld;
  float s = 0.f;
  for (int c = tid; c < a.q_rank; c += 256) s = fmaf(raw[c], raw[c], s);
  const float rq = 1.f / sqrtf(block_sum_256(s, red) / (float)a.q_rank + a.eps);
  T* cq = (T*)a.cq + (size_t)t * a.q_rank;
  for (int c = tid; c < a.q_rank; c += 256) El<T>::st(cq + c, raw[c] * rq * a.qn_w[c]);
  const int64_t slot = a.slots[t];
  if (slot < 0) return;
  const float* kv = raw + a.q_rank;
  s = 0.f;
  for (int c = tid; c < a.kv_rank; c += 256) s = fmaf(kv[c], kv[c], s);
  const float rk = 1.f / sqrtf(block_sum_256(s, red) / (float)a.kv_rank + a.eps);
  T* row = (T*)a.cache + slot * a.cache_ld;
  for (int c = tid; c < a.kv_rank; c += 256) El<T>::st(row + c, kv[c] * rk * a.kvn_w[c]);
  const float p = (float)a.positions[t];
  const float* r = kv + a.kv_rank;
  for (int i = tid; i < a.rot_dim / 2 + (a.rot_dim & 1); i += 256) {
    if (i < a.rot.pairs) {
      float c, sn;
      rot_cos_sin(a.rot, i, p, &c, &sn);
      const float u = r[2 * i], v = r[2 * i + 1];
      El<T>::st(row + a.kv_rank + 2 * i, u * c - v * sn);
      El<T>::st(row + a.kv_rank + 2 * i + 1, v * c + u * sn);
    } else {
      El<T>::st(row + a.kv_rank + 2 * i, r[2 * i]);
      if (2 * i + 1 < a.rot_dim) El<T>::st(row + a.kv_rank + 2 * i + 1, r[2 * i + 1]);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void stk_rope_heads_kernel(const T* in, int in_ld, int in_hs, int in_off, T* out, int out_ld, int out_hs, int out_off,
                                                             int n, int H, const int64_t* positions, StkRotary rot) {
  const int t = blockIdx.x;
  const float p = (float)positions[t];
  const int half = n / 2 + (n & 1);
  for (int e = threadIdx.x; e < H * half; e += 256) {
    const int h = e / half, i = e % half;
    const T* src = in + (size_t)t * in_ld + h * in_hs + in_off;
    T* dst = out + (size_t)t * out_ld + h * out_hs + out_off;
    if (i < rot.pairs) {
      float c, sn;
      rot_cos_sin(rot, i, p, &c, &sn);
      const float u = El<T>::ld(src + 2 * i), v = El<T>::ld(src + 2 * i + 1);
      El<T>::st(dst + 2 * i, u * c - v * sn);
      El<T>::st(dst + 2 * i + 1, v * c + u * sn);
    } else {
      El<T>::st(dst + 2 * i, El<T>::ld(src + 2 * i));
      if (2 * i + 1 < n) El<T>::st(dst + 2 * i + 1, El<T>::ld(src + 2 * i + 1));
    }
  }
}

// ------------------------------------------------------------------------------------------------ whole-projection q / k norm + cache rows
template <typename T>
__global__ __launch_bounds__(256) void stk_qk_norm_store_kernel(const float* raw, int ld, int nq, int nk, int nv, const float* q_w, const float* k_w,
                                                                float eps, T* q_out, T* kc, T* vc, const int64_t* slots) {
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float* r = raw + (size_t)t * ld;
  float rq = 1.f, rk = 1.f;
  if (q_w) {
    float s = 0.f;
    for (int c = tid; c < nq; c += 256) s = fmaf(r[c], r[c], s);
    rq = 1.f / sqrtf(block_sum_256(s, red) / (float)nq + eps);
  }
  for (int c = tid; c < nq; c += 256) El<T>::st(q_out + (size_t)t * nq + c, q_w ? r[c] * rq * q_w[c] : r[c]);
  const int64_t slot = slots[t];
  if (slot < 0) return;
  if (k_w) {
    float s = 0.f;
    for (int c = tid; c < nk; c += 256) s = fmaf(r[nq + c], r[nq + c], s);
    rk = 1.f / sqrtf(block_sum_256(s, red) / (float)nk + eps);
  }
  for (int c = tid; c < nk; c += 256) El<T>::st(kc + slot * nk + c, k_w ? r[nq + c] * rk * k_w[c] : r[nq + c]);
  for (int c = tid; c < nv; c += 256) El<T>::st(vc + slot * nv + c, r[nq + nk + c]);
}

// ------------------------------------------------------------------------------------------------ attention without softmax
// A workgroup owns QT query rows of one sequence and ALL heads (the mixing of the heads' weights needs every head's weight of a (query,
// key) pair in one place).  Key tiles of KT tokens, aligned to absolute positions; tiles that no row can see (between the kept first
// tokens and the window) are skipped.  Per tile: scores and weights head by head into LDS, the mix, then the value product with the
// accumulators in registers: thread = (row, every TPR-th output channel).
template <typename T, int QT, int NACC>
__global__ __launch_bounds__(256) void stk_sig_attn_kernel(StkSigAttnArgs a, int KT) {
  extern __shared__ float lds[];
  constexpr int TPR = 256 / QT;
  const int dim = a.dim, vdim = a.vdim, H = a.H, G = a.G, HG = H / G, kld = dim + 1, GV = G * vdim, HV = H * vdim;
  float* qs = lds;                       // [QT][dim]
  float* ks = qs + QT * dim;             // [KT][dim + 1]
  float* ws = ks + KT * kld;             // [H][QT][KT]
  float* ms = ws + H * QT * KT;          // [H][QT][KT] (mixed; aliases ws without a mixing matrix)
  float* vs = a.talk ? ms + H * QT * KT : ms;  // [KT][G * vdim]
  float* tk = vs + KT * GV;              // [H][H]
  if (!a.talk) ms = ws;
  const int b = blockIdx.y, tid = threadIdx.x;
  const int q0 = a.cu_q ? a.cu_q[b] : b, q1 = a.cu_q ? a.cu_q[b + 1] : b + 1;
  const int t0 = q0 + blockIdx.x * QT;
  if (t0 >= q1) return;
  const int nq = min(QT, q1 - t0);
  int64_t pmin = a.positions[t0], pmax = pmin;
  for (int r = 1; r < nq; r++) pmin = min(pmin, a.positions[t0 + r]), pmax = max(pmax, a.positions[t0 + r]);
  const int n_keys = (int)min((int64_t)a.context_lens[b], pmax + 1);
  if (a.talk)
    for (int i = tid; i < H * H; i += 256) tk[i] = a.talk[i];
  const T* q = (const T*)a.q;
  const T* kc = (const T*)a.kc;
  const T* vc = (const T*)a.vc;
  const uint32_t* bt = a.block_tables + (size_t)b * a.max_blocks;
  float acc[NACC];
#pragma unroll
  for (int i = 0; i < NACC; i++) acc[i] = 0.f;
  const int pr = tid / TPR, pl = tid % TPR;  // value phase: row, first channel
  const int win_first = a.window > 0 ? (int)(max((int64_t)0, pmin - a.window + 1) / KT) * KT : 0;
  const int keep_end = a.window > 0 ? (max(a.keep_first, 0) + KT - 1) / KT * KT : 0;
  for (int kt0 = 0; kt0 < n_keys; kt0 += KT) {
    if (a.window > 0 && kt0 >= keep_end && kt0 < win_first) {  // nothing between the kept tokens and the window is seen
      kt0 = win_first - KT;
      continue;
    }
    for (int g = 0; g < G; g++) {
      __syncthreads();
      for (int i = tid; i < KT * dim; i += 256) {
        const int j = i / dim, d = i % dim, key = kt0 + j;
        float v = 0.f;
        if (key < n_keys) {
          const int64_t slot = (int64_t)bt[key / a.BS] * a.BS + key % a.BS;
          v = El<T>::ld(kc + slot * (G * dim) + g * dim + d);
        }
        ks[j * kld + d] = v;
      }
      for (int hh = 0; hh < HG; hh++) {
        const int h = g * HG + hh;
        __syncthreads();
        for (int i = tid; i < QT * dim; i += 256) {
          const int r = i / dim, d = i % dim;
          qs[i] = r < nq ? El<T>::ld(q + (size_t)(t0 + r) * a.ldq + h * dim + d) : 0.f;
        }
        __syncthreads();
        const float slope = a.slopes ? a.slopes[h] : 0.f, hb = a.head_bias ? a.head_bias[h] : 0.f;
        for (int i = tid; i < QT * KT; i += 256) {
          const int r = i / KT, j = i % KT, key = kt0 + j;
          float w = 0.f;
          if (r < nq && key < n_keys) {
            const int64_t p = a.positions[t0 + r];
            if (key <= p && (a.window <= 0 || p - key < a.window || key < a.keep_first)) {
              float d0 = 0.f;
              for (int d = 0; d < dim; d++) d0 = fmaf(qs[r * dim + d], ks[j * kld + d], d0);
              w = sigmoidf_(d0 * a.scale - slope * (float)(p - key) + hb);
            }
          }
          ws[(h * QT + r) * KT + j] = w;
        }
      }
    }
    __syncthreads();
    if (a.talk) {
      for (int i = tid; i < QT * KT; i += 256) {
        const int r = i / KT, j = i % KT;
        for (int h = 0; h < H; h++) {
          float s = 0.f;
          for (int g2 = 0; g2 < H; g2++) s = fmaf(tk[h * H + g2], ws[(g2 * QT + r) * KT + j], s);
          ms[(h * QT + r) * KT + j] = s;
        }
      }
    }
    for (int i = tid; i < KT * GV; i += 256) {
      const int j = i / GV, c = i % GV, key = kt0 + j;
      float v = 0.f;
      if (key < n_keys) {
        const int64_t slot = (int64_t)bt[key / a.BS] * a.BS + key % a.BS;
        v = El<T>::ld(vc + slot * GV + c);
      }
      vs[i] = v;
    }
    __syncthreads();
    const int nj = min(KT, n_keys - kt0);
#pragma unroll
    for (int n = 0; n < NACC; n++) {
      const int c = pl + n * TPR;
      if (c < HV) {
        const int h = c / vdim, d = c % vdim, g = h / HG;
        const float* mw = ms + (h * QT + pr) * KT;
        const float* vv = vs + g * vdim + d;
        float o = acc[n];
        for (int j = 0; j < nj; j++) o = fmaf(mw[j], vv[j * GV], o);
        acc[n] = o;
      }
    }
  }
  if (pr >= nq) return;
  T* out = (T*)a.out + (size_t)(t0 + pr) * HV;
#pragma unroll
  for (int n = 0; n < NACC; n++) {
    const int c = pl + n * TPR;
    if (c < HV) {
      float o = acc[n];
      if (a.gate) o *= sigmoidf_(a.gate[(size_t)(t0 + pr) * a.gate_ld + c]);
      El<T>::st(out + c, o);
    }
  }
}


// ------------------------------------------------------------------------------------------------ the same on the matrix cores (bf16)
// The mixing of the heads is linear in the weights, so it commutes with the sum over keys:
//   out_h = sum_g talk[h, g] U[g, kv(h)],   U[g, kappa](i) = sum_j w_g(i, j) v_kappa(j).
// A workgroup of 4 waves owns 64 query rows of ONE head g and GC key/value heads: S^T = K . Q^T on MFMA (K fragments straight from the
// cache, one tile ahead), the sigmoid weights in f32 per lane, then U^T += V_kappa^T . W^T for each of its value heads with the weights
// split into a bf16 head and tail (w = hi + lo to 2^-17: f32 weights in effect).  Heads never meet inside the kernel; a second, element-wise
// launch mixes U and applies the gate.  32-key tiles aligned to absolute positions, ascending; tiles between the kept first tokens and the
// window are skipped.
template <int DC, int VT, int GC>
__global__ __launch_bounds__(256) void stk_sig_prefill_mfma_kernel(StkSigAttnArgs a, float* U) {
  constexpr int KT = 32, VLD = KT + 8;
  __shared__ __attribute__((aligned(16))) uint16_t vt[GC * VT * 16 * VLD];
  const int dim = a.dim, vdim = a.vdim, G = a.G;
  const int n_gc = (G + GC - 1) / GC;
  const int b = blockIdx.y, h = blockIdx.z / n_gc, kap0 = (blockIdx.z % n_gc) * GC, gk = h / (a.H / G);
  const int q0 = a.cu_q[b], q1 = a.cu_q[b + 1];
  const int t0 = q0 + ((int)gridDim.x - 1 - (int)blockIdx.x) * 64;
  if (t0 >= q1) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, rq = lane & 15, oct = lane >> 4;
  const int tq = t0 + wave * 16 + rq;
  const bool qv = tq < q1;
  const int64_t pq = qv ? a.positions[tq] : -1;
  const uint16_t* q = (const uint16_t*)a.q;
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  u32x4 qf[DC];
  for (int c = 0; c < DC; c++) {
    const int ch = c * 32 + oct * 8;
    const bool ok = qv && ch < dim;
    const u32x4 v = *(const u32x4*)(q + (size_t)(ok ? tq : q0) * a.ldq + h * dim + (ok ? ch : 0));
    qf[c] = ok ? v : zero4;
  }
  // the smallest and largest position of the wave's and of the workgroup's rows bound what they can see
  long long lo = qv ? pq : 0x7fffffffffffffffll, hi = pq;
  for (int o = 32; o > 0; o >>= 1) lo = min(lo, __shfl_xor(lo, o, 64)), hi = max(hi, __shfl_xor(hi, o, 64));
  __shared__ long long wlo[4], whi[4];
  if (lane == 0) wlo[wave] = lo, whi[wave] = hi;
  __syncthreads();
  const bool wave_has = hi >= 0;
  const int64_t wmin = lo, wmax = hi;
  const int64_t pmin = min(min(wlo[0], wlo[1]), min(wlo[2], wlo[3])), pmax = max(max(whi[0], whi[1]), max(whi[2], whi[3]));
  const int n_keys = (int)min((int64_t)a.context_lens[b], pmax + 1);
  const int win = a.window;
  const int keep_end = win > 0 ? (max(a.keep_first, 0) + KT - 1) / KT * KT : 0;
  const int win_first = win > 0 ? (int)(max((int64_t)0, pmin - win + 1) / KT) * KT : 0;
  const int wave_first = win > 0 ? (int)(max((int64_t)0, wmin - win + 1) / KT) * KT : 0;
  auto next_tile = [&](int kt0) {  // the tile after kt0 that some row of the workgroup may see
    int n = kt0 + KT;
    if (win > 0 && n >= keep_end && n < win_first) n = win_first;
    return n;
  };
  const uint16_t* kc = (const uint16_t*)a.kc;
  const uint16_t* vc = (const uint16_t*)a.vc;
  const uint32_t* bt = a.block_tables + (size_t)b * a.max_blocks;
  const int kdim = G * dim, vd_all = G * vdim;
  f32x4 acc[GC][VT];
#pragma unroll
  for (int e = 0; e < GC; e++)
#pragma unroll
    for (int t = 0; t < VT; t++) acc[e][t] = vra_zero_acc();
  const float slope = a.slopes ? a.slopes[h] : 0.f, hb = a.head_bias ? a.head_bias[h] : 0.f;
  // V item = (value head, pair of neighbouring keys, 8 channels): NV per thread, two 16-byte requests each
  constexpr int ITEMS = GC * (KT / 2) * VT * 2, NV = (ITEMS + 255) / 256;
  u32x4 kfn[2][DC], vgn[NV][2];
  auto page_slot = [&](int kt0) -> int64_t {  // first cache slot of the tile (a 32-key tile lies in one page: the page size is a multiple of 32)
    const int t = __builtin_amdgcn_readfirstlane(kt0);
    return t < n_keys ? (int64_t)bt[t / a.BS] * a.BS + t % a.BS : 0;
  };
  auto request_tile = [&](int kt0, int64_t slot0) {
    for (int u = 0; u < 2; u++) {
      const int key = kt0 + u * 16 + rq;
      const bool kv = key < n_keys;
      const uint16_t* kr = kc + (kv ? slot0 + (key - kt0) : 0) * kdim + gk * dim;
      for (int c = 0; c < DC; c++) {
        const int ch = c * 32 + oct * 8;
        const bool ok = kv && ch < dim;
        const u32x4 kf = *(const u32x4*)(kr + (ok ? ch : 0));
        kfn[u][c] = ok ? kf : zero4;
      }
    }
    for (int n = 0; n < NV; n++) {
      const int i = tid + n * 256;
      const int e = i / ((KT / 2) * VT * 2), r = i % ((KT / 2) * VT * 2);
      const int kp = r / (VT * 2), c8 = (r % (VT * 2)) * 8;
      for (int w2 = 0; w2 < 2; w2++) {
        const int key = kt0 + kp * 2 + w2;
        const bool ok = i < ITEMS && kap0 + e < G && key < n_keys && c8 < vdim;
        const u32x4 v = *(const u32x4*)(vc + (ok ? slot0 + (key - kt0) : 0) * vd_all + (ok ? (kap0 + e) * vdim + c8 : 0));
        vgn[n][w2] = ok ? v : zero4;
      }
    }
  };
  int kt0 = (win > 0 && keep_end == 0 && win_first > 0) ? win_first : 0;
  if (kt0 < n_keys) request_tile(kt0, page_slot(kt0));
  while (kt0 < n_keys) {
    const int ktn = next_tile(kt0);
    const int64_t slot_next = page_slot(ktn);
    u32x4 kfc[2][DC], vgc[NV][2];
    for (int u = 0; u < 2; u++)
      for (int c = 0; c < DC; c++) kfc[u][c] = kfn[u][c];
    for (int n = 0; n < NV; n++) vgc[n][0] = vgn[n][0], vgc[n][1] = vgn[n][1];
    __syncthreads();
    for (int n = 0; n < NV; n++) {
      const int i = tid + n * 256;
      if (i >= ITEMS) break;
      const int e = i / ((KT / 2) * VT * 2), r = i % ((KT / 2) * VT * 2);
      const int kl = (r / (VT * 2)) * 2, c8 = (r % (VT * 2)) * 8;
      const int pos = ((kl & 15) >> 2) * 8 + (kl >> 4) * 4 + (kl & 3);  // the order in which the lanes hold their weights
      uint32_t* row = (uint32_t*)(vt + e * VT * 16 * VLD);
      for (int x = 0; x < 4; x++) {
        const uint32_t lo0 = vgc[n][0][x] & 0xffffu, hi0 = vgc[n][0][x] >> 16, lo1 = vgc[n][1][x] & 0xffffu, hi1 = vgc[n][1][x] >> 16;
        row[((c8 + 2 * x) * VLD + pos) >> 1] = lo0 | (lo1 << 16);
        row[((c8 + 2 * x + 1) * VLD + pos) >> 1] = hi0 | (hi1 << 16);
      }
    }
    __syncthreads();
    if (ktn < n_keys) request_tile(ktn, slot_next);
    const int kt = kt0;
    kt0 = ktn;
    // (wave-uniform) nothing of this tile is visible to the wave's rows: behind its last row, or before its window and not kept
    if (!wave_has || kt > wmax || (win > 0 && kt >= keep_end && kt + KT <= wave_first)) continue;
    f32x4 s[2];
    s[0] = vra_zero_acc();
    s[1] = vra_zero_acc();
    for (int c = 0; c < DC; c++) {
      BF16::mfma(s[0], __builtin_bit_cast(s16x8, kfc[0][c]), __builtin_bit_cast(s16x8, qf[c]));
      BF16::mfma(s[1], __builtin_bit_cast(s16x8, kfc[1][c]), __builtin_bit_cast(s16x8, qf[c]));
    }
    VRA_MFMA_DRAIN();
    float pv[8];
    for (int u = 0; u < 2; u++)
      for (int j = 0; j < 4; j++) {
        const int key = kt + u * 16 + oct * 4 + j;
        const int dist = (int)pq - key;  // (no short-circuit evaluation: the weights of a tile are straight-line code)
        const bool seen = (dist >= 0) & (key < n_keys) & ((win <= 0) | (dist < win) | (key < a.keep_first));
        const float x = s[u][j] * a.scale - slope * (float)dist + hb;
        pv[u * 4 + j] = seen ? __builtin_amdgcn_rcpf(1.f + __expf(-x)) : 0.f;  // (hardware exponential and reciprocal: no branches)
      }
    u32x4 phi, plo;
    for (int e = 0; e < 4; e++) {
      const float a0 = pv[2 * e], a1 = pv[2 * e + 1];
      const uint32_t hi = BF16::pack2(a0, a1);
      phi[e] = hi;
      plo[e] = BF16::pack2(a0 - __uint_as_float(hi << 16), a1 - __uint_as_float(hi & 0xffff0000u));
    }
#pragma unroll
    for (int e = 0; e < GC; e++) {
      u32x4 vf[VT];
#pragma unroll
      for (int t = 0; t < VT; t++) vf[t] = *(const u32x4*)(vt + ((e * VT + t) * 16 + rq) * VLD + oct * 8);
#pragma unroll
      for (int t = 0; t < VT; t++) BF16::mfma(acc[e][t], __builtin_bit_cast(s16x8, vf[t]), __builtin_bit_cast(s16x8, phi));
#pragma unroll
      for (int t = 0; t < VT; t++) BF16::mfma(acc[e][t], __builtin_bit_cast(s16x8, vf[t]), __builtin_bit_cast(s16x8, plo));
    }
    VRA_MFMA_DRAIN();
  }
  if (!qv) return;
#pragma unroll
  for (int e = 0; e < GC; e++) {
    if (kap0 + e >= G) break;
    float* out = U + (((size_t)tq * a.H + h) * G + kap0 + e) * vdim;
#pragma unroll
    for (int t = 0; t < VT; t++)
      for (int j = 0; j < 4; j++) {
        const int c = t * 16 + oct * 4 + j;
        if (c < vdim) out[c] = acc[e][t][j];
      }
  }
}

// All heads in one workgroup of NW waves (H = NW HPW; a wave's HPW heads lie in one key/value group): 16 query rows, wave w owns
// the heads [w HPW, (w + 1) HPW).  (Eight waves of two heads for 16 heads measured slower than four waves of four: 357 against
// 290 us at 2048 tokens — more waves at the two meetings, every V tile transposed twice.)  Per 32-key tile every wave computes the weights of its own heads on MFMA and leaves them in LDS (f32,
// in the lanes' own key order), all waves meet, every wave mixes ALL heads' weights into those of its own heads (g ascending), and
// multiplies them — split hi + lo — with the V tile of its key/value head, which it transposed into its own part of LDS.  One value product
// per head instead of one per (head, key/value head): the kernel of choice when the shape allows it; it writes the gated output itself.
template <int DC, int VT, int HPW, int NW>
__global__ __launch_bounds__(64 * NW) void stk_sig_prefill_heads_kernel(StkSigAttnArgs a) {
  constexpr int KT = 32, VLD = KT + 8, QR = 16, WLD = KT + 4;  // (WLD: rows of the weight buffer 16 bytes apart in the banks)
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int dim = a.dim, vdim = a.vdim, H = a.H, G = a.G, HG = H / G;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, rq = lane & 15, oct = lane >> 4;
  float* wbuf = lds;                                   // [H][16 rows][WLD: 32 key places + 4]
  float* tk = wbuf + H * QR * WLD;                      // [H][H]
  uint16_t* vt = (uint16_t*)(tk + H * H) + wave * (VT * 16 * VLD);  // this wave's V tile, transposed: [VT * 16 channels][VLD]
  const int b = blockIdx.y;
  const int q0 = a.cu_q[b], q1 = a.cu_q[b + 1];
  const int t0 = q0 + ((int)gridDim.x - 1 - (int)blockIdx.x) * QR;
  if (t0 >= q1) return;
  const int tq = t0 + rq;
  const bool qv = tq < q1;
  const int64_t pq = qv ? a.positions[tq] : -1;
  const int h0 = wave * HPW, gk = h0 / HG;
  const uint16_t* q = (const uint16_t*)a.q;
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  u32x4 qf[HPW][DC];
#pragma unroll
  for (int hh = 0; hh < HPW; hh++)
#pragma unroll
    for (int c = 0; c < DC; c++) {
      const int ch = c * 32 + oct * 8;
      const bool ok = qv && ch < dim;
      const u32x4 v = *(const u32x4*)(q + (size_t)(ok ? tq : q0) * a.ldq + (h0 + hh) * dim + (ok ? ch : 0));
      qf[hh][c] = ok ? v : zero4;
    }
  long long lo = qv ? pq : 0x7fffffffffffffffll, hi = pq;  // (every wave holds the same 16 rows)
  for (int o = 32; o > 0; o >>= 1) lo = min(lo, __shfl_xor(lo, o, 64)), hi = max(hi, __shfl_xor(hi, o, 64));
  const int64_t pmin = lo, pmax = hi;
  const int n_keys = (int)min((int64_t)a.context_lens[b], pmax + 1);
  const int win = a.window;
  const int keep_end = win > 0 ? (max(a.keep_first, 0) + KT - 1) / KT * KT : 0;
  const int win_first = win > 0 ? (int)(max((int64_t)0, pmin - win + 1) / KT) * KT : 0;
  auto next_tile = [&](int kt0) {
    int n = kt0 + KT;
    if (win > 0 && n >= keep_end && n < win_first) n = win_first;
    return n;
  };
  for (int i = tid; i < H * H; i += 64 * NW) tk[i] = a.talk ? a.talk[i] : ((i / H == i % H) ? 1.f : 0.f);
  const uint16_t* kc = (const uint16_t*)a.kc;
  const uint16_t* vc = (const uint16_t*)a.vc;
  const uint32_t* bt = a.block_tables + (size_t)b * a.max_blocks;
  const int kdim = G * dim, vd_all = G * vdim;
  f32x4 acc[HPW][VT];
  float slope[HPW], hb[HPW];
#pragma unroll
  for (int hh = 0; hh < HPW; hh++) {
    slope[hh] = a.slopes ? a.slopes[h0 + hh] : 0.f, hb[hh] = a.head_bias ? a.head_bias[h0 + hh] : 0.f;
#pragma unroll
    for (int t = 0; t < VT; t++) acc[hh][t] = vra_zero_acc();
  }
  // the wave's share of a tile: K fragments of its key/value head and that head's V tile ((pair of keys, 8 channels) items, 64 lanes)
  constexpr int ITEMS = (KT / 2) * VT * 2, NV = ITEMS / 64;
  static_assert(ITEMS % 64 == 0, "a wave's V items come in whole rounds");
  u32x4 kfn[2][DC], vgn[NV][2];
  auto page_slot = [&](int kt0) -> int64_t {
    const int t = __builtin_amdgcn_readfirstlane(kt0);
    return t < n_keys ? (int64_t)bt[t / a.BS] * a.BS + t % a.BS : 0;
  };
  // Requests carry no select: what lies outside the tile or the head is read from a valid address instead (slot 0, channel 0: finite
  // numbers) and cannot reach a result — keys beyond the context get weight 0, channels beyond the key size meet zeros of the query
  // fragment, channels beyond the value size are never stored.  So nothing has to wait for a request before the next one is issued.
  auto request_tile = [&](int kt0, int64_t slot0) {
#pragma unroll
    for (int u = 0; u < 2; u++) {
      const int key = kt0 + u * 16 + rq;
      const uint16_t* kr = kc + (key < n_keys ? slot0 + (key - kt0) : 0) * kdim + gk * dim;
#pragma unroll
      for (int c = 0; c < DC; c++) {
        const int ch = c * 32 + oct * 8;
        kfn[u][c] = *(const u32x4*)(kr + (ch < dim ? ch : 0));
      }
    }
#pragma unroll
    for (int n = 0; n < NV; n++) {
      const int i = lane + n * 64;
      const int kp = i / (VT * 2), c8 = (i % (VT * 2)) * 8;
#pragma unroll
      for (int w2 = 0; w2 < 2; w2++) {
        const int key = kt0 + kp * 2 + w2;
        vgn[n][w2] = *(const u32x4*)(vc + (key < n_keys ? slot0 + (key - kt0) : 0) * vd_all + gk * vdim + (c8 < vdim ? c8 : 0));
      }
    }
  };
  int kt0 = (win > 0 && keep_end == 0 && win_first > 0) ? win_first : 0;
  if (kt0 < n_keys) request_tile(kt0, page_slot(kt0));
  while (kt0 < n_keys) {
    const int ktn = next_tile(kt0);
    const int64_t slot_next = page_slot(ktn);
    // V tile -> this wave's LDS part, transposed, keys in the order the lanes hold their weights (the wave's earlier reads of it are done:
    // LDS serves a wave's requests in order)
    for (int n = 0; n < NV; n++) {
      const int i = lane + n * 64;
      if (i >= ITEMS) break;
      const int kl = (i / (VT * 2)) * 2, c8 = (i % (VT * 2)) * 8;
      const int pos = ((kl & 15) >> 2) * 8 + (kl >> 4) * 4 + (kl & 3);
      uint32_t* row = (uint32_t*)vt;
      for (int x = 0; x < 4; x++) {
        const uint32_t lo0 = vgn[n][0][x] & 0xffffu, hi0 = vgn[n][0][x] >> 16, lo1 = vgn[n][1][x] & 0xffffu, hi1 = vgn[n][1][x] >> 16;
        row[((c8 + 2 * x) * VLD + pos) >> 1] = lo0 | (lo1 << 16);
        row[((c8 + 2 * x + 1) * VLD + pos) >> 1] = hi0 | (hi1 << 16);
      }
    }
    // weights of the wave's own heads -> LDS
#pragma unroll
    for (int hh = 0; hh < HPW; hh++) {
      f32x4 s[2];
      s[0] = vra_zero_acc();
      s[1] = vra_zero_acc();
      for (int c = 0; c < DC; c++) {
        BF16::mfma(s[0], __builtin_bit_cast(s16x8, kfn[0][c]), __builtin_bit_cast(s16x8, qf[hh][c]));
        BF16::mfma(s[1], __builtin_bit_cast(s16x8, kfn[1][c]), __builtin_bit_cast(s16x8, qf[hh][c]));
      }
      VRA_MFMA_DRAIN();
      f32x4 w4[2];
      for (int u = 0; u < 2; u++)
        for (int j = 0; j < 4; j++) {
          const int key = kt0 + u * 16 + oct * 4 + j;
          const int dist = (int)pq - key;  // (no short-circuit evaluation: the weights of a tile are straight-line code)
          const bool seen = (dist >= 0) & (key < n_keys) & ((win <= 0) | (dist < win) | (key < a.keep_first));
          const float x = s[u][j] * a.scale - slope[hh] * (float)dist + hb[hh];
          w4[u][j] = seen ? __builtin_amdgcn_rcpf(1.f + __expf(-x)) : 0.f;  // (hardware exponential and reciprocal: no branches)
        }
      float* wr = wbuf + ((h0 + hh) * QR + rq) * WLD + oct * 8;
      *(f32x4*)wr = w4[0];
      *(f32x4*)(wr + 4) = w4[1];
    }
    if (ktn < n_keys) request_tile(ktn, slot_next);  // (on its way from memory during the meeting, the mix and the value products)
    __syncthreads();
    // mix: the wave's heads take their share of EVERY head's weight of the lane's (row, 8 keys)
    float m[HPW][8];
#pragma unroll
    for (int hh = 0; hh < HPW; hh++)
      for (int i = 0; i < 8; i++) m[hh][i] = 0.f;
    for (int g = 0; g < H; g++) {
      const float* wr = wbuf + (g * QR + rq) * WLD + oct * 8;
      const f32x4 wa = *(const f32x4*)wr, wb = *(const f32x4*)(wr + 4);
#pragma unroll
      for (int hh = 0; hh < HPW; hh++) {
        const float t = tk[(h0 + hh) * H + g];
        for (int i = 0; i < 4; i++) m[hh][i] = fmaf(t, wa[i], m[hh][i]), m[hh][4 + i] = fmaf(t, wb[i], m[hh][4 + i]);
      }
    }
    __syncthreads();
    u32x4 vf[VT];
#pragma unroll
    for (int t = 0; t < VT; t++) vf[t] = *(const u32x4*)(vt + (t * 16 + rq) * VLD + oct * 8);
#pragma unroll
    for (int hh = 0; hh < HPW; hh++) {
      u32x4 phi, plo;
      for (int e = 0; e < 4; e++) {
        const float a0 = m[hh][2 * e], a1 = m[hh][2 * e + 1];
        const uint32_t hi2 = BF16::pack2(a0, a1);
        phi[e] = hi2;
        plo[e] = BF16::pack2(a0 - __uint_as_float(hi2 << 16), a1 - __uint_as_float(hi2 & 0xffff0000u));
      }
#pragma unroll
      for (int t = 0; t < VT; t++) BF16::mfma(acc[hh][t], __builtin_bit_cast(s16x8, vf[t]), __builtin_bit_cast(s16x8, phi));
#pragma unroll
      for (int t = 0; t < VT; t++) BF16::mfma(acc[hh][t], __builtin_bit_cast(s16x8, vf[t]), __builtin_bit_cast(s16x8, plo));
      VRA_MFMA_DRAIN();  // (per head: the compiler may park a head's accumulators elsewhere between tiles)
    }
    kt0 = ktn;
  }
  if (!qv) return;
  uint16_t* out = (uint16_t*)a.out + (size_t)tq * H * vdim;
#pragma unroll
  for (int hh = 0; hh < HPW; hh++)
#pragma unroll
    for (int t = 0; t < VT; t++)
      for (int j = 0; j < 4; j++) {
        const int c = t * 16 + oct * 4 + j;
        if (c >= vdim) continue;
        float o = acc[hh][t][j];
        if (a.gate) o *= sigmoidf_(a.gate[(size_t)tq * a.gate_ld + (h0 + hh) * vdim + c]);
        out[(h0 + hh) * vdim + c] = BF16::from_f32(o);
      }
}

// out[t, h, d] = sigmoid(gate[t, h, d]) * sum_g talk[h, g] U[t, g, kv(h), d]   (g ascending)
template <typename T>
__global__ __launch_bounds__(256) void stk_sig_mix_kernel(const float* U, const float* talk, const float* gate, int gate_ld, T* out, int H, int G, int vdim) {
  const int t = blockIdx.x, HV = H * vdim, HG = H / G;
  for (int c = threadIdx.x; c < HV; c += 256) {
    const int h = c / vdim, d = c % vdim, kap = h / HG;
    float s = 0.f;
    for (int g = 0; g < H; g++) s = fmaf(talk[h * H + g], U[(((size_t)t * H + g) * G + kap) * vdim + d], s);
    if (gate) s *= sigmoidf_(gate[(size_t)t * gate_ld + c]);
    El<T>::st(out + (size_t)t * HV + c, s);
  }
}

// ------------------------------------------------------------------------------------------------ one token per sequence
// The keys a token sees (its window and the kept first tokens) are cut into 64-key tiles aligned to absolute positions; workgroup (b, s)
// takes the tiles s, s + S, ... of sequence b, ALL heads: scores lane-per-key straight from the cache (a key row is read once for the
// query heads of its group), weights and their mix through LDS, the value product with 8 channels per thread.  Nothing is normalised
// over keys, so the workgroups' partial sums simply add: a second launch adds them in order s = 0 .. S-1 and applies the gate.
struct SigTiles {
  int n_keep, win_first, n;  // tiles [0, n_keep) and [win_first, ...): n in all
};
__device__ __forceinline__ SigTiles sig_tiles(int64_t p, int n_keys, int window, int keep_first, int KT) {
  SigTiles t;
  const int last = (n_keys - 1) / KT;
  if (window <= 0) {
    t.n_keep = 0, t.win_first = 0, t.n = last + 1;
  } else {
    t.win_first = (int)(max((int64_t)0, p - window + 1) / KT);
    t.n_keep = min((max(keep_first, 0) + KT - 1) / KT, t.win_first);
    t.n = t.n_keep + last - t.win_first + 1;
  }
  return t;
}
template <typename T>
__global__ __launch_bounds__(256) void stk_sig_decode_kernel(StkSigAttnArgs a, float* partial, int S) {
  extern __shared__ float lds[];
  constexpr int KT = 64;
  const int dim = a.dim, vdim = a.vdim, H = a.H, G = a.G, HG = H / G, HV = H * vdim, GV = G * vdim;
  float* qs = lds;                 // [H][dim]
  float* ws = qs + H * dim;        // [H][64]
  float* ms = ws + H * KT;         // [H][64]
  float* tk = ms + H * KT;         // [H][H]
  int* sl = (int*)(tk + H * H);    // [64] cache slots of the tile's keys
  const int b = blockIdx.x, sp = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t p = a.positions[b];
  const int n_keys = (int)min((int64_t)a.context_lens[b], p + 1);
  const T* q = (const T*)a.q + (size_t)b * a.ldq;
  for (int i = tid; i < H * dim; i += 256) qs[i] = El<T>::ld(q + i);
  for (int i = tid; i < H * H; i += 256) tk[i] = a.talk ? a.talk[i] : ((i / H == i % H) ? 1.f : 0.f);
  const T* kc = (const T*)a.kc;
  const T* vc = (const T*)a.vc;
  const uint32_t* bt = a.block_tables + (size_t)b * a.max_blocks;
  const bool vec = sizeof(T) == 2 && vdim % 8 == 0 && ((uintptr_t)vc % 16) == 0;
  float acc[16];
#pragma unroll
  for (int i = 0; i < 16; i++) acc[i] = 0.f;
  const SigTiles tl = sig_tiles(p, max(n_keys, 1), a.window, a.keep_first, KT);
  for (int ti = sp; ti < tl.n && n_keys > 0; ti += S) {
    const int kt0 = (ti < tl.n_keep ? ti : tl.win_first + ti - tl.n_keep) * KT;
    __syncthreads();
    if (tid < KT) {
      const int key = kt0 + tid;
      sl[tid] = key < n_keys ? (int)((int64_t)bt[key / a.BS] * a.BS + key % a.BS) : 0;
    }
    __syncthreads();
    {
      const int key = kt0 + lane;
      const int64_t dist = p - key;
      const bool seen = key < n_keys && dist >= 0 && (a.window <= 0 || dist < a.window || key < a.keep_first);
      for (int g = wave; g < G; g += 4) {
        const T* kr = kc + (int64_t)sl[lane] * (G * dim) + g * dim;
        for (int h0 = 0; h0 < HG; h0 += 4) {  // up to four query heads of the group share one pass over the key row
          float d4[4] = {0.f, 0.f, 0.f, 0.f};
          const float* q4 = qs + (g * HG + h0) * dim;
          const int nh = min(4, HG - h0);
          if (seen) {
            if (sizeof(T) == 2 && dim % 8 == 0 && ((uintptr_t)kr % 16) == 0) {
              for (int d0 = 0; d0 < dim; d0 += 32) {  // four 16-byte requests of the key row in flight, then their sums (d ascending)
                u32x4 kv4[4];
                for (int x = 0; x < 4; x++) kv4[x] = *(const u32x4*)((const uint16_t*)kr + (d0 + 8 * x < dim ? d0 + 8 * x : 0));
                for (int x = 0; x < 4; x++) {
                  const int d = d0 + 8 * x;
                  if (d >= dim) break;
                  for (int e = 0; e < 4; e++) {
                    const float k0 = __uint_as_float(kv4[x][e] << 16), k1 = __uint_as_float(kv4[x][e] & 0xffff0000u);
                    for (int u = 0; u < 4; u++)
                      if (u < nh) d4[u] = fmaf(q4[u * dim + d + 2 * e + 1], k1, fmaf(q4[u * dim + d + 2 * e], k0, d4[u]));
                  }
                }
              }
            } else {
              for (int d = 0; d < dim; d++) {
                const float kv = El<T>::ld(kr + d);
                for (int u = 0; u < 4; u++)
                  if (u < nh) d4[u] = fmaf(q4[u * dim + d], kv, d4[u]);
              }
            }
          }
          for (int u = 0; u < nh; u++) {
            const int h = g * HG + h0 + u;
            const float x = d4[u] * a.scale - (a.slopes ? a.slopes[h] : 0.f) * (float)dist + (a.head_bias ? a.head_bias[h] : 0.f);
            ws[h * KT + lane] = seen ? sigmoidf_(x) : 0.f;
          }
        }
      }
    }
    __syncthreads();
    for (int i = tid; i < H * KT; i += 256) {
      const int h = i / KT, j = i % KT;
      float s = 0.f;
      for (int g = 0; g < H; g++) s = fmaf(tk[h * H + g], ws[g * KT + j], s);
      ms[i] = s;
    }
    __syncthreads();
    const int nj = min(KT, n_keys - kt0);
    if (vec) {  // thread = 8 consecutive channels of one head per round: one 16-byte load per key
#pragma unroll
      for (int n = 0; n < 2; n++) {
        const int c8 = (tid + n * 256) * 8;
        if (c8 < HV) {
          const int h = c8 / vdim, d = c8 % vdim, g = h / HG;
          const float* mw = ms + h * KT;
          for (int j0 = 0; j0 < nj; j0 += 8) {  // eight value rows requested together; rows beyond the tile count with weight 0
            u32x4 v[8];
            float w[8];
            for (int u = 0; u < 8; u++) {
              const bool in = j0 + u < nj;
              v[u] = *(const u32x4*)((const uint16_t*)vc + (int64_t)sl[in ? j0 + u : j0] * GV + g * vdim + d);
              w[u] = in ? mw[j0 + u] : 0.f;
            }
            for (int u = 0; u < 8; u++)
              for (int e = 0; e < 4; e++) {
                acc[n * 8 + 2 * e] = fmaf(w[u], __uint_as_float(v[u][e] << 16), acc[n * 8 + 2 * e]);
                acc[n * 8 + 2 * e + 1] = fmaf(w[u], __uint_as_float(v[u][e] & 0xffff0000u), acc[n * 8 + 2 * e + 1]);
              }
          }
        }
      }
    } else {
#pragma unroll
      for (int n = 0; n < 16; n++) {
        const int c = tid + n * 256;
        if (c < HV) {
          const int h = c / vdim, d = c % vdim, g = h / HG;
          const float* mw = ms + h * KT;
          float o = acc[n];
          for (int j = 0; j < nj; j++) o = fmaf(mw[j], El<T>::ld(vc + (int64_t)sl[j] * GV + g * vdim + d), o);
          acc[n] = o;
        }
      }
    }
  }
  float* po = partial + ((size_t)b * S + sp) * HV;
  if (vec) {
    for (int n = 0; n < 2; n++) {
      const int c8 = (tid + n * 256) * 8;
      if (c8 < HV)
        for (int e = 0; e < 8; e++) po[c8 + e] = acc[n * 8 + e];
    }
  } else {
    for (int n = 0; n < 16; n++) {
      const int c = tid + n * 256;
      if (c < HV) po[c] = acc[n];
    }
  }
}
template <typename T>
__global__ __launch_bounds__(256) void stk_sig_decode_sum_kernel(const float* partial, int S, const float* gate, int gate_ld, T* out, int HV) {
  const int b = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= HV) return;
  const float* pp = partial + (size_t)b * S * HV + c;
  float s = 0.f;
  int i = 0;
  for (; i + 8 <= S; i += 8) {  // (eight requests in flight; the sum keeps the order i = 0 .. S-1)
    float v[8];
    for (int u = 0; u < 8; u++) v[u] = pp[(size_t)(i + u) * HV];
    for (int u = 0; u < 8; u++) s += v[u];
  }
  for (; i < S; i++) s += pp[(size_t)i * HV];
  if (gate) s *= sigmoidf_(gate[(size_t)b * gate_ld + c]);
  El<T>::st(out + (size_t)b * HV + c, s);
}

}  // namespace

// ================================================================================================ launchers
void vra_stack_dyt(float* x, const float* add, const float* w, const float* b, float alpha, void* h, int T, int W, int dtype, int64_t stream) {
  VRA_CHECK_ARG(x && w && b && h && T > 0 && W > 0, "stack dyt: null pointer or empty shape");
  const int64_t n = (int64_t)T * W;
  const int grid = (int)std::min<int64_t>((n + 255) / 256, 4096);
  if (dtype == VRA_F32) launch_checked("stack dyt", [&] { stk_dyt_kernel<float><<<grid, 256, 0, as_stream(stream)>>>(x, add, w, b, alpha, (float*)h, W, n); });
  else launch_checked("stack dyt", [&] { stk_dyt_kernel<uint16_t><<<grid, 256, 0, as_stream(stream)>>>(x, add, w, b, alpha, (uint16_t*)h, W, n); });
}

void vra_stack_latent_prep(const StkLatentPrepArgs& a, int dtype, int64_t stream) {
  VRA_CHECK_ARG(a.raw && a.qn_w && a.kvn_w && a.cq && a.cache && a.slots && a.positions && a.T > 0, "stack latent prep: null pointer or empty shape");
  VRA_CHECK_ARG(a.q_rank > 0 && a.kv_rank > 0 && a.rot_dim >= 0 && a.ld >= a.q_rank + a.kv_rank + a.rot_dim && a.cache_ld >= a.kv_rank + a.rot_dim,
                "stack latent prep: row shorter than its parts");
  VRA_CHECK_ARG(a.rot.pairs * 2 <= a.rot_dim && (a.rot.pairs == 0 || a.rot.freq_hi), "stack latent prep: more rotated pairs than the rotated part holds");
  if (dtype == VRA_F32) launch_checked("stack latent prep", [&] { stk_latent_prep_kernel<float><<<a.T, 256, 0, as_stream(stream)>>>(a); });
  else launch_checked("stack latent prep", [&] { stk_latent_prep_kernel<uint16_t><<<a.T, 256, 0, as_stream(stream)>>>(a); });
}

void vra_stack_rope_heads(const void* in, int in_ld, int in_hs, int in_off, void* out, int out_ld, int out_hs, int out_off, int n, int H,
                          const int64_t* positions, const StkRotary& rot, int T, int dtype, int64_t stream) {
  VRA_CHECK_ARG(in && out && positions && T > 0 && H > 0 && n > 0, "stack rope: null pointer or empty shape");
  VRA_CHECK_ARG(rot.pairs * 2 <= n && (rot.pairs == 0 || rot.freq_hi), "stack rope: more rotated pairs than the vector holds");
  if (dtype == VRA_F32)
    launch_checked("stack rope", [&] {
      stk_rope_heads_kernel<float><<<T, 256, 0, as_stream(stream)>>>((const float*)in, in_ld, in_hs, in_off, (float*)out, out_ld, out_hs, out_off, n, H, positions, rot);
    });
  else
    launch_checked("stack rope", [&] {
      stk_rope_heads_kernel<uint16_t><<<T, 256, 0, as_stream(stream)>>>((const uint16_t*)in, in_ld, in_hs, in_off, (uint16_t*)out, out_ld, out_hs, out_off, n, H,
                                                                        positions, rot);
    });
}

void vra_stack_qk_norm_store(const float* raw, int ld, int nq, int nk, int nv, const float* q_w, const float* k_w, float eps, void* q_out, void* kc,
                             void* vc, const int64_t* slots, int T, int dtype, int64_t stream) {
  VRA_CHECK_ARG(raw && q_out && kc && vc && slots && T > 0 && nq > 0 && nk > 0 && nv > 0 && ld >= nq + nk + nv, "stack qk norm: null pointer or empty shape");
  if (dtype == VRA_F32)
    launch_checked("stack qk norm", [&] {
      stk_qk_norm_store_kernel<float><<<T, 256, 0, as_stream(stream)>>>(raw, ld, nq, nk, nv, q_w, k_w, eps, (float*)q_out, (float*)kc, (float*)vc, slots);
    });
  else
    launch_checked("stack qk norm", [&] {
      stk_qk_norm_store_kernel<uint16_t><<<T, 256, 0, as_stream(stream)>>>(raw, ld, nq, nk, nv, q_w, k_w, eps, (uint16_t*)q_out, (uint16_t*)kc, (uint16_t*)vc, slots);
    });
}

void vra_stack_sigmoid_attention(const StkSigAttnArgs& a, int dtype, int64_t stream) {
  VRA_CHECK_ARG(a.q && a.out && a.kc && a.vc && a.positions && a.block_tables && a.context_lens, "stack sigmoid attention: null pointer");
  VRA_CHECK_ARG(a.B > 0 && a.H > 0 && a.G > 0 && a.H % a.G == 0 && a.dim > 0 && a.vdim > 0 && a.BS > 0 && a.max_blocks > 0 && a.max_q > 0,
                "stack sigmoid attention: heads must be a multiple of kv heads, sizes positive");
  VRA_CHECK_ARG(!a.gate || a.gate_ld >= a.H * a.vdim, "stack sigmoid attention: gate rows shorter than the output");
  hipStream_t st = as_stream(stream);
  const int HV = a.H * a.vdim;
  const bool decode = !a.cu_q;
  if (decode && a.scratch && HV <= 4096) {
    // tiles a token can see: the kept first tokens, its window and one more for the window's alignment; without a window, the context
    int S = a.window > 0 ? (std::max(a.keep_first, 0) + 63) / 64 + (a.window + 63) / 64 + 1 : std::max(1, (std::max(a.max_len, 1) + 63) / 64);
    S = std::min(S, 64);
    const size_t lds = ((size_t)a.H * a.dim + 2 * (size_t)a.H * 64 + (size_t)a.H * a.H + 64) * sizeof(float);
    if (lds <= 64 * 1024 && (size_t)a.B * S * HV * sizeof(float) <= a.scratch_bytes) {
      dim3 grid(a.B, S);
      if (dtype == VRA_F32) {
        launch_checked("stack sigmoid attention (decode)", [&] { stk_sig_decode_kernel<float><<<grid, 256, lds, st>>>(a, a.scratch, S); });
        launch_checked("stack sigmoid attention (decode sum)", [&] { stk_sig_decode_sum_kernel<float><<<dim3(a.B, (HV + 255) / 256), 256, 0, st>>>(a.scratch, S, a.gate, a.gate_ld, (float*)a.out, HV); });
      } else {
        launch_checked("stack sigmoid attention (decode)", [&] { stk_sig_decode_kernel<uint16_t><<<grid, 256, lds, st>>>(a, a.scratch, S); });
        launch_checked("stack sigmoid attention (decode sum)", [&] { stk_sig_decode_sum_kernel<uint16_t><<<dim3(a.B, (HV + 255) / 256), 256, 0, st>>>(a.scratch, S, a.gate, a.gate_ld, (uint16_t*)a.out, HV); });
      }
      return;
    }
  }
  const bool mfma_ok = !decode && dtype == VRA_BF16 && a.dim % 8 == 0 && a.vdim % 16 == 0 && a.dim <= 128 && a.vdim <= 128 && a.ldq % 8 == 0 &&
                       ((uintptr_t)a.q % 16 == 0) && ((uintptr_t)a.kc % 16 == 0) && ((uintptr_t)a.vc % 16 == 0) && a.BS % 32 == 0;
  // all heads in one workgroup: 4 waves of 1, 2 or 4 heads; a wave's heads share one key/value head
  const int nw = 4, hpw = a.H / nw;
  const bool per_head_ok = mfma_ok && a.scratch && a.talk && (size_t)a.T * a.H * a.G * a.vdim * sizeof(float) <= a.scratch_bytes;
  // Its time follows the longest row block's key tiles, whatever the step's size (16 rows a workgroup: a 2048-token step is 128
  // workgroups), the per-head kernel's follows the step's total work: measured at 16:4 heads of 128, 282 us against 395 at 2048 tokens,
  // 154 against 101 at 512 — so short steps go to the per-head kernel when its scratch is there.
  if (mfma_ok && (a.H == 4 || a.H == 8 || a.H == 16) && (a.H / a.G) % hpw == 0 && (a.T >= 1536 || !per_head_ok)) {
    const int vt = (a.dim <= 64 && a.vdim <= 64) ? 4 : 8;
    const size_t lds = ((size_t)a.H * 16 * 36 + (size_t)a.H * a.H) * sizeof(float) + (size_t)nw * vt * 16 * 40 * sizeof(uint16_t);
    dim3 grid((a.max_q + 15) / 16, a.B);
#define STK_SGH(DCV, VTV, HPWV, NWV)                                                                                                     \
  do {                                                                                                                                    \
    static bool attr = false;                                                                                                             \
    if (!attr) {                                                                                                                          \
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&stk_sig_prefill_heads_kernel<DCV, VTV, HPWV, NWV>),                        \
                                hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);                                                  \
      attr = true;                                                                                                                        \
    }                                                                                                                                     \
    launch_checked("stack sigmoid attention (prefill, all heads)",                                                                        \
                   [&] { stk_sig_prefill_heads_kernel<DCV, VTV, HPWV, NWV><<<grid, 64 * NWV, lds, st>>>(a); });                             \
  } while (0)
    if (vt == 4) {
      if (a.H == 4) STK_SGH(2, 4, 1, 4);
      else if (a.H == 8) STK_SGH(2, 4, 2, 4);
      else STK_SGH(2, 4, 4, 4);
    } else {
      if (a.H == 4) STK_SGH(4, 8, 1, 4);
      else if (a.H == 8) STK_SGH(4, 8, 2, 4);
      else STK_SGH(4, 8, 4, 4);
    }
#undef STK_SGH
    return;
  }
  if (per_head_ok) {
    const int gc = a.G >= 2 ? 2 : 1;  // value heads per workgroup: two keep the accumulators in registers, the scores are computed G / 2 times
    dim3 grid((a.max_q + 63) / 64, a.B, a.H * ((a.G + gc - 1) / gc));
#define STK_SGM(DCV, VTV, GCV) launch_checked("stack sigmoid attention (prefill, mfma)", [&] { stk_sig_prefill_mfma_kernel<DCV, VTV, GCV><<<grid, 256, 0, st>>>(a, a.scratch); })
    if (a.dim <= 64 && a.vdim <= 64) {
      if (gc == 2) STK_SGM(2, 4, 2);
      else STK_SGM(2, 4, 1);
    } else {
      if (gc == 2) STK_SGM(4, 8, 2);
      else STK_SGM(4, 8, 1);
    }
#undef STK_SGM
    launch_checked("stack sigmoid attention (mix)", [&] {
      stk_sig_mix_kernel<uint16_t><<<a.T, 256, 0, st>>>(a.scratch, a.talk, a.gate, a.gate_ld, (uint16_t*)a.out, a.H, a.G, a.vdim);
    });
    return;
  }
  int qt, nacc;
  if (decode) qt = 1, nacc = HV <= 4096 ? 16 : 64;
  else if (HV <= 256) qt = 16, nacc = 16;
  else if (HV <= 1024) qt = 16, nacc = 64;
  else if (HV <= 4096) qt = 4, nacc = 64;
  else qt = 1, nacc = 64;
  VRA_CHECK_ARG(HV <= (256 / qt) * nacc, "stack sigmoid attention: more output channels than the kernel's accumulators hold");
  auto need = [&](int kt) {
    return ((size_t)qt * a.dim + (size_t)kt * (a.dim + 1) + (size_t)(a.talk ? 2 : 1) * a.H * qt * kt + (size_t)kt * a.G * a.vdim + (size_t)a.H * a.H) * sizeof(float);
  };
  int kt = 64;
  while (kt > 8 && need(kt) > 64 * 1024) kt >>= 1;
  VRA_CHECK_ARG(need(kt) <= 64 * 1024, "stack sigmoid attention: heads do not fit LDS");
  const size_t lds = need(kt);
  dim3 grid(decode ? 1 : (a.max_q + qt - 1) / qt, a.B);
#define STK_SG(TT, QTV, NA) launch_checked("stack sigmoid attention", [&] { stk_sig_attn_kernel<TT, QTV, NA><<<grid, 256, lds, st>>>(a, kt); })
#define STK_SG_T(TT)                          \
  if (qt == 16 && nacc == 16) STK_SG(TT, 16, 16); \
  else if (qt == 16) STK_SG(TT, 16, 64);          \
  else if (qt == 4) STK_SG(TT, 4, 64);            \
  else if (nacc == 16) STK_SG(TT, 1, 16);         \
  else STK_SG(TT, 1, 64)
  if (dtype == VRA_F32) {
    STK_SG_T(float);
  } else {
    STK_SG_T(uint16_t);
  }
#undef STK_SG_T
#undef STK_SG
}

// ================================================================================================ C entry points (one operator each)
extern "C" void vra_stack_op_dyt(float* x, const float* add, const float* w, const float* b, float alpha, void* h, int32_t T, int32_t W, int32_t dtype,
                                 int64_t stream) {
  vra_stack_dyt(x, add, w, b, alpha, h, T, W, dtype, stream);
}
extern "C" void vra_stack_op_latent_prep(const float* raw, int32_t ld, int32_t q_rank, int32_t kv_rank, int32_t rot_dim, const float* qn_w,
                                         const float* kvn_w, float eps, void* cq, void* cache, int32_t cache_ld, const int64_t* slots,
                                         const int64_t* positions, const float* freq_hi, const float* freq_lo, int32_t pairs, float mag, int32_t T,
                                         int32_t dtype, int64_t stream) {
  StkLatentPrepArgs a;
  a.raw = raw, a.ld = ld, a.q_rank = q_rank, a.kv_rank = kv_rank, a.rot_dim = rot_dim, a.qn_w = qn_w, a.kvn_w = kvn_w, a.eps = eps, a.cq = cq;
  a.cache = cache, a.cache_ld = cache_ld, a.slots = slots, a.positions = positions, a.T = T;
  a.rot.freq_hi = freq_hi, a.rot.freq_lo = freq_lo, a.rot.pairs = pairs, a.rot.mag = mag;
  vra_stack_latent_prep(a, dtype, stream);
}
extern "C" void vra_stack_op_rope_heads(const void* in, int32_t in_ld, int32_t in_hs, int32_t in_off, void* out, int32_t out_ld, int32_t out_hs,
                                        int32_t out_off, int32_t n, int32_t H, const int64_t* positions, const float* freq_hi, const float* freq_lo,
                                        int32_t pairs, float mag, int32_t T, int32_t dtype, int64_t stream) {
  StkRotary r;
  r.freq_hi = freq_hi, r.freq_lo = freq_lo, r.pairs = pairs, r.mag = mag;
  vra_stack_rope_heads(in, in_ld, in_hs, in_off, out, out_ld, out_hs, out_off, n, H, positions, r, T, dtype, stream);
}
extern "C" void vra_stack_op_qk_norm_store(const float* raw, int32_t ld, int32_t nq, int32_t nk, int32_t nv, const float* q_w, const float* k_w, float eps,
                                           void* q_out, void* kc, void* vc, const int64_t* slots, int32_t T, int32_t dtype, int64_t stream) {
  vra_stack_qk_norm_store(raw, ld, nq, nk, nv, q_w, k_w, eps, q_out, kc, vc, slots, T, dtype, stream);
}
extern "C" void vra_stack_op_sigmoid_attention(const void* q, int32_t ldq, void* out, const void* kc, const void* vc, const int64_t* positions,
                                               const uint32_t* block_tables, const uint32_t* context_lens, const uint32_t* cu_q, int32_t B, int32_t T,
                                               int32_t max_q, int32_t H, int32_t G, int32_t dim, int32_t vdim, int32_t BS, int32_t max_blocks, float scale,
                                               int32_t window, int32_t keep_first, const float* slopes, const float* head_bias, const float* talk,
                                               const float* gate, int32_t gate_ld, float* scratch, int64_t scratch_bytes, int32_t max_len, int32_t dtype, int64_t stream) {
  StkSigAttnArgs a;
  a.q = q, a.ldq = ldq, a.out = out, a.kc = kc, a.vc = vc, a.positions = positions, a.block_tables = block_tables, a.context_lens = context_lens;
  a.cu_q = cu_q, a.B = B, a.T = T, a.max_q = max_q, a.H = H, a.G = G, a.dim = dim, a.vdim = vdim, a.BS = BS, a.max_blocks = max_blocks;
  a.scale = scale, a.window = window, a.keep_first = keep_first, a.slopes = slopes, a.head_bias = head_bias, a.talk = talk, a.gate = gate;
  a.gate_ld = gate_ld, a.scratch = scratch, a.scratch_bytes = (size_t)scratch_bytes, a.max_len = max_len;
  vra_stack_sigmoid_attention(a, dtype, stream);
}
// the matrix product with every option of StkGemmArgs: bias, batched form, kind of the gated pair
extern "C" void vra_stack_op_gemm_ex(const void* a, int32_t lda, const void* w, void* out, int32_t ldo, int32_t out_f32, int32_t M, int32_t N, int32_t K,
                                     float alpha, const float* bias, int32_t epi, int32_t act, int32_t batch, int64_t a_batch_stride,
                                     int64_t w_batch_stride, int64_t out_batch_stride, int32_t dtype, int64_t stream) {
  StkGemmArgs g;
  g.a = a, g.lda = lda, g.w = w, g.out = out, g.ldo = ldo, g.out_f32 = out_f32, g.M = M, g.N = N, g.K = K, g.alpha = alpha, g.bias = bias;
  g.epi = epi, g.act = act, g.batch = batch, g.a_batch_stride = a_batch_stride, g.w_batch_stride = w_batch_stride, g.out_batch_stride = out_batch_stride;
  vra_stack_gemm(g, dtype, stream);
}
// the softmax attention with a sink and a latent cache's row layout
extern "C" void vra_stack_op_attention_ex(const void* q, int32_t ldq, void* out, const void* kc, const void* vc, const int64_t* positions,
                                          const uint32_t* block_tables, const uint32_t* context_lens, const uint32_t* cu_q, int32_t B, int32_t T,
                                          int32_t max_q, int32_t H, int32_t G, int32_t dim, int32_t vdim, int32_t BS, int32_t max_blocks, float scale,
                                          const float* sink, int32_t k_ld, int32_t v_ld, int32_t dtype, int64_t stream) {
  StkAttnArgs a;
  a.q = q, a.ldq = ldq, a.out = out, a.kc = kc, a.vc = vc, a.positions = positions, a.block_tables = block_tables, a.context_lens = context_lens;
  a.cu_q = cu_q, a.B = B, a.T = T, a.max_q = max_q, a.H = H, a.G = G, a.dim = dim, a.vdim = vdim, a.BS = BS, a.max_blocks = max_blocks;
  a.scale = scale, a.sink = sink, a.k_ld = k_ld, a.v_ld = v_ld;
  vra_stack_attention(a, dtype, stream);
}
