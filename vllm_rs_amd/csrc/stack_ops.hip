// stack_ops.hip — operators of config-driven layer stacks (host/stack_model.cpp; every operator is specified in stack_launch.h), gfx950.
//
// What is kept in f32 whatever the storage type: positions and angles, norms, router logits and weights, attention scores and
// softmax weights (the value product included: p stays f32, v is widened), the residual stream and every sum into it.
// Matrix products: bf16 operands on v_mfma_f32_16x16x32_bf16 with f32 accumulation, or f32 operands on FMA (VRA_F32: no reduced
// matrix mode anywhere).  Every reduction has an order that depends on the shapes of the model alone — never on the number of rows
// of a step, on a row's place in the batch or on the pages it uses — so a token's result does not depend on how its prompt was cut.
#include <math.h>

#include "stack_common.cuh"
#include "stack_launch.h"

namespace {

__device__ __forceinline__ float gelu_tanh_(float z) { return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }
// act 0: min(g, L) * sigmoid(act_alpha * min(g, L)) * (clamp(u, +-L) + 1);  act 1: gelu_tanh(g) * u;  act 2: silu(g) * u
__device__ __forceinline__ float gated_pair(float g, float u, float limit, float act_alpha, int act = 0) {
  if (act == 1) return gelu_tanh_(g) * u;
  if (act == 2) return g * sigmoidf_(g) * u;
  if (limit > 0.f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  return g * sigmoidf_(act_alpha * g) * (u + 1.f);
}

// ------------------------------------------------------------------------------------------------ embedding + positions
template <typename T>
__global__ __launch_bounds__(256) void stk_embed_sinpos_kernel(const uint32_t* ids, const int64_t* pos, const T* embed, const float* inv_freq, float* x,
                                                               int W, int V) {
  const int t = blockIdx.x;
  uint32_t id = ids[t];
  if (id >= (uint32_t)V) id = 0;
  const float p = (float)pos[t];
  for (int c = threadIdx.x; c < W; c += 256) {
    float pe = 0.f;
    if (inv_freq) {
      const float ang = p * inv_freq[c >> 1];
      pe = (c & 1) ? cosf(ang) : sinf(ang);
    }
    x[(size_t)t * W + c] = El<T>::ld(embed + (size_t)id * W + c) + pe;
  }
}

// ------------------------------------------------------------------------------------------------ grouped RMS norm (+ router)
template <typename T>
__global__ __launch_bounds__(256) void stk_group_norm_kernel(StkNormArgs a) {
  extern __shared__ float lds[];
  float* xs = lds;                      // [W] the row, then the normalised row
  float* rs = lds + a.W;                // [groups] 1 / rms
  float* zs = rs + a.groups;            // [n_router + gate_row]
  const int t = blockIdx.x, W = a.W, gs = W / a.groups;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const float* x = a.x + (size_t)t * W;
  for (int c = threadIdx.x; c < W; c += 256) xs[c] = x[c];
  __syncthreads();
  for (int g = wave; g < a.groups; g += 4) {
    float s = 0.f;
    for (int c = lane; c < gs; c += 64) {
      const float v = xs[g * gs + c];
      s = fmaf(v, v, s);
    }
    s = wave_sum(s);
    if (lane == 0) rs[g] = 1.f / sqrtf(s / (float)gs + a.eps);
  }
  __syncthreads();
  T* h = (T*)a.h + (size_t)t * W;
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = xs[c] * rs[c / gs] * a.w[c];
    xs[c] = v;
    El<T>::st(h + c, v);
  }
  if (!a.router_w) return;
  __syncthreads();
  const int nz = a.n_router + (a.gate_row ? 1 : 0);
  const T* rw = (const T*)a.router_w;
  for (int e = wave; e < nz; e += 4) {
    float s = 0.f;
    if (sizeof(T) == 2 && W % 8 == 0 && ((uintptr_t)rw % 16) == 0) {  // 8 weights a load; the lane's partial sums keep one order for a given W
      for (int c = lane * 8; c < W; c += 64 * 8) {
        const u32x4 v = *(const u32x4*)((const uint16_t*)rw + (size_t)e * W + c);
        for (int i = 0; i < 4; i++) {
          s = fmaf(xs[c + 2 * i], __uint_as_float(v[i] << 16), s);
          s = fmaf(xs[c + 2 * i + 1], __uint_as_float(v[i] & 0xffff0000u), s);
        }
      }
    } else {
      for (int c = lane; c < W; c += 64) s = fmaf(xs[c], El<T>::ld(rw + (size_t)e * W + c), s);
    }
    s = wave_sum(s);
    if (lane == 0) zs[e] = s;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int j = 0; j < a.top; j++) {
      int best = -1;
      float bz = -INFINITY;
      for (int e = 0; e < a.n_router; e++) {
        bool taken = false;
        for (int q = 0; q < j; q++) taken = taken || a.pair_expert[(size_t)t * a.top + q] == e;
        if (!taken && (best < 0 || zs[e] > bz)) best = e, bz = zs[e];
      }
      a.pair_expert[(size_t)t * a.top + j] = best;
      a.pair_weight[(size_t)t * a.top + j] = sigmoidf_(bz);
    }
    if (a.gate_row) a.gate_out[t] = sigmoidf_(zs[a.n_router]);
  }
}

// ------------------------------------------------------------------------------------------------ MoE rows sorted by expert
__global__ __launch_bounds__(1024) void stk_moe_sort_kernel(const int* pair_expert, const float* pair_weight, int P, int top, int n_groups, int granule,
                                                            int max_rows, int* row_token, float* row_scale, int* row_pair, int* tile_group) {
  extern __shared__ int sl[];
  int* counts = sl;
  int* offs = sl + n_groups;
  int* cursor = offs + n_groups;
  const int tid = threadIdx.x;
  for (int e = tid; e < n_groups; e += 1024) counts[e] = 0, cursor[e] = 0;
  for (int r = tid; r < max_rows; r += 1024) row_token[r] = -1, row_pair[r] = -1, row_scale[r] = 0.f;
  for (int t = tid; t < max_rows / granule; t += 1024) tile_group[t] = -1;
  __syncthreads();
  for (int p = tid; p < P; p += 1024) {
    const int e = pair_expert[p];
    if (e >= 0 && e < n_groups) atomicAdd(&counts[e], 1);
  }
  __syncthreads();
  if (tid == 0) {
    int off = 0;
    for (int e = 0; e < n_groups; e++) {
      offs[e] = off;
      const int nt = (counts[e] + granule - 1) / granule;
      for (int t = 0; t < nt; t++) tile_group[off / granule + t] = e;
      off += nt * granule;
    }
  }
  __syncthreads();
  for (int p = tid; p < P; p += 1024) {
    const int e = pair_expert[p];
    if (e < 0 || e >= n_groups) continue;
    const int r = offs[e] + atomicAdd(&cursor[e], 1);
    row_token[r] = p / top;
    row_scale[r] = pair_weight[p];
    row_pair[r] = p;
  }
}

// ------------------------------------------------------------------------------------------------ GEMM, f32 FMA (any shape)
// 256 threads: 16 (m) x 16 (n) threads, RM rows x 4 columns each; K in steps of 16 through LDS; k ascending: one fixed order.
template <typename T, int RM>
__global__ __launch_bounds__(256) void stk_gemm_simple_kernel(StkGemmArgs g) {
  constexpr int TM = 16 * RM;
  __shared__ float As[16][TM + 1];
  __shared__ float Ws[16][65];
  __shared__ int a_idx[TM];
  __shared__ float a_sc[TM];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.x * TM, n0 = blockIdx.y * 64;
  int group = 0;
  if (g.tile_group) {
    group = g.tile_group[blockIdx.x];
    if (group < 0) return;
  }
  const T* A = (const T*)g.a + (int64_t)blockIdx.z * g.a_batch_stride;
  const T* Wt = (const T*)g.w + (int64_t)group * g.w_group_stride + (int64_t)blockIdx.z * g.w_batch_stride;
  const int64_t ob = (int64_t)blockIdx.z * g.out_batch_stride;
  if (tid < TM) {
    const int r = m0 + tid;
    int idx = r < g.M ? (g.a_row ? g.a_row[r] : r) : -1;
    a_idx[tid] = idx;
    a_sc[tid] = g.a_scale && idx >= 0 ? g.a_scale[r] : 1.f;
  }
  __syncthreads();
  float acc[RM][4];
  for (int i = 0; i < RM; i++)
    for (int j = 0; j < 4; j++) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < g.K; k0 += 16) {
    for (int i = tid; i < TM * 16; i += 256) {
      const int r = i >> 4, kk = i & 15, idx = a_idx[r];
      float v = 0.f;
      if (idx >= 0 && k0 + kk < g.K) {
        v = El<T>::ld(A + (int64_t)idx * g.lda + k0 + kk);
        if (g.a_scale) v = El<T>::rnd(v * a_sc[r]);
      }
      As[kk][r] = v;
    }
    for (int i = tid; i < 64 * 16; i += 256) {
      const int n = i >> 4, kk = i & 15;
      Ws[kk][n] = (n0 + n < g.N && k0 + kk < g.K) ? El<T>::ld(Wt + (int64_t)(n0 + n) * g.K + k0 + kk) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; kk++) {
      float av[RM], wv[4];
      for (int i = 0; i < RM; i++) av[i] = As[kk][ty * RM + i];
      for (int j = 0; j < 4; j++) wv[j] = Ws[kk][tx * 4 + j];
      for (int i = 0; i < RM; i++)
        for (int j = 0; j < 4; j++) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
  for (int i = 0; i < RM; i++) {
    const int r = m0 + ty * RM + i;
    if (r >= g.M || a_idx[ty * RM + i] < 0) continue;
    const int orow = g.out_row ? g.out_row[r] : r;
    if (orow < 0) continue;
    for (int j = 0; j < 4; j++) {
      const int n = n0 + tx * 4 + j;
      if (n >= g.N) continue;
      const float v = acc[i][j] * g.alpha + (g.bias ? g.bias[(int64_t)blockIdx.z * g.bias_batch_stride + n] : 0.f);
      if (g.out_f32) ((float*)g.out)[ob + (int64_t)orow * g.ldo + n] = v;
      else El<T>::st((T*)g.out + ob + (int64_t)orow * g.ldo + n, v);
    }
  }
}

// ------------------------------------------------------------------------------------------------ GEMM, bf16 MFMA (K % 8 == 0)
// A wave owns MT x NT tiles of 16 x 16; both operands come straight from global memory in the instruction's operand order (lane =
// (row rq = lane & 15, k octet oct = lane >> 4): 16 bytes of one row per lane and K-step of 32), the weights as the A operand and the
// activations as B, so a lane ends up with 4 consecutive output columns of ONE activation row.  K ascending in steps of 32.
template <int MT, int NT, int WM, int WN, bool SCALED>
__global__ __launch_bounds__(64 * WM * WN) void stk_gemm_mfma_kernel(StkGemmArgs g) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave % WM, wn = wave / WM, rq = lane & 15, oct = lane >> 4;
  int group = 0;
  if (g.tile_group) {
    group = g.tile_group[blockIdx.x];
    if (group < 0) return;
  }
  const uint16_t* A = (const uint16_t*)g.a + (int64_t)blockIdx.z * g.a_batch_stride;
  const uint16_t* Wt = (const uint16_t*)g.w + (int64_t)group * g.w_group_stride + (int64_t)blockIdx.z * g.w_batch_stride;
  const int64_t ob = (int64_t)blockIdx.z * g.out_batch_stride;
  const int m_base = blockIdx.x * (16 * MT * WM) + wm * 16 * MT;
  const int n_base = blockIdx.y * (16 * NT * WN) + wn * 16 * NT;
  const uint16_t* ap[MT];
  const uint16_t* wp[NT];
  bool av[MT], wv[NT];
  float asc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    const int r = m_base + mt * 16 + rq;
    const int idx = r < g.M ? (g.a_row ? g.a_row[r] : r) : -1;
    av[mt] = idx >= 0;
    ap[mt] = A + (int64_t)(idx >= 0 ? idx : 0) * g.lda;
    asc[mt] = SCALED && idx >= 0 ? g.a_scale[r] : 1.f;
  }
#pragma unroll
  for (int nt = 0; nt < NT; nt++) {
    const int n = n_base + nt * 16 + rq;
    wv[nt] = n < g.N;
    wp[nt] = Wt + (int64_t)(n < g.N ? n : 0) * g.K;
  }
  f32x4 acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++)
#pragma unroll
    for (int nt = 0; nt < NT; nt++) acc[mt][nt] = vra_zero_acc();
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  // the fragments of K-step k + 1 are requested before the MFMAs of step k run
  u32x4 af[MT], wf[NT], afn[MT], wfn[NT];
  auto request = [&](int k0, u32x4* ao, u32x4* wo) {
    const int k = k0 + oct * 8;
    const bool kin = k < g.K;
    const int kc = kin ? k : 0;
  #pragma unroll
  for (int mt = 0; mt < MT; mt++) {
      u32x4 v = *(const u32x4*)(ap[mt] + kc);
      if (SCALED) {
        const float s = asc[mt];
        for (int i = 0; i < 4; i++) {
          const float lo = __uint_as_float(v[i] << 16) * s, hi = __uint_as_float(v[i] & 0xffff0000u) * s;
          v[i] = BF16::pack2(lo, hi);
        }
      }
      ao[mt] = (av[mt] && kin) ? v : zero4;
    }
  #pragma unroll
  for (int nt = 0; nt < NT; nt++) {
      const u32x4 v = *(const u32x4*)(wp[nt] + kc);
      wo[nt] = (wv[nt] && kin) ? v : zero4;
    }
  };
  request(0, afn, wfn);
  for (int k0 = 0; k0 < g.K; k0 += 32) {
#pragma unroll
    for (int mt = 0; mt < MT; mt++) af[mt] = afn[mt];
#pragma unroll
    for (int nt = 0; nt < NT; nt++) wf[nt] = wfn[nt];
    request(k0 + 32, afn, wfn);  // (beyond K: loads from offset 0, counted as zeros)
#pragma unroll
    for (int mt = 0; mt < MT; mt++)
#pragma unroll
      for (int nt = 0; nt < NT; nt++) BF16::mfma(acc[mt][nt], __builtin_bit_cast(s16x8, wf[nt]), __builtin_bit_cast(s16x8, af[mt]));
  }
  VRA_MFMA_DRAIN();
  // lane: activation row rq of tile mt, output columns oct * 4 + j of tile nt
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    const int r = m_base + mt * 16 + rq;
    if (r >= g.M || !av[mt]) continue;
    const int orow = g.out_row ? g.out_row[r] : r;
    if (orow < 0) continue;
    if (g.epi == 1) {
#pragma unroll
      for (int nt = 0; nt + 1 < NT; nt += 2)
        for (int j = 0; j < 4; j++) {
          const int n = (n_base + nt * 16) / 2 + oct * 4 + j;
          if (n >= g.N / 2) continue;
          const float y = gated_pair(acc[mt][nt][j], acc[mt][nt + 1][j], g.limit, g.act_alpha, g.act);
          if (g.out_f32) ((float*)g.out)[ob + (int64_t)orow * g.ldo + n] = y;
          else ((uint16_t*)g.out)[ob + (int64_t)orow * g.ldo + n] = BF16::from_f32(y);
        }
    } else {
#pragma unroll
      for (int nt = 0; nt < NT; nt++)
        for (int j = 0; j < 4; j++) {
          const int n = n_base + nt * 16 + oct * 4 + j;
          if (n >= g.N) continue;
          const float v = acc[mt][nt][j] * g.alpha + (g.bias ? g.bias[(int64_t)blockIdx.z * g.bias_batch_stride + n] : 0.f);
          if (g.out_f32) ((float*)g.out)[ob + (int64_t)orow * g.ldo + n] = v;
          else ((uint16_t*)g.out)[ob + (int64_t)orow * g.ldo + n] = BF16::from_f32(v);
        }
    }
  }
}

// Steps of up to 32 rows (decoding): the weights are the whole traffic, so a workgroup takes only 32 output columns and its 8 waves
// take an eighth of K each (whole K-steps of 32, ascending inside a wave); the 8 partial tiles meet in LDS and are summed in wave order.
// One fixed order for a given K — another one than the large-M kernel's single chain, so the two agree to rounding, not to the bit.
template <bool SCALED>
__global__ __launch_bounds__(512) void stk_gemm_mfma_small_kernel(StkGemmArgs g) {
  __shared__ float part[8][16 * 32];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, rq = lane & 15, oct = lane >> 4;
  int group = 0;
  if (g.tile_group) {
    group = g.tile_group[blockIdx.x];
    if (group < 0) return;
  }
  const uint16_t* A = (const uint16_t*)g.a + (int64_t)blockIdx.z * g.a_batch_stride;
  const uint16_t* Wt = (const uint16_t*)g.w + (int64_t)group * g.w_group_stride + (int64_t)blockIdx.z * g.w_batch_stride;
  const int64_t ob = (int64_t)blockIdx.z * g.out_batch_stride;
  const int m_base = blockIdx.x * 16, n_base = blockIdx.y * 32;
  const int r = m_base + rq;
  const int idx = r < g.M ? (g.a_row ? g.a_row[r] : r) : -1;
  const uint16_t* ap = A + (int64_t)(idx >= 0 ? idx : 0) * g.lda;
  const float asc = SCALED && idx >= 0 ? g.a_scale[r] : 1.f;
  const uint16_t* wp[2];
  bool wv[2];
  for (int nt = 0; nt < 2; nt++) {
    const int n = n_base + nt * 16 + rq;
    wv[nt] = n < g.N;
    wp[nt] = Wt + (int64_t)(n < g.N ? n : 0) * g.K;
  }
  const int ksteps = (g.K + 31) / 32, per = (ksteps + 7) / 8;
  const int k_lo = wave * per * 32, k_hi = min(g.K, (wave + 1) * per * 32);
  f32x4 acc[2] = {vra_zero_acc(), vra_zero_acc()};
  const u32x4 zero4 = {0u, 0u, 0u, 0u};
  // four K-steps per round: their twelve 16-byte requests are in flight together, then the eight MFMAs (steps beyond the wave's range
  // load from offset 0 and count as zeros: same order of the sum, no branch between the MFMAs)
  for (int k0 = k_lo; k0 < k_hi; k0 += 4 * 32) {
    u32x4 af[4], wf[4][2];
    for (int u = 0; u < 4; u++) {
      const int k = k0 + u * 32 + oct * 8;
      const bool kin = k < k_hi;
      const int kc = kin ? k : 0;
      u32x4 a4 = *(const u32x4*)(ap + kc);
      if (SCALED) {
        for (int i = 0; i < 4; i++) a4[i] = BF16::pack2(__uint_as_float(a4[i] << 16) * asc, __uint_as_float(a4[i] & 0xffff0000u) * asc);
      }
      af[u] = (idx >= 0 && kin) ? a4 : zero4;
      for (int nt = 0; nt < 2; nt++) {
        const u32x4 v = *(const u32x4*)(wp[nt] + kc);
        wf[u][nt] = (wv[nt] && kin) ? v : zero4;
      }
    }
    for (int u = 0; u < 4; u++)
      for (int nt = 0; nt < 2; nt++) BF16::mfma(acc[nt], __builtin_bit_cast(s16x8, wf[u][nt]), __builtin_bit_cast(s16x8, af[u]));
  }
  VRA_MFMA_DRAIN();
  for (int nt = 0; nt < 2; nt++)
    for (int j = 0; j < 4; j++) part[wave][rq * 32 + nt * 16 + oct * 4 + j] = acc[nt][j];
  __syncthreads();
  const int e = threadIdx.x, m = e >> 5, c = e & 31;  // one output element per thread
  const int row = m_base + m;
  if (row >= g.M) return;
  const int ridx = g.a_row ? g.a_row[row] : row;
  if (ridx < 0) return;
  const int orow = g.out_row ? g.out_row[row] : row;
  if (orow < 0) return;
  auto total = [&](int col) {
    float s = part[0][m * 32 + col];
    for (int w = 1; w < 8; w++) s += part[w][m * 32 + col];
    return s;
  };
  if (g.epi == 1) {
    if (c >= 16) return;
    const int n = n_base / 2 + c;
    if (n >= g.N / 2) return;
    const float y = gated_pair(total(c), total(16 + c), g.limit, g.act_alpha, g.act);
    if (g.out_f32) ((float*)g.out)[ob + (int64_t)orow * g.ldo + n] = y;
    else ((uint16_t*)g.out)[ob + (int64_t)orow * g.ldo + n] = BF16::from_f32(y);
  } else {
    const int n = n_base + c;
    if (n >= g.N) return;
    const float v = total(c) * g.alpha + (g.bias ? g.bias[(int64_t)blockIdx.z * g.bias_batch_stride + n] : 0.f);
    if (g.out_f32) ((float*)g.out)[ob + (int64_t)orow * g.ldo + n] = v;
    else ((uint16_t*)g.out)[ob + (int64_t)orow * g.ldo + n] = BF16::from_f32(v);
  }
}

// ------------------------------------------------------------------------------------------------ activations
template <typename T>
__global__ __launch_bounds__(256) void stk_gated_act_kernel(const float* gu, T* out, int F, float limit, float act_alpha, int act) {
  const int m = blockIdx.x;
  const int Fp = (F + 15) / 16 * 16;
  for (int f = threadIdx.x; f < F; f += 256) {
    const int b = f >> 4, i = f & 15;
    const float gv = gu[(size_t)m * 2 * Fp + (2 * b) * 16 + i], uv = gu[(size_t)m * 2 * Fp + (2 * b + 1) * 16 + i];
    El<T>::st(out + (size_t)m * Fp + f, gated_pair(gv, uv, limit, act_alpha, act));
  }
  for (int f = F + threadIdx.x; f < Fp; f += 256) El<T>::st(out + (size_t)m * Fp + f, 0.f);
}

#define STK_PN_THREADS 1024
__device__ __forceinline__ float block_sum_pn(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
  for (int w = 0; w < STK_PN_THREADS / 64; w++) s += red[w];
  return s;
}
// one workgroup of 1024 threads per token: up to 8 values per thread stay in registers between the sums and the output
template <typename T>
__global__ __launch_bounds__(STK_PN_THREADS) void stk_polynorm_kernel(const float* z, T* out, const float* coef, int F, float eps) {
  __shared__ float red[STK_PN_THREADS / 64];
  const int m = blockIdx.x;
  const float* zr = z + (size_t)m * F;
  float keep[8];
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
  for (int n = 0; n < 8; n++) {  // the first 8192 values: one per thread and round, kept in registers
    const int f = threadIdx.x + n * STK_PN_THREADS;
    const float v = f < F ? zr[f] : 0.f, v2 = v * v, v3 = v2 * v;
    keep[n] = v;
    s1 = fmaf(v, v, s1), s2 = fmaf(v2, v2, s2), s3 = fmaf(v3, v3, s3);
  }
  for (int f = threadIdx.x + 8 * STK_PN_THREADS; f < F; f += STK_PN_THREADS) {
    const float v = zr[f], v2 = v * v, v3 = v2 * v;
    s1 = fmaf(v, v, s1), s2 = fmaf(v2, v2, s2), s3 = fmaf(v3, v3, s3);
  }
  s1 = block_sum_pn(s1, red);
  s2 = block_sum_pn(s2, red);
  s3 = block_sum_pn(s3, red);
  const float r1 = 1.f / sqrtf(s1 / (float)F + eps), r2 = 1.f / sqrtf(s2 / (float)F + eps), r3 = 1.f / sqrtf(s3 / (float)F + eps);
  const float ca = coef[0], cb = coef[1], cc = coef[2], ce = coef[3];
#pragma unroll
  for (int n = 0; n < 8; n++) {
    const int f = threadIdx.x + n * STK_PN_THREADS;
    const float v = keep[n], v2 = v * v, v3 = v2 * v;
    if (f < F) El<T>::st(out + (size_t)m * F + f, ca * (v * r1) + cb * (v2 * r2) + cc * (v3 * r3) + ce);
  }
  for (int f = threadIdx.x + 8 * STK_PN_THREADS; f < F; f += STK_PN_THREADS) {
    const float v = zr[f], v2 = v * v, v3 = v2 * v;
    El<T>::st(out + (size_t)m * F + f, ca * (v * r1) + cb * (v2 * r2) + cc * (v3 * r3) + ce);
  }
}

__global__ __launch_bounds__(256) void stk_residual_combine_kernel(float* x, const float* o, const float* p1, int n1, const float* p2, const float* gate,
                                                                   float mult, int W) {
  const int t = blockIdx.x;
  const float gt = gate ? gate[t] : 1.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    float s = o ? o[(size_t)t * W + c] : 0.f;
    for (int j = 0; j < n1; j++) s += p1[((size_t)t * n1 + j) * W + c];
    if (p2) s += gt * p2[(size_t)t * W + c];
    x[(size_t)t * W + c] += mult * s;
  }
}

__global__ __launch_bounds__(256) void stk_gather_rows_kernel(const float* src, const uint32_t* rows, float* dst, int W) {
  const int r = blockIdx.x;
  const float* s = src + (size_t)rows[r] * W;
  for (int c = threadIdx.x; c < W; c += 256) dst[(size_t)r * W + c] = s[c];
}

// ------------------------------------------------------------------------------------------------ paged KV cache
template <typename T>
__global__ __launch_bounds__(256) void stk_kv_store_kernel(const T* k, const T* v, int ld, T* kc, T* vc, const int64_t* slots, int kdim, int vdim) {
  const int t = blockIdx.x;
  const int64_t s = slots[t];
  if (s < 0) return;
  for (int c = threadIdx.x; c < kdim; c += 256) kc[s * kdim + c] = k[(size_t)t * ld + c];
  for (int c = threadIdx.x; c < vdim; c += 256) vc[s * vdim + c] = v[(size_t)t * ld + c];
}

__device__ __forceinline__ float q_temperature(int64_t p, float coef, int every) {
  if (every <= 0 || coef == 0.f) return 1.f;
  return 1.f + coef * logf((float)((p + 1) / every) + 1.f);
}
__device__ __forceinline__ float cap_score(float s, float softcap) { return softcap > 0.f ? softcap * tanhf(s / softcap) : s; }
// the same through the hardware exponential (f32 arithmetic, ~2^-21 relative in the exponential; |error| of the capped score below
// 2^-22 * softcap): the bf16 kernel's choice, where 16 library calls per lane and key tile would cost more than its matrix products
__device__ __forceinline__ float cap_score_fast(float s, float softcap) {
  if (!(softcap > 0.f)) return s;
  const float x = fminf(fmaxf(s / softcap, -15.f), 15.f);
  return softcap * (1.f - 2.f / (1.f + __expf(2.f * x)));
}

// Portions of prompts (and whatever else shares their step): 16 query rows of one head per workgroup, 4 per wave; key tiles of KT
// tokens staged once in LDS (f32) for all 16 rows; lane = key for the scores, lane = value channel for the weighted sum.
// Tiles start at key 0 of the sequence and a row's running maximum / sum go tile by tile: the order does not depend on the portion.
#define STK_QT 16
template <typename T, int KT>
__global__ __launch_bounds__(256) void stk_attn_prefill_kernel(StkAttnArgs a) {
  extern __shared__ float lds[];
  const int dim = a.dim, vdim = a.vdim, kld = dim + 1;
  float* qs = lds;                      // [16][dim]  q * temp
  float* ks = qs + STK_QT * dim;        // [KT][dim + 1]
  float* vs = ks + KT * kld;            // [KT][vdim]
  float* ps = vs + KT * vdim;           // [16][KT]
  const int b = blockIdx.y, h = blockIdx.z, g = h / (a.H / a.G);
  const int q0 = a.cu_q[b], q1 = a.cu_q[b + 1];
  const int t0 = q0 + blockIdx.x * STK_QT;
  if (t0 >= q1) return;
  const int nq = min(STK_QT, q1 - t0);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* q = (const T*)a.q;
  for (int i = tid; i < STK_QT * dim; i += 256) {
    const int r = i / dim, d = i % dim;
    float v = 0.f;
    if (r < nq) v = El<T>::ld(q + (size_t)(t0 + r) * a.ldq + h * dim + d) * q_temperature(a.positions[t0 + r], a.temp_coef, a.temp_every);
    qs[i] = v;
  }
  int64_t pq[4], plo[4];
  int64_t pmax = -1, lo_min = INT64_MAX;
  auto block_start = [&](int64_t p) {  // first key a query at p may see
    const int64_t lo = a.chunk > 0 ? p / a.chunk * a.chunk : (int64_t)0;
    return a.window > 0 ? max(lo, p - a.window + 1) : lo;
  };
  for (int i = 0; i < 4; i++) {
    const int r = wave * 4 + i;
    pq[i] = r < nq ? a.positions[t0 + r] : -1;
    plo[i] = pq[i] >= 0 ? block_start(pq[i]) : 0;
  }
  for (int r = 0; r < nq; r++) pmax = max(pmax, a.positions[t0 + r]), lo_min = min(lo_min, block_start(a.positions[t0 + r]));
  const int n_keys = (int)min((int64_t)a.context_lens[b], pmax + 1);
  const int kt_begin = (int)(lo_min / KT) * KT;  // (tiles stay aligned to absolute positions)
  float m[4], l[4], acc[4][4];
  for (int i = 0; i < 4; i++) {
    m[i] = -INFINITY, l[i] = 0.f;
    if (a.sink) m[i] = a.sink[h], l[i] = 1.f;  // the sink: one more term exp(sink - m) of the denominator, present from the start
    for (int r = 0; r < 4; r++) acc[i][r] = 0.f;
  }
  const T* kc = (const T*)a.kc;
  const T* vc = (const T*)a.vc;
  const uint32_t* bt = a.block_tables + (size_t)b * a.max_blocks;
  const int kdim = a.k_ld ? a.k_ld : a.G * dim, vd_all = a.v_ld ? a.v_ld : a.G * vdim;
  const float hscale = a.head_scale ? a.scale * a.head_scale[h] : a.scale;
  for (int kt0 = kt_begin; kt0 < n_keys; kt0 += KT) {
    __syncthreads();
    for (int i = tid; i < KT * dim; i += 256) {
      const int j = i / dim, d = i % dim, key = kt0 + j;
      float v = 0.f;
      if (key < n_keys) {
        const int64_t slot = (int64_t)bt[key / a.BS] * a.BS + key % a.BS;
        v = El<T>::ld(kc + slot * kdim + g * dim + d);
      }
      ks[j * kld + d] = v;
    }
    for (int i = tid; i < KT * vdim; i += 256) {
      const int j = i / vdim, d = i % vdim, key = kt0 + j;
      float v = 0.f;
      if (key < n_keys) {
        const int64_t slot = (int64_t)bt[key / a.BS] * a.BS + key % a.BS;
        v = El<T>::ld(vc + slot * vd_all + g * vdim + d);
      }
      vs[i] = v;
    }
    __syncthreads();
    for (int i = 0; i < 4; i++) {
      const int r = wave * 4 + i;
      float s = -INFINITY;
      if (lane < KT && pq[i] >= 0 && kt0 + lane <= pq[i] && kt0 + lane >= plo[i] && kt0 + lane < n_keys) {
        float d0 = 0.f;
        for (int d = 0; d < dim; d++) d0 = fmaf(qs[r * dim + d], ks[lane * kld + d], d0);
        s = cap_score(d0 * hscale, a.softcap);
      }
      const float mn = fmaxf(m[i], wave_max(s));
      float p = 0.f, corr = 1.f;
      if (mn > -INFINITY) {
        p = s > -INFINITY ? expf(s - mn) : 0.f;
        corr = m[i] > -INFINITY ? expf(m[i] - mn) : 0.f;
      }
      l[i] = l[i] * corr + wave_sum(p);
      m[i] = mn;
      for (int rr = 0; rr < 4; rr++) acc[i][rr] *= corr;
      if (lane < KT) ps[r * KT + lane] = p;
    }
    __syncthreads();
    for (int rr = 0; rr < 4; rr++) {
      const int d = lane + 64 * rr;
      if (d >= vdim) break;
#pragma unroll 4
      for (int j = 0; j < KT; j++) {
        const float v = vs[j * vdim + d];
        for (int i = 0; i < 4; i++) acc[i][rr] = fmaf(ps[(wave * 4 + i) * KT + j], v, acc[i][rr]);
      }
    }
  }
  T* out = (T*)a.out;
  for (int i = 0; i < 4; i++) {
    const int r = wave * 4 + i;
    if (r >= nq) continue;
    float inv = l[i] > 0.f ? 1.f / l[i] : 0.f;
    if (a.gate) inv *= sigmoidf_(a.gate[(size_t)(t0 + r) * a.gate_ld + h]);
    for (int rr = 0; rr < 4; rr++) {
      const int d = lane + 64 * rr;
      if (d < vdim) El<T>::st(out + (size_t)(t0 + r) * a.H * vdim + h * vdim + d, acc[i][rr] * inv);
    }
  }
}

// bf16 models, key size a multiple of 8 and value size a multiple of 16: the same operator on the matrix cores.
// A workgroup of 4 waves owns 64 query rows of one head (16 per wave) and walks the keys in tiles of 32 from key 0.
//   S^T = K . Q^T   A operand = K rows straight from the cache (lane = (key rq, channel octet oct)), B = Q fragments kept in registers;
//                   the lane ends up with query row rq and keys oct * 4 + j of both 16-key halves: 8 scores, all in f32 — temperature,
//                   scale, soft cap, mask, running maximum (two xor shuffles join the 4 lanes of a row) and exponentials;
//   O^T += V^T . P^T  A operand = the V tile, transposed once per workgroup into LDS with the keys in the order the lanes hold their
//                   scores (position = oct * 8 + half * 4 + j), B = the lane's own 8 weights.  The weights stay f32 in effect: each is
//                   split into a bf16 head and a bf16 tail (p = hi + lo to 2^-17) and the product runs twice.
// Every sum goes tile by tile from key 0 with a fixed lane pattern: the result of a row does not depend on the portion it came in.
template <int DC, int VT>
__global__ __launch_bounds__(256) void stk_attn_prefill_mfma_kernel(StkAttnArgs a) {
  constexpr int KT = 32, VLD = KT + 8;  // LDS row of a value channel: 32 positions + 8 (rows stay 16-byte aligned, lanes spread over banks)
  __shared__ __attribute__((aligned(16))) uint16_t vt[VT * 16 * VLD];
  const int dim = a.dim, vdim = a.vdim;
  const int b = blockIdx.y, h = blockIdx.z, g = h / (a.H / a.G);
  const int q0 = a.cu_q[b], q1 = a.cu_q[b + 1];
  // the last row blocks of a portion see the most keys: they are dispatched first, so that no long block is left to run alone at the end
  const int t0 = q0 + ((int)gridDim.x - 1 - (int)blockIdx.x) * 64;
  if (t0 >= q1) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, rq = lane & 15, oct = lane >> 4;
  const int tq = t0 + wave * 16 + rq;  // this lane's query row
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
  const float sc = a.scale * q_temperature(pq < 0 ? 0 : pq, a.temp_coef, a.temp_every) * (a.head_scale ? a.head_scale[h] : 1.f);
  // keys this workgroup needs: up to the largest position of its rows
  int64_t pmax = pq;
  for (int o = 32; o > 0; o >>= 1) pmax = max(pmax, (int64_t)__shfl_xor((long long)pmax, o, 64));
  // block mask: this row sees the keys from key_lo on; the workgroup's tiles start at the tile of its smallest key_lo
  int64_t key_lo = a.chunk > 0 && pq >= 0 ? pq / a.chunk * a.chunk : 0;
  if (a.window > 0 && pq >= 0) key_lo = max(key_lo, pq - a.window + 1);
  int64_t lmin = pq >= 0 ? key_lo : INT64_MAX;
  for (int o = 32; o > 0; o >>= 1) lmin = min(lmin, (int64_t)__shfl_xor((long long)lmin, o, 64));
  __shared__ long long wmax[4], wmin[4];
  if (lane == 0) wmax[wave] = pmax, wmin[wave] = lmin;
  __syncthreads();
  const int64_t gmax = max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3]));
  const int64_t gmin = min(min(wmin[0], wmin[1]), min(wmin[2], wmin[3]));
  const int kt_begin = gmin == INT64_MAX ? 0 : (int)(gmin / 32) * 32;
  const int n_keys = (int)min((int64_t)a.context_lens[b], gmax + 1);
  const int n_keys_wave = (int)min((int64_t)n_keys, pmax + 1);
  const uint16_t* kc = (const uint16_t*)a.kc;
  const uint16_t* vc = (const uint16_t*)a.vc;
  const uint32_t* bt = a.block_tables + (size_t)b * a.max_blocks;
  const int kdim = a.k_ld ? a.k_ld : a.G * dim, vd_all = a.v_ld ? a.v_ld : a.G * vdim;
  f32x4 acc[VT];
  for (int t = 0; t < VT; t++) acc[t] = vra_zero_acc();
  float m = -INFINITY, l = 0.f;
  if (a.sink) m = a.sink[h], l = oct == 0 ? 1.f : 0.f;  // (the four lanes of a row add their sums at the end: the sink counts once)
  const bool capped = a.softcap > 0.f;
  const float two_inv_cap = capped ? 2.f / a.softcap : 0.f, two_cap = 2.f * a.softcap;
  const int key_end = (int)min((int64_t)n_keys, pq + 1);  // this row sees the keys below key_end
  // The K fragments and this thread's share of the V tile are requested one tile ahead, so that their way from memory runs beside the
  // current tile's arithmetic.  V item = (key, 8 channels): NV per thread.
  // V item = (pair of neighbouring keys, 8 channels): NV per thread, two 16-byte requests each
  constexpr int NV = (KT / 2 * VT * 2 + 255) / 256;
  u32x4 kfn[2][DC], vgn[NV][2];
  // The page size is a multiple of 32 (the launcher sends other sizes to the FMA kernel), so a 32-key tile lies in ONE page: its first
  // slot is a scalar, read from the block table one tile ahead of the requests that use it — no request of a tile waits behind a
  // block-table read (vector loads return in order: a per-key read would also wait for everything issued before it).
  auto page_slot = [&](int kt0) -> int64_t {  // first cache slot of the tile that starts at key kt0 (uniform)
    const int t = __builtin_amdgcn_readfirstlane(kt0);
    return t < n_keys ? (int64_t)bt[t / a.BS] * a.BS + t % a.BS : 0;
  };
  auto request_tile = [&](int kt0, int64_t slot0) {
    auto slot_of = [&](int key) { return slot0 + (key - kt0); };
    for (int u = 0; u < 2; u++) {
      const int key = kt0 + u * 16 + rq;
      const bool kv = key < n_keys;
      const int64_t slot = kv ? slot_of(key) : 0;
      const uint16_t* kr = kc + slot * kdim + g * dim;
      for (int c = 0; c < DC; c++) {
        const int ch = c * 32 + oct * 8;
        const bool ok = kv && ch < dim;
        const u32x4 kf = *(const u32x4*)(kr + (ok ? ch : 0));
        kfn[u][c] = ok ? kf : zero4;
      }
    }
    for (int n = 0; n < NV; n++) {
      const int i = tid + n * 256;
      const int kp = i / (VT * 2), c8 = (i % (VT * 2)) * 8;
      for (int e = 0; e < 2; e++) {
        const int key = kt0 + kp * 2 + e;
        const bool ok = i < KT / 2 * VT * 2 && key < n_keys && c8 < vdim;
        const int64_t slot = ok ? slot_of(key) : 0;
        const u32x4 v = *(const u32x4*)(vc + slot * vd_all + g * vdim + (ok ? c8 : 0));
        vgn[n][e] = ok ? v : zero4;
      }
    }
  };
  request_tile(kt_begin, page_slot(kt_begin));
  int64_t slot_next = page_slot(kt_begin + KT);
  for (int kt0 = kt_begin; kt0 < n_keys; kt0 += KT) {
    u32x4 kfc[2][DC], vgc[NV][2];
    for (int u = 0; u < 2; u++)
      for (int c = 0; c < DC; c++) kfc[u][c] = kfn[u][c];
    for (int n = 0; n < NV; n++) vgc[n][0] = vgn[n][0], vgc[n][1] = vgn[n][1];
    __syncthreads();
    // V tile -> LDS, transposed, the keys in the order the lanes hold their scores: keys 2 kp and 2 kp + 1 are neighbours there too,
    // so one 32-bit store carries both for a channel
    for (int n = 0; n < NV; n++) {
      const int i = tid + n * 256;
      if (i >= KT / 2 * VT * 2) break;
      const int kl = (i / (VT * 2)) * 2, c8 = (i % (VT * 2)) * 8;
      const int pos = ((kl & 15) >> 2) * 8 + (kl >> 4) * 4 + (kl & 3);  // even
      uint32_t* row = (uint32_t*)vt;
      for (int e = 0; e < 4; e++) {
        const uint32_t lo0 = vgc[n][0][e] & 0xffffu, hi0 = vgc[n][0][e] >> 16, lo1 = vgc[n][1][e] & 0xffffu, hi1 = vgc[n][1][e] >> 16;
        row[((c8 + 2 * e) * VLD + pos) >> 1] = lo0 | (lo1 << 16);
        row[((c8 + 2 * e + 1) * VLD + pos) >> 1] = hi0 | (hi1 << 16);
      }
    }
    __syncthreads();
    if (kt0 + KT < n_keys) {
      request_tile(kt0 + KT, slot_next);
      slot_next = page_slot(kt0 + 2 * KT);
    }
    if (kt0 >= n_keys_wave) continue;  // (wave-uniform: nothing of this tile is visible to the wave's rows)
    // scores of the two 16-key halves
    f32x4 s[2];
    s[0] = vra_zero_acc();
    s[1] = vra_zero_acc();
    for (int c = 0; c < DC; c++) {  // (the two halves' chains alternate: an MFMA never waits for the one issued just before it)
      BF16::mfma(s[0], __builtin_bit_cast(s16x8, kfc[0][c]), __builtin_bit_cast(s16x8, qf[c]));
      BF16::mfma(s[1], __builtin_bit_cast(s16x8, kfc[1][c]), __builtin_bit_cast(s16x8, qf[c]));
    }
    VRA_MFMA_DRAIN();
    float sv[8];
    float tmax = -INFINITY;
    for (int u = 0; u < 2; u++)
      for (int j = 0; j < 4; j++) {
        const int key = kt0 + u * 16 + oct * 4 + j;
        float x = s[u][j] * sc;
        if (capped) {  // softcap * tanh(x / softcap) = softcap - 2 softcap / (1 + e^(2 x / softcap)), hardware exponential and reciprocal
          const float y = fminf(fmaxf(x * two_inv_cap, -30.f), 30.f);
          x = a.softcap - two_cap * __builtin_amdgcn_rcpf(1.f + __expf(y));
        }
        x = key < key_end && key >= key_lo ? x : -INFINITY;
        sv[u * 4 + j] = x;
        tmax = fmaxf(tmax, x);
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float mn = fmaxf(m, tmax);
    float corr = 1.f, psum = 0.f, pv[8];
    for (int i = 0; i < 8; i++) pv[i] = 0.f;
    if (mn > -INFINITY) {
      corr = m > -INFINITY ? __expf(m - mn) : 0.f;
      for (int i = 0; i < 8; i++) {
        pv[i] = sv[i] > -INFINITY ? __expf(sv[i] - mn) : 0.f;
        psum += pv[i];
      }
    }
    l = l * corr + psum;
    m = mn;
    u32x4 phi, plo;
    for (int e = 0; e < 4; e++) {
      const float a0 = pv[2 * e], a1 = pv[2 * e + 1];
      const uint32_t hi = BF16::pack2(a0, a1);
      phi[e] = hi;
      plo[e] = BF16::pack2(a0 - __uint_as_float(hi << 16), a1 - __uint_as_float(hi & 0xffff0000u));
    }
    for (int t = 0; t < VT; t++) {
      acc[t][0] *= corr, acc[t][1] *= corr, acc[t][2] *= corr, acc[t][3] *= corr;
    }
    u32x4 vf[VT];
#pragma unroll
    for (int t = 0; t < VT; t++) vf[t] = *(const u32x4*)(vt + (t * 16 + rq) * VLD + oct * 8);
    // heads of all channel tiles first, then the tails: the two MFMAs into one accumulator are VT instructions apart
    // (fully unrolled: every accumulator keeps its registers, no indexed register moves next to an MFMA)
#pragma unroll
    for (int t = 0; t < VT; t++) BF16::mfma(acc[t], __builtin_bit_cast(s16x8, vf[t]), __builtin_bit_cast(s16x8, phi));
#pragma unroll
    for (int t = 0; t < VT; t++) BF16::mfma(acc[t], __builtin_bit_cast(s16x8, vf[t]), __builtin_bit_cast(s16x8, plo));
    VRA_MFMA_DRAIN();
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!qv) return;
  float inv = l > 0.f ? 1.f / l : 0.f;
  if (a.gate) inv *= sigmoidf_(a.gate[(size_t)tq * a.gate_ld + h]);
  uint16_t* out = (uint16_t*)a.out + (size_t)tq * a.H * vdim + h * vdim;
  for (int t = 0; t < VT; t++)
    for (int j = 0; j < 4; j++) {
      const int c = t * 16 + oct * 4 + j;
      if (c < vdim) out[c] = BF16::from_f32(acc[t][j] * inv);
    }
}

// One decoded token per sequence: a workgroup per (sequence, query head); its 8 waves take the 64-key tiles of the context in turn,
// read K rows straight from the cache (lane = key, 16 bytes a load where the row allows) and V rows channel-wise (lane = channel), and
// meet once in LDS.  The order of the sums depends on the context length alone.
#define STK_DW 8
template <typename T>
__device__ __forceinline__ float stk_dot_row(const float* qs, const T* kr, int dim) {
  float d0 = 0.f;
  for (int d = 0; d < dim; d++) d0 = fmaf(qs[d], El<T>::ld(kr + d), d0);
  return d0;
}
template <>
__device__ __forceinline__ float stk_dot_row<uint16_t>(const float* qs, const uint16_t* kr, int dim) {
  float d0 = 0.f;
  if (dim % 8 == 0 && ((uintptr_t)kr % 16) == 0) {
    for (int d = 0; d < dim; d += 8) {
      const u32x4 v = *(const u32x4*)(kr + d);
      for (int e = 0; e < 4; e++) {
        d0 = fmaf(qs[d + 2 * e], __uint_as_float(v[e] << 16), d0);
        d0 = fmaf(qs[d + 2 * e + 1], __uint_as_float(v[e] & 0xffff0000u), d0);
      }
    }
    return d0;
  }
  for (int d = 0; d < dim; d++) d0 = fmaf(qs[d], BF16::to_f32(kr[d]), d0);
  return d0;
}
template <typename T>
__global__ __launch_bounds__(64 * STK_DW) void stk_attn_decode_kernel(StkAttnArgs a) {
  extern __shared__ float lds[];
  const int dim = a.dim, vdim = a.vdim;
  float* qs = lds;                     // [dim]
  float* ps = qs + dim;                // [waves][64]
  float* ms = ps + STK_DW * 64;        // [waves] max, [waves] sum
  float* os = ms + 2 * STK_DW;         // [waves][vdim]
  int* ss = (int*)(os + STK_DW * vdim);  // [waves][64] cache slot of each key of the wave's current tile
  const int b = blockIdx.x, h = blockIdx.y, g = h / (a.H / a.G);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t p = a.positions[b];
  const int n_keys = (int)min((int64_t)a.context_lens[b], p + 1);
  const T* q = (const T*)a.q + (size_t)b * a.ldq + h * dim;
  const float temp = q_temperature(p, a.temp_coef, a.temp_every);
  for (int d = tid; d < dim; d += 64 * STK_DW) qs[d] = El<T>::ld(q + d) * temp;
  __syncthreads();
  const T* kc = (const T*)a.kc;
  const T* vc = (const T*)a.vc;
  const uint32_t* bt = a.block_tables + (size_t)b * a.max_blocks;
  const int kdim = a.k_ld ? a.k_ld : a.G * dim, vd_all = a.v_ld ? a.v_ld : a.G * vdim;
  float m = -INFINITY, l = 0.f, acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (a.sink && wave == 0) m = a.sink[h], l = 1.f;
  // 16-bit values in whole octets: the value phase reads 16 bytes a lane (oc = channel octets rounded up to a power of two)
  const bool vec = sizeof(T) == 2 && vdim % 8 == 0 && vd_all % 8 == 0 && ((uintptr_t)vc % 16) == 0;
  int oc = 1;
  while (oc * 8 < vdim) oc <<= 1;
  const int co = lane & (oc - 1), kg = lane / oc, kpar = 64 / oc;
  float vacc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // block mask: the keys from key_lo on; tiles stay aligned to absolute positions (the first one may begin below key_lo: those keys
  // count with weight 0)
  int key_lo = a.chunk > 0 ? (int)(p / a.chunk * a.chunk) : 0;
  if (a.window > 0) key_lo = max(key_lo, (int)(p - a.window + 1));
  const float hscale = a.head_scale ? a.scale * a.head_scale[h] : a.scale;
  for (int kt0 = key_lo / 64 * 64 + wave * 64; kt0 < n_keys; kt0 += STK_DW * 64) {
    const int key = kt0 + lane;
    float s = -INFINITY;
    if (key < n_keys) {
      const int64_t slot = (int64_t)bt[key / a.BS] * a.BS + key % a.BS;
      ss[wave * 64 + lane] = (int)slot;
      if (key >= key_lo) s = cap_score(stk_dot_row<T>(qs, kc + slot * kdim + g * dim, dim) * hscale, a.softcap);
    }
    const float mn = fmaxf(m, wave_max(s));  // (the tile's first key exists: mn is finite)
    const float pj = s > -INFINITY ? expf(s - mn) : 0.f;
    const float corr = m > -INFINITY ? expf(m - mn) : 0.f;
    l = l * corr + wave_sum(pj);
    m = mn;
    ps[wave * 64 + lane] = pj;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const int nj = min(64, n_keys - kt0);
    if (vec) {
      // lane = (key group kg, channel octet co): one 16-byte load covers 8 channels of one key, 64 / OC keys are in flight per step;
      // the groups' partial sums meet after the last tile
      for (int i = 0; i < 8; i++) vacc[i] *= corr;
      // four keys of a group per step, their rows requested together (the slots come from LDS, where the score phase left them, so no
      // request waits for a block-table read); keys beyond the tile count with weight 0
      for (int j = kg; j < nj && co * 8 < vdim; j += 4 * kpar) {
        u32x4 v[4];
        float pw[4];
        for (int u = 0; u < 4; u++) {
          const int ju = j + u * kpar;
          const bool in = ju < nj;
          const int64_t sl = ss[wave * 64 + (in ? ju : j)];
          v[u] = *(const u32x4*)((const uint16_t*)vc + sl * vd_all + g * vdim + co * 8);
          pw[u] = in ? ps[wave * 64 + ju] : 0.f;
        }
        for (int u = 0; u < 4; u++)
          for (int i = 0; i < 4; i++) {
            vacc[2 * i] = fmaf(pw[u], __uint_as_float(v[u][i] << 16), vacc[2 * i]);
            vacc[2 * i + 1] = fmaf(pw[u], __uint_as_float(v[u][i] & 0xffff0000u), vacc[2 * i + 1]);
          }
      }
    } else {
      for (int rr = 0; rr < 4; rr++) {
        const int d = lane + 64 * rr;
        if (d >= vdim) break;
        float o = acc[rr] * corr;
        for (int j = 0; j < nj; j++) o = fmaf(ps[wave * 64 + j], El<T>::ld(vc + (int64_t)ss[wave * 64 + j] * vd_all + g * vdim + d), o);
        acc[rr] = o;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  if (vec) {
    for (int o = oc; o < 64; o <<= 1)
      for (int i = 0; i < 8; i++) vacc[i] += __shfl_xor(vacc[i], o, 64);
    if (lane < oc && co * 8 < vdim)
      for (int i = 0; i < 8; i++) os[wave * vdim + co * 8 + i] = vacc[i];
  } else {
    for (int rr = 0; rr < 4; rr++) {
      const int d = lane + 64 * rr;
      if (d < vdim) os[wave * vdim + d] = acc[rr];
    }
  }
  if (lane == 0) ms[wave] = m, ms[STK_DW + wave] = l;
  __syncthreads();
  float M = ms[0];
  for (int w = 1; w < STK_DW; w++) M = fmaxf(M, ms[w]);
  T* out = (T*)a.out + (size_t)b * a.H * vdim + h * vdim;
  const float og = a.gate ? sigmoidf_(a.gate[(size_t)b * a.gate_ld + h]) : 1.f;
  for (int d = tid; d < vdim; d += 64 * STK_DW) {
    float L = 0.f, o = 0.f;
    for (int w = 0; w < STK_DW; w++) {
      const float c = ms[w] > -INFINITY ? expf(ms[w] - M) : 0.f;
      L += ms[STK_DW + w] * c;
      o += os[w * vdim + d] * c;
    }
    El<T>::st(out + d, L > 0.f ? o / L * og : 0.f);
  }
}

}  // namespace

// ================================================================================================ launchers
int vra_stack_gemm_granule(int rows, int groups) { return groups > 0 && rows / groups >= 128 ? 64 : 16; }

void vra_stack_gemm(const StkGemmArgs& g, int dtype, int64_t stream) {
  VRA_CHECK_ARG(g.a && g.w && g.out && g.M > 0 && g.N > 0 && g.K > 0, "stack gemm: null pointer or empty shape");
  VRA_CHECK_ARG(dtype == VRA_BF16 || dtype == VRA_F32, "stack gemm: dtype must be bf16 or f32");
  VRA_CHECK_ARG(!g.tile_group || g.granule == 16 || g.granule == 64, "stack gemm: granule must be 16 or 64");
  VRA_CHECK_ARG(g.batch >= 1 && (g.batch == 1 || !g.tile_group), "stack gemm: a batched product has no row groups");
  hipStream_t st = as_stream(stream);
  const int nb = g.batch;
  const bool big = g.tile_group ? g.granule == 64 : g.M > 32;
  const bool mfma = dtype == VRA_BF16 && g.K % 8 == 0 && g.lda % 8 == 0 && ((uintptr_t)g.a % 16 == 0) && ((uintptr_t)g.w % 16 == 0) &&
                    (g.w_group_stride % 8 == 0) && (g.a_batch_stride % 8 == 0) && (g.w_batch_stride % 8 == 0);
  VRA_CHECK_ARG(g.epi == 0 || (mfma && g.N % 32 == 0), "stack gemm: the gated epilogue needs the bf16 MFMA path and whole gate / up blocks");
  if (mfma) {
    if (big && !g.tile_group && !g.a_scale && g.M >= 256 && (int64_t)((g.M + 127) / 128) * ((g.N + 127) / 128) * nb >= 256) {
      // enough 128 x 128 tiles to fill the chip: a wave owns 64 x 64 (16 MFMAs per 8 fragment requests instead of 8 per 6)
      dim3 grid((g.M + 127) / 128, (g.N + 127) / 128, nb);
      launch_checked("stack gemm", [&] { stk_gemm_mfma_kernel<4, 4, 2, 2, false><<<grid, 256, 0, st>>>(g); });
    } else if (big) {
      dim3 grid((g.M + 63) / 64, (g.N + 127) / 128, nb);
      if (g.a_scale) launch_checked("stack gemm", [&] { stk_gemm_mfma_kernel<2, 4, 2, 2, true><<<grid, 256, 0, st>>>(g); });
      else launch_checked("stack gemm", [&] { stk_gemm_mfma_kernel<2, 4, 2, 2, false><<<grid, 256, 0, st>>>(g); });
    } else {
      dim3 grid((g.M + 15) / 16, (g.N + 31) / 32, nb);
      if (g.a_scale) launch_checked("stack gemm", [&] { stk_gemm_mfma_small_kernel<true><<<grid, 512, 0, st>>>(g); });
      else launch_checked("stack gemm", [&] { stk_gemm_mfma_small_kernel<false><<<grid, 512, 0, st>>>(g); });
    }
    return;
  }
  if (big) {
    dim3 grid((g.M + 63) / 64, (g.N + 63) / 64, nb);
    if (dtype == VRA_F32) launch_checked("stack gemm", [&] { stk_gemm_simple_kernel<float, 4><<<grid, 256, 0, st>>>(g); });
    else launch_checked("stack gemm", [&] { stk_gemm_simple_kernel<uint16_t, 4><<<grid, 256, 0, st>>>(g); });
  } else {
    dim3 grid((g.M + 15) / 16, (g.N + 63) / 64, nb);
    if (dtype == VRA_F32) launch_checked("stack gemm", [&] { stk_gemm_simple_kernel<float, 1><<<grid, 256, 0, st>>>(g); });
    else launch_checked("stack gemm", [&] { stk_gemm_simple_kernel<uint16_t, 1><<<grid, 256, 0, st>>>(g); });
  }
}

void vra_stack_embed_sinpos(const uint32_t* ids, const int64_t* positions, const void* embed, const float* inv_freq, float* x, int T, int W, int V,
                            int dtype, int64_t stream) {
  VRA_CHECK_ARG(ids && positions && embed && x && T > 0 && W > 0, "stack embed: null pointer or empty shape");
  if (dtype == VRA_F32)
    launch_checked("stack embed", [&] { stk_embed_sinpos_kernel<float><<<T, 256, 0, as_stream(stream)>>>(ids, positions, (const float*)embed, inv_freq, x, W, V); });
  else
    launch_checked("stack embed", [&] { stk_embed_sinpos_kernel<uint16_t><<<T, 256, 0, as_stream(stream)>>>(ids, positions, (const uint16_t*)embed, inv_freq, x, W, V); });
}

void vra_stack_group_norm(const StkNormArgs& a, int dtype, int64_t stream) {
  VRA_CHECK_ARG(a.x && a.w && a.h && a.T > 0 && a.W > 0, "stack norm: null pointer or empty shape");
  VRA_CHECK_ARG(a.groups >= 1 && a.W % a.groups == 0, "stack norm: the width must split into equal groups");
  VRA_CHECK_ARG(!a.router_w || (a.pair_expert && a.pair_weight && a.top >= 1 && a.top <= a.n_router && (!a.gate_row || a.gate_out)), "stack norm: router outputs");
  const size_t lds = ((size_t)a.W + a.groups + a.n_router + 2) * sizeof(float);
  VRA_CHECK_ARG(lds <= 64 * 1024, "stack norm: row does not fit LDS");
  if (dtype == VRA_F32) launch_checked("stack norm", [&] { stk_group_norm_kernel<float><<<a.T, 256, lds, as_stream(stream)>>>(a); });
  else launch_checked("stack norm", [&] { stk_group_norm_kernel<uint16_t><<<a.T, 256, lds, as_stream(stream)>>>(a); });
}

void vra_stack_moe_sort(const int* pair_expert, const float* pair_weight, int P, int top, int n_groups, int granule, int max_rows, int* row_token,
                        float* row_scale, int* row_pair, int* tile_group, int64_t stream) {
  VRA_CHECK_ARG(pair_expert && pair_weight && row_token && row_scale && row_pair && tile_group && P > 0 && top > 0, "stack moe sort: null pointer");
  VRA_CHECK_ARG((granule == 16 || granule == 64) && max_rows % granule == 0 && max_rows >= P + n_groups * (granule - 1), "stack moe sort: row space too small");
  const size_t lds = (size_t)n_groups * 3 * sizeof(int);
  VRA_CHECK_ARG(lds <= 48 * 1024, "stack moe sort: too many experts");
  launch_checked("stack moe sort", [&] {
    stk_moe_sort_kernel<<<1, 1024, lds, as_stream(stream)>>>(pair_expert, pair_weight, P, top, n_groups, granule, max_rows, row_token, row_scale, row_pair, tile_group);
  });
}

void vra_stack_gated_act(const float* gu, void* out, int M, int F, float limit, float act_alpha, int dtype, int64_t stream, int act) {
  VRA_CHECK_ARG(gu && out && M > 0 && F > 0, "stack gated act: null pointer or empty shape");
  if (dtype == VRA_F32) launch_checked("stack gated act", [&] { stk_gated_act_kernel<float><<<M, 256, 0, as_stream(stream)>>>(gu, (float*)out, F, limit, act_alpha, act); });
  else launch_checked("stack gated act", [&] { stk_gated_act_kernel<uint16_t><<<M, 256, 0, as_stream(stream)>>>(gu, (uint16_t*)out, F, limit, act_alpha, act); });
}

void vra_stack_polynorm(const float* z, void* out, const float* coef, int M, int F, float eps, int dtype, int64_t stream) {
  VRA_CHECK_ARG(z && out && coef && M > 0 && F > 0, "stack polynorm: null pointer or empty shape");
  if (dtype == VRA_F32) launch_checked("stack polynorm", [&] { stk_polynorm_kernel<float><<<M, STK_PN_THREADS, 0, as_stream(stream)>>>(z, (float*)out, coef, F, eps); });
  else launch_checked("stack polynorm", [&] { stk_polynorm_kernel<uint16_t><<<M, STK_PN_THREADS, 0, as_stream(stream)>>>(z, (uint16_t*)out, coef, F, eps); });
}

void vra_stack_residual_combine(float* x, const float* o, const float* p1, int n1, const float* p2, const float* gate, float mult, int T, int W,
                                int64_t stream) {
  VRA_CHECK_ARG(x && T > 0 && W > 0 && (n1 == 0 || p1), "stack combine: null pointer or empty shape");
  launch_checked("stack combine", [&] { stk_residual_combine_kernel<<<T, 256, 0, as_stream(stream)>>>(x, o, p1, n1, p2, gate, mult, W); });
}

void vra_stack_gather_rows_f32(const float* src, const uint32_t* rows, float* dst, int n, int W, int64_t stream) {
  VRA_CHECK_ARG(src && rows && dst && n > 0 && W > 0, "stack gather: null pointer or empty shape");
  launch_checked("stack gather", [&] { stk_gather_rows_kernel<<<n, 256, 0, as_stream(stream)>>>(src, rows, dst, W); });
}

void vra_stack_kv_store(const void* k, const void* v, int ld, void* kc, void* vc, const int64_t* slots, int T, int kdim, int vdim, int dtype,
                        int64_t stream) {
  VRA_CHECK_ARG(k && v && kc && vc && slots && T > 0, "stack kv store: null pointer or empty shape");
  if (dtype == VRA_F32)
    launch_checked("stack kv store", [&] { stk_kv_store_kernel<float><<<T, 256, 0, as_stream(stream)>>>((const float*)k, (const float*)v, ld, (float*)kc, (float*)vc, slots, kdim, vdim); });
  else
    launch_checked("stack kv store", [&] {
      stk_kv_store_kernel<uint16_t><<<T, 256, 0, as_stream(stream)>>>((const uint16_t*)k, (const uint16_t*)v, ld, (uint16_t*)kc, (uint16_t*)vc, slots, kdim, vdim);
    });
}

void vra_stack_attention(const StkAttnArgs& a, int dtype, int64_t stream) {
  VRA_CHECK_ARG(a.q && a.out && a.kc && a.vc && a.positions && a.block_tables && a.context_lens, "stack attention: null pointer");
  VRA_CHECK_ARG(a.B > 0 && a.H > 0 && a.G > 0 && a.H % a.G == 0 && a.dim > 0 && a.vdim > 0 && a.vdim <= 256 && a.BS > 0 && a.max_blocks > 0,
                "stack attention: heads must be a multiple of kv heads, value size at most 256");
  hipStream_t st = as_stream(stream);
  if (!a.cu_q) {
    const size_t lds = ((size_t)a.dim + 2 * STK_DW * 64 + 2 * STK_DW + STK_DW * (size_t)a.vdim) * sizeof(float);
    VRA_CHECK_ARG(lds <= 64 * 1024, "stack attention: head does not fit LDS");
    dim3 grid(a.B, a.H);
    if (dtype == VRA_F32) launch_checked("stack attention (decode)", [&] { stk_attn_decode_kernel<float><<<grid, 64 * STK_DW, lds, st>>>(a); });
    else launch_checked("stack attention (decode)", [&] { stk_attn_decode_kernel<uint16_t><<<grid, 64 * STK_DW, lds, st>>>(a); });
    return;
  }
  if (dtype == VRA_BF16 && a.dim % 8 == 0 && a.vdim % 16 == 0 && a.dim <= 256 && a.ldq % 8 == 0 && ((uintptr_t)a.q % 16 == 0) && a.BS % 32 == 0 &&
      a.k_ld % 8 == 0 && a.v_ld % 8 == 0 && ((uintptr_t)a.vc % 16 == 0)) {
    dim3 grid((a.max_q + 63) / 64, a.B, a.H);
#define STK_PFM(DCV, VTV) launch_checked("stack attention (prefill, mfma)", [&] { stk_attn_prefill_mfma_kernel<DCV, VTV><<<grid, 256, 0, st>>>(a); })
    if (a.dim <= 64 && a.vdim <= 64) STK_PFM(2, 4);
    else if (a.dim <= 128 && a.vdim <= 128) STK_PFM(4, 8);
    else if (a.vdim <= 192) STK_PFM(8, 12);  // (a latent cache's rows: 192 value channels do not pay for 256)
    else STK_PFM(8, 16);
#undef STK_PFM
    return;
  }
  auto need = [&](int kt) { return ((size_t)STK_QT * a.dim + (size_t)kt * (a.dim + 1) + (size_t)kt * a.vdim + (size_t)STK_QT * kt) * sizeof(float); };
  dim3 grid((a.max_q + STK_QT - 1) / STK_QT, a.B, a.H);
  const int kt = need(64) <= 64 * 1024 ? 64 : (need(32) <= 64 * 1024 ? 32 : 16);
  VRA_CHECK_ARG(need(kt) <= 64 * 1024, "stack attention: head does not fit LDS");
  const size_t lds = need(kt);
#define STK_PF(TT, KTV) launch_checked("stack attention (prefill)", [&] { stk_attn_prefill_kernel<TT, KTV><<<grid, 256, lds, st>>>(a); })
  if (dtype == VRA_F32) {
    if (kt == 64) STK_PF(float, 64);
    else if (kt == 32) STK_PF(float, 32);
    else STK_PF(float, 16);
  } else {
    if (kt == 64) STK_PF(uint16_t, 64);
    else if (kt == 32) STK_PF(uint16_t, 32);
    else STK_PF(uint16_t, 16);
  }
#undef STK_PF
}

// ================================================================================================ C entry points (one operator each)
extern "C" void vra_stack_op_embed_sinpos(const uint32_t* ids, const int64_t* positions, const void* embed, const float* inv_freq, float* x, int32_t T,
                                          int32_t W, int32_t V, int32_t dtype, int64_t stream) {
  vra_stack_embed_sinpos(ids, positions, embed, inv_freq, x, T, W, V, dtype, stream);
}
extern "C" void vra_stack_op_group_norm(const float* x, const float* w, void* h, int32_t T, int32_t W, int32_t groups, float eps, const void* router_w,
                                        int32_t n_router, int32_t top, int32_t gate_row, int32_t* pair_expert, float* pair_weight, float* gate_out,
                                        int32_t dtype, int64_t stream) {
  StkNormArgs a;
  a.x = x, a.w = w, a.h = h, a.T = T, a.W = W, a.groups = groups, a.eps = eps;
  a.router_w = router_w, a.n_router = n_router, a.top = top, a.gate_row = gate_row;
  a.pair_expert = pair_expert, a.pair_weight = pair_weight, a.gate_out = gate_out;
  vra_stack_group_norm(a, dtype, stream);
}
extern "C" void vra_stack_op_gemm(const void* a, int32_t lda, const void* w, int64_t w_group_stride, void* out, int32_t ldo, int32_t out_f32, int32_t M,
                                  int32_t N, int32_t K, float alpha, const int32_t* tile_group, int32_t granule, const int32_t* a_row,
                                  const float* a_scale, const int32_t* out_row, int32_t epi, float limit, int32_t dtype, int64_t stream) {
  StkGemmArgs g;
  g.a = a, g.lda = lda, g.w = w, g.w_group_stride = w_group_stride, g.out = out, g.ldo = ldo, g.out_f32 = out_f32, g.M = M, g.N = N, g.K = K;
  g.alpha = alpha, g.tile_group = tile_group, g.granule = granule, g.a_row = a_row, g.a_scale = a_scale, g.out_row = out_row, g.epi = epi, g.limit = limit;
  vra_stack_gemm(g, dtype, stream);
}
extern "C" void vra_stack_op_moe_sort(const int32_t* pair_expert, const float* pair_weight, int32_t P, int32_t top, int32_t n_groups, int32_t granule,
                                      int32_t max_rows, int32_t* row_token, float* row_scale, int32_t* row_pair, int32_t* tile_group, int64_t stream) {
  vra_stack_moe_sort(pair_expert, pair_weight, P, top, n_groups, granule, max_rows, row_token, row_scale, row_pair, tile_group, stream);
}
extern "C" void vra_stack_op_gated_act(const float* gu, void* out, int32_t M, int32_t F, float limit, float act_alpha, int32_t dtype, int64_t stream) {
  vra_stack_gated_act(gu, out, M, F, limit, act_alpha, dtype, stream, 0);
}
extern "C" void vra_stack_op_polynorm(const float* z, void* out, const float* coef, int32_t M, int32_t F, float eps, int32_t dtype, int64_t stream) {
  vra_stack_polynorm(z, out, coef, M, F, eps, dtype, stream);
}
extern "C" void vra_stack_op_residual_combine(float* x, const float* o, const float* p1, int32_t n1, const float* p2, const float* gate, float mult,
                                              int32_t T, int32_t W, int64_t stream) {
  vra_stack_residual_combine(x, o, p1, n1, p2, gate, mult, T, W, stream);
}
extern "C" void vra_stack_op_kv_store(const void* k, const void* v, int32_t ld, void* kc, void* vc, const int64_t* slots, int32_t T, int32_t kdim,
                                      int32_t vdim, int32_t dtype, int64_t stream) {
  vra_stack_kv_store(k, v, ld, kc, vc, slots, T, kdim, vdim, dtype, stream);
}
extern "C" void vra_stack_op_attention(const void* q, int32_t ldq, void* out, const void* kc, const void* vc, const int64_t* positions,
                                       const uint32_t* block_tables, const uint32_t* context_lens, const uint32_t* cu_q, int32_t B, int32_t T,
                                       int32_t max_q, int32_t H, int32_t G, int32_t dim, int32_t vdim, int32_t BS, int32_t max_blocks, float scale,
                                       float softcap, float temp_coef, int32_t temp_every, int32_t dtype, int64_t stream) {
  StkAttnArgs a;
  a.q = q, a.ldq = ldq, a.out = out, a.kc = kc, a.vc = vc, a.positions = positions, a.block_tables = block_tables, a.context_lens = context_lens;
  a.cu_q = cu_q, a.B = B, a.T = T, a.max_q = max_q, a.H = H, a.G = G, a.dim = dim, a.vdim = vdim, a.BS = BS, a.max_blocks = max_blocks;
  a.scale = scale, a.softcap = softcap, a.temp_coef = temp_coef, a.temp_every = temp_every;
  vra_stack_attention(a, dtype, stream);
}
