// MFMA path of decode attention over the mid rows (gfx950, wave64).
//
// One workgroup (4 waves, one per SIMD, up to 512 VGPRs each) owns one KV head, one group
// of batch elements whose query rows fill the 16 MFMA columns (R = nb * G <= 16), and one
// contiguous range of 32-token pages.  Per page:
//
//   scores  S[32 x 16] = E[32 x 2N] . W'[2N x 16]      (f16 MFMA; E = cos/sin of the token offset
//                        + K_mn[32 x dims] . Q_n        inside the page, W' = coefficient-domain
//                                                        query rotated to the page start)
//   softmax P = exp2(S - m)                              (online, base 2)
//   g'[2N x 16] += E^T[2N x 32] . P                      (f16 MFMA, accumulated in the frame of the
//                                                        current page: rotated by one page step first)
//   o_n[dims x 16] += V_mn^T[dims x 32] . P              (bf16 / f16 MFMA on the stored dims)
//
// The 2N coefficient rows are split over the 4 waves (each keeps its slice of E, E^T, W' and
// g' in registers); the partial scores are summed through LDS with one barrier per page.
// Wave w also streams the stored dims of batch element w of the group.  K/V pages arrive as
// ready-made MFMA A operands (see the page layout in the public header).
#pragma once

#include "fa_common.h"

namespace fa_mfma {

typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float2v __attribute__((ext_vector_type(2)));

constexpr int kPart = 36;  // padded row (tokens) of the LDS score partials, floats

template <typename E> struct Mma;
template <> struct Mma<bf16_t> {
  using vec8 = bf16x8;
  using elem = __bf16;
  static __device__ __forceinline__ float4v mma(vec8 a, vec8 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ elem from_bits(bf16_t x) { return __builtin_bit_cast(__bf16, x.bits); }
};
template <> struct Mma<f16_t> {
  using vec8 = half8;
  using elem = _Float16;
  static __device__ __forceinline__ float4v mma(vec8 a, vec8 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ elem from_bits(f16_t x) { return x.v; }
};

// frequency owned by (kstep s, lane group lg, register v) of the score GEMM's K dimension and by
// (row tile rt = 2s + v/2, lane group lg, pair v%2) of the g GEMM's rows: per lane the same set
__device__ __forceinline__ int freq_of(int rt, int lg, int fi2) { return rt * 8 + lg * 2 + fi2; }

constexpr int kFreqWaves = 4;  // the coefficient rows are split four ways (one slice per SIMD)

// ---------------------------------------------------------------------------
// constant operand tables (depend on T and N only); KS = N / 64 ksteps per frequency slice
//   tabE  [4 slices][2 row blocks][KS][64 lanes] x half8 : A operand of the score GEMM
//   tabET [4 slices][2*KS row tiles][64 lanes]  x half8 : A operand of the g GEMM
//   rot   [N] float2 : (cos, sin)(2 pi f 32 / T), the per-page frame rotation
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void decode_tables_kernel(half8* __restrict__ tabE, half8* __restrict__ tabET,
                                                            float2v* __restrict__ rot, int KS, int T, int N) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  const int nE = kFreqWaves * 2 * KS * 64, nET = kFreqWaves * 2 * KS * 64;
  if (idx < nE) {
    const int lane = idx & 63, s = (idx >> 6) % KS, rb = ((idx >> 6) / KS) & 1, w = (idx >> 6) / (2 * KS);
    const int lg = lane >> 4, lc = lane & 15;
    const int i = rb * 16 + lc;
    half8 out;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int v = e >> 1, cs = e & 1;
      const int f = w * 16 * KS + freq_of(2 * s + (v >> 1), lg, v & 1);
      float sn, co;
      fa_sincos_phase(f, i, T, &sn, &co);
      out[e] = (_Float16)(cs ? sn : co);
    }
    tabE[idx] = out;
  } else if (idx < nE + nET) {
    const int k = idx - nE;
    const int lane = k & 63, rt = (k >> 6) % (2 * KS), w = (k >> 6) / (2 * KS);
    const int lg = lane >> 4, rho = lane & 15;
    const int f = w * 16 * KS + freq_of(rt, rho >> 2, (rho & 3) >> 1);
    const int cs = rho & 1;
    half8 out;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float sn, co;
      fa_sincos_phase(f, 8 * lg + e, T, &sn, &co);
      out[e] = (_Float16)(cs ? sn : co);
    }
    tabET[k] = out;
  } else if (idx < nE + nET + N) {
    const int f = idx - nE - nET;
    float sn, co;
    fa_sincos_phase(f, 32, T, &sn, &co);
    rot[f] = float2v{co, sn};
  }
}

static inline size_t tables_bytes(int N) {
  const int KS = N / 64;
  return (size_t)(2 * kFreqWaves * 2 * KS * 64) * 16 + (size_t)N * 8;
}

template <typename E>
struct MidParams {
  const E* q;
  const float* W;       // [B][Hq][2N] fp32, already carrying sm_scale*log2e/N
  const float* c0;      // [B][Hq]
  const E* k_mid;
  const E* v_mid;
  int64_t k_bs, v_bs;
  int cap_pages;
  const int32_t* kn_list;
  const int32_t* kn_h;
  const int32_t* kpad_h;
  const int32_t* vn_h;
  const int32_t* vpad_h;
  const half8* tabE;
  const half8* tabET;
  const float2v* rot;
  float* pm;
  float* pd;
  float* pg;
  float* pon;
  int B, Hq, Hkv, D, G, nbpg, N, L_m, T, n_split, tiles_per_split;
  float sm_log2e;
  int dbg;  // profiling aid: bit 0 skips the stored-dim stream
};

// native sin/cos of 2*pi*((a*b) mod T)/T (hardware takes the angle in revolutions)
__device__ __forceinline__ void fast_sincos_phase(int64_t a, int64_t b, int T, float* s, float* c) {
  const float x = (float)((a * b) % (int64_t)T) / (float)T;
  *s = __builtin_amdgcn_sinf(x);
  *c = __builtin_amdgcn_cosf(x);
}

// The workgroup is a two-stage pipeline over the pages of its split, one barrier per page:
//   waves 0-3 ("score waves")  page t+1: S partial = E . W' (their frequency slice) + K_mn . Q_n (their batch
//                              element) -> LDS; then advance W' by one page step
//   waves 4-7 ("value waves")  page t  : sum the four partials, online softmax, rotate/rescale the g history,
//                              g' += E^T . P (their frequency slice), o_n += V_mn^T . P (their batch element)
// Score wave i and value wave i own the same frequencies and stream the same batch element of the group.
// KS: ksteps (32 coefficient rows) per slice = N / 64.  KMAX: ksteps of stored K dims a head may have
// (dp_k / 32).  VMAX: V dim groups of 16 (dp_v / 16).
template <typename E, int KS, int KMAX, int VMAX>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void decode_mid_mfma_kernel(
    const MidParams<E> p) {
  using M = Mma<E>;
  using vec8 = typename M::vec8;
  __shared__ float s_part[2][kFreqWaves][16 * kPart];
  __shared__ float s_max[kFreqWaves][16];
  __shared__ float4v s_rot[kFreqWaves * 2 * KS * 4];  // [slice][row tile][lane group] = (c, s) pair 0, (c, s) pair 1

  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, lg = lane >> 4, lc = lane & 15;
  const bool score_wave = w < kFreqWaves;
  const int sl = w & 3;  // frequency slice and batch element of the group
  const int split = blockIdx.x, h = blockIdx.y, grp = blockIdx.z;
  const int G = p.G, N = p.N;
  const int b0 = grp * p.nbpg;
  const int nb = min(p.nbpg, p.B - b0);
  const int R = nb * G;
  const bool valid_r = lc < R;
  const int bb_r = lc / G, g_r = lc - bb_r * G;
  const int64_t qrow = valid_r ? ((int64_t)(b0 + bb_r) * p.Hq + h * G + g_r) : 0;
  const int fbase = sl * 16 * KS;
  const bool has_mn = sl < nb && !(p.dbg & 1);
  const int my_b = b0 + (sl < nb ? sl : 0);

  const int n_tiles = (p.L_m + 31) >> 5;
  const int t_beg = split * p.tiles_per_split;
  const int t_end = min(n_tiles, t_beg + p.tiles_per_split);
  const int n_it = t_end > t_beg ? t_end - t_beg : 0;

  if (score_wave && lc == 0) {
#pragma unroll
    for (int rt = 0; rt < 2 * KS; ++rt) {
      const float2v a = p.rot[fbase + freq_of(rt, lg, 0)];
      const float2v b = p.rot[fbase + freq_of(rt, lg, 1)];
      s_rot[(sl * 2 * KS + rt) * 4 + lg] = float4v{a[0], a[1], b[0], b[1]};
    }
  }

  if (score_wave) {
    // =============================== score waves ===============================
    half8 Ea[2][KS];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int s = 0; s < KS; ++s) Ea[rb][s] = p.tabE[((sl * 2 + rb) * KS + s) * 64 + lane];

    // coefficient-domain query: Wc/Ws[rt][f2] = (cos-row, sin-row) weights of frequency
    // freq_of(rt, lg, f2) for column lc; normalised per column, rotated to the first page
    float Wc[2 * KS][2], Ws[2 * KS][2];
    float wmax = 0.f;
    {
      const float* wr = p.W + qrow * 2 * N;
#pragma unroll
      for (int rt = 0; rt < 2 * KS; ++rt) {
        const int f = fbase + freq_of(rt, lg, 0);
        float2v c2 = valid_r ? *(const float2v*)(wr + f) : float2v{0.f, 0.f};
        float2v s2 = valid_r ? *(const float2v*)(wr + N + f) : float2v{0.f, 0.f};
        Wc[rt][0] = c2[0]; Wc[rt][1] = c2[1];
        Ws[rt][0] = s2[0]; Ws[rt][1] = s2[1];
        wmax = fmaxf(wmax, fmaxf(fmaxf(fabsf(c2[0]), fabsf(c2[1])), fmaxf(fabsf(s2[0]), fabsf(s2[1]))));
      }
    }
    wmax = fa_rows_max(wmax);
    if (lg == 0) s_max[sl][lc] = wmax;
    __syncthreads();
    wmax = fmaxf(fmaxf(s_max[0][lc], s_max[1][lc]), fmaxf(s_max[2][lc], s_max[3][lc]));
    // power-of-two column scale keeps the f16 operand in [-1, 1] without rounding
    const float colscale = wmax > 0.f ? exp2f(ceilf(log2f(wmax))) : 1.f;
    const float colinv = 1.0f / colscale;
    const float c0col = (valid_r && sl == 0) ? p.c0[qrow] : 0.f;
#pragma unroll
    for (int rt = 0; rt < 2 * KS; ++rt)
#pragma unroll
      for (int f2 = 0; f2 < 2; ++f2) {
        float sn, co;
        fast_sincos_phase(fbase + freq_of(rt, lg, f2), (int64_t)32 * t_beg, p.T, &sn, &co);
        const float wc = Wc[rt][f2] * colinv, ws = Ws[rt][f2] * colinv;
        Wc[rt][f2] = co * wc + sn * ws;    // rotation by -phi: W'c = cos(phi) wc + sin(phi) ws
        Ws[rt][f2] = -sn * wc + co * ws;   //                   W's = -sin(phi) wc + cos(phi) ws
      }

    // stored K dims of batch element sl: both 16-token blocks of the page
    const int kn0 = p.kn_h[h], kn_len = p.kn_h[h + 1] - kn0;
    const int kp0 = p.kpad_h[h], dpk = p.kpad_h[h + 1] - kp0;
    const int nks = dpk >> 5;
    vec8 Qb[KMAX];
#pragma unroll
    for (int s = 0; s < KMAX; ++s)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = s * 32 + 8 * lg + e;
        typename M::elem val = (typename M::elem)0.f;
        if (has_mn && valid_r && bb_r == sl && j < kn_len)
          val = M::from_bits(p.q[qrow * p.D + (p.kn_list[kn0 + j] - h * p.D)]);
        Qb[s][e] = val;
      }
    const E* kbase = p.k_mid + (int64_t)my_b * p.k_bs + (int64_t)kp0 * 32 * p.cap_pages + lane * 8;
    vec8 K0[2 * KMAX], K1[2 * KMAX], K2[2 * KMAX];
    auto load_k = [&](int t, vec8* kf) {
      const E* kp = kbase + (int64_t)t * dpk * 32;
#pragma unroll
      for (int tb = 0; tb < 2; ++tb)
#pragma unroll
        for (int s = 0; s < KMAX; ++s)
          if (s < nks) kf[tb * KMAX + s] = *(const vec8*)(kp + (tb * nks + s) * 512);
    };
    if (has_mn && n_it > 0) load_k(t_beg, K0);
    if (has_mn && n_it > 1) load_k(t_beg + 1, K1);

    for (int it = 0; it <= n_it; ++it) {
      if (it < n_it) {
        const int t = t_beg + it;
        if (has_mn && it + 2 < n_it) load_k(t + 2, K2);
        float4v accf[2] = {float4v{0.f, 0.f, 0.f, 0.f}, float4v{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
        for (int s = 0; s < KS; ++s) {
          half8 wb;
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            wb[2 * v] = (_Float16)Wc[2 * s + (v >> 1)][v & 1];
            wb[2 * v + 1] = (_Float16)Ws[2 * s + (v >> 1)][v & 1];
          }
          accf[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ea[0][s], wb, accf[0], 0, 0, 0);
          accf[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ea[1][s], wb, accf[1], 0, 0, 0);
        }
        float4v accm[2] = {float4v{0.f, 0.f, 0.f, 0.f}, float4v{0.f, 0.f, 0.f, 0.f}};
        if (has_mn) {
#pragma unroll
          for (int s = 0; s < KMAX; ++s)
            if (s < nks) {
              accm[0] = M::mma(K0[s], Qb[s], accm[0]);
              accm[1] = M::mma(K0[KMAX + s], Qb[s], accm[1]);
            }
        }
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
          float4v o;
#pragma unroll
          for (int v = 0; v < 4; ++v) o[v] = accf[rb][v] * colscale + accm[rb][v] * p.sm_log2e + c0col;
          *(float4v*)&s_part[it & 1][sl][lc * kPart + rb * 16 + 4 * lg] = o;
        }
        // advance W' by one page step
#pragma unroll
        for (int rt = 0; rt < 2 * KS; ++rt) {
          const float4v cs = s_rot[(sl * 2 * KS + rt) * 4 + lg];
#pragma unroll
          for (int f2 = 0; f2 < 2; ++f2) {
            const float c = cs[2 * f2], s = cs[2 * f2 + 1];
            const float x = Wc[rt][f2], y = Ws[rt][f2];
            Wc[rt][f2] = c * x + s * y;
            Ws[rt][f2] = c * y - s * x;
          }
        }
        if (has_mn) {
#pragma unroll
          for (int f = 0; f < 2 * KMAX; ++f) {
            K0[f] = K1[f];
            K1[f] = K2[f];
          }
        }
      }
      __syncthreads();
    }
  } else {
    // =============================== value waves ===============================
    half8 ETa[2 * KS];
#pragma unroll
    for (int rt = 0; rt < 2 * KS; ++rt) ETa[rt] = p.tabET[(sl * 2 * KS + rt) * 64 + lane];
    const int vp0 = p.vpad_h[h], dpv = p.vpad_h[h + 1] - vp0;
    const int ndg = dpv >> 4;
    const E* vbase = p.v_mid + (int64_t)my_b * p.v_bs + (int64_t)vp0 * 32 * p.cap_pages + lane * 8;
    vec8 V0[VMAX], V1[VMAX], V2[VMAX];
    auto load_v = [&](int t, vec8* vf) {
      const E* vp = vbase + (int64_t)t * dpv * 32;
#pragma unroll
      for (int f = 0; f < VMAX; ++f)
        if (f < ndg) vf[f] = *(const vec8*)(vp + f * 512);
    };
    if (has_mn && n_it > 0) load_v(t_beg, V0);
    if (has_mn && n_it > 1) load_v(t_beg + 1, V1);
    float4v hacc[2 * KS], oacc[VMAX];
#pragma unroll
    for (int rt = 0; rt < 2 * KS; ++rt) hacc[rt] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int f = 0; f < VMAX; ++f) oacc[f] = float4v{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, d_run = 0.f;
    const bool ragged_tail = (p.L_m & 31) != 0;
    __syncthreads();  // pairs with the score waves' column-scale exchange

    for (int it = 0; it <= n_it; ++it) {
      if (it > 0) {
        const int t = t_beg + it - 1, buf = (it - 1) & 1;
        if (has_mn && it + 1 < n_it) load_v(t + 2, V2);
        // scores of the page in B-operand layout: column lc, tokens 8*lg + e
        float4v a0 = *(const float4v*)&s_part[buf][0][lc * kPart + 8 * lg];
        float4v a1 = *(const float4v*)&s_part[buf][0][lc * kPart + 8 * lg + 4];
#pragma unroll
        for (int ww = 1; ww < kFreqWaves; ++ww) {
          a0 += *(const float4v*)&s_part[buf][ww][lc * kPart + 8 * lg];
          a1 += *(const float4v*)&s_part[buf][ww][lc * kPart + 8 * lg + 4];
        }
        float sc[8] = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
        if (ragged_tail && t == n_tiles - 1) {
          const int tok0 = t * 32 + 8 * lg;
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (tok0 + e >= p.L_m) sc[e] = -INFINITY;
        }
        float tmax = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
        tmax = fa_rows_max(tmax);
        const float m_new = fmaxf(m_run, tmax);
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // 0 on the first page (m_run = -inf)
        float psum = 0.f;
        half8 pf;
        vec8 pe;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float pv = __builtin_amdgcn_exp2f(sc[e] - m_new);
          psum += pv;
          pf[e] = (_Float16)pv;
          pe[e] = (typename M::elem)pv;
        }
        d_run = d_run * alpha + psum;
        m_run = m_new;
        const bool rescale = __any(alpha != 1.0f);
        // the g history (rescaled by alpha) moves into the frame of this page
        if (rescale) {
#pragma unroll
          for (int rt = 0; rt < 2 * KS; ++rt) hacc[rt] *= alpha;
        }
#pragma unroll
        for (int rt = 0; rt < 2 * KS; ++rt) {
          const float4v cs = s_rot[(sl * 2 * KS + rt) * 4 + lg];
#pragma unroll
          for (int f2 = 0; f2 < 2; ++f2) {
            const float c = cs[2 * f2], s = cs[2 * f2 + 1];
            const float hx = hacc[rt][2 * f2], hy = hacc[rt][2 * f2 + 1];
            hacc[rt][2 * f2] = c * hx + s * hy;
            hacc[rt][2 * f2 + 1] = c * hy - s * hx;
          }
        }
#pragma unroll
        for (int rt = 0; rt < 2 * KS; ++rt)
          hacc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ETa[rt], pf, hacc[rt], 0, 0, 0);
        if (has_mn) {
#pragma unroll
          for (int f = 0; f < VMAX; ++f)
            if (f < ndg) {
              if (rescale) oacc[f] *= alpha;
              oacc[f] = M::mma(V0[f], pe, oacc[f]);
            }
#pragma unroll
          for (int f = 0; f < VMAX; ++f) {
            V0[f] = V1[f];
            V1[f] = V2[f];
          }
        }
      }
      __syncthreads();
    }

    // ---- partials of this split ------------------------------------------------------
    const float dsum = fa_rows_sum(d_run);
    if (valid_r) {
      const int64_t base = qrow * p.n_split + split;
      if (sl == 0 && lg == 0) {
        p.pm[base] = m_run;
        p.pd[base] = dsum;
      }
      float* g = p.pg + base * 2 * N;
      const int64_t last = (int64_t)32 * (t_end > t_beg ? t_end - 1 : t_beg);
#pragma unroll
      for (int rt = 0; rt < 2 * KS; ++rt)
#pragma unroll
        for (int f2 = 0; f2 < 2; ++f2) {
          const int f = fbase + freq_of(rt, lg, f2);
          float sn, co;
          fast_sincos_phase(f, last, p.T, &sn, &co);
          const float x = hacc[rt][2 * f2], y = hacc[rt][2 * f2 + 1];
          g[f] = co * x - sn * y;       // back from the page frame: rotation by +phi
          g[N + f] = sn * x + co * y;
        }
      if (has_mn && bb_r == sl) {
        const int vn_len = p.vn_h[h + 1] - p.vn_h[h];
        float* on = p.pon + base * p.D;
#pragma unroll
        for (int f = 0; f < VMAX; ++f)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            const int j = f * 16 + 4 * lg + v;
            if (f < ndg && j < vn_len) on[j] = oacc[f][v];
          }
      }
    }
  }
}

}  // namespace fa_mfma
