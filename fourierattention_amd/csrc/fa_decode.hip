// Decode attention over [sink ; local window ; mid rows]: the generic VALU kernels that accept any
// shape, the vectorised sink/window kernel, and the dispatch to the MFMA path (fa_decode_mfma.h).
//
// The compressed dims of the mid rows are never rebuilt.  With s = scale,
// a = avg_u - avg_d * s and F[l, n] = cos / sin(2 pi n l / T):
//   score[l]  = F[l, :] . w + q_c . a + q_n . K_mn[l, :],  w = (1/N) K_coef (q_c * s)
//   out_c     = s_v * ((1/N) V_coef^T (F^T p) - avg_d_v * P) + avg_u_v * P,  P = sum_l p[l]
// so one pass over the coefficients before (prep) and one after (merge) replace the
// per-token reconstruction, and the token loop only touches the stored dims.
// All exponentials are base 2 (scores carry log2(e)).
#include <stdlib.h>
#include <string.h>

#include "fa_common.h"
#include <mutex>
#include "fa_decode_mid_launch.h"

namespace {

constexpr int kGMax = 8;      // query heads per KV head handled by the generic kernels
constexpr int kTile = 256;    // tokens per tile = threads per block
constexpr int kFreqIters = 4; // frequencies per thread in the g accumulation (N <= 1024)
constexpr float kLog2e = 1.4426950408889634f;
// fused step: how long a workgroup waits for the rest of its team before it gives up and writes NaN rows, in ticks
// of the 100 MHz wall clock (0.2 s; the wait normally lasts a few microseconds)
constexpr unsigned kTeamWaitTicks = 20u * 1000u * 1000u;

struct Seg {
  const void* k;
  const void* v;
  int rows;
  int64_t bs, rs;
};

// ---------------------------------------------------------------------------
// prep: W[b, hq, n] = (sm*log2e/N) sum_j coef[b, n, kc0 + j] q[b, hq, d_j] s[b, kc0 + j]
//       c0[b, hq]   = sm*log2e * sum_j q[b, hq, d_j] (avg_u - avg_d s)[b, kc0 + j]
// block = 64 coefficient rows of one (b, KV head); thread = (row, one of 4 column classes):
// a thread reads every 4th compressed dim of its row (up to 32 independent loads in flight),
// four neighbouring lanes finish the dot product.
// ---------------------------------------------------------------------------
constexpr int kPrepRows = 64;

template <typename E>
struct PrepArgs {
  const E* q;
  const float* k_mc;
  const float* avg_u;
  const float* avg_d;
  const float* scale;
  const int32_t* kc_list;
  const int32_t* kc_h;
  float* W;
  float* c0;
  int Hq, Hkv, D, N, Ck;
  float sm_log2e;
  // matrix-core mid rows: W goes out in the register layout of that kernel's score waves instead,
  // [batch group][KV head][frequency slice][row tile][cos | sin][column][pair of frequencies] x 2 frequencies, so
  // that each of its loads is one contiguous 512-byte line
  float* W_lane;
  int nbpg, n_slices, ks;
  // and the stored query dims of a column go out as that kernel's B operands (16-bit, zeros where a lane holds
  // nothing): [batch group][KV head][batch element of the group, 4][kstep, 4][64 lanes] x 8 values, lane
  // (lg, lc) of kstep s holding the dims kn_list[32 s + 8 lg + 0 .. 7] of column lc if the column belongs to
  // that batch element.  The mid-row launch then starts with one load per kstep instead of an index load and a
  // gather that depends on it.
  E* q_stored;
  const int32_t* kn_list;
  const int32_t* kn_h;
  // fused step: the two meeting counters of every (batch group, KV head), cleared here for the launch behind
  unsigned* team_cnt;
  // a batch of one sequence whose mid rows run as four sub-splits per workgroup (SUB instances of the mid-row kernel):
  // the stored query dims go out four times, once for the columns of each sub-split
  int sub;
  // A rank-1 update the K coefficients are still owed (the row that left the window, see fa_decode_args.upd_*): every
  // coefficient is read here by exactly one thread, which adds the row's term, writes the coefficient back and goes
  // on with the new value.  upd_row == nullptr: nothing pending.
  const E* upd_row;
  int64_t upd_bs, upd_phase;
  int upd_T;
};

// LDS of the query preparation: the gathered query dims times the scale / the mean terms, per query head; the
// compressed dims of a row the coefficients are still owed
constexpr int kPrepLdsBytes = (2 * kGMax * 128 + 128) * (int)sizeof(float);

// bx: block index along x (row chunk of kPrepRows coefficient rows); y, z come from blockIdx; lds: kPrepLdsBytes
// UPD: a rank-1 update of the K coefficients is pending (an instance of its own: the code for it costs the launch
// 2 us even when it does not run)
template <typename E, bool UPD>
__device__ __forceinline__ void decode_prep_body(const PrepArgs<E>& pa, int bx, void* lds) {
  const E* __restrict__ q = pa.q;
  const float* __restrict__ k_mc = pa.k_mc;
  const float* __restrict__ avg_u = pa.avg_u;
  const float* __restrict__ avg_d = pa.avg_d;
  const float* __restrict__ scale = pa.scale;
  const int32_t* __restrict__ kc_list = pa.kc_list;
  const int32_t* __restrict__ kc_h = pa.kc_h;
  float* __restrict__ W = pa.W;
  float* __restrict__ c0 = pa.c0;
  const int Hq = pa.Hq, Hkv = pa.Hkv, D = pa.D, N = pa.N, Ck = pa.Ck;
  const float sm_log2e = pa.sm_log2e;
  float (&s_qs)[kGMax][128] = *reinterpret_cast<float (*)[kGMax][128]>(lds);
  float (&s_qa)[kGMax][128] = *reinterpret_cast<float (*)[kGMax][128]>((float*)lds + kGMax * 128);
  float* s_ue = (float*)lds + 2 * kGMax * 128;
  const int tid = threadIdx.x;
  const int h = blockIdx.y, b = blockIdx.z;
  const int G = Hq / Hkv;
  const int kc0 = kc_h[h], kc_len = kc_h[h + 1] - kc0;
  for (int e = tid; e < kGMax * 128; e += 256) {
    const int g = e >> 7, j = e & 127;
    float qs = 0.f, qa = 0.f;
    if (g < G && j < kc_len) {
      const int d = kc_list[kc0 + j] - h * D;
      const float sc = scale[(int64_t)b * Ck + kc0 + j];
      const float a = avg_u[(int64_t)b * Ck + kc0 + j] - avg_d[(int64_t)b * Ck + kc0 + j] * sc;
      const float qv = fa_to_float(q[((int64_t)b * Hq + h * G + g) * D + d]);
      qs = qv * sc;
      qa = qv * a;
    }
    s_qs[g][j] = qs;
    s_qa[g][j] = qa;
    if constexpr (UPD)
      if (g == 0) s_ue[j] = j < kc_len ? fa_to_float(pa.upd_row[(int64_t)b * pa.upd_bs + kc_list[kc0 + j]]) : 0.f;
  }
  __syncthreads();
  if (bx == 0 && tid < 2 && pa.team_cnt && b % pa.nbpg == 0) pa.team_cnt[((int64_t)(b / pa.nbpg) * Hkv + h) * 2 + tid] = 0u;
  if (bx == 0 && tid < 64) {
    for (int g = 0; g < G; ++g) {
      float v = fa_wave_sum(s_qa[g][tid] + s_qa[g][tid + 64]);
      if (tid == 0) c0[(int64_t)b * Hq + h * G + g] = v * sm_log2e;
    }
  }
  if constexpr (sizeof(E) == 2) if (bx == 1 && pa.q_stored) {
    const int kn0 = pa.kn_h[h], kn_len = pa.kn_h[h + 1] - kn0;
    const int s = tid >> 6, lane = tid & 63, lg = lane >> 4, lc = lane & 15;
    const int grp = b / pa.nbpg;
    // (a head that stores no K dims has no entries in the list and nobody reads its operands)
    for (int sl = pa.sub ? 0 : b - grp * pa.nbpg, last = pa.sub ? 3 : sl; sl <= last && kn_len > 0; ++sl) {
      const int g = lc - sl * G;   // the column's query head if the column is this batch element's (this sub-split's)
      const bool mine = g >= 0 && g < G;
      const E* qr = q + ((int64_t)b * Hq + h * G + (mine ? g : 0)) * D - h * D;
      union { E e[8]; uint4 raw; } o;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = s * 32 + 8 * lg + e;
        const E qv = qr[pa.kn_list[kn0 + min(j, kn_len - 1)]];   // clamped: no load under a per-lane condition
        o.e[e] = (mine && j < kn_len) ? qv : E();
      }
      *(uint4*)(pa.q_stored + ((((int64_t)(grp * Hkv + h) * 4 + sl) * 4 + s) * 64 + lane) * 8) = o.raw;
    }
  }
  const int n = bx * kPrepRows + (tid >> 2), jq = tid & 3;
  if (n >= 2 * N) return;
  const float* row = k_mc + ((int64_t)b * 2 * N + n) * Ck + kc0;
  float v[32];
#pragma unroll
  for (int i = 0; i < 32; ++i) {
    const int j = jq + 4 * i;
    v[i] = j < kc_len ? row[j] : 0.f;
  }
  if constexpr (UPD) {
    // the pending rank-1 update of this row (the arithmetic of fa_stream_update / fa_coeff_update)
    float sn, co;
    fa_sincos_phase(n >= N ? n - N : n, pa.upd_phase, pa.upd_T, &sn, &co);
    const float f = n >= N ? sn : co;
    float* wrow = const_cast<float*>(row);
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      const int j = jq + 4 * i;
      if (j < kc_len) {
        v[i] = v[i] + f * s_ue[j];
        wrow[j] = v[i];
      }
    }
  }
  const float mul = sm_log2e / (float)N;
#pragma unroll
  for (int g = 0; g < kGMax; ++g) {
    if (g >= G) break;
    float a = 0.f;
#pragma unroll
    for (int i = 0; i < 32; ++i) a = fmaf(v[i], s_qs[g][jq + 4 * i], a);
    a = fa_group_sum<4>(a);
    if (jq == 0) {
      if (pa.W_lane) {
        const int cs = n >= N, nn = n - cs * N;
        const int per = 16 * pa.ks, sl = nn / per, r = nn - sl * per;
        const int grp = b / pa.nbpg, lc = (b - grp * pa.nbpg) * G + g;
        const int lane = lc * 4 + ((r & 7) >> 1);
        const int64_t tile = ((int64_t)(grp * Hkv + h) * pa.n_slices + sl) * 2 * pa.ks + (r >> 3);
        pa.W_lane[((tile * 2 + cs) * 64 + lane) * 2 + (r & 1)] = a * mul;
      } else {
        W[((int64_t)b * Hq + h * G + g) * 2 * N + n] = a * mul;
      }
    }
  }
}

template <typename E, bool UPD>
__global__ __launch_bounds__(256) void decode_prep_kernel(const PrepArgs<E> pa) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[kPrepLdsBytes];
  decode_prep_body<E, UPD>(pa, blockIdx.x, lds);
}

// ---------------------------------------------------------------------------
// sink + local window: one tile of up to 256 full-width rows per block
// ---------------------------------------------------------------------------
template <typename E>
__global__ __launch_bounds__(256) void decode_il_kernel(
    const E* __restrict__ q, Seg s0, Seg s1, float* __restrict__ pm, float* __restrict__ pd,
    float* __restrict__ po, int Hq, int Hkv, int D, int n_split, float sm_log2e) {
  extern __shared__ float smem[];
  const int G = Hq / Hkv;
  float* s_q = smem;                 // [G][D]
  float* s_p = s_q + G * D;          // [G][kTile]
  float* s_red = s_p + G * kTile;    // [4][kGMax]
  float* s_o = s_red + 4 * kGMax;    // [G][D] (second half accumulators)
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int n_il = s0.rows + s1.rows;
  for (int e = tid; e < G * D; e += 256)
    s_q[e] = fa_to_float(q[((int64_t)b * Hq + h * G) * D + e]) * sm_log2e;
  __syncthreads();

  const int i = split * kTile + tid;
  const bool ok = i < n_il;
  const E* krow = nullptr;
  if (ok) {
    krow = (i < s0.rows) ? (const E*)s0.k + (int64_t)b * s0.bs + (int64_t)i * s0.rs
                         : (const E*)s1.k + (int64_t)b * s1.bs + (int64_t)(i - s0.rows) * s1.rs;
    krow += h * D;
  }
  float sc[kGMax];
#pragma unroll
  for (int g = 0; g < kGMax; ++g) sc[g] = 0.f;
  if (ok) {
    for (int d = 0; d < D; ++d) {
      float kv = fa_to_float(krow[d]);
#pragma unroll
      for (int g = 0; g < kGMax; ++g)
        if (g < G) sc[g] = fmaf(kv, s_q[g * D + d], sc[g]);
    }
  }
  // tile max
#pragma unroll
  for (int g = 0; g < kGMax; ++g) {
    float v = fa_wave_max(ok ? sc[g] : -INFINITY);
    if (lane == 0) s_red[w * kGMax + g] = v;
  }
  __syncthreads();
  float mx[kGMax];
#pragma unroll
  for (int g = 0; g < kGMax; ++g)
    mx[g] = fmaxf(fmaxf(s_red[g], s_red[kGMax + g]), fmaxf(s_red[2 * kGMax + g], s_red[3 * kGMax + g]));
  __syncthreads();
  float dsum[kGMax];
#pragma unroll
  for (int g = 0; g < kGMax; ++g) {
    float p = (ok && g < G) ? exp2f(sc[g] - mx[g]) : 0.f;
    if (g < G) s_p[g * kTile + tid] = p;
    float v = fa_wave_sum(p);
    if (lane == 0) s_red[w * kGMax + g] = v;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < kGMax; ++g)
    dsum[g] = s_red[g] + s_red[kGMax + g] + s_red[2 * kGMax + g] + s_red[3 * kGMax + g];

  // PV: thread = (dim, half of the tile)
  const int dim = tid % 128, half = tid / 128;
  float o[kGMax];
#pragma unroll
  for (int g = 0; g < kGMax; ++g) o[g] = 0.f;
  const int t_end = min(kTile, n_il - split * kTile);
  if (dim < D) {
    for (int tt = half; tt < t_end; tt += 2) {
      int ii = split * kTile + tt;
      const E* vrow = (ii < s0.rows) ? (const E*)s0.v + (int64_t)b * s0.bs + (int64_t)ii * s0.rs
                                     : (const E*)s1.v + (int64_t)b * s1.bs + (int64_t)(ii - s0.rows) * s1.rs;
      float vv = fa_to_float(vrow[h * D + dim]);
#pragma unroll
      for (int g = 0; g < kGMax; ++g)
        if (g < G) o[g] = fmaf(s_p[g * kTile + tt], vv, o[g]);
    }
  }
  if (half == 1 && dim < D) {
#pragma unroll
    for (int g = 0; g < kGMax; ++g)
      if (g < G) s_o[g * D + dim] = o[g];
  }
  __syncthreads();
  if (half == 0 && dim < D) {
#pragma unroll
    for (int g = 0; g < kGMax; ++g)
      if (g < G) {
        int64_t r = ((int64_t)b * Hq + h * G + g) * n_split + split;
        po[r * D + dim] = o[g] + s_o[g * D + dim];
      }
  }
  if (tid < G) {
    int64_t r = ((int64_t)b * Hq + h * G + tid) * n_split + split;
    float m = -INFINITY, dd = 0.f;
#pragma unroll
    for (int g = 0; g < kGMax; ++g)
      if (g == tid) {
        m = mx[g];
        dd = dsum[g];
      }
    pm[r] = m;
    pd[r] = dd;
  }
}

// ---------------------------------------------------------------------------
// mid rows: split over tokens; per split partial (m, d, g[2N], o_n[vn_len])
// ---------------------------------------------------------------------------
// element offset of (token, stored dim j) inside one (batch, head) run of pages
__device__ __forceinline__ int64_t paged_offset(bool is_v, int dp, int64_t token, int j) {
  const int64_t page = token >> 5;
  const int t = (int)(token & 31);
  if (!is_v) return page * dp * 32 + (int64_t)((t >> 4) * (dp >> 5) + (j >> 5)) * 512 + (((j & 31) >> 3) * 16 + (t & 15)) * 8 + (j & 7);
  return page * dp * 32 + (int64_t)(j >> 4) * 512 + ((t >> 3) * 16 + (j & 15)) * 8 + (t & 7);
}

template <typename E, bool PAGED>
__global__ __launch_bounds__(256) void decode_mid_kernel(
    const E* __restrict__ q, const E* __restrict__ k_mn, int64_t k_bs, int64_t k_rs,
    const E* __restrict__ v_mn, int64_t v_bs, int64_t v_rs, int cap_pages, const int32_t* __restrict__ kpad_h,
    const int32_t* __restrict__ vpad_h, const float* __restrict__ W,
    const float* __restrict__ c0, const int32_t* __restrict__ kn_list, const int32_t* __restrict__ kn_h,
    const int32_t* __restrict__ vn_h, float* __restrict__ pm, float* __restrict__ pd,
    float* __restrict__ pg, float* __restrict__ pon, int Hq, int Hkv, int D, int N, int L_m, int T,
    int n_split, int tiles_per_split, float sm_log2e) {
  extern __shared__ float smem[];
  const int G = Hq / Hkv;
  float* s_w = smem;                   // [G][2N]
  float* s_qn = s_w + G * 2 * N;       // [G][D]
  float* s_p = s_qn + G * D;           // [G][kTile]
  float* s_red = s_p + G * kTile;      // [4][kGMax]
  float* s_o = s_red + 4 * kGMax;      // [G][D]
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int split = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int kn0 = kn_h[h], kn_len = kn_h[h + 1] - kn0;
  const int vn0 = vn_h[h], vn_len = vn_h[h + 1] - vn0;

  for (int e = tid; e < G * 2 * N; e += 256) s_w[e] = W[((int64_t)b * Hq + h * G) * 2 * N + e];
  for (int e = tid; e < G * D; e += 256) {
    int g = e / D, j = e % D;
    float v = 0.f;
    if (j < kn_len) v = fa_to_float(q[((int64_t)b * Hq + h * G + g) * D + (kn_list[kn0 + j] - h * D)]) * sm_log2e;
    s_qn[e] = v;
  }
  float cz[kGMax], m_run[kGMax], d_run[kGMax];
#pragma unroll
  for (int g = 0; g < kGMax; ++g) {
    cz[g] = g < G ? c0[(int64_t)b * Hq + h * G + g] : 0.f;
    m_run[g] = -INFINITY;
    d_run[g] = 0.f;
  }
  float gc[kFreqIters][kGMax], gs[kFreqIters][kGMax], on[kGMax];
#pragma unroll
  for (int i = 0; i < kFreqIters; ++i)
#pragma unroll
    for (int g = 0; g < kGMax; ++g) gc[i][g] = gs[i][g] = 0.f;
#pragma unroll
  for (int g = 0; g < kGMax; ++g) on[g] = 0.f;
  __syncthreads();

  const int l_beg = split * tiles_per_split * kTile;
  const int l_end = min(L_m, l_beg + tiles_per_split * kTile);
  int dpk = 0, dpv = 0;
  const E* kb;
  const E* vb;
  if (PAGED) {
    dpk = kpad_h[h + 1] - kpad_h[h];
    dpv = vpad_h[h + 1] - vpad_h[h];
    kb = k_mn + (int64_t)b * k_bs + (int64_t)kpad_h[h] * 32 * cap_pages;
    vb = v_mn + (int64_t)b * v_bs + (int64_t)vpad_h[h] * 32 * cap_pages;
  } else {
    kb = k_mn + (int64_t)b * k_bs + kn0;
    vb = v_mn + (int64_t)b * v_bs + vn0;
  }
  const int dim = tid % 128, half = tid / 128;

  for (int l0 = l_beg; l0 < l_end; l0 += kTile) {
    const int t_len = min(kTile, l_end - l0);
    // ---- phase 1: scores, thread = token --------------------------------
    const int l = l0 + tid;
    const bool ok = tid < t_len;
    float sc[kGMax];
#pragma unroll
    for (int g = 0; g < kGMax; ++g) sc[g] = cz[g];
    if (ok) {
      float sr, si, zr = 1.f, zi = 0.f;
      fa_sincos_phase(l, 1, T, &si, &sr);
      for (int n = 0; n < N; ++n) {
        if ((n & 63) == 0) fa_sincos_phase(l, n, T, &zi, &zr);
#pragma unroll
        for (int g = 0; g < kGMax; ++g)
          if (g < G) sc[g] = fmaf(zr, s_w[g * 2 * N + n], fmaf(zi, s_w[g * 2 * N + N + n], sc[g]));
        float nr = zr * sr - zi * si;
        float ni = zr * si + zi * sr;
        zr = nr;
        zi = ni;
      }
      for (int j = 0; j < kn_len; ++j) {
        float kv = fa_to_float(PAGED ? kb[paged_offset(false, dpk, l, j)] : kb[(int64_t)l * k_rs + j]);
#pragma unroll
        for (int g = 0; g < kGMax; ++g)
          if (g < G) sc[g] = fmaf(kv, s_qn[g * D + j], sc[g]);
      }
    }
    // ---- phase 2: online softmax over the tile --------------------------
#pragma unroll
    for (int g = 0; g < kGMax; ++g) {
      float v = fa_wave_max(ok ? sc[g] : -INFINITY);
      if (lane == 0) s_red[w * kGMax + g] = v;
    }
    __syncthreads();
    float alpha[kGMax];
#pragma unroll
    for (int g = 0; g < kGMax; ++g) {
      float tm = fmaxf(fmaxf(s_red[g], s_red[kGMax + g]), fmaxf(s_red[2 * kGMax + g], s_red[3 * kGMax + g]));
      float mn = fmaxf(m_run[g], tm);
      alpha[g] = (m_run[g] == -INFINITY) ? 0.f : exp2f(m_run[g] - mn);
      m_run[g] = mn;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < kGMax; ++g) {
      float p = (ok && g < G) ? exp2f(sc[g] - m_run[g]) : 0.f;
      if (g < G) s_p[g * kTile + tid] = p;
      float v = fa_wave_sum(p);
      if (lane == 0) s_red[w * kGMax + g] = v;
    }
    __syncthreads();
#pragma unroll
    for (int g = 0; g < kGMax; ++g)
      d_run[g] = d_run[g] * alpha[g] + (s_red[g] + s_red[kGMax + g] + s_red[2 * kGMax + g] + s_red[3 * kGMax + g]);
    // ---- phase 3: g[n] += sum_t p[t] e^{i theta n (l0 + t)}, thread = frequency
#pragma unroll
    for (int i = 0; i < kFreqIters; ++i) {
      const int n = tid + 256 * i;
      if (n < N) {
#pragma unroll
        for (int g = 0; g < kGMax; ++g) {
          gc[i][g] *= alpha[g];
          gs[i][g] *= alpha[g];
        }
        float sr, si, zr, zi;
        fa_sincos_phase(n, 1, T, &si, &sr);
        for (int tt = 0; tt < t_len; ++tt) {
          if ((tt & 63) == 0) fa_sincos_phase(n, l0 + tt, T, &zi, &zr);
#pragma unroll
          for (int g = 0; g < kGMax; ++g)
            if (g < G) {
              float p = s_p[g * kTile + tt];
              gc[i][g] = fmaf(p, zr, gc[i][g]);
              gs[i][g] = fmaf(p, zi, gs[i][g]);
            }
          float nr = zr * sr - zi * si;
          float ni = zr * si + zi * sr;
          zr = nr;
          zi = ni;
        }
      }
    }
    // ---- phase 4: stored V dims, thread = (dim, tile half) ----------------
#pragma unroll
    for (int g = 0; g < kGMax; ++g) on[g] *= alpha[g];
    if (dim < vn_len) {
      for (int tt = half; tt < t_len; tt += 2) {
        float vv = fa_to_float(PAGED ? vb[paged_offset(true, dpv, l0 + tt, dim)] : vb[(int64_t)(l0 + tt) * v_rs + dim]);
#pragma unroll
        for (int g = 0; g < kGMax; ++g)
          if (g < G) on[g] = fmaf(s_p[g * kTile + tt], vv, on[g]);
      }
    }
    __syncthreads();
  }

  // ---- write the split's partials ---------------------------------------
  if (half == 1 && dim < vn_len) {
#pragma unroll
    for (int g = 0; g < kGMax; ++g)
      if (g < G) s_o[g * D + dim] = on[g];
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < kGMax; ++g) {
    if (g >= G) continue;
    const int64_t r = ((int64_t)b * Hq + h * G + g) * n_split + split;
    if (half == 0 && dim < vn_len) pon[r * D + dim] = on[g] + s_o[g * D + dim];
#pragma unroll
    for (int i = 0; i < kFreqIters; ++i) {
      const int n = tid + 256 * i;
      if (n < N) {
        pg[r * 2 * N + n] = gc[i][g];
        pg[r * 2 * N + N + n] = gs[i][g];
      }
    }
    if (tid == 0) {
      pm[r] = m_run[g];
      pd[r] = d_run[g];
    }
  }
}

// ---------------------------------------------------------------------------
// merge: one block of 1024 threads per (b, KV head) combines, for the G query heads of that head,
// the partials of every split and applies the V coefficients once:
//   out_c = s_v * ((1/N) V_coef^T g - avg_d_v * P) + avg_u_v * P
// The kernel is a chain of short dependent phases, so its time is memory latency: every thread first
// issues the loads of ALL phases (split maxima, its g / o partials, its V-coefficient rows) into
// registers and only then starts the first phase; what does not fit the prefetch is looped afterwards.
// ---------------------------------------------------------------------------
constexpr int kMergePre = 16;    // splits held in registers per prefetched element
constexpr int kMergeRows = 16;   // V-coefficient rows held in registers per thread
constexpr int kMergeIl = 20;     // sink/window splits held in registers per output element

// n > 0 loads from ptr[min(u, n - 1) * stride], u < CNT: clamped, so that none of them is conditional
template <int CNT>
__device__ __forceinline__ void prefetch_strided(float (&v)[CNT], const float* __restrict__ ptr, int64_t stride, int n) {
#pragma unroll
  for (int u = 0; u < CNT; ++u) v[u] = ptr[(int64_t)min(u, n - 1) * stride];
}
// sum_s w[s] * x[s] over the prefetched head of a strided vector, the tail read from memory
template <int CNT>
__device__ __forceinline__ float weighted_sum_pre(const float (&v)[CNT], const float* __restrict__ ptr, int64_t stride,
                                                  const float* w, int n) {
  float a = 0.f;
#pragma unroll
  for (int u = 0; u < CNT; ++u)
    if (u < n) a = fmaf(w[u], v[u], a);
  for (int s0 = CNT; s0 < n; s0 += 16) {
    float t[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) t[u] = ptr[(int64_t)min(s0 + u, n - 1) * stride];
#pragma unroll
    for (int u = 0; u < 16; ++u)
      if (s0 + u < n) a = fmaf(w[s0 + u], t[u], a);
  }
  return a;
}
// the same without a prefetched head
__device__ __forceinline__ float weighted_sum(const float* __restrict__ ptr, int64_t stride, const float* w, int n) {
  float a = 0.f;
  for (int s0 = 0; s0 < n; s0 += 16) {
    float t[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) t[u] = ptr[(int64_t)min(s0 + u, n - 1) * stride];
#pragma unroll
    for (int u = 0; u < 16; ++u)
      if (s0 + u < n) a = fmaf(w[s0 + u], t[u], a);
  }
  return a;
}

constexpr int kMergeChunksMax = 8;  // blocks per (b, KV head): each applies the V coefficients of its share of the dims

// n_mid_stride: splits the partial buffers of the mid rows have room for per query head; the head's own number of
// splits comes from the table (heads that store more dims are cut into more splits)
__global__ __launch_bounds__(1024) void decode_merge_kernel(
    const float* __restrict__ il_m, const float* __restrict__ il_d, const float* __restrict__ il_o, int n_il_split,
    const float* __restrict__ md_m, const float* __restrict__ md_d, const float* __restrict__ md_g,
    const float* __restrict__ md_on, int n_mid_stride, const fa_mfma::SplitTable st, const float* __restrict__ v_mc,
    const float* __restrict__ avg_u, const float* __restrict__ avg_d, const float* __restrict__ scale,
    const int32_t* __restrict__ vc_list, const int32_t* __restrict__ vc_h, const int32_t* __restrict__ vn_list,
    const int32_t* __restrict__ vn_h, float* __restrict__ out, void* __restrict__ out_cast, int cast_dtype, int Hq, int Hkv,
    int D, int N, int Cv, int g_nbpg) {
  // the result goes out as fp32 (out) and / or rounded to the storage type of the model (out_cast)
  auto put = [&](int64_t at, float v) {
    if (out) out[at] = v;
    if (out_cast) {
      if (cast_dtype == FA_BF16) ((bf16_t*)out_cast)[at] = bf16_t{fa_f32_to_bf16_bits(v)};
      else if (cast_dtype == FA_FP16) ((f16_t*)out_cast)[at] = f16_t{(_Float16)v};
      else ((float*)out_cast)[at] = v;
    }
  };
  // g_nbpg > 0: the g partials come from the matrix-core kernel in its own layout, per (batch group of g_nbpg,
  // KV head, split) N/8 tiles of [column][pair of frequencies] x {cos f, sin f, cos f+1, sin f+1},
  // column = (batch element within the group) * G + query head within the KV head; otherwise one row of 2N per
  // (query head, split)
  extern __shared__ float smem[];
  const int G = Hq / Hkv;
  const int n_mid_split = (int)blockIdx.x < fa_mfma::kSplitHeads ? min(st.n[blockIdx.x], n_mid_stride) : n_mid_stride;
  const int n_all = n_il_split + n_mid_split;
  float* s_g = smem;                     // [G][2N]
  float* s_w = s_g + G * 2 * N;          // [G][n_all]
  float* s_d = s_w + G * n_all;          // [G][n_all]
  float* s_sc = s_d + G * n_all;         // [2][kGMax]: sum of d, sum of d over the mid rows
  float* s_part = s_sc + 2 * kGMax;      // [parts][G][cwp] = 1024 * G
  float* s_o = s_part + 1024 * G;        // [G][D]
  int* s_own = (int*)(s_o + G * D);      // [D]: bit 0 = some list holds the dim, bit 1 = this block writes it
  const int tid = threadIdx.x;
  const int h = blockIdx.x, b = blockIdx.y, z = blockIdx.z, n_chunks = gridDim.z;
  const int64_t r0 = (int64_t)b * Hq + h * G;
  const int vc0 = vc_h[h], vc_len = vc_h[h + 1] - vc0;
  const int vn0 = vn_h[h], vn_len = vn_h[h + 1] - vn0;
  // this block's share of the compressed and of the stored dims (by position in the head's lists)
  const int cw = (vc_len + n_chunks - 1) / n_chunks;
  const int c_lo = min(vc_len, z * cw), cn = min(vc_len, c_lo + cw) - c_lo;
  const int nw = (vn_len + n_chunks - 1) / n_chunks;
  const int n_lo = min(vn_len, z * nw), nn = min(vn_len, n_lo + nw) - n_lo;
  const bool has_coef = n_mid_split > 0 && cn > 0;
  int cwp = 1;                           // power of two >= cw: threads = (dim, row class)
  while (cwp < cw) cwp <<= 1;
  const int parts = 1024 / cwp;          // cw <= 128 for head dims up to 512

  // ---- every load this thread will need, issued before anything is waited for --------------------------
  float m_raw = -INFINITY, d_raw = 0.f;            // split maxima / denominators (first G * n_all threads)
  if (tid < G * n_all) {
    const int g = tid / n_all, s_ = tid - g * n_all;
    const int64_t r = r0 + g;
    const bool il = s_ < n_il_split;
    m_raw = il ? il_m[r * n_il_split + s_] : md_m[r * n_mid_stride + (s_ - n_il_split)];
    d_raw = il ? il_d[r * n_il_split + s_] : md_d[r * n_mid_stride + (s_ - n_il_split)];
  }
  // g partials: two neighbouring threads share four consecutive coefficient rows of one head, one takes the even
  // splits, the other the odd ones (16-byte loads: a quarter of the load instructions of a row-per-thread map)
  constexpr int kGPre = kMergePre / 2;
  // (a row-per-head g whose rows of 2N values are not multiples of 16 bytes is read value by value: E4 = 1)
  const int E4 = (g_nbpg > 0 || (2 * N) % 4 == 0) ? 4 : 1;
  const int g_items = G * (2 * N / E4);
  auto g_load = [&](const float* ptr) { return E4 == 4 ? *(const float4*)ptr : make_float4(*ptr, 0.f, 0.f, 0.f); };
  const int g_item = tid >> 1, g_half = tid & 1;
  const int64_t g_split_stride = g_nbpg > 0 ? (int64_t)16 * 2 * N : (int64_t)2 * N;
  // item -> (query head g, group of four values n4) and the address of its values in split 0
  auto g_locate = [&](int item, int& g, int& n4) -> const float* {
    if (g_nbpg > 0) {   // consecutive items walk through the 64 * G contiguous bytes this block owns in a tile
      g = (item >> 2) % G;
      n4 = (item / (4 * G)) * 4 + (item & 3);
      const int grp = b / g_nbpg, lc = (b - grp * g_nbpg) * G + g;
      return md_g + (int64_t)(grp * Hkv + h) * n_mid_stride * g_split_stride + (int64_t)(n4 >> 2) * 256 + (lc * 4 + (n4 & 3)) * 4;
    }
    g = item / (2 * N / E4);
    n4 = item - g * (2 * N / E4);
    return md_g + (r0 + g) * n_mid_stride * 2 * N + E4 * n4;
  };
  float4 g_pre[kGPre];
  if (has_coef && g_item < g_items) {
    int g, n4;
    const float* gp = g_locate(g_item, g, n4);
#pragma unroll
    for (int u = 0; u < kGPre; ++u) g_pre[u] = g_load(gp + (int64_t)min(g_half + 2 * u, n_mid_split - 1) * g_split_stride);
  }
  // V coefficients: rows part, part + parts, ... of dim c_lo + j
  const int j = tid & (cwp - 1), part = tid / cwp;
  const float* vp = v_mc + (int64_t)b * 2 * N * Cv + vc0 + c_lo + j;
  float v_pre[kMergeRows];
  if (has_coef && j < cn) {
#pragma unroll
    for (int u = 0; u < kMergeRows; ++u) v_pre[u] = vp[(int64_t)min(part + u * parts, 2 * N - 1) * Cv];
  }
  float n_pre[kMergePre];                           // stored-dim outputs of the mid rows
  if (n_mid_split > 0 && tid < G * nn) {
    const int g = tid / nn, jj = n_lo + (tid - g * nn);
    prefetch_strided(n_pre, md_on + (r0 + g) * n_mid_stride * D + jj, D, n_mid_split);
  }
  float il_pre[kMergeIl];                           // sink/window outputs of element tid
  if (n_il_split > 0 && tid < G * D) {
    const int g = tid / D, d = tid - g * D;
    prefetch_strided(il_pre, il_o + (r0 + g) * n_il_split * D + d, D, n_il_split);
  }

  // ---- split weights: one wave per query head ----------------------------------------------------------
  for (int idx = tid; idx < G * n_all; idx += 1024) {
    if (idx == tid) {
      s_w[idx] = m_raw;
      s_d[idx] = d_raw;
    } else {
      const int g = idx / n_all, s_ = idx - g * n_all;
      const int64_t r = r0 + g;
      const bool il = s_ < n_il_split;
      s_w[idx] = il ? il_m[r * n_il_split + s_] : md_m[r * n_mid_stride + (s_ - n_il_split)];
      s_d[idx] = il ? il_d[r * n_il_split + s_] : md_d[r * n_mid_stride + (s_ - n_il_split)];
    }
  }
  for (int idx = tid; idx < G * D; idx += 1024) s_o[idx] = 0.f;
  for (int idx = tid; idx < D; idx += 1024) s_own[idx] = 0;
  __syncthreads();
  // which dims this block writes: its list shares; block 0 also takes dims that no list names
  for (int idx = tid; idx < vc_len + vn_len; idx += 1024) {
    const bool c = idx < vc_len;
    const int pos = c ? idx : idx - vc_len;
    const int d = (c ? vc_list[vc0 + pos] : vn_list[vn0 + pos]) - h * D;
    const bool mine = c ? (pos >= c_lo && pos < c_lo + cn) : (pos >= n_lo && pos < n_lo + nn);
    s_own[d] = mine ? 3 : 1;
  }
  {
    const int g = tid >> 6, lane = tid & 63;
    if (g < G) {
      float mstar = -INFINITY;
      for (int s_ = lane; s_ < n_all; s_ += 64) mstar = fmaxf(mstar, s_w[g * n_all + s_]);
      mstar = fa_wave_max(mstar);
      float dsum = 0.f, pmid = 0.f;
      for (int s_ = lane; s_ < n_all; s_ += 64) {
        const float m = s_w[g * n_all + s_];
        const float wgt = m == -INFINITY ? 0.f : exp2f(m - mstar);
        s_w[g * n_all + s_] = wgt;
        if (s_ < n_il_split) dsum += wgt * s_d[g * n_all + s_]; else pmid += wgt * s_d[g * n_all + s_];
      }
      dsum = fa_wave_sum(dsum);
      pmid = fa_wave_sum(pmid);
      if (lane == 0) {
        s_sc[g] = dsum + pmid;
        s_sc[kGMax + g] = pmid;
      }
    }
  }
  __syncthreads();

  if (n_mid_split > 0) {
    if (cn > 0) {
      // g summed over the splits
      auto fold1 = [&](const float4& v, int sp, const float* wg, float4& a) {
        if (sp < n_mid_split) {
          const float wt = wg[sp];
          a.x = fmaf(wt, v.x, a.x); a.y = fmaf(wt, v.y, a.y);
          a.z = fmaf(wt, v.z, a.z); a.w = fmaf(wt, v.w, a.w);
        }
      };
      for (int item = g_item; item < g_items; item += 512) {   // same trip count for both threads of a pair
        int g, n4;
        const float* gp = g_locate(item, g, n4);
        const float* wg = s_w + g * n_all + n_il_split;
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
        int u0 = 0;
        if (item == g_item) {   // the prefetched head
#pragma unroll
          for (int u = 0; u < kGPre; ++u) fold1(g_pre[u], g_half + 2 * u, wg, a);
          u0 = kGPre;
        }
        for (; g_half + 2 * u0 < n_mid_split; u0 += 4) {
          float4 v[4];
#pragma unroll
          for (int u = 0; u < 4; ++u)
            v[u] = g_load(gp + (int64_t)min(g_half + 2 * (u0 + u), n_mid_split - 1) * g_split_stride);
#pragma unroll
          for (int u = 0; u < 4; ++u) fold1(v[u], g_half + 2 * (u0 + u), wg, a);
        }
        a.x += fa_dpp<FA_DPP_XOR1>(a.x); a.y += fa_dpp<FA_DPP_XOR1>(a.y);
        a.z += fa_dpp<FA_DPP_XOR1>(a.z); a.w += fa_dpp<FA_DPP_XOR1>(a.w);
        if (g_half == 0) {
          if (g_nbpg > 0) {   // {cos f, sin f, cos f+1, sin f+1} with f = 2 * n4
            *(float2*)(s_g + g * 2 * N + 2 * n4) = make_float2(a.x, a.z);
            *(float2*)(s_g + g * 2 * N + N + 2 * n4) = make_float2(a.y, a.w);
          } else if (E4 == 4) {
            *(float4*)(s_g + g * 2 * N + 4 * n4) = a;
          } else {
            s_g[g * 2 * N + n4] = a.x;
          }
        }
      }
      __syncthreads();
      // g . V_coef
      float acc[kGMax];
#pragma unroll
      for (int g = 0; g < kGMax; ++g) acc[g] = 0.f;
      if (j < cn) {
#pragma unroll
        for (int u = 0; u < kMergeRows; ++u) {
          const int n = part + u * parts;
          if (n < 2 * N) {
#pragma unroll
            for (int g = 0; g < kGMax; ++g)
              if (g < G) acc[g] = fmaf(s_g[g * 2 * N + n], v_pre[u], acc[g]);
          }
        }
        for (int n0 = part + kMergeRows * parts; n0 < 2 * N; n0 += 16 * parts) {
          float v[16];
#pragma unroll
          for (int u = 0; u < 16; ++u) v[u] = vp[(int64_t)min(n0 + u * parts, 2 * N - 1) * Cv];
#pragma unroll
          for (int u = 0; u < 16; ++u)
            if (n0 + u * parts < 2 * N) {
#pragma unroll
              for (int g = 0; g < kGMax; ++g)
                if (g < G) acc[g] = fmaf(s_g[g * 2 * N + n0 + u * parts], v[u], acc[g]);
            }
        }
      }
      // the row classes of one dim meet in LDS
#pragma unroll
      for (int g = 0; g < kGMax; ++g)
        if (g < G) s_part[(part * G + g) * cwp + j] = acc[g];
      __syncthreads();
      // 16 lanes per (head, dim) fold the row classes
      for (int idx = tid; idx < G * cwp * 16; idx += 1024) {
        const int sub = idx & 15, gj = idx >> 4;
        const int g = gj / cwp, jj = gj - g * cwp;
        float a = 0.f;
        for (int pp = sub; pp < parts; pp += 16) a += s_part[(pp * G + g) * cwp + jj];
        a = fa_group_sum<16>(a);
        if (sub == 0 && jj < cn) {
          a /= (float)N;
          const int64_t o = (int64_t)b * Cv + vc0 + c_lo + jj;
          const float pmid = s_sc[kGMax + g];
          s_o[g * D + (vc_list[vc0 + c_lo + jj] - h * D)] = scale[o] * (a - avg_d[o] * pmid) + avg_u[o] * pmid;
        }
      }
    }
    if (tid < G * nn) {
      const int g = tid / nn, jj = n_lo + (tid - g * nn);
      s_o[g * D + (vn_list[vn0 + jj] - h * D)] = weighted_sum_pre(n_pre, md_on + (r0 + g) * n_mid_stride * D + jj, D,
                                                                  s_w + g * n_all + n_il_split, n_mid_split);
    }
    for (int idx = tid + 1024; idx < G * nn; idx += 1024) {
      const int g = idx / nn, jj = n_lo + (idx - g * nn);
      s_o[g * D + (vn_list[vn0 + jj] - h * D)] =
          weighted_sum(md_on + (r0 + g) * n_mid_stride * D + jj, D, s_w + g * n_all + n_il_split, n_mid_split);
    }
  }
  __syncthreads();
  if (tid < G * D) {
    const int g = tid / D, d = tid - g * D;
    const int own = s_own[d];
    if ((own & 2) || (z == 0 && own == 0)) {
      float a = s_o[tid];
      if (n_il_split > 0) a += weighted_sum_pre(il_pre, il_o + (r0 + g) * n_il_split * D + d, D, s_w + g * n_all, n_il_split);
      put((r0 + g) * D + d, a / s_sc[g]);
    }
  }
  for (int idx = tid + 1024; idx < G * D; idx += 1024) {
    const int g = idx / D, d = idx - g * D;
    const int own = s_own[d];
    if ((own & 2) || (z == 0 && own == 0)) {
      float a = s_o[idx];
      if (n_il_split > 0) a += weighted_sum(il_o + (r0 + g) * n_il_split * D + d, D, s_w + g * n_all, n_il_split);
      put((r0 + g) * D + d, a / s_sc[g]);
    }
  }
}

// ---------------------------------------------------------------------------
// merge after the matrix-core mid rows: the same result as decode_merge_kernel, cut along the coefficient rows.
// Block (z, KV head, b) of 256 threads owns 64 frequencies = 128 coefficient rows: it folds the g partials of every
// split for those rows (each read by exactly one block), multiplies them with its 128 rows of the V coefficients
// (each read by exactly one block) and leaves the contribution to every compressed dim of the head in part_c.  It
// also folds, for its share of the head's dims, the sink/window partial outputs (stage_il, by dim) and the
// stored-dim partial outputs of the mid rows (stage_on, by position in the head's list).  The block that finishes
// last for a (b, KV head) - a counter tells, cleared by the mid-row kernel in front - adds the row blocks up in a
// fixed order, applies the column statistics, normalises and writes the G output rows.
// Every load of the first phases is requested before the first barrier.
// ---------------------------------------------------------------------------
constexpr int kMrTiles = 8;               // g tiles of 8 frequencies per block
constexpr int kMrRows = kMrTiles * 16;    // coefficient rows per block (cos and sin of 64 frequencies)
constexpr int kMrGPre = 8;                // g partials (16 bytes each) a thread requests ahead
constexpr int kMrVPre = 8;                // V-coefficient groups of four dims a thread requests ahead
constexpr int kMrSub = 4;                 // lanes that share one (query head, dim) of the staged sums
constexpr int kMrIlPre = 6, kMrOnPre = 4; // sink/window and mid partial outputs requested ahead per lane

// What the blocks of one launch hand to the block that finishes last goes through device-scope accesses: stores that
// write through to memory, loads that do not stop at a cache another block's data has never been in.  The stores of a
// block have completed when it counts itself (the barrier in front of the count waits for them), and the last block
// loads after it has seen the count, so no cache write-back or invalidate is needed around the counter.
__device__ __forceinline__ void st_device(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float ld_device(const float* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }

template <int CTRL>
__device__ __forceinline__ float4 fa_dpp4_add(float4 v) {
  v.x += fa_dpp<CTRL>(v.x); v.y += fa_dpp<CTRL>(v.y); v.z += fa_dpp<CTRL>(v.z); v.w += fa_dpp<CTRL>(v.w);
  return v;
}
// sum over the lanes q, q + nqp, q + 2 nqp, ... of a wave (nqp a power of two up to 32, uniform over the wave); every
// lane gets the sum of its class
__device__ __forceinline__ float4 fa_sum_lane_classes(float4 v, int nqp) {
  if (nqp <= 1) v = fa_dpp4_add<0x121>(v);   // row_ror:1
  if (nqp <= 2) v = fa_dpp4_add<0x122>(v);   // row_ror:2
  if (nqp <= 4) v = fa_dpp4_add<0x124>(v);   // row_ror:4
  if (nqp <= 8) v = fa_dpp4_add<0x128>(v);   // row_ror:8
  float lo, hi;
  if (nqp <= 16) {
    fa_swap16(v.x, &lo, &hi); v.x = lo + hi; fa_swap16(v.y, &lo, &hi); v.y = lo + hi;
    fa_swap16(v.z, &lo, &hi); v.z = lo + hi; fa_swap16(v.w, &lo, &hi); v.w = lo + hi;
  }
  fa_swap32(v.x, &lo, &hi); v.x = lo + hi; fa_swap32(v.y, &lo, &hi); v.y = lo + hi;
  fa_swap32(v.z, &lo, &hi); v.z = lo + hi; fa_swap32(v.w, &lo, &hi); v.w = lo + hi;
  return v;
}

struct MergeRowsArgs {
  const float* il_m; const float* il_d; const float* il_o; int n_il_split;
  const float* md_m; const float* md_d; const float* md_g; const float* md_on; int n_mid_stride;
  const float* v_mc; const float* avg_u; const float* avg_d; const float* scale;
  const int32_t* vc_list; const int32_t* vc_h; const int32_t* vn_list; const int32_t* vn_h;
  float* out; void* out_cast; int cast_dtype;
  float* part_c;      // [B][Hkv][row blocks][G][128]
  float* stage_il;    // [B][Hq][D]
  float* stage_on;    // [B][Hq][D]
  unsigned* count;    // [B][Hkv]
  int Hq, Hkv, D, N, Cv, nbpg;
  fa_mfma::SplitTable st;
};

__global__ __launch_bounds__(256) void decode_merge_rows_kernel(const MergeRowsArgs a) {
  extern __shared__ float smem[];
  const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int z = blockIdx.x, R = gridDim.x, h = blockIdx.y, b = blockIdx.z;
  const int G = a.Hq / a.Hkv, D = a.D, N = a.N, Hkv = a.Hkv;
  const int n_il = a.n_il_split, n_mid = min(a.st.n[h], a.n_mid_stride), n_all = n_il + n_mid;
  const int64_t r0 = (int64_t)b * a.Hq + h * G;
  float* s_w = smem;                        // [G][n_all]
  float* s_d = s_w + G * n_all;             // [G][n_all]
  float* s_sc = s_d + G * n_all;            // [2][kGMax]
  float* s_g = s_sc + 2 * kGMax;            // [G][128]: cos rows of the block's 64 frequencies, then sin rows
  float* s_x = s_g + G * kMrRows;           // max(1024, 512 * G): g per split class, then the four waves' sums of the product
  float* s_o = s_x + (512 * G > 1024 ? 512 * G : 1024);   // [G][D], last block
  __shared__ int s_last;

  // ---- requests: first those whose addresses do not wait for the head's entries of the index lists ------------
  float m_raw = -INFINITY, d_raw = 0.f;
  if (tid < G * n_all) {
    const int g = tid / n_all, s_ = tid - g * n_all;
    const bool il = s_ < n_il;
    m_raw = il ? a.il_m[(r0 + g) * n_il + s_] : a.md_m[(r0 + g) * a.n_mid_stride + (s_ - n_il)];
    d_raw = il ? a.il_d[(r0 + g) * n_il + s_] : a.md_d[(r0 + g) * a.n_mid_stride + (s_ - n_il)];
  }
  // g partials: item = (tile, query head, pair of frequencies) = 16 bytes {cos f, sin f, cos f+1, sin f+1};
  // consecutive items walk through the 64 G contiguous bytes this (b, KV head) owns in a tile
  const int n_items = kMrTiles * G * 4;                  // <= 256 (G <= kGMax)
  const int n_cls = 256 / n_items;                       // split classes
  const int item = tid % n_items, cls = tid / n_items;
  const bool g_on = cls < n_cls;
  const int64_t g_split_stride = (int64_t)16 * 2 * N;
  const int it_g = (item >> 2) % G, it_t = item / (4 * G), it_q = item & 3;
  const float* gp;
  {
    const int grp = b / a.nbpg, lc = (b - grp * a.nbpg) * G + it_g;
    gp = a.md_g + (int64_t)(grp * Hkv + h) * a.n_mid_stride * g_split_stride + (int64_t)(z * kMrTiles + it_t) * 256 +
         (lc * 4 + it_q) * 4;
  }
  float4 g_pre[kMrGPre];
  if (g_on) {
#pragma unroll
    for (int u = 0; u < kMrGPre; ++u) g_pre[u] = *(const float4*)(gp + (int64_t)min(cls + u * n_cls, n_mid - 1) * g_split_stride);
  }
  const int dsh = (D + R - 1) / R, d_lo = min(D, z * dsh), d_n = min(D, d_lo + dsh) - d_lo;   // this block's dims
  const int sub = tid & (kMrSub - 1), sit = tid / kMrSub;   // 64 (head, dim) items at a time
  float il_pre[kMrIlPre], on_pre[kMrOnPre];
  const bool il_on = n_il > 0 && sit < G * d_n;
  if (il_on) {
    const int g = sit / d_n, d = d_lo + (sit - g * d_n);
#pragma unroll
    for (int u = 0; u < kMrIlPre; ++u) il_pre[u] = a.il_o[((r0 + g) * n_il + min(sub + u * kMrSub, n_il - 1)) * D + d];
  }
  const int vc0 = a.vc_h[h], vc_len = a.vc_h[h + 1] - vc0;
  const int vn0 = a.vn_h[h], vn_len = a.vn_h[h + 1] - vn0;
  int nqp = 2;                              // groups of four dims, a power of two (at least two: no more row classes
                                            // than rows): threads = (group, row class)
  while (4 * nqp < vc_len) nqp <<= 1;
  const int cwp = 4 * nqp;
  const int parts = 256 / nqp;              // vc_len <= D <= 128: at least eight row classes
  const bool has_coef = vc_len > 0;
  // V coefficients: local row rr < 64 is the cos row of frequency 64 z + rr, rr >= 64 the sin row of 64 z + rr - 64;
  // 16 bytes per load where the head's columns allow it (the address path takes one load instruction of a wave per
  // 16 clocks whatever its width)
  const int vq = tid & (nqp - 1), part = tid / nqp;
  const int rows_per_thread = kMrRows / parts;           // parts divides 128
  auto v_row = [&](int rr) { return rr < 64 ? 64 * z + rr : N + 64 * z + (rr - 64); };
  const float* vp = a.v_mc + (int64_t)b * 2 * N * a.Cv + vc0 + 4 * vq;
  const bool v_on = has_coef && 4 * vq < vc_len;
  const int v_lim = vc_len - 4 * vq - 1;    // last valid offset within the group of four
  const bool v_wide = v_lim >= 3 && ((vc0 | a.Cv) & 3) == 0 && ((uintptr_t)a.v_mc & 15) == 0;
  auto v_load = [&](int rr) {
    const float* p4 = vp + (int64_t)v_row(min(rr, kMrRows - 1)) * a.Cv;
    if (v_wide) return *(const float4*)p4;
    return make_float4(p4[0], p4[min(1, v_lim)], p4[min(2, v_lim)], p4[min(3, v_lim)]);   // dims past the head's: unused
  };
  float4 v_pre[kMrVPre];
  if (v_on) {
#pragma unroll
    for (int u = 0; u < kMrVPre; ++u) v_pre[u] = v_load(part + u * parts);
  }
  // this block's share of the stored positions of the mid rows
  const int nsh = (vn_len + R - 1) / R, n_lo = min(vn_len, z * nsh), n_n = min(vn_len, n_lo + nsh) - n_lo;
  const bool on_on = sit < G * n_n;
  if (on_on) {
    const int g = sit / n_n, jj = n_lo + (sit - g * n_n);
#pragma unroll
    for (int u = 0; u < kMrOnPre; ++u) on_pre[u] = a.md_on[((r0 + g) * a.n_mid_stride + min(sub + u * kMrSub, n_mid - 1)) * D + jj];
  }

  // ---- split weights: one wave per query head -----------------------------------------------------------
  for (int idx = tid; idx < G * n_all; idx += 256) {
    if (idx == tid) {
      s_w[idx] = m_raw;
      s_d[idx] = d_raw;
    } else {
      const int g = idx / n_all, s_ = idx - g * n_all;
      const bool il = s_ < n_il;
      s_w[idx] = il ? a.il_m[(r0 + g) * n_il + s_] : a.md_m[(r0 + g) * a.n_mid_stride + (s_ - n_il)];
      s_d[idx] = il ? a.il_d[(r0 + g) * n_il + s_] : a.md_d[(r0 + g) * a.n_mid_stride + (s_ - n_il)];
    }
  }
  __syncthreads();
  for (int g = wv; g < G; g += 4) {
    float mstar = -INFINITY;
    for (int s_ = lane; s_ < n_all; s_ += 64) mstar = fmaxf(mstar, s_w[g * n_all + s_]);
    mstar = fa_wave_max(mstar);
    float dsum = 0.f, pmid = 0.f;
    for (int s_ = lane; s_ < n_all; s_ += 64) {
      const float m = s_w[g * n_all + s_];
      const float wgt = m == -INFINITY ? 0.f : exp2f(m - mstar);
      s_w[g * n_all + s_] = wgt;
      if (s_ < n_il) dsum += wgt * s_d[g * n_all + s_]; else pmid += wgt * s_d[g * n_all + s_];
    }
    dsum = fa_wave_sum(dsum);
    pmid = fa_wave_sum(pmid);
    if (lane == 0) {
      s_sc[g] = dsum + pmid;
      s_sc[kGMax + g] = pmid;
    }
  }
  __syncthreads();

  // ---- g of the block's rows, summed over the splits ------------------------------------------------------
  if (has_coef) {
    if (g_on) {
      const float* wg = s_w + it_g * n_all + n_il;
      float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
      auto fold = [&](const float4& v, int sp) {
        if (sp < n_mid) {
          const float wt = wg[sp];
          acc.x = fmaf(wt, v.x, acc.x); acc.y = fmaf(wt, v.y, acc.y);
          acc.z = fmaf(wt, v.z, acc.z); acc.w = fmaf(wt, v.w, acc.w);
        }
      };
#pragma unroll
      for (int u = 0; u < kMrGPre; ++u) fold(g_pre[u], cls + u * n_cls);
      for (int u0 = kMrGPre; cls + u0 * n_cls < n_mid; u0 += 4) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = *(const float4*)(gp + (int64_t)min(cls + (u0 + u) * n_cls, n_mid - 1) * g_split_stride);
#pragma unroll
        for (int u = 0; u < 4; ++u) fold(v[u], cls + (u0 + u) * n_cls);
      }
      *(float4*)(s_x + (cls * n_items + item) * 4) = acc;
    }
    __syncthreads();
    for (int idx = tid; idx < n_items * 4; idx += 256) {
      float v = 0.f;
      for (int c = 0; c < n_cls; ++c) v += s_x[c * n_items * 4 + idx];
      const int it = idx >> 2, e = idx & 3;          // e: cos f, sin f, cos f + 1, sin f + 1 with f = 8 tile + 2 pair
      const int g = (it >> 2) % G, t = it / (4 * G), q = it & 3;
      s_g[g * kMrRows + (e & 1) * 64 + t * 8 + 2 * q + (e >> 1)] = v;
    }
    __syncthreads();
    // ---- times the block's rows of the V coefficients
    float4 acc[kGMax];
#pragma unroll
    for (int g = 0; g < kGMax; ++g) acc[g] = make_float4(0.f, 0.f, 0.f, 0.f);
    auto fma_row = [&](int rr, const float4& v) {
#pragma unroll
      for (int g = 0; g < kGMax; ++g)
        if (g < G) {
          const float gg = s_g[g * kMrRows + rr];
          acc[g].x = fmaf(gg, v.x, acc[g].x); acc[g].y = fmaf(gg, v.y, acc[g].y);
          acc[g].z = fmaf(gg, v.z, acc[g].z); acc[g].w = fmaf(gg, v.w, acc[g].w);
        }
    };
    if (v_on) {
#pragma unroll
      for (int u = 0; u < kMrVPre; ++u)
        if (u < rows_per_thread) fma_row(part + u * parts, v_pre[u]);
      for (int u = kMrVPre; u < rows_per_thread; ++u) fma_row(part + u * parts, v_load(part + u * parts));
    }
    // the row classes of a wave meet through lane exchanges, the four waves in LDS
#pragma unroll
    for (int g = 0; g < kGMax; ++g)
      if (g < G) {
        const float4 v = fa_sum_lane_classes(acc[g], nqp);
        if (lane < nqp) {
          float* dst = s_x + (wv * G + g) * cwp + 4 * lane;
          dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
        }
      }
    __syncthreads();
    float* pc = a.part_c + (((int64_t)b * Hkv + h) * R + z) * G * 128;
    for (int idx = tid; idx < G * cwp; idx += 256) {
      const int g = idx / cwp, jj = idx - g * cwp;
      if (jj < vc_len) {
        float v = 0.f;
#pragma unroll
        for (int ww = 0; ww < 4; ++ww) v += s_x[(ww * G + g) * cwp + jj];
        st_device(pc + g * 128 + jj, v);
      }
    }
  }
  // ---- staged sums of this block's share of the dims --------------------------------------------------
  for (int it0 = 0; it0 < G * d_n && n_il > 0; it0 += 256 / kMrSub) {
    const int it = it0 + sit;
    float v = 0.f;
    if (it < G * d_n) {
      const int g = it / d_n, d = d_lo + (it - g * d_n);
      const float* wg = s_w + g * n_all;
      const float* src = a.il_o + (r0 + g) * n_il * D + d;
      int u0 = 0;
      if (it0 == 0) {
#pragma unroll
        for (int u = 0; u < kMrIlPre; ++u)
          if (sub + u * kMrSub < n_il) v = fmaf(wg[sub + u * kMrSub], il_pre[u], v);
        u0 = kMrIlPre;
      }
      for (int sp = sub + u0 * kMrSub; sp < n_il; sp += kMrSub) v = fmaf(wg[sp], src[(int64_t)sp * D], v);
    }
    v = fa_group_sum<kMrSub>(v);
    if (it < G * d_n && sub == 0) {
      const int g = it / d_n, d = d_lo + (it - g * d_n);
      st_device(a.stage_il + (r0 + g) * D + d, v);
    }
  }
  for (int it0 = 0; it0 < G * n_n; it0 += 256 / kMrSub) {
    const int it = it0 + sit;
    float v = 0.f;
    if (it < G * n_n) {
      const int g = it / n_n, jj = n_lo + (it - g * n_n);
      const float* wg = s_w + g * n_all + n_il;
      const float* src = a.md_on + (r0 + g) * a.n_mid_stride * D + jj;
      int u0 = 0;
      if (it0 == 0) {
#pragma unroll
        for (int u = 0; u < kMrOnPre; ++u)
          if (sub + u * kMrSub < n_mid) v = fmaf(wg[sub + u * kMrSub], on_pre[u], v);
        u0 = kMrOnPre;
      }
      for (int sp = sub + u0 * kMrSub; sp < n_mid; sp += kMrSub) v = fmaf(wg[sp], src[(int64_t)sp * D], v);
    }
    v = fa_group_sum<kMrSub>(v);
    if (it < G * n_n && sub == 0) {
      const int g = it / n_n, jj = n_lo + (it - g * n_n);
      st_device(a.stage_on + (r0 + g) * D + jj, v);
    }
  }

  // ---- the block that finishes last for this (b, KV head) puts the rows together ----------------------------
  // Everything handed to that block went out through st_device (written through to memory) and is read back through
  // ld_device (past the caches); a plain store or load on this path would be a hand-over that works most of the
  // time.  The build checks in the generated assembly that no store follows the wait below in front of the counter.
  __builtin_amdgcn_s_waitcnt(0);   // vmcnt(0) expcnt(0) lgkmcnt(0): this thread's stores have been acknowledged
  __syncthreads();
  if (tid == 0) s_last = atomicAdd(a.count + (int64_t)b * Hkv + h, 1u) == (unsigned)(R - 1);
  __syncthreads();
  if (!s_last) return;
  for (int idx = tid; idx < G * D; idx += 256) s_o[idx] = n_il > 0 ? ld_device(a.stage_il + r0 * D + idx) : 0.f;
  __syncthreads();
  const float* pc0 = a.part_c + ((int64_t)b * Hkv + h) * R * G * 128;
  for (int idx = tid; idx < G * vc_len; idx += 256) {
    const int g = idx / vc_len, jj = idx - g * vc_len;
    float v = 0.f;
    for (int z0 = 0; z0 < R; z0 += 8) {       // eight loads in flight, added in the order of the row blocks
      float t[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) t[u] = ld_device(pc0 + ((int64_t)min(z0 + u, R - 1) * G + g) * 128 + jj);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (z0 + u < R) v += t[u];
    }
    v /= (float)N;
    const int64_t o = (int64_t)b * a.Cv + vc0 + jj;
    const float pmid = s_sc[kGMax + g];
    s_o[g * D + (a.vc_list[vc0 + jj] - h * D)] += a.scale[o] * (v - a.avg_d[o] * pmid) + a.avg_u[o] * pmid;
  }
  for (int idx = tid; idx < G * vn_len; idx += 256) {
    const int g = idx / vn_len, jj = idx - g * vn_len;
    s_o[g * D + (a.vn_list[vn0 + jj] - h * D)] += ld_device(a.stage_on + (r0 + g) * D + jj);
  }
  __syncthreads();
  for (int idx = tid; idx < G * D; idx += 256) {
    const int g = idx / D;
    const float v = s_o[idx] / s_sc[g];
    const int64_t at = r0 * D + idx;
    if (a.out) a.out[at] = v;
    if (a.out_cast) {
      if (a.cast_dtype == FA_BF16) ((bf16_t*)a.out_cast)[at] = bf16_t{fa_f32_to_bf16_bits(v)};
      else if (a.cast_dtype == FA_FP16) ((f16_t*)a.out_cast)[at] = f16_t{(_Float16)v};
      else ((float*)a.out_cast)[at] = v;
    }
  }
}

// ---------------------------------------------------------------------------
// merge after the matrix-core mid rows, up to four query heads per KV head: the result of decode_merge_kernel with
// the loads laid out for the address path.  A compute unit takes one load instruction of a wave every 16 clocks
// whatever its width, and this kernel's time is the number of such instructions: every thread therefore reads 16
// bytes per load wherever the data allow it, and nothing is loaded after the first barrier on the common shapes.
//   g partials     one thread per group of four values {cos f, sin f, cos f+1, sin f+1} of one query head, GPRE
//                  splits requested ahead (all of them for an even share of the mid rows)
//   V coefficients thread = (four neighbouring dims of the block's share, row class): 16-byte loads where the head's
//                  columns allow it; the row classes of a wave are folded with lane exchanges, the waves in LDS
//   sink/window    thread = (query head, four neighbouring dims, one of eight split groups)
//   stored dims    thread = (query head, position in the head's list, split group)
// Block (KV head, b, z) applies the V coefficients of share z of the head's dims, like decode_merge_kernel.
// ---------------------------------------------------------------------------
constexpr int kMfG = 4;        // query heads per KV head (one 16-byte row of the folded g per coefficient row)
constexpr int kMfIlPre = 3;    // sink/window partial outputs (16 bytes each) a thread requests ahead
constexpr int kMfOnPre = 2;    // stored-dim partial outputs a thread requests ahead

template <int GPRE, int VPRE>
__global__ __launch_bounds__(1024) void decode_merge_fast_kernel(const MergeRowsArgs a) {
  auto put = [&](int64_t at, float v) {
    if (a.out) a.out[at] = v;
    if (a.out_cast) {
      if (a.cast_dtype == FA_BF16) ((bf16_t*)a.out_cast)[at] = bf16_t{fa_f32_to_bf16_bits(v)};
      else if (a.cast_dtype == FA_FP16) ((f16_t*)a.out_cast)[at] = f16_t{(_Float16)v};
      else ((float*)a.out_cast)[at] = v;
    }
  };
  extern __shared__ float smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int h = blockIdx.x, b = blockIdx.y, z = blockIdx.z, n_chunks = gridDim.z;
  const int Hq = a.Hq, Hkv = a.Hkv, D = a.D, N = a.N, Cv = a.Cv, G = Hq / Hkv;
  const int n_il = a.n_il_split, n_mid = min(a.st.n[h], a.n_mid_stride), n_all = n_il + n_mid;
  const int WM = (a.n_mid_stride + 3) & ~3;   // row of the mid-split weights, 16-byte aligned
  const int64_t r0 = (int64_t)b * Hq + h * G;
  const int vc0 = a.vc_h[h], vc_len = a.vc_h[h + 1] - vc0;
  const int vn0 = a.vn_h[h], vn_len = a.vn_h[h + 1] - vn0;
  // this block's share of the compressed and of the stored dims (by position in the head's lists)
  const int cw = (vc_len + n_chunks - 1) / n_chunks;
  const int c_lo = min(vc_len, z * cw), cn = min(vc_len, c_lo + cw) - c_lo;
  const int nw = (vn_len + n_chunks - 1) / n_chunks;
  const int n_lo = min(vn_len, z * nw), nn = min(vn_len, n_lo + nw) - n_lo;
  const bool has_coef = n_mid > 0 && cn > 0;
  int nqp = 1;   // groups of four dims in the share, rounded up to a power of two (at most 32: 128 dims)
  while (4 * nqp < cw) nqp <<= 1;
  const int CWP = 4 * nqp;

  // (what is read 16 bytes at a time comes first)
  float* s_g = smem;                           // [2N][4]: folded g, one 16-byte row per coefficient row
  float* s_wm = s_g + 2 * N * kMfG;            // [4][WM]: weights of the mid splits (zero past the head's count)
  float* s_part = s_wm + kMfG * WM;            // [16 waves][4][CWP]
  float* s_w = s_part + 16 * kMfG * CWP;       // [G][n_all]
  float* s_d = s_w + G * n_all;                // [G][n_all]
  float* s_sc = s_d + G * n_all;               // [2][kGMax]: sum of d, sum of d over the mid rows
  float* s_o = s_sc + 2 * kGMax;               // [G][D]
  int* s_own = (int*)(s_o + G * D);            // [D]: bit 0 = some list holds the dim, bit 1 = this block writes it

  // ---- every load of the common shapes, issued before anything is waited for ---------------------------------
  // (first the dim that position tid of the head's lists names: G * D <= 512 threads cover both lists)
  int own_dim = -1;
  if (tid < vc_len + vn_len) own_dim = (tid < vc_len ? a.vc_list[vc0 + tid] : a.vn_list[vn0 + tid - vc_len]) - h * D;
  float m_raw = -INFINITY, d_raw = 0.f;
  if (tid < G * n_all) {
    const int g = tid / n_all, s_ = tid - g * n_all;
    const int64_t r = r0 + g;
    const bool il = s_ < n_il;
    m_raw = il ? a.il_m[r * n_il + s_] : a.md_m[r * a.n_mid_stride + (s_ - n_il)];
    d_raw = il ? a.il_d[r * n_il + s_] : a.md_d[r * a.n_mid_stride + (s_ - n_il)];
  }
  // g partials: item = (tile of 8 frequencies, query head, pair of frequencies within the tile); consecutive items
  // walk through the 64 * G contiguous bytes this block owns in a tile of a split
  const int n_items = G * (N / 2);
  const int64_t g_stride = (int64_t)16 * 2 * N;   // floats between two splits
  const int g_of = (tid >> 2) % G, n4 = (tid / (4 * G)) * 4 + (tid & 3);
  const float* gp = nullptr;
  float4 gv[GPRE];
  const bool g_on = has_coef && tid < n_items;
  if (g_on) {
    const int grp = b / a.nbpg, lc = (b - grp * a.nbpg) * G + g_of;
    gp = a.md_g + (int64_t)(grp * Hkv + h) * a.n_mid_stride * g_stride + (int64_t)(n4 >> 2) * 256 + (lc * 4 + (n4 & 3)) * 4;
#pragma unroll
    for (int u = 0; u < GPRE; ++u) gv[u] = *(const float4*)(gp + (int64_t)min(u, n_mid - 1) * g_stride);
  }
  // V coefficients: dims c_lo + 4 q .. + 3 of the head's list, rows cls, cls + classes, ...
  const int q = tid & (nqp - 1), cls = tid / nqp, classes = 1024 / nqp;
  const bool v_on = has_coef && 4 * q < cn;
  const int v_lim = cn - 4 * q - 1;   // last valid offset within the group of four
  const float* vp = a.v_mc + (int64_t)b * 2 * N * Cv + vc0 + c_lo + 4 * q;
  const bool v_wide = v_lim >= 3 && ((vc0 + c_lo) & 3) == 0 && (Cv & 3) == 0 && ((uintptr_t)a.v_mc & 15) == 0;
  auto v_load = [&](int n) {
    const float* p4 = vp + (int64_t)min(n, 2 * N - 1) * Cv;
    if (v_wide) return *(const float4*)p4;
    return make_float4(p4[0], p4[min(1, v_lim)], p4[min(2, v_lim)], p4[min(3, v_lim)]);   // dims past the share: unused
  };
  float4 vv[VPRE];
  if (v_on) {
#pragma unroll
    for (int u = 0; u < VPRE; ++u) vv[u] = v_load(cls + u * classes);
  }
  // what the last step of the compressed dims needs: thread = (query head, dim of the share)
  const int fin_g = tid / CWP, fin_j = tid - fin_g * CWP;
  const bool fin_on = has_coef && fin_g < G && fin_j < cn;
  float fin_scale = 0.f, fin_au = 0.f, fin_ad = 0.f;
  int fin_dim = 0;
  if (fin_on) {
    const int64_t o = (int64_t)b * Cv + vc0 + c_lo + fin_j;
    fin_scale = a.scale[o]; fin_au = a.avg_u[o]; fin_ad = a.avg_d[o];
    fin_dim = a.vc_list[vc0 + c_lo + fin_j] - h * D;
  }

  // ---- split weights: one wave per query head ------------------------------------------------------------------
  if (tid < G * n_all) {
    s_w[tid] = m_raw;
    s_d[tid] = d_raw;
  }
  for (int idx = tid; idx < kMfG * WM; idx += 1024) s_wm[idx] = 0.f;
  for (int idx = tid; idx < G * D; idx += 1024) s_o[idx] = 0.f;
  for (int idx = tid; idx < D; idx += 1024) s_own[idx] = 0;
  __syncthreads();
  // which dims this block writes: its list shares; block 0 also takes dims that no list names
  if (own_dim >= 0) {
    const bool c = tid < vc_len;
    const int pos = c ? tid : tid - vc_len;
    const bool mine = c ? (pos >= c_lo && pos < c_lo + cn) : (pos >= n_lo && pos < n_lo + nn);
    s_own[own_dim] = mine ? 3 : 1;
  }
  if (wave < G) {
    const int g = wave;
    float mstar = -INFINITY;
    for (int s_ = lane; s_ < n_all; s_ += 64) mstar = fmaxf(mstar, s_w[g * n_all + s_]);
    mstar = fa_wave_max(mstar);
    float dsum = 0.f, pmid = 0.f;
    for (int s_ = lane; s_ < n_all; s_ += 64) {
      const float m = s_w[g * n_all + s_];
      const float wgt = m == -INFINITY ? 0.f : exp2f(m - mstar);
      s_w[g * n_all + s_] = wgt;
      if (s_ < n_il) {
        dsum += wgt * s_d[g * n_all + s_];
      } else {
        pmid += wgt * s_d[g * n_all + s_];
        s_wm[g * WM + (s_ - n_il)] = wgt;
      }
    }
    dsum = fa_wave_sum(dsum);
    pmid = fa_wave_sum(pmid);
    if (lane == 0) {
      s_sc[g] = dsum + pmid;
      s_sc[kGMax + g] = pmid;
    }
  }
  __syncthreads();

  // ---- g summed over the splits, left as one row of the query heads' values per coefficient row ---------------
  if (g_on) {
    const float* wg = s_wm + g_of * WM;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    auto fold = [&](const float4& v, float wt) {
      acc.x = fmaf(wt, v.x, acc.x); acc.y = fmaf(wt, v.y, acc.y);
      acc.z = fmaf(wt, v.z, acc.z); acc.w = fmaf(wt, v.w, acc.w);
    };
#pragma unroll
    for (int u = 0; u < GPRE; u += 4) {
      if (u < WM) {   // (splits past the head's count: the clamped loads meet a weight of zero)
        const float4 w4 = *(const float4*)(wg + u);
        fold(gv[u], w4.x); fold(gv[u + 1], w4.y); fold(gv[u + 2], w4.z); fold(gv[u + 3], w4.w);
      }
    }
    for (int u = GPRE; u < n_mid; ++u) fold(*(const float4*)(gp + (int64_t)u * g_stride), wg[u]);
    // {cos f, sin f, cos f+1, sin f+1} with f = 2 * n4
    s_g[(2 * n4) * kMfG + g_of] = acc.x;
    s_g[(N + 2 * n4) * kMfG + g_of] = acc.y;
    s_g[(2 * n4 + 1) * kMfG + g_of] = acc.z;
    s_g[(N + 2 * n4 + 1) * kMfG + g_of] = acc.w;
  }
  // The loads of the last two steps go out here: their results are not needed before the products below are done,
  // and the registers of the g partials are free now.
  // sink/window partial outputs: thread = (query head, four dims, split group); needs 2 G D <= 1024
  const int QD = D >> 2;
  const int il_sg = tid & 7, il_d4 = (tid >> 3) % QD, il_g = tid / (8 * QD);
  const bool il_on = n_il > 0 && il_g < G;
  const float* ip = nullptr;
  float4 iv[kMfIlPre];
  if (il_on) {
    ip = a.il_o + (r0 + il_g) * n_il * D + 4 * il_d4;
#pragma unroll
    for (int u = 0; u < kMfIlPre; ++u) iv[u] = *(const float4*)(ip + (int64_t)min(il_sg + 8 * u, n_il - 1) * D);
  }
  // stored-dim partial outputs of the mid rows: thread = (query head, position in the share, split group), taken
  // from the far end of the block so that they do not add to the loads of the sink/window threads
  int SP = 16;
  while (SP > 1 && G * nn * SP > 1024) SP >>= 1;
  const int on_t = 1023 - tid;
  const int on_sp = on_t & (SP - 1), on_j = (on_t / SP) % max(nn, 1), on_g = on_t / (SP * max(nn, 1));
  const bool on_on = n_mid > 0 && nn > 0 && on_g < G;
  const float* op = nullptr;
  float ov[kMfOnPre];
  int on_dim = 0;
  if (on_on) {
    op = a.md_on + (r0 + on_g) * a.n_mid_stride * D + n_lo + on_j;
#pragma unroll
    for (int u = 0; u < kMfOnPre; ++u) ov[u] = op[(int64_t)min(on_sp + SP * u, n_mid - 1) * D];
    on_dim = a.vn_list[vn0 + n_lo + on_j] - h * D;
  }
  __syncthreads();

  // ---- g . V_coef: rows of this thread's class, then the classes of the wave, then the waves ------------------
  if (has_coef) {
    float4 acc[kMfG];
#pragma unroll
    for (int g = 0; g < kMfG; ++g) acc[g] = make_float4(0.f, 0.f, 0.f, 0.f);
    auto fma_row = [&](int n, const float4& v) {
      const float4 gq = *(const float4*)(s_g + n * kMfG);
      const float gg[kMfG] = {gq.x, gq.y, gq.z, gq.w};
#pragma unroll
      for (int g = 0; g < kMfG; ++g) {
        acc[g].x = fmaf(gg[g], v.x, acc[g].x); acc[g].y = fmaf(gg[g], v.y, acc[g].y);
        acc[g].z = fmaf(gg[g], v.z, acc[g].z); acc[g].w = fmaf(gg[g], v.w, acc[g].w);
      }
    };
    if (v_on) {
#pragma unroll
      for (int u = 0; u < VPRE; ++u)
        if (cls + u * classes < 2 * N) fma_row(cls + u * classes, vv[u]);
      for (int n = cls + VPRE * classes; n < 2 * N; n += classes) fma_row(n, v_load(n));
    }
    // lanes q, q + nqp, q + 2 nqp, ... of the wave hold the same dims
#pragma unroll
    for (int g = 0; g < kMfG; ++g) {
      if (g < G) {
        const float4 v = fa_sum_lane_classes(acc[g], nqp);
        if (lane < nqp) *(float4*)(s_part + (wave * kMfG + g) * CWP + 4 * lane) = v;
      }
    }
    __syncthreads();
    if (fin_on) {
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < 16; ++w) s += s_part[(w * kMfG + fin_g) * CWP + fin_j];
      s /= (float)N;
      const float pmid = s_sc[kGMax + fin_g];
      s_o[fin_g * D + fin_dim] = fin_scale * (s - fin_ad * pmid) + fin_au * pmid;
    }
  }
  // stored dims of the mid rows
  {
    float s = 0.f;
    if (on_on) {
      const float* wg = s_w + on_g * n_all + n_il;
#pragma unroll
      for (int u = 0; u < kMfOnPre; ++u)
        if (on_sp + SP * u < n_mid) s = fmaf(wg[on_sp + SP * u], ov[u], s);
      for (int sp = on_sp + SP * kMfOnPre; sp < n_mid; sp += SP) s = fmaf(wg[sp], op[(int64_t)sp * D], s);
    }
    // (the split groups of an element are neighbouring lanes)
    if (SP >= 2) s += fa_dpp<FA_DPP_XOR1>(s);
    if (SP >= 4) s += fa_dpp<FA_DPP_XOR2>(s);
    if (SP >= 8) s += fa_dpp<FA_DPP_HALF_MIRROR>(s);
    if (SP >= 16) s += fa_dpp<FA_DPP_MIRROR>(s);
    if (on_on && on_sp == 0) s_o[on_g * D + on_dim] = s;
  }
  __syncthreads();
  // ---- sink/window rows, sum, normalisation ---------------------------------------------------------------------
  {
    float4 s4 = make_float4(0.f, 0.f, 0.f, 0.f);
    if (il_on) {
      const float* wg = s_w + il_g * n_all;
      auto fold = [&](const float4& v, float wt) {
        s4.x = fmaf(wt, v.x, s4.x); s4.y = fmaf(wt, v.y, s4.y); s4.z = fmaf(wt, v.z, s4.z); s4.w = fmaf(wt, v.w, s4.w);
      };
#pragma unroll
      for (int u = 0; u < kMfIlPre; ++u)
        if (il_sg + 8 * u < n_il) fold(iv[u], wg[il_sg + 8 * u]);
      for (int sp = il_sg + 8 * kMfIlPre; sp < n_il; sp += 8) fold(*(const float4*)(ip + (int64_t)sp * D), wg[sp]);
    }
    s4 = fa_dpp4_add<FA_DPP_XOR1>(s4);
    s4 = fa_dpp4_add<FA_DPP_XOR2>(s4);
    s4 = fa_dpp4_add<FA_DPP_HALF_MIRROR>(s4);
    if (il_g < G && il_sg < 4) {   // lane il_sg writes dim 4 * il_d4 + il_sg
      const int d = 4 * il_d4 + il_sg;
      const int own = s_own[d];
      if ((own & 2) || (z == 0 && own == 0)) {
        const float mine = il_sg == 0 ? s4.x : il_sg == 1 ? s4.y : il_sg == 2 ? s4.z : s4.w;
        put((r0 + il_g) * D + d, (s_o[il_g * D + d] + mine) / s_sc[il_g]);
      }
    }
  }
}


// ---------------------------------------------------------------------------
// sink + local window, vectorised (16-bit storage, head_dim 64 or 128, 16-byte aligned rows):
// a block takes kIlFastTile rows; LPT = D/8 lanes share one row, each holding 8 dims; every wave
// issues all of its loads first, then runs an online softmax of its own; the four waves of the
// block are merged through LDS.
// ---------------------------------------------------------------------------
constexpr int kIlFastTile = 64;

template <typename E>
struct IlArgs {
  const E* q;
  Seg s0, s1;
  float* pm;
  float* pd;
  float* po;
  int Hq, Hkv, n_split;
  float sm_log2e;
};

// LDS of a sink/window block: the four waves' maxima, denominators and outputs meet here
template <int D, int GM>
struct IlFastLds {
  float m[4][GM];
  float d[4][(64 / (D / 8)) / 2][GM];
  __attribute__((aligned(16))) float o[4][(64 / (D / 8)) / 2][GM][D];
};

// bx: block index along x (tile of kIlFastTile rows); y, z come from blockIdx; lds: an IlFastLds<D, GM>
template <typename E, int D, int GM>
__device__ __forceinline__ void decode_il_fast_body(const IlArgs<E>& ia, int bx, void* lds) {
  const E* __restrict__ q = ia.q;
  const Seg s0 = ia.s0, s1 = ia.s1;
  float* __restrict__ pm = ia.pm;
  float* __restrict__ pd = ia.pd;
  float* __restrict__ po = ia.po;
  const int Hq = ia.Hq, Hkv = ia.Hkv, n_split = ia.n_split;
  const float sm_log2e = ia.sm_log2e;
  constexpr int LPT = D / 8, TPW = 64 / LPT, ITERS = kIlFastTile / 4 / TPW;
  IlFastLds<D, GM>& sh = *reinterpret_cast<IlFastLds<D, GM>*>(lds);
  auto& s_m = sh.m;
  auto& s_d = sh.d;
  auto& s_o = sh.o;
  const int G = Hq / Hkv;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
  const int sub = lane % LPT, tl = lane / LPT;
  const int split = bx, h = blockIdx.y, b = blockIdx.z;
  const int n_il = s0.rows + s1.rows;
  const int base = split * kIlFastTile + w * (kIlFastTile / 4);
  uint4 kraw[ITERS], vraw[ITERS];
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int i = base + it * TPW + tl;
    const int ii = i < n_il ? i : 0;
    const bool in0 = ii < s0.rows;
    const int64_t off = in0 ? (int64_t)b * s0.bs + (int64_t)ii * s0.rs : (int64_t)b * s1.bs + (int64_t)(ii - s0.rows) * s1.rs;
    kraw[it] = *(const uint4*)((in0 ? (const E*)s0.k : (const E*)s1.k) + off + h * D + sub * 8);
    vraw[it] = *(const uint4*)((in0 ? (const E*)s0.v : (const E*)s1.v) + off + h * D + sub * 8);
  }
  // the query slices: one unconditional 16-byte load per head (a head index past G repeats the last one)
  uint4 qraw[GM];
#pragma unroll
  for (int g = 0; g < GM; ++g)
    qraw[g] = *(const uint4*)(q + ((int64_t)b * Hq + h * G + min(g, G - 1)) * D + sub * 8);
  // (the query stays packed: the scores are sums of pair products, v_dot2c, scaled once per score)
  // The wave holds only ITERS * TPW rows, so it takes one softmax block: all scores first, one maximum,
  // then the weighted sum (no running maximum, no rescaling).
  float sc[ITERS][GM], m[GM];
#pragma unroll
  for (int g = 0; g < GM; ++g) m[g] = -INFINITY;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const bool ok = base + it * TPW + tl < n_il;
    const uint4 kr = kraw[it];
#pragma unroll
    for (int g = 0; g < GM; ++g) {
      float a = fa_dot2<E>(kr.x, qraw[g].x, 0.f);
      a = fa_dot2<E>(kr.y, qraw[g].y, a);
      a = fa_dot2<E>(kr.z, qraw[g].z, a);
      a = fa_dot2<E>(kr.w, qraw[g].w, a);
      a = fa_group_sum<LPT>(a) * sm_log2e;
      sc[it][g] = (ok && g < G) ? a : -INFINITY;
      m[g] = fmaxf(m[g], sc[it][g]);
    }
  }
#pragma unroll
  for (int g = 0; g < GM; ++g) {
    if (LPT == 8) m[g] = fmaxf(m[g], fa_dpp<FA_DPP_ROR8>(m[g]));
    m[g] = fa_rows_max(m[g]);
  }
  // The weighted sums take the query heads two at a time (the rows' V values are converted once per pair): sixteen
  // accumulators live instead of eight per head, which is what lets six waves share a SIMD.
  // Rows held side by side in the wave: lanes i and i + 32 meet in registers, the rest in LDS together with the
  // four waves.
#pragma unroll
  for (int g0 = 0; g0 < GM; g0 += 2) {
    float d[2] = {0.f, 0.f}, o[2][8];
#pragma unroll
    for (int gg = 0; gg < 2; ++gg)
#pragma unroll
      for (int e = 0; e < 8; ++e) o[gg][e] = 0.f;
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const E* ve = (const E*)&vraw[it];
      float vf[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) vf[e] = fa_to_float(ve[e]);
#pragma unroll
      for (int gg = 0; gg < 2; ++gg) {
        const int g = g0 + gg;
        const float pv = m[g] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(sc[it][g] - m[g]);
        d[gg] += pv;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[gg][e] = fmaf(pv, vf[e], o[gg][e]);
      }
    }
#pragma unroll
    for (int gg = 0; gg < 2; ++gg) {
      const int g = g0 + gg;
      float lo, hi;
      fa_swap32(d[gg], &lo, &hi);
      d[gg] = lo + hi;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        fa_swap32(o[gg][e], &lo, &hi);
        o[gg][e] = lo + hi;
      }
      if (lane < 32) {
        *(float4*)&s_o[w][tl][g][sub * 8] = make_float4(o[gg][0], o[gg][1], o[gg][2], o[gg][3]);
        *(float4*)&s_o[w][tl][g][sub * 8 + 4] = make_float4(o[gg][4], o[gg][5], o[gg][6], o[gg][7]);
        if (sub == 0) s_d[w][tl][g] = d[gg];
      }
    }
  }
  if (lane == 0) {
#pragma unroll
    for (int g = 0; g < GM; ++g) s_m[w][g] = m[g];
  }
  __syncthreads();
  for (int idx = tid; idx < G * D; idx += 256) {
    const int g = idx / D, dim = idx % D;
    const float mm = fmaxf(fmaxf(s_m[0][g], s_m[1][g]), fmaxf(s_m[2][g], s_m[3][g]));
    float acc = 0.f, dd = 0.f;
#pragma unroll
    for (int ww = 0; ww < 4; ++ww) {
      const float wgt = s_m[ww][g] == -INFINITY ? 0.f : exp2f(s_m[ww][g] - mm);
      float os = 0.f, ds = 0.f;
#pragma unroll
      for (int t = 0; t < TPW / 2; ++t) {
        os += s_o[ww][t][g][dim];
        ds += s_d[ww][t][g];
      }
      acc = fmaf(wgt, os, acc);
      dd = fmaf(wgt, ds, dd);
    }
    const int64_t r = ((int64_t)b * Hq + h * G + g) * n_split + split;
    po[r * D + dim] = acc;
    if (dim == 0) {
      pm[r] = mm;
      pd[r] = dd;
    }
  }
}

template <typename E, int D, int GM>
__global__ __launch_bounds__(256) void decode_il_fast_kernel(const IlArgs<E> ia) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[sizeof(IlFastLds<D, GM>)];
  decode_il_fast_body<E, D, GM>(ia, blockIdx.x, lds);
}

// The coefficient-domain query and the sink/window rows do not depend on each other and are both short,
// latency-bound pieces of work: one launch runs them side by side (blocks [0, n_prep) prepare the query,
// the rest attend over sink/window tiles).
template <typename E, int D, int GM, bool UPD>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(GM <= 4 ? 6 : 4, GM <= 4 ? 6 : 4)))
void decode_prep_il_kernel(const PrepArgs<E> pa, const IlArgs<E> ia, int n_prep) {
  // one buffer for whichever piece the block runs: what a block holds in LDS decides how many run side by side
  constexpr int kLds = (int)sizeof(IlFastLds<D, GM>) > kPrepLdsBytes ? (int)sizeof(IlFastLds<D, GM>) : kPrepLdsBytes;
  __shared__ __attribute__((aligned(16))) unsigned char lds[kLds];
  if ((int)blockIdx.x < n_prep) decode_prep_body<E, UPD>(pa, blockIdx.x, lds);
  else decode_il_fast_body<E, D, GM>(ia, blockIdx.x - n_prep, lds);
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
int device_cu_count() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess && n > 0)
      cus = n;
    else
      cus = 256;
  }
  return cus;
}

// which implementation handles the mid rows
enum class Path { Generic, Mfma };

struct Plan {
  Path path;
  // n_mid_split: splits the partial buffers of the mid rows have room for per head (with the matrix-core kernels the
  // heads may differ, see st; tiles_per_split then belongs to the generic kernels only)
  int n_il_split, n_mid_split, tiles_per_split, nbpg, n_groups, ks;
  int n_wg;   // matrix-core mid rows: workgroups per batch group
  fa_mfma::SplitTable st;
  int heads_per_bin;                        // > 0: the splits were shared out so that the teams fill the dies exactly
  int bin_of_head[fa_mfma::kSplitHeads];
  int n_merge_chunks;
  size_t off_W, off_c0, off_ilm, off_ild, off_ilo, off_mm, off_md, off_mg, off_mon, off_tab, off_scores, total;
  // merge after the matrix-core mid rows: contributions per block of coefficient rows, staged sums, counters
  int n_row_blocks;
  size_t off_pc, off_sil, off_son, off_cnt;
  size_t off_qn;   // stored query dims as B operands of the mid-row kernel
};

bool mfma_shape_ok(int Hq, int Hkv, int D, int N, int dtype, int layout) {
  const int G = Hq / Hkv;
  return layout == FA_MID_PAGED && (dtype == FA_BF16 || dtype == FA_FP16) && G <= 16 && D <= 128 &&
         (N == 128 || N == 256 || N == 512 || N == 1024);
}

// Splits per head of the matrix-core mid rows.  Without the per-head padded dim counts (kpad / vpad, host copies of the
// cumulative lists) every head gets the same number.  With them the same total is shared out so that the slowest
// workgroup is as fast as possible: a page of a head costs a fixed part for the coefficient-domain arithmetic (54) plus
// 1 per 1 KiB fragment of stored K dims and 3 per fragment of stored V dims (the value waves are the slower role;
// weights fitted on the kernel's time with the per-head counts of three layers of the reference's mask for
// Llama-3.1-8B), a workgroup takes ceil(pages / splits) pages, and single splits move from the head that finishes first to
// the head that finishes last while that shortens the longest time.  No head gets more than `room` splits (half as
// many again as the even share: the partial buffers are sized for that).  Returns the largest count.
// heads_per_bin > 0 (the merge may run inside the mid-row launch, whose teams must fill the dies exactly): the heads
// are put into bins of that many, expensive heads with cheap ones, and splits only move between the heads of a bin,
// so that every bin keeps heads_per_bin * ns splits; bin_of_head[h] receives the bin.  Splits that no page is left
// for are then kept (their workgroups find nothing to do).
int share_out_splits(fa_mfma::SplitTable& st, int Hkv, int tiles, int ns, int room, const int32_t* kpad, const int32_t* vpad,
                     int heads_per_bin = 0, int* bin_of_head = nullptr) {
  using fa_mfma::kSplitHeads;
  for (int h = 0; h < kSplitHeads; ++h) st.n[h] = ns;
  const bool binned = heads_per_bin > 0 && bin_of_head && Hkv <= kSplitHeads && Hkv % heads_per_bin == 0;
  if (bin_of_head)
    for (int h = 0; h < Hkv && h < kSplitHeads; ++h) bin_of_head[h] = binned ? h / heads_per_bin : -1;
  if (kpad && vpad && ns > 1 && Hkv > 1 && Hkv <= kSplitHeads) {
    int cost[kSplitHeads];
    for (int h = 0; h < Hkv; ++h) cost[h] = 54 + 2 * ((kpad[h + 1] - kpad[h]) / 32) + 3 * ((vpad[h + 1] - vpad[h]) / 16);
    auto time_of = [&](int h, int n) { return (int64_t)cost[h] * fa_cdiv(tiles, n); };
    const int n_bins = binned ? Hkv / heads_per_bin : 1;
    if (binned) {   // heads by falling cost, dealt out to the bins there and back
      int order[kSplitHeads];
      for (int h = 0; h < Hkv; ++h) order[h] = h;
      for (int i = 1; i < Hkv; ++i)
        for (int j = i; j > 0 && cost[order[j]] > cost[order[j - 1]]; --j) {
          const int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t;
        }
      for (int i = 0; i < Hkv; ++i) {
        const int pass = i / n_bins, at = i % n_bins;
        bin_of_head[order[i]] = (pass & 1) ? n_bins - 1 - at : at;
      }
    }
    for (int bin = 0; bin < n_bins; ++bin) {
      auto in_bin = [&](int h) { return !binned || bin_of_head[h] == bin; };
      for (int moves = 0; moves < ns * Hkv; ++moves) {
        int slow = -1;
        for (int h = 0; h < Hkv; ++h)
          if (in_bin(h) && (slow < 0 || time_of(h, st.n[h]) > time_of(slow, st.n[slow]))) slow = h;
        if (slow < 0 || st.n[slow] >= room) break;
        const int64_t worst = time_of(slow, st.n[slow]);
        int donor = -1;   // the head that is fastest even with one split fewer
        for (int h = 0; h < Hkv; ++h)
          if (in_bin(h) && h != slow && st.n[h] > 1 &&
              (donor < 0 || time_of(h, st.n[h] - 1) < time_of(donor, st.n[donor] - 1))) donor = h;
        if (donor < 0 || time_of(donor, st.n[donor] - 1) >= worst) break;   // nothing gained: the donor would be as slow
        // the step must shorten the longest time or leave it to another head that is no slower than before
        --st.n[donor];
        ++st.n[slow];
      }
    }
  }
  int largest = 0;
  st.first[0] = 0;
  for (int h = 0; h < kSplitHeads; ++h) {
    if (h < Hkv) {
      // (as many splits as pages of the resulting length really fill)
      const int per = fa_cdiv(tiles, st.n[h] > 0 ? st.n[h] : 1);
      if (!binned) st.n[h] = st.n[h] > 0 ? fa_cdiv(tiles, per) : 0;
      if (st.n[h] > largest) largest = st.n[h];
    }
    st.first[h + 1] = st.first[h] + (h < Hkv ? st.n[h] : 0);
  }
  return largest;
}

// kpad / vpad: see share_out_splits.  full_room: size the partial buffers for the most uneven share a call with those
// lists could ask for (the workspace query, which does not see them).
Plan make_plan(int B, int Hq, int Hkv, int D, int N, int n_il, int L_m, bool mfma, bool il_fast,
               const int32_t* kpad = nullptr, const int32_t* vpad = nullptr, bool full_room = false,
               bool fill_dies = true) {
  Plan p{};
  p.path = mfma ? Path::Mfma : Path::Generic;
  p.n_il_split = fa_cdiv(n_il, il_fast ? kIlFastTile : kTile);
  if (mfma) {
    const int G = Hq / Hkv;
    p.nbpg = 16 / G < 4 ? 16 / G : 4;       // one wave streams one batch element of the group
    if (p.nbpg > B) p.nbpg = B;
    p.n_groups = fa_cdiv(B, p.nbpg);
    p.ks = N / (16 * fa_mfma::table_slices(N));
    const int tiles = fa_cdiv(L_m, 32);
    // one workgroup per compute unit; rounded down where rounding up would leave a second round of a few workgroups
    int want = fa_cdiv(device_cu_count(), (int64_t)Hkv * p.n_groups);
    if ((int64_t)want * Hkv * p.n_groups > device_cu_count() && want > 1) --want;
    if (want < 1) want = 1;
    int ns = tiles < want ? tiles : want;
    p.tiles_per_split = ns > 0 ? fa_cdiv(tiles, ns) : 0;
    const int even = ns > 0 ? fa_cdiv(tiles, p.tiles_per_split) : 0;
    int room = fa_cdiv(3 * even, 2);
    if (room > tiles) room = tiles;
    // Teams of the launch per die, if the merge may run inside it (see fused_merge_plan): a whole number of heads of
    // one batch group, or whole batch groups
    p.heads_per_bin = 0;
    {
      const int teams = Hkv * p.n_groups;
      if (fill_dies && D == fa_mfma::kFusedD && G <= fa_mfma::kFusedG && teams % fa_mfma::kFusedXcds == 0 &&
          teams / fa_mfma::kFusedXcds < Hkv && Hkv % (teams / fa_mfma::kFusedXcds) == 0)
        p.heads_per_bin = teams / fa_mfma::kFusedXcds;
    }
    const int largest = share_out_splits(p.st, Hkv, tiles, even, room, kpad, vpad, p.heads_per_bin, p.bin_of_head);
    p.n_mid_split = full_room && Hkv > 1 && Hkv <= fa_mfma::kSplitHeads ? room : largest;
    p.n_wg = p.st.first[Hkv <= fa_mfma::kSplitHeads ? Hkv : fa_mfma::kSplitHeads];
  } else {
    const int tiles = fa_cdiv(L_m, kTile);
    int want = fa_cdiv(1024, (int64_t)B * Hkv);
    if (want < 1) want = 1;
    int ns = tiles < want ? tiles : want;
    if (ns > 64) ns = 64;
    p.tiles_per_split = ns > 0 ? fa_cdiv(tiles, ns) : 0;
    p.n_mid_split = ns > 0 ? fa_cdiv(tiles, p.tiles_per_split) : 0;
    for (int h = 0; h < fa_mfma::kSplitHeads; ++h) p.st.n[h] = p.n_mid_split;
  }
  const size_t rows = (size_t)B * Hq;
  size_t o = 0;
  auto take = [&](size_t bytes) {
    size_t at = o;
    o += fa_align_up(bytes, 256);
    return at;
  };
  // W: one row of 2N per query head; the matrix-core path keeps 16 columns per (batch group, KV head) instead
  p.off_W = take(mfma ? (size_t)p.n_groups * Hkv * 16 * 2 * N * 4 : rows * 2 * N * 4);
  p.off_c0 = take(rows * 4);
  p.off_ilm = take(rows * p.n_il_split * 4);
  p.off_ild = take(rows * p.n_il_split * 4);
  p.off_ilo = take(rows * p.n_il_split * D * 4);
  // (a single sequence on the matrix-core path may run as four sub-splits per workgroup, each with partials of its own)
  const size_t prows = mfma && B == 1 ? 4 * rows : rows;
  p.off_mm = take(prows * p.n_mid_split * 4);
  p.off_md = take(prows * p.n_mid_split * 4);
  // g partials: a row of 2N per (query head, split); the matrix-core path stores 16 columns per (batch group, KV head, split)
  p.off_mg = take((mfma ? (size_t)p.n_groups * Hkv * 16 : rows) * p.n_mid_split * 2 * N * 4);
  p.off_mon = take(prows * p.n_mid_split * D * 4);
  p.off_tab = take(mfma ? fa_mfma::tables_bytes(N) : 0);
  // merge: as many blocks per (b, KV head) as still run side by side on the device (a block fills one compute unit)
  p.n_merge_chunks = kMergeChunksMax;
  while (p.n_merge_chunks > 1 && (int64_t)B * Hkv * p.n_merge_chunks > device_cu_count()) p.n_merge_chunks >>= 1;
  // two-pass mid rows (eight frequency slices): the scores of every page travel through memory
  p.off_scores = take(mfma && fa_mfma::table_slices(N) > 4 ? (size_t)p.n_groups * Hkv * fa_cdiv(L_m, 32) * 512 * 4 : 0);
  p.n_row_blocks = mfma ? N / (kMrTiles * 8) : 0;
  {
    const size_t by_rows = (size_t)B * Hkv * p.n_row_blocks * (Hq / Hkv) * 128 * 4;
    const size_t by_team = (size_t)p.n_groups * Hkv * p.n_mid_split * 16 * 128 * 4;   // fused step
    p.off_pc = take(mfma ? (by_rows > by_team ? by_rows : by_team) : 0);
  }
  p.off_sil = take(mfma ? rows * D * 4 : 0);
  p.off_son = take(mfma ? rows * D * 4 : 0);
  p.off_cnt = take(mfma ? ((size_t)B * Hkv + (size_t)p.n_groups * Hkv * 2) * 4 : 0);
  p.off_qn = take(mfma ? (size_t)p.n_groups * Hkv * 4 * 4 * 64 * 16 : 0);
  p.total = o;
  return p;
}

bool il_fast_ok(const fa_decode_args& a) {
  if (a.dtype == FA_FP32 || (a.D != 64 && a.D != 128)) return false;
  if ((uintptr_t)a.q & 15) return false;   // query rows are read 16 bytes at a time
  for (int i = 0; i < 2; ++i) {
    if (a.il_rows[i] == 0) continue;
    if (((uintptr_t)a.k_il[i] & 15) || ((uintptr_t)a.v_il[i] & 15)) return false;
    if ((a.il_batch_stride[i] & 7) || (a.il_row_stride[i] & 7)) return false;
  }
  return true;
}

void launch_tables(void* tables, int N, int T, hipStream_t st) {
  using namespace fa_mfma;
  const int NSL = table_slices(N), KS = N / (16 * NSL);
  half8* tabE = (half8*)tables;
  half8* tabET = tabE + NSL * 2 * KS * 64;
  float2v* rot = (float2v*)(tabET + NSL * 2 * KS * 64);
  const int total = tables_entries(N) + N;
  decode_tables_kernel<<<fa_cdiv(total, 256), 256, 0, st>>>(tabE, tabET, rot, KS, T, N, NSL);
}

// The fused merge relies on the workgroups of a launch being dealt out to the dies in turn (workgroup L on die
// L % 8).  Checked once per device by a launch of the same shape that records the die of every workgroup; a device
// (or partition mode) that deals them out differently keeps the merge in a launch of its own.
static __device__ unsigned xcc_probe_out[fa_mfma::kFusedMaxWgs];
__global__ __launch_bounds__(512) void xcc_probe_kernel(unsigned* out) {
  if (threadIdx.x == 0) out[blockIdx.x] = fa_mfma::xcc_id();
}
// (set around the call by the entry point that must not allocate: the probe copies its result to pageable host memory,
// for which the runtime may set up a staging buffer; that entry point keeps the merge launch until another call has
// probed the device)
thread_local bool g_no_layout_probe = false;
bool fused_layout_ok(hipStream_t st) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static int known[kMaxDevices] = {};   // 0: not probed, 1: in turn, -1: not
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return false;
  std::lock_guard<std::mutex> lock(mu);
  if (known[dev] != 0) return known[dev] > 0;
  if (g_no_layout_probe) return false;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(st, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) return false;   // (ask again later)
  void* out = nullptr;
  unsigned host[fa_mfma::kFusedMaxWgs];
  bool ok = hipGetSymbolAddress(&out, HIP_SYMBOL(xcc_probe_out)) == hipSuccess && out;
  if (ok) {
    xcc_probe_kernel<<<fa_mfma::kFusedMaxWgs, 512, 0, st>>>((unsigned*)out);
    ok = hipMemcpyAsync(host, out, sizeof(host), hipMemcpyDeviceToHost, st) == hipSuccess &&
         hipStreamSynchronize(st) == hipSuccess;
  }
  for (int l = 0; ok && l < fa_mfma::kFusedMaxWgs; ++l) ok = host[l] == host[l % fa_mfma::kFusedXcds];
  for (int i = 0; ok && i < fa_mfma::kFusedXcds; ++i)
    for (int j = 0; j < i; ++j) ok = ok && host[i] != host[j];
  known[dev] = ok ? 1 : -1;
  return ok;
}

thread_local int g_last_call_fused = 0;   // what the last fa_decode_attn call of this thread did (a measurement aid)

// Whether the merge can run inside the mid-row launch (fa_decode_fused.h): the one-pass matrix-core pipeline, heads
// of 128 dims with at most four query heads per KV head, every workgroup of the launch resident at once (the
// workgroups of a team wait for each other), and the teams dealt out so that each sits on one die.  Fills wg_map.
bool fused_merge_plan(const fa_decode_args& a, const Plan& p, uint16_t* wg_map, hipStream_t st) {
  using namespace fa_mfma;
  if (p.path != Path::Mfma || (a.no_fuse & 1) || p.n_mid_split <= 0) return false;
  if (a.D != kFusedD || a.Hq / a.Hkv > kFusedG) return false;
  if (a.dtype != FA_BF16 && a.dtype != FA_FP16) return false;
  const int total = p.n_wg * p.n_groups, n_teams = p.n_groups * a.Hkv;
  if (total > device_cu_count() || total > kFusedMaxWgs || total % kFusedXcds != 0 || n_teams > (1 << (16 - kFusedSplitBits)))
    return false;
  if (p.n_mid_split + p.n_il_split > kFusedMaxParts || p.n_mid_split >= (1 << kFusedSplitBits)) return false;
  // a workgroup finishes ceil(R / splits) columns of its team's R = nb * G: they must belong to one batch element
  {
    const int G = a.Hq / a.Hkv;
    for (int h = 0; h < a.Hkv; ++h)
      for (int nb = p.nbpg; nb > 0; nb = (nb == p.nbpg && a.B % p.nbpg) ? a.B % p.nbpg : 0) {   // full groups, the last one
        const int per = fa_cdiv(nb * G, p.st.n[h]);
        if (per > G || G % per != 0) return false;
      }
  }
  if (!fused_layout_ok(st)) return false;
  // Workgroup L of the launch runs on die L % 8; the workgroups of die c are L = c, c + 8, c + 16, ...  Teams go
  // to the dies bin by bin (the bins the splits were shared out in, or whole batch groups), largest first otherwise.
  const int cap = total / kFusedXcds;
  int order[kFusedMaxWgs], fill[kFusedXcds] = {};
  for (int t = 0; t < n_teams; ++t) order[t] = t;
  auto size_of = [&](int t) { return p.st.n[t % a.Hkv]; };
  if (p.heads_per_bin == 0) {
    for (int i = 1; i < n_teams; ++i)   // insertion sort by size, descending, stable
      for (int j = i; j > 0 && size_of(order[j]) > size_of(order[j - 1]); --j) {
        const int tmp = order[j]; order[j] = order[j - 1]; order[j - 1] = tmp;
      }
  }
  for (int i = 0; i < n_teams; ++i) {
    const int t = order[i], n = size_of(t);
    if (n <= 0) return false;
    int c = 0;
    if (p.heads_per_bin > 0) {
      c = (t / a.Hkv) * (a.Hkv / p.heads_per_bin) + p.bin_of_head[t % a.Hkv];
      if (c >= kFusedXcds || fill[c] + n > cap) return false;
    } else {
      while (c < kFusedXcds && fill[c] + n > cap) ++c;
      if (c == kFusedXcds) return false;
    }
    for (int s = 0; s < n; ++s) wg_map[kFusedXcds * (fill[c] + s) + c] = (uint16_t)((t << kFusedSplitBits) | s);
    fill[c] += n;
  }
  return true;
}

// bytes of LDS decode_merge_fast_kernel needs for this call, 0 where it does not apply (then decode_merge_kernel runs)
static size_t merge_fast_lds(const fa_decode_args& a, const Plan& p, int G) {
  const int n_all = p.n_il_split + p.n_mid_split;
  if (p.path != Path::Mfma || p.n_mid_split <= 0 || G > kMfG || G * (a.N / 2) > 1024 || a.N % 8 != 0 || a.D % 4 != 0 ||
      2 * G * a.D > 1024 || a.D > 128 * p.n_merge_chunks || G * n_all > 1024)
    return 0;
  int nqp = 1;
  while (4 * nqp * p.n_merge_chunks < a.D) nqp <<= 1;   // the largest share of dims a head can have
  const size_t lds = ((size_t)2 * a.N * kMfG + (size_t)kMfG * ((p.n_mid_split + 3) & ~3) + (size_t)16 * kMfG * 4 * nqp +
                      2 * (size_t)G * n_all + 2 * kGMax + (size_t)G * a.D + a.D) * sizeof(float);
  return lds <= 64 * 1024 ? lds : 0;
}

// ev (optional): five events recorded before the first kernel and after each of prep (+ tables),
// mid, sink/window and merge
template <typename E>
int launch_all(const fa_decode_args& a, const Plan& p, bool p_il_fast, float sm_scale, hipStream_t st, hipEvent_t* ev) {
  if (ev) hipEventRecord(ev[0], st);
  char* ws = (char*)a.workspace;
  float* W = (float*)(ws + p.off_W);
  float* c0 = (float*)(ws + p.off_c0);
  float* ilm = (float*)(ws + p.off_ilm);
  float* ild = (float*)(ws + p.off_ild);
  float* ilo = (float*)(ws + p.off_ilo);
  float* mm = (float*)(ws + p.off_mm);
  float* md = (float*)(ws + p.off_md);
  float* mg = (float*)(ws + p.off_mg);
  float* mon = (float*)(ws + p.off_mon);
  const int G = a.Hq / a.Hkv;
  const float sm_log2e = sm_scale * kLog2e;
  Seg s0{a.k_il[0], a.v_il[0], a.il_rows[0], a.il_batch_stride[0], a.il_row_stride[0]};
  Seg s1{a.k_il[1], a.v_il[1], a.il_rows[1], a.il_batch_stride[1], a.il_row_stride[1]};
  IlArgs<E> ia{(const E*)a.q, s0, s1, ilm, ild, ilo, a.Hq, a.Hkv, p.n_il_split, sm_log2e};
  // sink/window tiles ride in the query-preparation launch when both exist and the fast tile kernel applies
  const bool fuse_il = sizeof(E) == 2 && p_il_fast && p.n_il_split > 0 && p.n_mid_split > 0;
  uint16_t wg_map[fa_mfma::kFusedMaxWgs] = {};
  // (the sink/window tiles must be in front of the mid rows for the merge to run inside that launch)
  const bool fused = sizeof(E) == 2 && (fuse_il || p.n_il_split == 0) && fused_merge_plan(a, p, wg_map, st);
  // one sequence: its mid rows as four sub-splits per workgroup in the places of four batch elements
  const bool one_pass = p.path == Path::Mfma && fa_mfma::table_slices(a.N) == 4;
  const bool sub = fused && one_pass && a.B == 1 && !(a.no_fuse & 2);
  g_last_call_fused = fused ? (sub ? 2 : 1) : 0;
  // A rank-1 update the coefficients are still owed: the query preparation applies it to the K coefficients it streams,
  // the merge inside the mid-row launch to the V coefficients; where those do not run it gets a launch of its own
  if (a.upd_k_row && a.Ck > 0 && p.n_mid_split <= 0) {
    const int rc = fa_coeff_update(const_cast<float*>(a.k_mc), a.upd_k_row, a.dtype, a.upd_batch_stride, a.kc_list, a.B, a.N,
                                   a.Ck, a.upd_phase, a.upd_T, (fa_stream_t)st);
    if (rc != FA_OK) return rc;
  }
  // (the tail of the mid-row launch reduces its phases in 32 bits)
  const bool upd_v_in_tail = fused && one_pass && a.upd_v_row && (uint64_t)a.N * (uint64_t)a.upd_T < (1ull << 32);
  if (a.upd_v_row && a.Cv > 0 && !upd_v_in_tail) {
    const int rc = fa_coeff_update(const_cast<float*>(a.v_mc), a.upd_v_row, a.dtype, a.upd_batch_stride, a.vc_list, a.B, a.N,
                                   a.Cv, a.upd_phase, a.upd_T, (fa_stream_t)st);
    if (rc != FA_OK) return rc;
  }
  if (p.n_mid_split > 0) {
    PrepArgs<E> pa{(const E*)a.q, a.k_mc, a.avg_k_u, a.avg_k_d, a.scale_k, a.kc_list, a.kc_h_list, W, c0,
                   a.Hq, a.Hkv, a.D, a.N, a.Ck, sm_log2e,
                   p.path == Path::Mfma ? W : nullptr, p.nbpg, p.path == Path::Mfma ? fa_mfma::table_slices(a.N) : 0, p.ks,
                   p.path == Path::Mfma ? (E*)(ws + p.off_qn) : nullptr, a.kn_list, a.kn_h_list,
                   fused ? (unsigned*)(ws + p.off_cnt) + (size_t)a.B * a.Hkv : nullptr, sub ? 1 : 0,
                   a.Ck > 0 ? (const E*)a.upd_k_row : nullptr, a.upd_batch_stride, a.upd_phase, a.upd_T};
    const int n_prep = fa_cdiv(2 * a.N, kPrepRows);
    if (fuse_il) {
      if constexpr (sizeof(E) == 2) {
        dim3 grid(n_prep + p.n_il_split, a.Hkv, a.B);
        if (pa.upd_row) {
          if (a.D == 128 && G <= 4) decode_prep_il_kernel<E, 128, 4, true><<<grid, 256, 0, st>>>(pa, ia, n_prep);
          else if (a.D == 128) decode_prep_il_kernel<E, 128, kGMax, true><<<grid, 256, 0, st>>>(pa, ia, n_prep);
          else if (G <= 4) decode_prep_il_kernel<E, 64, 4, true><<<grid, 256, 0, st>>>(pa, ia, n_prep);
          else decode_prep_il_kernel<E, 64, kGMax, true><<<grid, 256, 0, st>>>(pa, ia, n_prep);
        } else {
          if (a.D == 128 && G <= 4) decode_prep_il_kernel<E, 128, 4, false><<<grid, 256, 0, st>>>(pa, ia, n_prep);
          else if (a.D == 128) decode_prep_il_kernel<E, 128, kGMax, false><<<grid, 256, 0, st>>>(pa, ia, n_prep);
          else if (G <= 4) decode_prep_il_kernel<E, 64, 4, false><<<grid, 256, 0, st>>>(pa, ia, n_prep);
          else decode_prep_il_kernel<E, 64, kGMax, false><<<grid, 256, 0, st>>>(pa, ia, n_prep);
        }
      }
    } else if (pa.upd_row) {
      decode_prep_kernel<E, true><<<dim3(n_prep, a.Hkv, a.B), 256, 0, st>>>(pa);
    } else {
      decode_prep_kernel<E, false><<<dim3(n_prep, a.Hkv, a.B), 256, 0, st>>>(pa);
    }
    if (p.path == Path::Mfma) {
      if constexpr (sizeof(E) == 2) {
        using namespace fa_mfma;
        void* tables = a.tables ? (void*)a.tables : (void*)(ws + p.off_tab);
        if (!a.tables) launch_tables(tables, a.N, a.T, st);
        const int KS = p.ks;
        MidParams<E> mp{};
        mp.q = (const E*)a.q; mp.W = W; mp.c0 = c0;
        mp.k_mid = (const E*)a.k_mn; mp.v_mid = (const E*)a.v_mn;
        mp.k_bs = a.k_mn_batch_stride; mp.v_bs = a.v_mn_batch_stride; mp.cap_pages = a.mid_cap_pages;
        mp.kn_list = a.kn_list; mp.kn_h = a.kn_h_list; mp.kpad_h = a.k_pad_h_list;
        mp.vn_h = a.vn_h_list; mp.vpad_h = a.v_pad_h_list;
        mp.tabE = (const half8*)tables;
        const int NSL = table_slices(a.N);
        mp.tabET = mp.tabE + NSL * 2 * KS * 64;
        mp.rot = (const float2v*)(mp.tabET + NSL * 2 * KS * 64);
        mp.pm = mm; mp.pd = md; mp.pg = mg; mp.pon = mon;
        mp.scores = (float*)(ws + p.off_scores);
        mp.merge_count = fused ? nullptr : (unsigned*)(ws + p.off_cnt);
        if (fused) {
          auto& fz = mp.fz;
          fz.il_m = ilm; fz.il_d = ild; fz.il_o = ilo; fz.n_il = p.n_il_split;
          fz.part_c = (float*)(ws + p.off_pc);
          fz.cnt = (unsigned*)(ws + p.off_cnt) + (size_t)a.B * a.Hkv;
          fz.v_mc = a.v_mc; fz.avg_u = a.avg_v_u; fz.avg_d = a.avg_v_d; fz.scale = a.scale_v;
          fz.vc_list = a.vc_list; fz.vc_h = a.vc_h_list; fz.vn_list = a.vn_list;
          fz.out = a.out; fz.out_cast = (E*)a.out_cast; fz.Cv = a.Cv;
          fz.upd_row = a.Cv > 0 && upd_v_in_tail ? (const E*)a.upd_v_row : nullptr;
          fz.upd_bs = a.upd_batch_stride; fz.upd_T = a.upd_T;
          fz.upd_phase = a.upd_T > 0 ? (unsigned)(a.upd_phase % a.upd_T) : 0u;
          fz.wait_ticks = kTeamWaitTicks;
          memcpy(fz.wg_map, wg_map, sizeof(wg_map));
        }
        mp.q_stored = (const E*)(ws + p.off_qn);
        mp.B = a.B; mp.Hq = a.Hq; mp.Hkv = a.Hkv; mp.D = a.D; mp.G = G; mp.nbpg = p.nbpg; mp.N = a.N;
        mp.L_m = a.L_m; mp.T = a.T; mp.n_split = p.n_mid_split; mp.st = p.st;
        mp.sm_log2e = sm_log2e;
        if (ev) hipEventRecord(ev[1], st);
        const bool wide = a.mid_max_k_pad > 64 || a.mid_max_v_pad > 64;
        launch_mid_rows<E>(mp, MidLaunch{p.n_wg, p.n_groups, KS, wide, NSL > 4, fused, sub}, st);
      }
    } else {
      size_t lds = ((size_t)G * 2 * a.N + 2 * (size_t)G * a.D + (size_t)G * kTile + 4 * kGMax) * sizeof(float);
      const bool paged = a.mid_layout == FA_MID_PAGED;
      const void* fn = paged ? reinterpret_cast<const void*>(&decode_mid_kernel<E, true>)
                             : reinterpret_cast<const void*>(&decode_mid_kernel<E, false>);
      if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        FA_REQUIRE(e == hipSuccess, FA_ERR_UNSUPPORTED, "fa_decode_attn: %zu bytes of LDS refused", lds);
      }
      dim3 grid(p.n_mid_split, a.Hkv, a.B);
      if (paged)
        decode_mid_kernel<E, true><<<grid, 256, lds, st>>>(
            (const E*)a.q, (const E*)a.k_mn, a.k_mn_batch_stride, 0, (const E*)a.v_mn, a.v_mn_batch_stride, 0,
            a.mid_cap_pages, a.k_pad_h_list, a.v_pad_h_list, W, c0, a.kn_list, a.kn_h_list, a.vn_h_list, mm, md, mg,
            mon, a.Hq, a.Hkv, a.D, a.N, a.L_m, a.T, p.n_mid_split, p.tiles_per_split, sm_log2e);
      else
        decode_mid_kernel<E, false><<<grid, 256, lds, st>>>(
            (const E*)a.q, (const E*)a.k_mn, a.k_mn_batch_stride, a.k_mn_row_stride, (const E*)a.v_mn,
            a.v_mn_batch_stride, a.v_mn_row_stride, 0, nullptr, nullptr, W, c0, a.kn_list, a.kn_h_list, a.vn_h_list,
            mm, md, mg, mon, a.Hq, a.Hkv, a.D, a.N, a.L_m, a.T, p.n_mid_split, p.tiles_per_split, sm_log2e);
    }
  }
  if (ev && (p.n_mid_split == 0 || p.path != Path::Mfma)) hipEventRecord(ev[1], st);
  if (ev) hipEventRecord(ev[2], st);
  if (fused) {   // the launch above has written the output rows
    if (ev) {
      hipEventRecord(ev[3], st);
      hipEventRecord(ev[4], st);
    }
    return fa_check_launch("fa_decode_attn");
  }
  if (p.n_il_split > 0 && !fuse_il) {
    dim3 grid(p.n_il_split, a.Hkv, a.B);
    bool launched = false;
    if constexpr (sizeof(E) == 2) {
      if (p_il_fast) {
        launched = true;
        if (a.D == 128 && G <= 4) decode_il_fast_kernel<E, 128, 4><<<grid, 256, 0, st>>>(ia);
        else if (a.D == 128) decode_il_fast_kernel<E, 128, kGMax><<<grid, 256, 0, st>>>(ia);
        else if (G <= 4) decode_il_fast_kernel<E, 64, 4><<<grid, 256, 0, st>>>(ia);
        else decode_il_fast_kernel<E, 64, kGMax><<<grid, 256, 0, st>>>(ia);
      }
    }
    if (!launched) {
      size_t lds = (2 * (size_t)G * a.D + (size_t)G * kTile + 4 * kGMax) * sizeof(float);
      decode_il_kernel<E><<<grid, 256, lds, st>>>((const E*)a.q, s0, s1, ilm, ild, ilo, a.Hq, a.Hkv, a.D, p.n_il_split, sm_log2e);
    }
  }
  if (ev) hipEventRecord(ev[3], st);
  // 1024 frequencies: blocks per 128 coefficient rows read every partial once (26 against 35 us at B = 4, 130000 mid
  // rows, 32 splits); up to 512 frequencies the blocks per share of dims below are as fast or 1 us faster
  if (p.path == Path::Mfma && p.n_mid_split > 0 && a.N >= 1024) {
    const int n_all = p.n_il_split + p.n_mid_split;
    const size_t lds = (2 * (size_t)G * n_all + 2 * kGMax + (size_t)G * kMrRows + (512 * (size_t)G > 1024 ? 512 * (size_t)G : 1024) +
                        (size_t)G * a.D) * sizeof(float);
    MergeRowsArgs ma{};
    ma.il_m = ilm; ma.il_d = ild; ma.il_o = ilo; ma.n_il_split = p.n_il_split;
    ma.md_m = mm; ma.md_d = md; ma.md_g = mg; ma.md_on = mon; ma.n_mid_stride = p.n_mid_split;
    ma.v_mc = a.v_mc; ma.avg_u = a.avg_v_u; ma.avg_d = a.avg_v_d; ma.scale = a.scale_v;
    ma.vc_list = a.vc_list; ma.vc_h = a.vc_h_list; ma.vn_list = a.vn_list; ma.vn_h = a.vn_h_list;
    ma.out = a.out; ma.out_cast = a.out_cast; ma.cast_dtype = a.dtype;
    ma.part_c = (float*)(ws + p.off_pc); ma.stage_il = (float*)(ws + p.off_sil); ma.stage_on = (float*)(ws + p.off_son);
    ma.count = (unsigned*)(ws + p.off_cnt);
    ma.Hq = a.Hq; ma.Hkv = a.Hkv; ma.D = a.D; ma.N = a.N; ma.Cv = a.Cv; ma.nbpg = p.nbpg;
    ma.st = p.st;
    decode_merge_rows_kernel<<<dim3(p.n_row_blocks, a.Hkv, a.B), 256, lds, st>>>(ma);
  } else if (merge_fast_lds(a, p, G) > 0) {
    const size_t lds = merge_fast_lds(a, p, G);
    MergeRowsArgs ma{};
    ma.il_m = ilm; ma.il_d = ild; ma.il_o = ilo; ma.n_il_split = p.n_il_split;
    ma.md_m = mm; ma.md_d = md; ma.md_g = mg; ma.md_on = mon; ma.n_mid_stride = p.n_mid_split;
    ma.v_mc = a.v_mc; ma.avg_u = a.avg_v_u; ma.avg_d = a.avg_v_d; ma.scale = a.scale_v;
    ma.vc_list = a.vc_list; ma.vc_h = a.vc_h_list; ma.vn_list = a.vn_list; ma.vn_h = a.vn_h_list;
    ma.out = a.out; ma.out_cast = a.out_cast; ma.cast_dtype = a.dtype;
    ma.Hq = a.Hq; ma.Hkv = a.Hkv; ma.D = a.D; ma.N = a.N; ma.Cv = a.Cv; ma.nbpg = p.nbpg;
    ma.st = p.st;
    const dim3 grid(a.Hkv, a.B, p.n_merge_chunks);
    // (with few splits the registers go to more rows of the V coefficients per thread instead)
    if (p.n_mid_split <= 8) decode_merge_fast_kernel<8, 8><<<grid, 1024, lds, st>>>(ma);
    else decode_merge_fast_kernel<16, 4><<<grid, 1024, lds, st>>>(ma);
  } else {
    const int n_all = p.n_il_split + p.n_mid_split;
    size_t lds = ((size_t)G * 2 * a.N + 2 * (size_t)G * n_all + 2 * kGMax + 1024 * (size_t)G + (size_t)G * a.D + a.D) * sizeof(float);
    if (lds > 64 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&decode_merge_kernel),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
      FA_REQUIRE(e == hipSuccess, FA_ERR_UNSUPPORTED, "fa_decode_attn: %zu bytes of LDS refused", lds);
    }
    decode_merge_kernel<<<dim3(a.Hkv, a.B, p.n_merge_chunks), 1024, lds, st>>>(
        ilm, ild, ilo, p.n_il_split, mm, md, mg, mon, p.n_mid_split, p.st, a.v_mc, a.avg_v_u, a.avg_v_d, a.scale_v,
        a.vc_list, a.vc_h_list, a.vn_list, a.vn_h_list, a.out, a.out_cast, a.dtype, a.Hq, a.Hkv, a.D, a.N, a.Cv,
        p.path == Path::Mfma ? p.nbpg : 0);
  }
  if (ev) hipEventRecord(ev[4], st);
  return fa_check_launch("fa_decode_attn");
}

bool use_mfma(const fa_decode_args& a) {
  return a.L_m > 0 && !a.force_generic && mfma_shape_ok(a.Hq, a.Hkv, a.D, a.N, a.dtype, a.mid_layout) &&
         a.Hq / a.Hkv <= kGMax && a.mid_max_k_pad <= 128 && a.mid_max_v_pad <= 128 && a.Hkv <= fa_mfma::kSplitHeads;
}

}  // namespace

// full_room: room for the uneven shares that a call with the per-head lists on the host side may ask for
static size_t workspace_bytes_for(int B, int Hq, int Hkv, int D, int N, int il_rows_total, int L_m, bool full_room) {
  if (B <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || N < 0 || il_rows_total < 0 || L_m < 0 || Hq % Hkv) return 0;
  const int n = N > 0 ? N : 1;
  // large enough for either path
  size_t a = 0;
  for (int il_fast = 0; il_fast < 2; ++il_fast) {
    size_t b = make_plan(B, Hq, Hkv, D, n, il_rows_total, L_m, false, il_fast != 0).total;
    if (b > a) a = b;
    if (mfma_shape_ok(Hq, Hkv, D, n, FA_BF16, FA_MID_PAGED)) {
      b = make_plan(B, Hq, Hkv, D, n, il_rows_total, L_m, true, il_fast != 0, nullptr, nullptr, full_room).total;
      if (b > a) a = b;
    }
  }
  return a;
}

extern "C" size_t fa_decode_attn_workspace_bytes(int B, int Hq, int Hkv, int D, int N, int il_rows_total, int L_m) {
  return workspace_bytes_for(B, Hq, Hkv, D, N, il_rows_total, L_m, true);
}

extern "C" int fa_decode_split_plan(int B, int Hq, int Hkv, int D, int N, int il_rows_total, int L_m,
                                    const int32_t* k_pad_h_host, const int32_t* v_pad_h_host, int32_t* splits_out,
                                    int32_t* room_out) {
  FA_REQUIRE(splits_out, FA_ERR_NULL_POINTER, "fa_decode_split_plan: null pointer");
  FA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && D > 0 && N > 0 && il_rows_total >= 0 && L_m > 0 && Hq % Hkv == 0, FA_ERR_BAD_SHAPE,
             "fa_decode_split_plan: bad shape");
  FA_REQUIRE(mfma_shape_ok(Hq, Hkv, D, N, FA_BF16, FA_MID_PAGED) && Hq / Hkv <= kGMax && Hkv <= fa_mfma::kSplitHeads,
             FA_ERR_UNSUPPORTED, "fa_decode_split_plan: this shape does not take the matrix-core kernels");
  const Plan p = make_plan(B, Hq, Hkv, D, N, il_rows_total, L_m, true, true, k_pad_h_host, v_pad_h_host);
  for (int h = 0; h < Hkv; ++h) splits_out[h] = p.st.n[h];
  if (room_out) *room_out = make_plan(B, Hq, Hkv, D, N, il_rows_total, L_m, true, true, nullptr, nullptr, true).n_mid_split;
  return FA_OK;
}

extern "C" size_t fa_decode_tables_bytes(int N) { return (N > 0 && N % 64 == 0) ? fa_mfma::tables_bytes(N) : 0; }

extern "C" int fa_decode_tables_build(void* tables, size_t tables_bytes, int N, int T, fa_stream_t stream) {
  FA_REQUIRE(tables, FA_ERR_NULL_POINTER, "fa_decode_tables_build: null pointer");
  FA_REQUIRE(N > 0 && N % 64 == 0 && T > 0, FA_ERR_BAD_SHAPE, "fa_decode_tables_build: N=%d T=%d", N, T);
  FA_REQUIRE(tables_bytes >= fa_mfma::tables_bytes(N), FA_ERR_WORKSPACE, "fa_decode_tables_build: %zu < %zu bytes",
             tables_bytes, fa_mfma::tables_bytes(N));
  FA_REQUIRE(((uintptr_t)tables & 15) == 0, FA_ERR_MISALIGNED, "fa_decode_tables_build: tables not 16-byte aligned");
  launch_tables(tables, N, T, fa_hip_stream(stream));
  return fa_check_launch("fa_decode_tables_build");
}

static int decode_attn_impl(const fa_decode_args* a, fa_stream_t stream, hipEvent_t* ev) {
  FA_REQUIRE(a, FA_ERR_NULL_POINTER, "fa_decode_attn: null argument block");
  FA_REQUIRE(a->q_len == 1, FA_ERR_BAD_SHAPE, "fa_decode_attn: q_len = %d, decode needs exactly one query row", a->q_len);
  FA_REQUIRE(a->B > 0 && a->Hq > 0 && a->Hkv > 0 && a->D > 0, FA_ERR_BAD_SHAPE, "fa_decode_attn: bad B/Hq/Hkv/D");
  FA_REQUIRE(a->Hq % a->Hkv == 0, FA_ERR_BAD_SHAPE, "fa_decode_attn: Hq %d not a multiple of Hkv %d", a->Hq, a->Hkv);
  FA_REQUIRE(a->il_rows[0] >= 0 && a->il_rows[1] >= 0 && a->L_m >= 0, FA_ERR_BAD_SHAPE, "fa_decode_attn: negative row count");
  FA_REQUIRE(a->il_rows[0] + a->il_rows[1] + a->L_m > 0, FA_ERR_BAD_SHAPE, "fa_decode_attn: no keys");
  FA_REQUIRE(a->q && (a->out || a->out_cast), FA_ERR_NULL_POINTER, "fa_decode_attn: q/out null");
  FA_REQUIRE(a->dtype == FA_BF16 || a->dtype == FA_FP16 || a->dtype == FA_FP32, FA_ERR_BAD_DTYPE, "fa_decode_attn: dtype %d", a->dtype);
  for (int i = 0; i < 2; ++i)
    FA_REQUIRE(a->il_rows[i] == 0 || (a->k_il[i] && a->v_il[i]), FA_ERR_NULL_POINTER, "fa_decode_attn: il segment %d null", i);
  const int G = a->Hq / a->Hkv;
  FA_REQUIRE(G <= kGMax, FA_ERR_UNSUPPORTED, "fa_decode_attn: %d query heads per KV head (max %d)", G, kGMax);
  FA_REQUIRE(a->D <= 128, FA_ERR_UNSUPPORTED, "fa_decode_attn: head_dim %d (max 128)", a->D);
  if (a->L_m > 0) {
    FA_REQUIRE(a->N > 0 && a->T > 0, FA_ERR_BAD_SHAPE, "fa_decode_attn: N=%d T=%d", a->N, a->T);
    FA_REQUIRE(a->N <= 256 * kFreqIters, FA_ERR_UNSUPPORTED, "fa_decode_attn: N=%d (max %d)", a->N, 256 * kFreqIters);
    FA_REQUIRE(a->Ck >= 0 && a->Cv >= 0 && a->Cnk >= 0 && a->Cnv >= 0, FA_ERR_BAD_SHAPE, "fa_decode_attn: negative dim count");
    FA_REQUIRE(a->Ck + a->Cnk == a->Hkv * a->D && a->Cv + a->Cnv == a->Hkv * a->D, FA_ERR_BAD_SHAPE,
               "fa_decode_attn: compressed + stored dims must equal Hkv*D");
    FA_REQUIRE(a->kc_h_list && a->kn_h_list && a->vc_h_list && a->vn_h_list, FA_ERR_NULL_POINTER,
               "fa_decode_attn: per-head offset list null");
    FA_REQUIRE((a->Ck == 0 || a->kc_list) && (a->Cnk == 0 || a->kn_list) && (a->Cv == 0 || a->vc_list) &&
                   (a->Cnv == 0 || a->vn_list), FA_ERR_NULL_POINTER, "fa_decode_attn: index list null");
    FA_REQUIRE((a->Ck == 0 || (a->k_mc && a->avg_k_u && a->avg_k_d && a->scale_k)) &&
                   (a->Cv == 0 || (a->v_mc && a->avg_v_u && a->avg_v_d && a->scale_v)),
               FA_ERR_NULL_POINTER, "fa_decode_attn: coefficient/statistics pointer null");
    FA_REQUIRE((a->Cnk == 0 || a->k_mn) && (a->Cnv == 0 || a->v_mn), FA_ERR_NULL_POINTER, "fa_decode_attn: k_mn/v_mn null");
    FA_REQUIRE(a->mid_layout == FA_MID_TOKEN_MAJOR || a->mid_layout == FA_MID_PAGED, FA_ERR_BAD_SHAPE,
               "fa_decode_attn: mid_layout %d", a->mid_layout);
    if (a->mid_layout == FA_MID_PAGED) {
      FA_REQUIRE(a->k_pad_h_list && a->v_pad_h_list, FA_ERR_NULL_POINTER, "fa_decode_attn: padded offset list null");
      FA_REQUIRE((int64_t)a->mid_cap_pages * FA_PAGE_TOKENS >= a->L_m, FA_ERR_BAD_SHAPE,
                 "fa_decode_attn: %d mid rows beyond %d pages", a->L_m, a->mid_cap_pages);
      FA_REQUIRE(a->k_mn && a->v_mn, FA_ERR_NULL_POINTER, "fa_decode_attn: paged store null");
      FA_REQUIRE((((uintptr_t)a->k_mn | (uintptr_t)a->v_mn) & 15) == 0 && (a->k_mn_batch_stride & 7) == 0 &&
                     (a->v_mn_batch_stride & 7) == 0, FA_ERR_MISALIGNED, "fa_decode_attn: paged store not 16-byte aligned");
    }
  }
  if (a->upd_k_row || a->upd_v_row) {
    FA_REQUIRE(a->upd_T > 0 && a->upd_phase >= 0 && a->N > 0, FA_ERR_BAD_SHAPE, "fa_decode_attn: pending update with N=%d T=%d phase=%lld",
               a->N, a->upd_T, (long long)a->upd_phase);
    FA_REQUIRE(a->Ck >= 0 && a->Cv >= 0, FA_ERR_BAD_SHAPE, "fa_decode_attn: negative dim count");
    FA_REQUIRE((a->Ck == 0 || !a->upd_k_row || (a->k_mc && a->kc_list)) && (a->Cv == 0 || !a->upd_v_row || (a->v_mc && a->vc_list)),
               FA_ERR_NULL_POINTER, "fa_decode_attn: pending update without coefficients / column list");
  }
  const bool mfma = use_mfma(*a);
  const bool il_fast = il_fast_ok(*a);
  const Plan p = make_plan(a->B, a->Hq, a->Hkv, a->D, a->N > 0 ? a->N : 1, a->il_rows[0] + a->il_rows[1], a->L_m, mfma,
                           il_fast, a->k_pad_h_host, a->v_pad_h_host, false, !(a->no_fuse & 1));
  FA_REQUIRE(a->workspace && a->workspace_bytes >= p.total, FA_ERR_WORKSPACE, "fa_decode_attn: workspace %zu < %zu",
             a->workspace_bytes, p.total);
  FA_REQUIRE(((uintptr_t)a->workspace & 255) == 0, FA_ERR_MISALIGNED, "fa_decode_attn: workspace not 256-byte aligned");
  FA_REQUIRE(!a->tables || ((uintptr_t)a->tables & 15) == 0, FA_ERR_MISALIGNED, "fa_decode_attn: tables not 16-byte aligned");
  const float sm = a->sm_scale > 0.f ? a->sm_scale : 1.0f / sqrtf((float)a->D);
  hipStream_t st = fa_hip_stream(stream);
  switch (a->dtype) {
    case FA_BF16: return launch_all<bf16_t>(*a, p, il_fast, sm, st, ev);
    case FA_FP16: return launch_all<f16_t>(*a, p, il_fast, sm, st, ev);
    default: return launch_all<float>(*a, p, il_fast, sm, st, ev);
  }
}

extern "C" int fa_decode_attn(const fa_decode_args* a, fa_stream_t stream) { return decode_attn_impl(a, stream, nullptr); }

// ---- the entry point that allocates nothing -------------------------------------------------------------------
// Device memory for the partial results of one decode call (what `workspace` brings in for fa_decode_attn), held
// by every GPU the library runs on until the process ends.  In host code the array's name is a stand-in, not a
// device address: the address on the current device comes from hipGetSymbolAddress, once per device.
static __device__ __align__(256) unsigned char scratch[FA_DECODE_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

int scratch_on_current_device(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fa_set_error("fa_decode_attn_noalloc: no current device (or device index above %d)", kMaxDevices - 1);
    return FA_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      fa_set_error("fa_decode_attn_noalloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return FA_ERR_LAUNCH;
    }
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return FA_OK;
}
}  // namespace

extern "C" int fa_decode_attn_noalloc(const fa_decode_args* a, fa_stream_t stream) {
  FA_REQUIRE(a, FA_ERR_NULL_POINTER, "fa_decode_attn_noalloc: null argument block");
  // (every head the same number of splits here: the built-in buffer is not sized for uneven shares)
  const size_t need = workspace_bytes_for(a->B, a->Hq, a->Hkv, a->D, a->N, a->il_rows[0] + a->il_rows[1], a->L_m, false);
  FA_REQUIRE(need > 0, FA_ERR_BAD_SHAPE, "fa_decode_attn_noalloc: bad B/Hq/Hkv/D/N/row counts");
  FA_REQUIRE(need <= (size_t)FA_DECODE_NOALLOC_SCRATCH_BYTES, FA_ERR_WORKSPACE,
             "fa_decode_attn_noalloc: this shape needs %zu bytes of scratch, the built-in buffer holds %zu; use "
             "fa_decode_attn with a workspace of the caller's", need, (size_t)FA_DECODE_NOALLOC_SCRATCH_BYTES);
  void* ptr = nullptr;
  int rc = scratch_on_current_device(&ptr);
  if (rc != FA_OK) return rc;
  fa_decode_args b = *a;
  b.k_pad_h_host = b.v_pad_h_host = nullptr;
  b.workspace = ptr;
  b.workspace_bytes = (size_t)FA_DECODE_NOALLOC_SCRATCH_BYTES;
  g_no_layout_probe = true;
  rc = decode_attn_impl(&b, stream, nullptr);
  g_no_layout_probe = false;
  return rc;
}

extern "C" int fa_decode_attn_last_fused(void) { return g_last_call_fused; }

extern "C" int fa_decode_attn_timed(const fa_decode_args* a, fa_stream_t stream, float* ms_out) {
  FA_REQUIRE(ms_out, FA_ERR_NULL_POINTER, "fa_decode_attn_timed: ms_out null");
  hipEvent_t ev[5];
  for (int i = 0; i < 5; ++i)
    if (hipEventCreate(&ev[i]) != hipSuccess) {
      fa_set_error("fa_decode_attn_timed: hipEventCreate failed");
      return FA_ERR_LAUNCH;
    }
  int rc = decode_attn_impl(a, stream, ev);
  if (rc == FA_OK && hipEventSynchronize(ev[4]) != hipSuccess) {
    fa_set_error("fa_decode_attn_timed: hipEventSynchronize failed");
    rc = FA_ERR_LAUNCH;
  }
  if (rc == FA_OK)
    for (int i = 0; i < 4; ++i) hipEventElapsedTime(&ms_out[i], ev[i], ev[i + 1]);
  for (int i = 0; i < 5; ++i) hipEventDestroy(ev[i]);
  return rc;
}
