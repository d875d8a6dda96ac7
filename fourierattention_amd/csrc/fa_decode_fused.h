// The tail of the fused decode step: what the workgroups of the matrix-core mid-row kernel do after their last
// page when the merge runs inside the same launch (gfx950, wave64).
//
// As launches of their own, a step is [query preparation + sink/window tiles] -> mid rows -> merge, and the merge
// costs its chain of dependent loads plus the gap between two launches.  Here the workgroups of a (batch group, KV
// head) - the "team", one workgroup per split of the head's mid rows, all resident at once because the launch has
// no more workgroups than the device has compute units - finish the step themselves:
//
//   value waves   write the partials of the split (m, d, g, o_n) as before
//   meeting 1     the workgroup counts itself in and waits until the whole team has (a bounded wait)
//   merge share   split weights; the workgroup's share of the coefficient rows: g summed over the team's splits
//                 times those rows of the V coefficients (requested before the meeting) -> a partial output per
//                 column; its share of the dims of the sink/window and stored-dim partial outputs
//   meeting 2     every workgroup of the team has stored its partial output
//   column share  for its share of the team's columns the workgroup adds those partial outputs up in a fixed order,
//                 applies the column statistics, normalises and writes the output rows
//
// The workgroups of a team all run on ONE accelerator die (XCD): the hardware deals the workgroups of a launch out to
// the eight dies in turn (linear workgroup index modulo 8), and the host numbers the workgroups so that a team's
// splits share that residue.  What they hand to each other therefore meets in that die's L2 cache: plain stores
// (the vector L1 writes through), waited for before the workgroup counts itself in with an atomic that executes
// in the L2; plain loads behind the meeting (nothing of these buffers can be in the reader's L1: it is empty when
// the launch starts and the reader touches them here for the first time).  A round trip through memory with
// device scope (`sc1`) takes about 3 us on a loaded device against well under 1 us through the L2, and the tail is
// a chain of eight such trips.  (With 1024 frequencies the same tail runs behind the value pass of the two passes.)  Every workgroup adds the number of its die to the upper half of the meeting
// counter and checks the sum: a team that does not sit on one die (or a workgroup that never arrives) ends the
// wait without a result and leaves NaN rows, never plausible numbers.
#pragma once

#include "fa_mfma_util.h"
#include <type_traits>

// a . b of two pairs of 16-bit values plus c, in one instruction
typedef __bf16 fa_bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 fa_f16x2 __attribute__((ext_vector_type(2)));
template <typename E>
__device__ __forceinline__ float fa_dot2(unsigned a, unsigned b, float c);
template <>
__device__ __forceinline__ float fa_dot2<bf16_t>(unsigned a, unsigned b, float c) {
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(fa_bf16x2, a), __builtin_bit_cast(fa_bf16x2, b), c, false);
}
template <>
__device__ __forceinline__ float fa_dot2<f16_t>(unsigned a, unsigned b, float c) {
  return __builtin_amdgcn_fdot2(__builtin_bit_cast(fa_f16x2, a), __builtin_bit_cast(fa_f16x2, b), c, false);
}
template <>
__device__ __forceinline__ float fa_dot2<float>(unsigned, unsigned, float c) { return c; }   // never run: 16-bit rows only

namespace fa_mfma {

// ---- accesses that meet in the L2 of the team's die ------------------------------------------------------------
// read-modify-write executed in the L2 (returns the value before): the counters of the meetings
__device__ __forceinline__ unsigned team_atomic_add(unsigned* p, unsigned v) {
  unsigned old;
  asm volatile("global_atomic_add %0, %1, %2, off sc0\n\ts_waitcnt vmcnt(0)" : "=v"(old) : "v"(p), "v"(v) : "memory");
  return old;
}
// the die this wave runs on (HW_REG_XCC_ID, bits 3:0)
__device__ __forceinline__ unsigned xcc_id() { return __builtin_amdgcn_s_getreg(20 | (31 << 11)) & 15u; }

constexpr int kFusedMaxWgs = 256;   // workgroups of a fused launch (one per compute unit)
constexpr int kFusedXcds = 8;       // dies the workgroups of a launch are dealt out to in turn
constexpr int kFusedG = 4;          // query heads per KV head the fused tail handles (column slot = 4 * batch element + head)
constexpr int kFusedD = 128;        // head dim
constexpr int kFusedVPre = 8;       // V-coefficient rows a thread requests while it waits for the team
constexpr int kFusedTileBlock = 8;  // g tiles (8 frequencies each) summed and multiplied at a time
constexpr int kFusedGPre = 8;       // g partials (16 bytes each) a thread requests at once
constexpr int kFusedMaxParts = 120; // mid splits + sink/window tiles per query head the tail's LDS has room for
constexpr int kFusedSplitBits = 6;  // wg_map: team << 6 | split

// what the fused tail needs beyond the mid-row kernel's own parameters
template <typename E>
struct FusedParams {
  const float* il_m;  // [B * Hq][n_il]     sink/window partials, one per tile of the launch in front
  const float* il_d;
  const float* il_o;  // [B * Hq][n_il][D]
  int n_il;
  float* part_c;      // [groups][Hkv][n_split][16 column slots][128]  g . V_coef of a workgroup's coefficient rows
  unsigned* cnt;      // [groups][Hkv][2]  the two meetings; zero when the launch starts
  const float* v_mc;
  const float* avg_u;
  const float* avg_d;
  const float* scale;
  const int32_t* vc_list;
  const int32_t* vc_h;
  const int32_t* vn_list;
  float* out;         // fp32 rows and / or rows of the storage type
  E* out_cast;
  int Cv;
  // A rank-1 update the V coefficients are still owed (the row that left the window, see fa_decode_args.upd_*): the
  // thread that reads a coefficient for the row share - exactly one per coefficient - adds the row's term, writes the
  // coefficient back and multiplies with the new value.  upd_row == nullptr: nothing pending.
  const E* upd_row;
  int64_t upd_bs;
  unsigned upd_phase;   // already reduced modulo upd_T
  int upd_T;
  unsigned wait_ticks;   // bound of a meeting's wait, in ticks of the 100 MHz wall clock
  // workgroup of the launch (linear index) -> team << 6 | split, numbered so that a team shares its index modulo 8
  uint16_t wg_map[kFusedMaxWgs];
};

// One meeting of a team, in two halves so that loads can be requested in between and travel while the workgroup
// waits.  Every thread's stores must have been issued before team_count_in; it counts this workgroup in (lower half
// of the counter: workgroups; upper half: the sum of the numbers of their dies).  team_wait then waits (bounded)
// until `n` have counted in; false if the wait ran out (some workgroup of the team never arrived) or the team does
// not sit on one die.
__device__ __forceinline__ void team_count_in(unsigned* counter, int tid, unsigned* s_seen) {
  __builtin_amdgcn_s_waitcnt(0);   // vmcnt(0) expcnt(0) lgkmcnt(0): this thread's stores have reached the L2
  __syncthreads();
  if (tid == 0) {
    const unsigned inc = 1u | (xcc_id() << 16);
    *s_seen = team_atomic_add(counter, inc) + inc;
  }
}
__device__ __forceinline__ bool team_wait(unsigned* counter, unsigned n, unsigned wait_ticks, int tid, unsigned* s_seen) {
  if (tid == 0) {
    unsigned seen = *s_seen;
    const unsigned long long t0 = wall_clock64();
    while ((seen & 0xffffu) < n) {
      __builtin_amdgcn_s_sleep(2);
      if (wall_clock64() - t0 > (unsigned long long)wait_ticks) break;
      seen = team_atomic_add(counter, 0u);
    }
    *s_seen = (seen & 0xffffu) == n && (seen >> 16) == n * xcc_id();
  }
  __syncthreads();
  return *s_seen != 0;
}

// ---- the merge share (see the head of this file) -----------------------------------------------------------------
// What a workgroup of a team does behind the first meeting.  Two shares, each an even cut of the team's work:
//   rows     its tiles [t0, t1) of the N / 8 tiles of 8 frequencies (8 cosine + 8 sine coefficient rows each): g of
//            those rows summed over the team's splits, times those rows of the V coefficients of every batch element
//            of the group -> one partial output per column (every byte of g and of the V coefficients is read by
//            exactly one workgroup);
//   columns  (behind the second meeting) its columns [u_lo, u_hi) of the team's R = nb * G (unit u = batch element *
//            G + query head, the matrix-core column; all of one batch element): the partial outputs of all row shares
//            added up in a fixed order, the column statistics, the sink/window and stored-dim outputs summed over
//            their parts, normalisation, the output row.
struct FusedShare {
  int t0, t1;          // row share: tiles
  int u_lo, u_hi;      // column share
  int vc0, vc_len;     // the head's compressed V dims: offset into the lists, count
  int nqp, lq;         // groups of four compressed dims, rounded up to a power of two, and its logarithm
  int q, bbslot, rc, n_rc;   // this thread in the g . V_coef product: dim group, batch element, row class
  bool v_on;           // this thread's (dim group, batch element) exists
  int v_back;          // dims the last, incomplete group of four starts early by (its loads stay inside the head's columns)
  const float* vp;     // V coefficients of this thread's batch element at its dim group, row 0
};
// LDS of the tail, in floats: weights and denominators of the parts of sixteen column slots, their sums, g of a
// block of tiles (later the stored-dim sums of the column share), the row classes of the product (before that the
// split classes of the g sums and the sink/window sums), where each dim comes from, statistics of the compressed dims
__host__ __device__ __forceinline__ int fused_tail_lds_floats(int n_parts) { return 2 * 16 * n_parts + 32 + 2048 + 8192 + 128 + 384; }

// SUB: the team belongs to one batch element whose mid rows were cut into four sub-splits per workgroup (see the
// mid-row kernel): the sixteen column slots are (sub-split, query head), all of them multiply with the V coefficients
// of that one batch element, so the product first adds the four sub-splits of a head and the threads that would
// have taken the other batch elements take further row classes instead.
template <bool SUB, typename P>
__device__ __forceinline__ FusedShare fused_share(const P& p, int vc0, int vc_len, int split, int n_s, int b0, int nb, int KS,
                                                  int tid) {
  FusedShare f;
  const int NT = p.N / 8;   // tiles of 8 frequencies (2 KS per frequency slice)
  const int tper = (NT + n_s - 1) / n_s;
  f.t0 = min(NT, split * tper);
  f.t1 = min(NT, f.t0 + tper);
  const int R = nb * p.G;
  const int uper = (R + n_s - 1) / n_s;
  f.u_lo = min(R, split * uper);
  f.u_hi = min(R, f.u_lo + uper);
  f.vc0 = vc0;
  f.vc_len = vc_len;
  int nqp = 1, lq = 0;
  while (4 * nqp < f.vc_len) { nqp <<= 1; ++lq; }
  f.nqp = nqp;
  f.lq = lq;
  f.q = tid & (nqp - 1);
  f.bbslot = SUB ? 0 : (tid >> lq) & 3;
  f.rc = SUB ? tid >> lq : tid >> (lq + 2);
  f.n_rc = (SUB ? 512 : 128) >> lq;
  f.v_on = f.vc_len > 0 && f.bbslot < nb && 4 * f.q < f.vc_len && f.t1 > f.t0;
  // every thread reads 16 bytes per row (4-byte aligned: the head's columns start anywhere); the group that would
  // reach past the head's columns starts early instead and its values are moved down when they are used
  f.v_back = f.v_on && f.vc_len >= 4 ? max(0, 4 * f.q + 4 - f.vc_len) : 0;
  f.vp = p.fz.v_mc + (int64_t)(b0 + (f.bbslot < nb ? f.bbslot : 0)) * 2 * p.N * p.fz.Cv + f.vc0 + 4 * f.q - f.v_back;
  return f;
}
typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));
// V-coefficient row of local row r of a tile block that starts at tile tb: r = (tile * 2 + cos|sin) * 8 + frequency
__device__ __forceinline__ int fused_v_row(int tb, int r, int N) { return ((r >> 3) & 1) * N + 8 * (tb + (r >> 4)) + (r & 7); }
template <typename P>
__device__ __forceinline__ float4v fused_v_load(const P& p, const FusedShare& f, int tb, int r) {
  const float* p4 = f.vp + (int64_t)fused_v_row(tb, r, p.N) * p.fz.Cv;
  if (f.vc_len >= 4) return *(const float4u*)p4;   // (uniform over the workgroup)
  return float4v{p4[0], p4[min(1, f.vc_len - 1)], p4[min(2, f.vc_len - 1)], 0.f};   // a head with one to three such dims
}
// the values of a group that started `back` dims early, moved down to their places (the rest is never used)
__device__ __forceinline__ float4v fused_v_place(float4v v, int back) {
  if (back == 1) return float4v{v[1], v[2], v[3], 0.f};
  if (back == 2) return float4v{v[2], v[3], 0.f, 0.f};
  if (back == 3) return float4v{v[3], 0.f, 0.f, 0.f};
  return v;
}

// Called by every thread of the workgroup behind the page loops, with the workgroup's partials stored but not yet
// waited for.  P: the mid-row kernel's parameter block (pm, pd, pg, pon, n_split, shape) with the FusedParams in
// P::fz.  sm: LDS of at least fused_tail_lds_floats(n_split + n_il) floats that no wave uses any more.  KS: ksteps per
// frequency slice.  s_own: four more floats of LDS per thread (free behind the page loops as well).
template <typename E, bool SUB, bool UPD, typename P>
__device__ __forceinline__ void fused_merge_tail(const P& p, float* sm, float* s_own, int* s_flag, const FusedShare& f, int grp,
                                                 int h, int split, int n_s, int b0, int nb, int KS) {
  constexpr int D = kFusedD, GS = kFusedG;
  const int tid = threadIdx.x;
  const int G = p.G, N = p.N, NS = p.n_split, n_il = p.fz.n_il, WS = NS + n_il;
  float* s_w = sm;                    // [16 column slots][WS]: mid splits at [0, NS), sink/window tiles at [NS, NS + n_il)
  float* s_d = s_w + 16 * WS;
  float* s_sc = s_d + 16 * WS;        // [2][16]: sum of d over all parts, over the mid rows
  float* s_g = s_sc + 32;             // [128 rows][16 column slots]; later [4 classes][4 columns][128] stored-dim sums
  float* s_red = s_g + 2048;          // [row class][batch element][head][4 nqp]; before that the split classes of the g
                                      // sums, then [4 classes][4 columns][128] sink/window sums
  int* s_src = (int*)(s_red + 8192);  // [128] where dim d comes from: position in the compressed list, or 128 + position
                                      // in the stored list
  float* s_stat = (float*)(s_src + 128);   // [3][128] scale, avg_u, avg_d of the compressed dims of the column share
  unsigned* cnt = p.fz.cnt + (int64_t)(grp * p.Hkv + h) * 2;
  const int vn0 = p.vn_h[h], vn_len = p.vn_h[h + 1] - vn0;
  // column slot c16 = 4 * batch element of the group + query head; SUB: 4 * sub-split + query head, the partials of
  // sub-split j being those of the virtual batch element 4 b0 + j and the sink/window tiles belonging to slot j = 0
  auto slot_ok = [&](int c16) { return (SUB || (c16 >> 2) < nb) && (c16 & 3) < G; };
  auto qrow_of = [&](int c16) { return (int64_t)(b0 + (SUB ? 0 : c16 >> 2)) * p.Hq + h * G + (c16 & 3); };   // the query row
  auto prow_of = [&](int c16) { return (int64_t)((SUB ? 4 * b0 : b0) + (c16 >> 2)) * p.Hq + h * G + (c16 & 3); };   // its mid partials
  // column share: the columns are query heads g_lo .. g_lo + ncol - 1 of batch element cbb (the host only fuses when
  // the columns of a workgroup belong to one batch element)
  const int ncol = f.u_hi - f.u_lo, cbb = f.u_lo / G, g_lo = f.u_lo - cbb * G;
  const int c16_0 = cbb * 4 + g_lo;   // column slot of the share's first column
  const int64_t qrow0 = (int64_t)(b0 + cbb) * p.Hq + h * G + g_lo;
  const bool has_coef = f.vc_len > 0 && f.t1 > f.t0;

  // ---- meeting 1: the team's partials are complete; this workgroup's V-coefficient rows travel while it waits ----
  team_count_in(cnt, tid, (unsigned*)s_flag);
  float4v v_pre[kFusedVPre];
  if (f.v_on) {
    const int rows = 16 * min(kFusedTileBlock, f.t1 - f.t0);
#pragma unroll
    for (int u = 0; u < kFusedVPre; ++u) v_pre[u] = fused_v_load(p, f, f.t0, min(f.rc + u * f.n_rc, rows - 1));
  }
  // a pending rank-1 update of the V coefficients: this thread's four dims of the row that left the window, which of
  // the four loaded values are its own (a group that started early overlaps its neighbour's; a head with one to
  // three such dims repeats its last), and the update itself for local row r of the tile block at tb
  constexpr bool upd = UPD;   // (an instance of its own: p.fz.upd_row is set)
  int ue_own = 0;
  if (upd && f.v_on) {
    const E* ur = p.fz.upd_row + (int64_t)(b0 + f.bbslot) * p.fz.upd_bs;
    const int d0 = 4 * f.q - f.v_back;
    float4v ue;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      ue[c] = fa_to_float(ur[p.fz.vc_list[f.vc0 + min(d0 + c, f.vc_len - 1)]]);
      if (c >= f.v_back && d0 + c < f.vc_len) ue_own |= 1 << c;
    }
    *(float4v*)(s_own + 4 * tid) = ue;   // (kept in LDS until the row share: registers are scarce in between)
  }
  // (the host hands over the phase reduced modulo the period and only when N * period fits 32 bits)
  // cos or sin(2 pi n p / T) for local row r of the tile block at tb, by the hardware's sine / cosine of revolutions
  // (within 1e-7 of the library routine that fa_coeff_update calls)
  auto owed_factor = [&](int tb, int r) -> float {
    const int grow = fused_v_row(tb, r, N), fr = grow >= N ? grow - N : grow;
    const float x = (float)(((unsigned)fr * p.fz.upd_phase) % (unsigned)p.fz.upd_T) / (float)p.fz.upd_T;
    return grow >= N ? __builtin_amdgcn_sinf(x) : __builtin_amdgcn_cosf(x);
  };
  // the coefficient with the row's term added, written back where the thread owns it (no wait: nobody reads it again
  // in this launch).  Applied where the row is used, behind the meeting: the wait for the team does not start behind
  // the arrival of the rows requested ahead.
  auto owed = [&](int tb, int r, float4v v, float fct, const float4v& ue) -> float4v {
    float* wp = const_cast<float*>(f.vp) + (int64_t)fused_v_row(tb, r, N) * p.fz.Cv;
    if (ue_own == 15) {
      v = v + fct * ue;
      *(float4u*)wp = v;
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c)
        if ((ue_own >> c) & 1) {
          v[c] = v[c] + fct * ue[c];
          wp[c] = v[c];
        }
    }
    return v;
  };
  // where the dims of the head come from, and the statistics of the compressed dims of the column share
  int src_dim = -1;
  float st_scale = 0.f, st_au = 0.f, st_ad = 0.f;
  if (ncol > 0) {
    if (tid < f.vc_len) {
      src_dim = p.fz.vc_list[f.vc0 + tid] - h * D;
      const int64_t o = (int64_t)(b0 + cbb) * p.fz.Cv + f.vc0 + tid;
      st_scale = p.fz.scale[o]; st_au = p.fz.avg_u[o]; st_ad = p.fz.avg_d[o];
    } else if (tid >= 128 && tid < 128 + vn_len) {
      src_dim = p.fz.vn_list[vn0 + tid - 128] - h * D;
    }
  }
  if (!team_wait(cnt, (unsigned)n_s, p.fz.wait_ticks, tid, (unsigned*)s_flag)) {
    // some workgroup of the team never arrived, or the team is spread over several dies: no plausible numbers
    for (int idx = tid; idx < ncol * D; idx += 512) {
      const int64_t at = (qrow0 + idx / D) * D + idx % D;
      if (p.fz.out) p.fz.out[at] = __builtin_nanf("");
      if constexpr (sizeof(E) == 2)
        if (p.fz.out_cast) ((uint16_t*)p.fz.out_cast)[at] = 0x7fc0;   // a NaN in bf16 and in f16
    }
    return;
  }

  // ---- requests: everything the shares need goes out before the first result is used -----------------------------
  const int64_t g_split_floats = (int64_t)16 * 2 * N;
  const float* g_team = p.pg + (int64_t)(grp * p.Hkv + h) * NS * g_split_floats;
  // maxima and denominators of the parts (requested first: the weights are computed while the rest arrives)
  float m_raw[4], d_raw[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int idx = tid + 512 * u;
    const int c16 = idx / WS, e = idx - c16 * WS;
    m_raw[u] = -INFINITY;
    d_raw[u] = 0.f;
    if (idx < 16 * WS && slot_ok(c16)) {
      if (e < n_s) {
        m_raw[u] = p.pm[prow_of(c16) * NS + e];
        d_raw[u] = p.pd[prow_of(c16) * NS + e];
      } else if (e >= NS && (!SUB || c16 < 4)) {
        m_raw[u] = p.fz.il_m[qrow_of(c16) * n_il + (e - NS)];
        d_raw[u] = p.fz.il_d[qrow_of(c16) * n_il + (e - NS)];
      }
    }
  }
  // g partials of the first tile block: item = (tile of the block, column, pair of frequencies) = 16 bytes
  // {cos f, sin f, cos f+1, sin f+1}; the team's splits go round the split classes
  float4v gv[kFusedGPre];
  if (has_coef) {
    const int ntb = min(kFusedTileBlock, f.t1 - f.t0);
    const int n_items = 64 * ntb, n_cls = 512 / n_items;
    const int item = tid % n_items, cls = tid / n_items;
    if (cls < n_cls && ((item & 63) >> 2) < (SUB ? 4 : nb) * G) {
      const float* gp = g_team + (f.t0 + (item >> 6)) * 256 + (item & 63) * 4;
#pragma unroll
      for (int u = 0; u < kFusedGPre; ++u) gv[u] = *(const float4v*)(gp + (int64_t)min(cls + u * n_cls, n_s - 1) * g_split_floats);
    }
  }
#pragma unroll
  for (int u = 0; u < 4; ++u)
    if (tid + 512 * u < 16 * WS) {
      s_w[tid + 512 * u] = m_raw[u];
      s_d[tid + 512 * u] = d_raw[u];
    }
  if (tid < 128) s_src[tid] = 0;
  __syncthreads();
  if (src_dim >= 0) s_src[src_dim] = tid;   // compressed: position; stored: 128 + position
  if (tid < f.vc_len) {
    s_stat[tid] = st_scale;
    s_stat[128 + tid] = st_au;
    s_stat[256 + tid] = st_ad;
  }
  // Weights of the parts: thread (column slot, e), e + 32, ... takes the maximum of its own entries, the 32 lanes of
  // the column find the column's maximum with lane exchanges (a loop over all entries in every thread is a chain of
  // dependent LDS reads: 1.4 us at config 3), and each thread turns its entries into weights in place
  {
    const int c16 = tid >> 5, e0 = tid & 31;
    const float* mrow = s_w + c16 * WS;
    float mstar = -INFINITY;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = e0 + 32 * u;
      if (e < WS) {
        if constexpr (SUB) {   // one reference for the four sub-splits of the query head
#pragma unroll
          for (int j = 0; j < 4; ++j) mstar = fa_fmax(mstar, s_w[(4 * j + (c16 & 3)) * WS + e]);
        } else {
          mstar = fa_fmax(mstar, mrow[e]);
        }
      }
    }
    mstar = fa_fmax(mstar, fa_dpp<FA_DPP_XOR1>(mstar));
    mstar = fa_fmax(mstar, fa_dpp<FA_DPP_XOR2>(mstar));
    mstar = fa_fmax(mstar, fa_dpp<FA_DPP_HALF_MIRROR>(mstar));
    mstar = fa_fmax(mstar, fa_dpp<FA_DPP_MIRROR>(mstar));
    {
      float lo, hi;
      fa_swap16(mstar, &lo, &hi);
      mstar = fa_fmax(lo, hi);
    }
    float wgt[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = e0 + 32 * u;
      const float mv = e < WS ? mrow[e] : -INFINITY;
      wgt[u] = mv == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mv - mstar);
    }
    // the column's denominators (all parts / the mid rows alone): sums over the 32 lanes of the column
    float den = 0.f, pmid = 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int e = e0 + 32 * u;
      if (e < WS) {
        const float t = wgt[u] * s_d[c16 * WS + e];
        den += t;
        if (e < NS) pmid += t;
      }
    }
    den = fa_group_sum<16>(den);
    pmid = fa_group_sum<16>(pmid);
    float lo, hi;
    fa_swap16(den, &lo, &hi); den = lo + hi;
    fa_swap16(pmid, &lo, &hi); pmid = lo + hi;
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (e0 + 32 * u < WS) s_w[c16 * WS + e0 + 32 * u] = wgt[u];
    if (e0 == 0) {
      s_sc[c16] = den;
      s_sc[16 + c16] = pmid;
    }
  }
  __syncthreads();

  // column share: sink/window partial outputs, thread = (four dims, class of parts, column); stored dims likewise by
  // position in the head's list
  constexpr int kPre = 5;
  const int x_d4 = tid & 31, x_cls = (tid >> 5) & 3, x_cl = tid >> 7;
  float4v il_pre[kPre], on_pre[kPre];
  const bool il_on = n_il > 0 && x_cl < ncol;
  const float* il_src = p.fz.il_o + (qrow0 + x_cl) * n_il * D + 4 * x_d4;
  if (il_on) {
#pragma unroll
    for (int u = 0; u < kPre; ++u) il_pre[u] = *(const float4v*)(il_src + (int64_t)min(x_cls + 4 * u, n_il - 1) * D);
  }
  // (SUB: class j takes all splits of sub-split j, whose partials are those of virtual batch element 4 b0 + j - up to
  // 32 of them, a chain of dependent loads if one thread walks them all.  A workgroup with one or two columns has
  // threads for four: the spare ones help, thread column x_cl working for column x_cl % ncol on every on_h-th split.)
  const int on_h = (SUB && (ncol == 1 || ncol == 2)) ? 4 / ncol : 1;
  const int on_col = on_h > 1 ? x_cl % ncol : x_cl, on_hlp = on_h > 1 ? x_cl / ncol : 0;
  const bool on_on = on_col < ncol && 4 * x_d4 < vn_len;
  const int on_first = SUB ? on_hlp : x_cls, on_step = SUB ? on_h : 4;
  const int on_slot = SUB ? 4 * x_cls + c16_0 + on_col : c16_0 + on_col;
  const float* on_src = p.pon + (SUB ? prow_of(on_slot) : qrow0 + on_col) * NS * D + 4 * x_d4;
  if (on_on) {
#pragma unroll
    for (int u = 0; u < kPre; ++u) on_pre[u] = *(const float4v*)(on_src + (int64_t)min(on_first + on_step * u, n_s - 1) * D);
  }
  // ---- row share: g over the team's splits, times the V coefficients -----------------------------------------------
  float4v acc[GS];
#pragma unroll
  for (int g = 0; g < GS; ++g) acc[g] = float4v{0.f, 0.f, 0.f, 0.f};
  if (has_coef) {
    const bool ragged = (f.vc_len & 3) != 0;   // (uniform: only then some group of four started early)
    float4v ue = float4v{0.f, 0.f, 0.f, 0.f};
    if (upd && f.v_on) ue = *(const float4v*)(s_own + 4 * tid);
    for (int tb = f.t0; tb < f.t1; tb += kFusedTileBlock) {
      const int ntb = min(kFusedTileBlock, f.t1 - tb);
      const int n_items = 64 * ntb, n_cls = 512 / n_items;
      const int item = tid % n_items, cls = tid / n_items;
      const int tl = item >> 6, rem = item & 63, lc = rem >> 2, lgp = rem & 3;
      const int c16 = (lc / G) * 4 + (lc % G);
      if (tb > f.t0) __syncthreads();   // the block before is done with s_g and s_red
      const bool col_ok = lc < (SUB ? 4 : nb) * G;   // (columns past the group hold nothing; their slots of s_g are never read)
      auto put_g = [&](const float4v& a4) {
        const int rb = tl * 16 + 2 * lgp;
        s_g[rb * 16 + c16] = a4[0]; s_g[(rb + 8) * 16 + c16] = a4[1];
        s_g[(rb + 1) * 16 + c16] = a4[2]; s_g[(rb + 9) * 16 + c16] = a4[3];
      };
      if (cls < n_cls && col_ok) {
        const float* wg = s_w + c16 * WS;
        const float* gp = g_team + (tb + tl) * 256 + rem * 4;
        float4v a4 = float4v{0.f, 0.f, 0.f, 0.f};
        int s0 = cls;
        if (tb == f.t0) {
#pragma unroll
          for (int u = 0; u < kFusedGPre; ++u)
            if (cls + u * n_cls < n_s) a4 += gv[u] * wg[cls + u * n_cls];
          s0 = cls + kFusedGPre * n_cls;
        }
        for (; s0 < n_s; s0 += 4 * n_cls) {
          float4v v[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) v[u] = *(const float4v*)(gp + (int64_t)min(s0 + u * n_cls, n_s - 1) * g_split_floats);
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (s0 + u * n_cls < n_s) a4 += v[u] * wg[s0 + u * n_cls];
        }
        if (n_cls > 1) *(float4v*)(s_red + (cls * n_items + item) * 4) = a4;
        else put_g(a4);
      }
      if (n_cls > 1) {
        __syncthreads();
        if (cls == 0 && col_ok) {
          float4v a4 = *(const float4v*)(s_red + item * 4);
          for (int c = 1; c < n_cls; ++c) a4 += *(const float4v*)(s_red + (c * n_items + item) * 4);
          put_g(a4);
        }
      }
      __syncthreads();
      if (f.v_on) {
        const int rows = 16 * ntb;
        auto fma_row = [&](int r, float4v v) {
          if (ragged) v = fused_v_place(v, f.v_back);
          float4v gq = *(const float4v*)(s_g + r * 16 + f.bbslot * 4);
          if constexpr (SUB)   // the four sub-splits of a query head meet here
            gq = (gq + *(const float4v*)(s_g + r * 16 + 4)) + (*(const float4v*)(s_g + r * 16 + 8) + *(const float4v*)(s_g + r * 16 + 12));
#pragma unroll
          for (int g = 0; g < GS; ++g) acc[g] += v * gq[g];
        };
        int r = f.rc;
        if (tb == f.t0) {   // the rows requested ahead
#pragma unroll
          for (int u = 0; u < kFusedVPre; ++u)
            if (f.rc + u * f.n_rc < rows) {
              // (opaque here: otherwise every way fused_v_place can move these rows is worked out ahead of the loop
              // and held in registers)
              asm volatile("" : "+v"(v_pre[u]));
              if (upd) {
                int tbo = tb;   // (opaque as well: the factors are not to be worked out ahead of the loop either)
                asm volatile("" : "+s"(tbo));
                v_pre[u] = owed(tbo, f.rc + u * f.n_rc, v_pre[u], owed_factor(tbo, f.rc + u * f.n_rc), ue);
              }
              fma_row(f.rc + u * f.n_rc, v_pre[u]);
            }
          r = f.rc + kFusedVPre * f.n_rc;
        }
        for (; r < rows; r += 4 * f.n_rc) {
          float4v v[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) v[u] = fused_v_load(p, f, tb, min(r + u * f.n_rc, rows - 1));
#pragma unroll
          for (int u = 0; u < 4; ++u)
            if (r + u * f.n_rc < rows) {
              if (upd) v[u] = owed(tb, r + u * f.n_rc, v[u], owed_factor(tb, r + u * f.n_rc), ue);
              fma_row(r + u * f.n_rc, v[u]);
            }
        }
      }
    }
  }
  __syncthreads();   // s_red held the split classes of the last block; s_g is free
  // column share: sink/window outputs summed over their tiles, by class -> s_red; stored dims -> s_g
  {
    float4v a4 = float4v{0.f, 0.f, 0.f, 0.f};
    if (il_on) {
      const float* wg = s_w + (c16_0 + x_cl) * WS + NS;
#pragma unroll
      for (int u = 0; u < kPre; ++u)
        if (x_cls + 4 * u < n_il) a4 += il_pre[u] * wg[x_cls + 4 * u];
      for (int sp = x_cls + 4 * kPre; sp < n_il; sp += 4) a4 += *(const float4v*)(il_src + (int64_t)sp * D) * wg[sp];
    }
    *(float4v*)(s_red + ((x_cls * 4 + x_cl) * 32 + x_d4) * 4) = a4;
    a4 = float4v{0.f, 0.f, 0.f, 0.f};
    if (on_on) {
      const float* wg = s_w + on_slot * WS;
#pragma unroll
      for (int u = 0; u < kPre; ++u)
        if (on_first + on_step * u < n_s) a4 += on_pre[u] * wg[on_first + on_step * u];
      for (int sp = on_first + on_step * kPre; sp < n_s; sp += on_step) a4 += *(const float4v*)(on_src + (int64_t)sp * D) * wg[sp];
    }
    *(float4v*)(s_g + ((x_cls * 4 + x_cl) * 32 + x_d4) * 4) = a4;
  }
  __syncthreads();
  // this thread's output element of the column share: thread = (column, dim); the sink/window part of it
  const int o_cl = tid >> 7, o_d = tid & 127;
  float o_val = (s_red[((0 * 4 + o_cl) * 32) * 4 + o_d] + s_red[((1 * 4 + o_cl) * 32) * 4 + o_d]) +
                (s_red[((2 * 4 + o_cl) * 32) * 4 + o_d] + s_red[((3 * 4 + o_cl) * 32) * 4 + o_d]);
  const int o_src = s_src[o_d];
  if (o_src >= 128) {   // a stored dim: its sum (over the classes, and over the helpers of the column)
    const int jj = o_src - 128;
    for (int hh = 0; hh < on_h; ++hh) {
      const int sl = min(o_cl + hh * ncol, 3);
      o_val += (s_g[((0 * 4 + sl) * 32) * 4 + jj] + s_g[((1 * 4 + sl) * 32) * 4 + jj]) +
               (s_g[((2 * 4 + sl) * 32) * 4 + jj] + s_g[((3 * 4 + sl) * 32) * 4 + jj]);
    }
  }
  __syncthreads();
  // the row classes of the product meet -> the row share's partial output per column, by position in the head's list
  float* pc_team = p.fz.part_c + (int64_t)(grp * p.Hkv + h) * NS * 16 * 128;
  if (has_coef) {
    if (f.v_on) {
#pragma unroll
      for (int g = 0; g < GS; ++g) *(float4v*)(s_red + ((f.rc * (SUB ? 1 : 4) + f.bbslot) * GS + g) * 4 * f.nqp + 4 * f.q) = acc[g];
    }
    __syncthreads();
    float* pc = pc_team + (int64_t)split * 16 * 128;
    // (SUB: the row classes hold four slots each, those of the query heads)
    constexpr int kSlots = SUB ? 4 : 16;
    const int n_out = kSlots * f.nqp;
    // the row classes [r0, r1) of one output (column slot, four dims) added up: four reads in flight, fixed order
    // (the number of classes is a power of two, at least four)
    auto class_sum = [&](int c16, int q, int r0, int r1) -> float4v {
      float4v a4 = float4v{0.f, 0.f, 0.f, 0.f};
      for (int rc = r0; rc < r1; rc += 4) {
        float4v t[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) t[u] = *(const float4v*)(s_red + ((rc + u) * kSlots + c16) * 4 * f.nqp + 4 * q);
        a4 += (t[0] + t[1]) + (t[2] + t[3]);
      }
      return a4;
    };
    // A head with few compressed dims has few outputs and many row classes (256 for eight dims of a single sequence):
    // one thread per output walking them all is a chain of n_rc / 4 LDS round trips, 6 us there.  Then the classes are
    // added up in `parts` pieces by as many threads per output, and the pieces by one (through s_g, free by now).
    const int parts = f.n_rc >= 256 ? 16 : f.n_rc >= 64 ? 8 : f.n_rc >= 32 ? 4 : 1;
    if (parts == 1) {
      for (int idx = tid; idx < n_out; idx += 512) {
        const int c16 = idx >> f.lq, q = idx & (f.nqp - 1);
        if (4 * q < f.vc_len && slot_ok(c16)) *(float4v*)(pc + c16 * 128 + 4 * q) = class_sum(c16, q, 0, f.n_rc);
      }
    } else {
      const int per = f.n_rc / parts;
      const int o = tid & (n_out - 1), part = tid / n_out;   // (parts * n_out <= n_rc / 4 * n_out = 512)
      const int c16 = o >> f.lq, q = o & (f.nqp - 1);
      const bool live = 4 * q < f.vc_len && slot_ok(c16);
      if (part < parts && live) *(float4v*)(s_g + (part * n_out + o) * 4) = class_sum(c16, q, part * per, (part + 1) * per);
      __syncthreads();
      if (part == 0 && live) {
        float4v a4 = float4v{0.f, 0.f, 0.f, 0.f};
        for (int pp = 0; pp < parts; pp += 4) {
          float4v t[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) t[u] = *(const float4v*)(s_g + ((pp + u) * n_out + o) * 4);
          a4 += (t[0] + t[1]) + (t[2] + t[3]);
        }
        *(float4v*)(pc + c16 * 128 + 4 * q) = a4;
      }
    }
  }

  // ---- meeting 2: every row share of the team is out -------------------------------------------------------------
  team_count_in(cnt + 1, tid, (unsigned*)s_flag);
  if (!team_wait(cnt + 1, (unsigned)n_s, p.fz.wait_ticks, tid, (unsigned*)s_flag)) return;   // (cannot happen behind meeting 1)
  // ---- column share: the output element -------------------------------------------------------------------------------
  if (o_cl < ncol) {
    if (o_src < 128) {
      const int NT = N / 8, tper = (NT + n_s - 1) / n_s;
      const int n_blocks = (NT + tper - 1) / tper;   // workgroups of the team that own coefficient rows
      const float* src = pc_team + (c16_0 + o_cl) * 128 + o_src;
      float sum = 0.f;
      for (int z0 = 0; z0 < n_blocks; z0 += 16) {   // sixteen loads in flight, added in the order of the workgroups
        float t[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) t[u] = src[(int64_t)min(z0 + u, n_blocks - 1) * 16 * 128];
#pragma unroll
        for (int u = 0; u < 16; ++u)
          if (z0 + u < n_blocks) sum += t[u];
      }
      float pmid = s_sc[16 + c16_0 + o_cl];
      if constexpr (SUB) pmid = (pmid + s_sc[20 + c16_0 + o_cl]) + (s_sc[24 + c16_0 + o_cl] + s_sc[28 + c16_0 + o_cl]);
      o_val += s_stat[o_src] * (sum * (1.0f / (float)N) - s_stat[256 + o_src] * pmid) + s_stat[128 + o_src] * pmid;
    }
    float den = s_sc[c16_0 + o_cl];
    if constexpr (SUB) den = (den + s_sc[4 + c16_0 + o_cl]) + (s_sc[8 + c16_0 + o_cl] + s_sc[12 + c16_0 + o_cl]);
    o_val *= 1.0f / den;
    const int64_t at = (qrow0 + o_cl) * D + o_d;
    if (p.fz.out) p.fz.out[at] = o_val;
    if constexpr (sizeof(E) == 2) {
      if (p.fz.out_cast) {
        if constexpr (std::is_same<E, bf16_t>::value) p.fz.out_cast[at] = bf16_t{fa_f32_to_bf16_bits(o_val)};
        else p.fz.out_cast[at] = E{(_Float16)o_val};
      }
    }
  }
}

}  // namespace fa_mfma
