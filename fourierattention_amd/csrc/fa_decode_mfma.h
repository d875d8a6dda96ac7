// MFMA path of decode attention over the mid rows (gfx950, wave64).
//
// One workgroup (8 waves, two per SIMD, 256 VGPRs each) owns one KV head, one group of batch
// elements whose query rows fill the 16 MFMA columns (R = nb * G <= 16), and one contiguous
// range of 32-token pages.  Per page:
//
//   scores  S[32 x 16] = E[32 x 2N] . W'[2N x 16]      (f16 MFMA; E = cos/sin of the token offset
//                        + K_mn[32 x dims] . Q_n        from the centre of the frame, W' = coefficient-domain
//                                                        query rotated to that centre)
//   softmax P = exp2(S - m)                              (online, base 2)
//   g'[2N x 16] += E^T[2N x 32] . P                      (f16 MFMA, accumulated in the frame of the
//                                                        current pair of pages)
//   o_n[dims x 16] += V_mn^T[dims x 32] . P              (bf16 / f16 MFMA on the stored dims)
//
// Frames.  Two pages share one frame whose centre lies half a token before the first token of the second
// page: its tokens sit at the offsets +(i + 1/2), those of the first page at -(i + 1/2), i = 0 .. 31.  Cosine is
// even and sine is odd, so ONE constant operand E (offsets i + 1/2) serves both pages, and so does one product:
// with C = E_cos . W'_cos and S = E_sin . W'_sin (cosine and sine ksteps in separate accumulators) the scores of
// the second page are C + S and those of the first ("mirrored") page C - S, row i being token 31 - i there; g of
// the frame takes E_cos^T (P2 + P1) and E_sin^T (P2 - P1), P1 / P2 being the probabilities of the first and of
// the second page.  The coefficient-domain products are thus issued once per frame, and W' and the g history are
// rotated once per frame (64 tokens), not once per page.  On a mirrored page every
// position-indexed quantity (score partials in LDS, probabilities) is held in the mirrored order; the K and V
// pages come into LDS through per-lane addresses, so fetching a K fragment with its 16 rows reversed (and the two
// 16-token blocks exchanged) or a V fragment with its four groups of 8 tokens exchanged costs nothing.
//
// The 2N coefficient rows are split four ways; slice i belongs to score wave i (E, W') and to
// value wave i (E^T, g'), which share a SIMD.  The score waves work one page ahead of the value
// waves; the partial scores cross through LDS with one barrier per page.  Waves i and 4 + i also
// stream the stored K resp. V dims of batch element i of the group.  K/V pages arrive as
// ready-made MFMA A operands (see the page layout in the public header).
#pragma once

#include "fa_mfma_util.h"
#include "fa_decode_fused.h"
#include <type_traits>

namespace fa_mfma {

constexpr int kPart = 36;  // padded row (tokens) of the LDS score partials, floats

// frequency owned by (kstep s, lane group lg, register v) of the score GEMM's K dimension and by
// (row tile rt = 2s + v/2, lane group lg, pair v%2) of the g GEMM's rows: per lane the same set
__device__ __forceinline__ int freq_of(int rt, int lg, int fi2) { return rt * 8 + lg * 2 + fi2; }

constexpr float kLazyLog2 = 8.0f;   // slack of the running softmax reference, in powers of two
constexpr int kFreqWaves = 4;  // the coefficient rows are split four ways (one slice per SIMD)
constexpr int kScoreFrames = 4;  // value pass: frames (two pages) of scores a workgroup keeps in LDS

// ---------------------------------------------------------------------------
// constant operand tables (depend on T and N only); KS = N / (16 * slices) ksteps per frequency slice
//   tabE  [slices][2 row blocks][KS][64 lanes] x half8 : A operand of the score GEMM, row i = offset i + 1/2; kstep
//         2j holds the cosines and kstep 2j + 1 the sines of the frequencies of the row tiles 4j .. 4j + 3
//   tabET [slices][2*KS tiles][64 lanes] x half8 : A operand of the g GEMM; tile 2j holds the cosines and tile
//         2j + 1 the sines of the 16 frequencies 16j .. 16j + 15 of the slice (row = frequency), columns = the
//         offsets i + 1/2
//   rot   [N] float2 : (cos, sin)(2 pi f 64 / T), the rotation from one frame to the next
// Half-token offsets: phase f (2i + 1) / (2T), reduced exactly in integers.
// ---------------------------------------------------------------------------
static __global__ __launch_bounds__(256) void decode_tables_kernel(half8* __restrict__ tabE, half8* __restrict__ tabET,
                                                            float2v* __restrict__ rot, int KS, int T, int N, int NSL) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  const int nE = NSL * 2 * KS * 64, nET = NSL * 2 * KS * 64;
  if (idx < nE) {
    const int lane = idx & 63, s = (idx >> 6) % KS, rb = ((idx >> 6) / KS) & 1, w = (idx >> 6) / (2 * KS);
    const int lg = lane >> 4, lc = lane & 15;
    const int i = rb * 16 + lc;
    // kstep s = 2j + cs: the cosines (cs = 0) or the sines (cs = 1) of the eight frequencies of the row tiles
    // 4j .. 4j + 3 that this lane group owns
    const int j = s >> 1, cs = s & 1;
    half8 out;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int f = w * 16 * KS + freq_of(4 * j + (e >> 1), lg, e & 1);
      float sn, co;
      fa_sincos_phase(f, 2 * i + 1, 2 * T, &sn, &co);
      out[e] = (_Float16)(cs ? sn : co);
    }
    tabE[idx] = out;
  } else if (idx < nE + nET) {
    const int k = idx - nE;
    const int lane = k & 63, tile = (k >> 6) % (2 * KS), w = (k >> 6) / (2 * KS);
    const int lg = lane >> 4;
    const int f = w * 16 * KS + 16 * (tile >> 1) + (lane & 15);
    const int cs = tile & 1;
    half8 out;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float sn, co;
      fa_sincos_phase(f, 2 * (8 * lg + e) + 1, 2 * T, &sn, &co);
      out[e] = (_Float16)(cs ? sn : co);
    }
    tabET[k] = out;
  } else if (idx < nE + nET + N) {
    const int f = idx - nE - nET;
    float sn, co;
    fa_sincos_phase(f, 64, T, &sn, &co);
    rot[f] = float2v{co, sn};
  }
}

// frequency slices: four (one per SIMD, score and value wave of a slice side by side) up to N = 512; eight for
// N = 1024, whose per-wave state only fits when a pass runs one role on all eight waves
static inline int table_slices(int N) { return N > 512 ? 8 : 4; }
static inline int tables_entries(int N) {
  const int NSL = table_slices(N), KS = N / (16 * NSL);
  return 2 * NSL * 2 * KS * 64;   // half8 operands of tabE and tabET together
}
static inline size_t tables_bytes(int N) { return (size_t)tables_entries(N) * 16 + (size_t)N * 8; }


// ---- frame-to-frame rotation of coefficient-domain state ---------------------------------------------------
// Both wave roles turn 2*KS row tiles of (cos, sin) pairs by the per-frequency angle of one frame (64 tokens).  The
// constants sit in LDS as float4 {c, s, c', s'} per (row tile, lane group), 64 bytes between row tiles.
// They are fetched in batches of four tiles, two batches in flight, so that the LDS latency hides behind
// the arithmetic of the previous batch instead of being paid once per tile.
template <int BATCH>
__device__ __forceinline__ void rot_issue(unsigned lane_base, uint4v (&buf)[4]) {
  buf[0] = lds_read_b128_async_at<(BATCH * 4 + 0) * 64>(lane_base);
  buf[1] = lds_read_b128_async_at<(BATCH * 4 + 1) * 64>(lane_base);
  buf[2] = lds_read_b128_async_at<(BATCH * 4 + 2) * 64>(lane_base);
  buf[3] = lds_read_b128_async_at<(BATCH * 4 + 3) * 64>(lane_base);
}
// the same, issued only once `after` has been computed: keeps a refill of a constant buffer behind the
// arithmetic that consumed its previous contents (otherwise all batches are hoisted and held at once)
template <int BATCH>
__device__ __forceinline__ void rot_issue_after(unsigned lane_base, uint4v (&buf)[4], float after) {
  asm volatile("ds_read_b128 %0, %1 offset:%3 ; after %2" : "=v"(buf[0]) : "v"(lane_base), "v"(after), "n"((BATCH * 4 + 0) * 64));
  asm volatile("ds_read_b128 %0, %1 offset:%3 ; after %2" : "=v"(buf[1]) : "v"(lane_base), "v"(after), "n"((BATCH * 4 + 1) * 64));
  asm volatile("ds_read_b128 %0, %1 offset:%3 ; after %2" : "=v"(buf[2]) : "v"(lane_base), "v"(after), "n"((BATCH * 4 + 2) * 64));
  asm volatile("ds_read_b128 %0, %1 offset:%3 ; after %2" : "=v"(buf[3]) : "v"(lane_base), "v"(after), "n"((BATCH * 4 + 3) * 64));
}
__device__ __forceinline__ void rot_pair(float c, float s, float& x, float& y) {
  const float sy = s * y, sx = s * x;
  x = __builtin_fmaf(c, x, sy);
  y = __builtin_fmaf(c, y, -sx);
}
// The same for the four pairs of two row tiles with the results in the registers of the operands.  State that lives
// across loop iterations in plain registers (not in accumulators of the matrix unit) is otherwise left wherever the
// last instruction of a rotation put it, and every iteration ends with one move per value to bring the registers
// back in order.  Four pairs per statement: the compiler separates every asm statement from what follows by a
// wait state, so one statement per pair would cost as many idle issue slots as it saves moves.
// k0, k1: {c, s, c', s'} of the two row tiles; x*, y*: (cos-row, sin-row) values of the pairs (tile, 0), (tile, 1).
__device__ __forceinline__ void rot_two_tiles_in_place(uint4v k0, uint4v k1, float& x00, float& y00, float& x01, float& y01,
                                                       float& x10, float& y10, float& x11, float& y11) {
  const unsigned c00 = k0[0], s00 = k0[1], c01 = k0[2], s01 = k0[3];   // scalars first: see fa_swap16
  const unsigned c10 = k1[0], s10 = k1[1], c11 = k1[2], s11 = k1[3];
  float t0, t1;
  asm volatile(
      "v_mul_f32 %0, %11, %3\n\tv_mul_f32 %1, %11, %2\n\tv_fma_f32 %2, %10, %2, %0\n\tv_fma_f32 %3, %10, %3, -%1\n\t"
      "v_mul_f32 %0, %13, %5\n\tv_mul_f32 %1, %13, %4\n\tv_fma_f32 %4, %12, %4, %0\n\tv_fma_f32 %5, %12, %5, -%1\n\t"
      "v_mul_f32 %0, %15, %7\n\tv_mul_f32 %1, %15, %6\n\tv_fma_f32 %6, %14, %6, %0\n\tv_fma_f32 %7, %14, %7, -%1\n\t"
      "v_mul_f32 %0, %17, %9\n\tv_mul_f32 %1, %17, %8\n\tv_fma_f32 %8, %16, %8, %0\n\tv_fma_f32 %9, %16, %9, -%1"
      : "=&v"(t0), "=&v"(t1), "+v"(x00), "+v"(y00), "+v"(x01), "+v"(y01), "+v"(x10), "+v"(y10), "+v"(x11), "+v"(y11)
      : "v"(c00), "v"(s00), "v"(c01), "v"(s01), "v"(c10), "v"(s10), "v"(c11), "v"(s11));
}
// The page-step rotation of the 2*KS row tiles held in x[rt][f2], y[rt][f2] with that helper; the first two batches
// of constants must be in flight in rc[0], rc[1]
template <int NT, int B>
__device__ __forceinline__ void rot_apply_in_place_from(unsigned lane_base, uint4v (&rc)[2][4], float (&x)[NT][2], float (&y)[NT][2]) {
  constexpr int NB = NT / 4;
  if constexpr (B < NB) {
    if (B + 1 < NB) lds_wait_for4<4>(rc[B % 2]);
    else lds_wait_for4<0>(rc[B % 2]);
    rot_two_tiles_in_place(rc[B % 2][0], rc[B % 2][1], x[4 * B][0], y[4 * B][0], x[4 * B][1], y[4 * B][1],
                           x[4 * B + 1][0], y[4 * B + 1][0], x[4 * B + 1][1], y[4 * B + 1][1]);
    rot_two_tiles_in_place(rc[B % 2][2], rc[B % 2][3], x[4 * B + 2][0], y[4 * B + 2][0], x[4 * B + 2][1], y[4 * B + 2][1],
                           x[4 * B + 3][0], y[4 * B + 3][0], x[4 * B + 3][1], y[4 * B + 3][1]);
    if constexpr (B + 2 < NB) rot_issue_after<B + 2>(lane_base, rc[B % 2], y[4 * B + 3][1]);
    rot_apply_in_place_from<NT, B + 1>(lane_base, rc, x, y);
  }
}
// pair(rt, f2, c, s) applies one rotation and returns one of its results; pin(b) passes the results of
// batch b (row tiles 4b .. 4b+3) through an empty asm volatile, which keeps their arithmetic above the
// next wait (it is otherwise sunk to its uses, and every batch of constants is then held at once);
// the first NBUF batches must already be in flight in rc[0 .. NBUF-1] (NBUF = 2 hides the LDS latency of a batch
// behind the arithmetic of the one before; NBUF = 1 saves 16 registers and pays the latency)
template <int NT, int NBUF, int B, typename F, typename P>
__device__ __forceinline__ void rot_apply_from(unsigned lane_base, uint4v (&rc)[NBUF][4], F&& pair, P&& pin) {
  constexpr int NB = NT / 4;
  if constexpr (B < NB) {
    if (NBUF == 2 && B + 1 < NB) lds_wait_for4<4>(rc[B % NBUF]);
    else lds_wait_for4<0>(rc[B % NBUF]);
    float last = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint4v raw = rc[B % NBUF][j];
      const unsigned c0 = raw[0], s0 = raw[1], c1 = raw[2], s1 = raw[3];  // scalars first: see fa_swap16
      pair(B * 4 + j, 0, __builtin_bit_cast(float, c0), __builtin_bit_cast(float, s0));
      last = pair(B * 4 + j, 1, __builtin_bit_cast(float, c1), __builtin_bit_cast(float, s1));
    }
    pin(B);
    if constexpr (B + NBUF < NB) rot_issue_after<B + NBUF>(lane_base, rc[B % NBUF], last);
    rot_apply_from<NT, NBUF, B + 1>(lane_base, rc, pair, pin);
  }
}
template <int NT, int NBUF, typename F, typename P>
__device__ __forceinline__ void rot_apply(unsigned lane_base, uint4v (&rc)[NBUF][4], F&& pair, P&& pin) {
  rot_apply_from<NT, NBUF, 0>(lane_base, rc, pair, pin);
}

// Wait until at most AHEAD pages of PER * n fragment loads each are still in flight (n is uniform over the wave,
// 1 .. NMAX; the count of the wait instruction is an immediate, hence one branch per possible value).
template <int AHEAD, int NMAX, int PER, int F = 1>
__device__ __forceinline__ void wait_pages_in_flight(int n) {
  if constexpr (AHEAD == 0) {
    wait_vmcnt<0>();
  } else if constexpr (F >= NMAX) {
    wait_vmcnt<AHEAD * PER * NMAX>();
  } else {
    if (n == F) wait_vmcnt<AHEAD * PER * F>();
    else wait_pages_in_flight<AHEAD, NMAX, PER, F + 1>(n);
  }
}

// The mid rows of KV head h are cut into n[h] splits (heads that store more dims take longer per page and get more);
// the workgroups of one batch group are numbered head by head, first[h] being the first one of head h.
constexpr int kSplitHeads = 64;
struct SplitTable {
  int n[kSplitHeads];
  int first[kSplitHeads + 1];
};

template <typename E>
struct MidParams {
  const E* q;
  const E* q_stored;    // the stored query dims as B operands: [batch group][KV head][batch element, 4][kstep, 4][lane] x 8
  const float* W;       // fp32, already carrying sm_scale*log2e/N, in the lane layout of the score waves:
                        // [batch group][KV head][slice][row tile][cos | sin][column][pair of frequencies] x float2
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
  float* scores;   // two-pass mode: [groups][Hkv][pages][16 columns][32 tokens] fp32
  unsigned* merge_count;   // [B][Hkv] counters of the merge launch behind this one: cleared here
  int B, Hq, Hkv, D, G, nbpg, N, L_m, T;
  int n_split;   // splits the partial buffers have room for per head (the largest n[h])
  float sm_log2e;
  SplitTable st;
  FusedParams<E> fz;   // the fused merge only (FUSE instances of the kernel)
};

// The workgroup is a two-stage pipeline over the pages of its split, one barrier per page:
//   waves 0-3 ("score waves")  page t+1: S partial = E . W' (their frequency slice; the product itself on the first
//                              page of a frame, see above) + K_mn . Q_n (their batch element) -> LDS; after the second
//                              page of a frame, W' moves on to the next frame
//   waves 4-7 ("value waves")  page t  : sum the four partials, online softmax, before the first page of a frame
//                              rotate the g history into it, rescale, on the second page g' += E^T . (P2 +- P1)
//                              (their frequency slice), on both o_n += V_mn^T . P (their batch element)
// Pages at an even distance from the first page of the split are the mirrored pages of their frames.
// Score wave i and value wave i own the same frequencies and stream the same batch element of the group.
// KS: ksteps (32 coefficient rows) per slice = N / (16 * slices).  KMAX: ksteps of stored K dims a head may have
// (dp_k / 32).  VMAX: V dim groups of 16 (dp_v / 16).
// NST: page stages per wave in LDS; the K / V pages travel HBM -> LDS with global_load_lds (no registers
// held while in flight), NST - 1 pages ahead of their use.
// MODE 0: the fused pipeline above (N <= 512).  For N = 1024 a wave cannot hold twice the state, so the work is cut
// into two passes over the same pages, each running ONE role on all eight waves (eight frequency slices):
// MODE 1, scores: eight partials per page meet in LDS, their sum (the complete score of the page) goes to
//         memory (2 KiB per page and workgroup, against 16 KiB of K/V);
// MODE 2, values: every wave reads the page's scores back, runs the softmax and keeps its slice of the g
//         history; waves 0-3 stream V, waves 4-7 bring the scores of a frame into LDS for all eight; one meeting
//         per frame.
// FUSE (MODE 0 and the value pass, MODE 2): the launch merges its own partials and writes the output rows, see fa_decode_fused.h; the
// workgroups are then numbered through p.fz.wg_map so that the splits of a (batch group, KV head) share one die.
// SUB (FUSE only, a batch of one sequence, at most four query heads per KV head): a single batch element would
// leave twelve of the sixteen matrix-core columns and three of the four page streams of a workgroup idle.  The
// workgroup's pages are cut into four sub-splits instead, which take the places of four batch elements: wave i
// streams the pages of sub-split i, column 4 j' + g (j' = sub-split, as a batch element would be) holds query head g
// with its weights W' rotated to the first frame of sub-split j', and every column keeps its own softmax reference,
// g history and outputs, i.e. each sub-split ends as a partial result of its own ("virtual batch element" j' of the
// partial buffers).  The page loop has a quarter of the trips.  Pages past the end of a sub-split are fetched from a
// valid page and masked.
// UPD (FUSE only): the tail also applies a pending rank-1 update to the V coefficients of its row share.
template <typename E, int KS, int KMAX, int VMAX, int NST, int MODE = 0, bool FUSE = false, bool SUB = false, bool UPD = false>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void decode_mid_mfma_kernel(
    const MidParams<E> p) {
  static_assert(!FUSE || MODE == 0 || MODE == 2, "the fused merge runs behind the one-pass pipeline or behind the value pass");
  static_assert(!SUB || MODE == 0, "sub-splits belong to the one-pass pipeline");
  static_assert(!UPD || MODE == 0, "the pending update keeps its row in the LDS of the score partials");
  static_assert(!SUB || FUSE, "sub-splits end in the fused merge");
  static_assert(!UPD || FUSE, "the pending update rides in the fused merge");
  constexpr int NSL = MODE == 0 ? kFreqWaves : 2 * kFreqWaves;   // frequency slices
  using M = Mma<E>;
  using vec8 = typename M::vec8;
  constexpr int kFragsMax = (2 * KMAX > VMAX ? 2 * KMAX : VMAX);   // fragments (1 KiB) of one page of one wave
  // in the two-pass modes only waves 0-3 stream pages
  __shared__ __attribute__((aligned(16))) unsigned char s_stage[MODE == 0 ? 8 : 4][NST][kFragsMax * 1024];
  __shared__ float s_part[MODE == 2 ? 1 : 2][MODE == 2 ? 1 : NSL][16 * kPart];
  // value pass: the scores of a page travel like its V fragments, memory -> LDS without registers (two fragments per
  // page: positions 8 lg .. 8 lg + 3 and 8 lg + 4 .. 8 lg + 7 of column lc at lane * 16), so that the only accesses
  // to vector memory inside the loop are page requests, whose arrival can be counted.  One copy per workgroup, frame
  // by frame: waves 4-7, which stream no V, bring one of the frame's four fragments each, and the workgroup meets
  // once per frame.
  __shared__ __attribute__((aligned(16))) unsigned char s_sc[MODE == 2 ? kScoreFrames : 1][MODE == 2 ? 4096 : 16];
  // frame-to-frame rotation constants, float4 = (c, s) of two neighbouring frequencies, [slice][unit][lane group]:
  // for the score waves unit = row tile rt, frequencies freq_of(rt, lg, 0 / 1); for the value waves unit u covers
  // the frequencies 16 (u / 2) + 4 lg + 2 (u % 2) + 0 / 1, the rows 4 lg + 2 (u % 2) + 0 / 1 of tile pair u / 2
  __shared__ float4v s_rot[MODE == 2 ? 1 : NSL * 2 * KS * 4];
  __shared__ float4v s_rotv[MODE == 1 ? 1 : NSL * 2 * KS * 4];
  __shared__ int s_team_flag;
  const int tid = threadIdx.x, lane = tid & 63, lg = lane >> 4, lc = lane & 15;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps role and page addressing scalar
  const bool score_wave = MODE == 0 ? w < kFreqWaves : MODE == 1;
  const int sl = MODE == 0 ? (w & 3) : w;  // frequency slice; below 4 also the batch element of the group
  // workgroup -> (batch group, KV head, split of that head)
  int grp = blockIdx.y, h = 0, split = 0;
  if constexpr (FUSE) {
    const int code = p.fz.wg_map[blockIdx.x];   // (a one-dimensional grid)
    const int team = code >> kFusedSplitBits;
    grp = team / p.Hkv;
    h = team - grp * p.Hkv;
    split = code & ((1 << kFusedSplitBits) - 1);
  } else {
    // (the first sixteen entries are compared at once: they arrive with one load of the argument block, where a
    // scan waits for one dependent load per head)
#pragma unroll
    for (int i = 1; i < 16; ++i) h += (int)blockIdx.x >= p.st.first[i] ? 1 : 0;
    if (p.Hkv > 16)
      while (h + 1 < p.Hkv && (int)blockIdx.x >= p.st.first[h + 1]) ++h;
    split = blockIdx.x - p.st.first[h];
  }
  const int G = p.G, N = p.N;
  const int b0 = grp * p.nbpg;
  const int nb_real = min(p.nbpg, p.B - b0);
  const int nb = SUB ? 4 : nb_real;   // SUB: four sub-splits of the one batch element in the places of batch elements
  const int R = nb * G;
  const bool valid_r = lc < R;
  const int bb_r = lc / G, g_r = lc - bb_r * G;
  // the query row of this lane's column; the row of its partial results (SUB: virtual batch element 4 b + sub-split)
  const int64_t qrow = valid_r ? ((int64_t)(b0 + (SUB ? 0 : bb_r)) * p.Hq + h * G + g_r) : 0;
  const int64_t prow = !SUB ? qrow : valid_r ? ((int64_t)(b0 * 4 + bb_r) * p.Hq + h * G + g_r) : 0;
  if (MODE != 1 && split == 0 && tid < nb_real && p.merge_count) p.merge_count[(b0 + tid) * p.Hkv + h] = 0u;
  const int fbase = sl * 16 * KS;
  const bool has_mn = sl < nb && sl < kFreqWaves;
  const int my_b = b0 + (has_mn && !SUB ? sl : 0);
  const int stw = has_mn ? w & 3 : 0;   // page stage of this wave

  const int n_tiles = (p.L_m + 31) >> 5;
  const int tiles_per_split = (n_tiles + p.st.n[h] - 1) / p.st.n[h];
  const int t_beg = split * tiles_per_split;
  const int t_end = min(n_tiles, t_beg + tiles_per_split);
  const int n_pages = t_end > t_beg ? t_end - t_beg : 0;
  // trips of the page loop; SUB: a quarter of the pages per sub-split, the sub-split of this wave (wave-uniform) and
  // of this lane's column start at page w_beg / c_beg of the split, and the column's has c_n pages
  const int n_it = SUB ? (n_pages + 3) >> 2 : n_pages;
  const int w_beg = SUB ? min(n_pages, (w & 3) * n_it) : 0;
  const int c_beg = SUB ? min(n_pages, min(bb_r, 3) * n_it) : 0;
  const int c_n = SUB ? min(n_pages, c_beg + n_it) - c_beg : n_pages;
  const int t_beg_w = t_beg + w_beg;
  // fused merge: the head's compressed V dims (offset into the lists, count), needed behind the page loop
  int fz_vc0 = 0, fz_vc_len = 0;
  if constexpr (FUSE) {
    fz_vc0 = p.fz.vc_h[h];
    fz_vc_len = p.fz.vc_h[h + 1] - fz_vc0;
  }

  // Rotation constants of slice sl into LDS: one entry (unit, lane group) per lane, requested early and stored once
  // the other loads of the prologue are on their way.  Every wave stores the constants it reads itself (in the
  // order of its own role), so no wave waits for another one here.
  float4v rot_c = float4v{0.f, 0.f, 0.f, 0.f};
  const bool rot_lane_ok = lane < 2 * KS * 4;
  auto rot_fetch = [&]() {
    if (rot_lane_ok) {
      const int u = lane >> 2, ulg = lane & 3;
      // even: (c, s)(f), (c, s)(f + 1) are 16 aligned bytes
      const int f = fbase + (score_wave ? freq_of(u, ulg, 0) : 16 * (u >> 1) + 4 * ulg + 2 * (u & 1));
      rot_c = *(const float4v*)&p.rot[f];
    }
  };
  auto rot_store = [&]() {
    if (rot_lane_ok) {
      if (score_wave) s_rot[(MODE == 2 ? 0 : sl * 2 * KS) * 4 + lane] = rot_c;
      else s_rotv[(MODE == 1 ? 0 : sl * 2 * KS) * 4 + lane] = rot_c;
    }
    asm volatile("" ::: "memory");   // the reads of these constants are asm statements the compiler cannot order
  };
  // per-lane element offsets of a fragment load: as stored, with the 16 rows of a K fragment reversed, with the four
  // token groups of a V fragment exchanged
  const int lane_nat = lane * 8, lane_krev = (lg * 16 + 15 - lc) * 8, lane_vrev = ((3 - lg) * 16 + lc) * 8;

  if (score_wave) {
    // =============================== score waves ===============================
    // stored K dims of batch element sl: both 16-token blocks of the page
    const int kp0 = p.kpad_h[h], dpk = p.kpad_h[h + 1] - kp0;
    const int nks = dpk >> 5;
    const E* kbase = p.k_mid + (int64_t)my_b * p.k_bs + (int64_t)kp0 * 32 * p.cap_pages;  // wave-uniform
    const bool has_k = has_mn && nks > 0;
    // a page moves the fragments the head really has
    // (mirrored page: token 31 - i becomes row i, i.e. the blocks change places and their rows are reversed)
    auto issue_k = [&](int t, bool mir) {   // page t -> stage (t - t_beg_w) % NST
      const int tp = SUB ? min(t, n_tiles - 1) : t;   // (a page past the sub-split: any valid page, masked later)
      const E* kp = kbase + (int64_t)tp * dpk * 32 + (mir ? lane_krev : lane_nat);
      unsigned char* st = &s_stage[MODE == 0 ? w : stw][(t - t_beg_w) % NST][0];
#pragma unroll
      for (int tb = 0; tb < 2; ++tb)
#pragma unroll
        for (int ks = 0; ks < KMAX; ++ks)
          if (ks < nks) load_frag_to_lds<2>(kp + ((mir ? 1 - tb : tb) * nks + ks) * 512, st + (tb * KMAX + ks) * 1024);
    };
    rot_fetch();
    half8 Ea[2][KS];

    // coefficient-domain query: Wc/Ws[rt][f2] = (cos-row, sin-row) weights of frequency
    // freq_of(rt, lg, f2) for column lc; normalised per column, rotated to the centre of the first frame
    float Wc[2 * KS][2], Ws[2 * KS][2];
    float wmax = 0.f;
    // the stored query dims of this wave's batch element, laid out as B operands by the launch in front (zeros in
    // the lanes of other batch elements and past the head's count): requested behind the weights
    vec8 Qb[KMAX];
    {
      // (SUB: every sub-split starts from the weights of its query head, column g of the one batch element)
      const float2v* wl = (const float2v*)p.W + ((int64_t)((grp * p.Hkv + h) * NSL + sl) * 2 * KS * 2) * 64 + ((SUB ? g_r : lc) * 4 + lg);
      float2v wc2[2 * KS], ws2[2 * KS];
#pragma unroll
      for (int rt = 0; rt < 2 * KS; ++rt) {
        wc2[rt] = wl[(rt * 2 + 0) * 64];
        ws2[rt] = wl[(rt * 2 + 1) * 64];
      }
      // the table operand goes out behind the weights: loads return in order, so the arithmetic on the weights
      // below runs while the (four times larger) table is still arriving
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int s = 0; s < KS; ++s) Ea[rb][s] = p.tabE[((sl * 2 + rb) * KS + s) * 64 + lane];
      {
        const vec8* qs = (const vec8*)p.q_stored + ((int64_t)((grp * p.Hkv + h) * 4 + stw) * 4) * 64 + lane;
#pragma unroll
        for (int s = 0; s < KMAX; ++s) Qb[s] = qs[s * 64];   // used by waves that stream K pages only
      }
      // The first pages go out behind the operand loads: loads return in order, and a first access to a page of
      // the store takes about twice as long as the operands, which the weights below would otherwise wait for.
      if (has_k) {
#pragma unroll
        for (int i = 0; i < NST - 1; ++i)
          if (i < n_it) issue_k(t_beg_w + i, (i & 1) == 0);
      }
#pragma unroll
      for (int rt = 0; rt < 2 * KS; ++rt) {
        float2v c2 = wc2[rt], s2 = ws2[rt];
        if (!valid_r) c2 = s2 = float2v{0.f, 0.f};   // lanes of columns past the group hold nothing
        Wc[rt][0] = c2[0]; Wc[rt][1] = c2[1];
        Ws[rt][0] = s2[0]; Ws[rt][1] = s2[1];
        wmax = fa_fmax(fa_fmax(fa_fmax(fa_fmax(wmax, fabsf(c2[0])), fabsf(c2[1])), fabsf(s2[0])), fabsf(s2[1]));
      }
    }
    wmax = fa_rows_max(wmax);
    // power-of-two scale per column and frequency slice (the partial scores are rescaled in fp32 before they
    // are summed): keeps the f16 operand in [-1, 1] without rounding
    const float colscale = wmax > 0.f ? exp2f(ceilf(log2f(wmax))) : 1.f;
    const float colinv = 1.0f / colscale;
    const float c0col = (valid_r && sl == 0) ? p.c0[qrow] : 0.f;
    {
      // phases of the first frame centre (token 32 (t_beg + 1) - 1/2, as a count of half tokens against 2T): exact
      // for row tile 0, then stepped by the (exact) phase of 8 frequencies
      const int64_t c2 = (int64_t)64 * (t_beg + c_beg + 1) - 1;   // (SUB: of the column's sub-split)
      float sn[2], co[2], s8, c8;
      fast_sincos_phase(8, c2, 2 * p.T, &s8, &c8);
#pragma unroll
      for (int f2 = 0; f2 < 2; ++f2) fast_sincos_phase(fbase + freq_of(0, lg, f2), c2, 2 * p.T, &sn[f2], &co[f2]);
#pragma unroll
      for (int rt = 0; rt < 2 * KS; ++rt)
#pragma unroll
        for (int f2 = 0; f2 < 2; ++f2) {
          const float wc = Wc[rt][f2] * colinv, ws = Ws[rt][f2] * colinv;
          Wc[rt][f2] = co[f2] * wc + sn[f2] * ws;    // rotation by -phi: W'c = cos(phi) wc + sin(phi) ws
          Ws[rt][f2] = -sn[f2] * wc + co[f2] * ws;   //                   W's = -sin(phi) wc + cos(phi) ws
          const float cn = co[f2] * c8 - sn[f2] * s8;
          sn[f2] = sn[f2] * c8 + co[f2] * s8;
          co[f2] = cn;
        }
    }

    // every table and weight load above must have landed before the loop starts: inside it the only
    // waits on vector memory in this wave are the explicit page waits
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) asm volatile("" ::"v"(Ea[rb][ks]));
    rot_store();
    const unsigned rot_lane = lds_addr_of(&s_rot[(MODE == 2 ? 0 : sl * 2 * KS) * 4 + lg]);
    // score pass: the complete scores of page pg of the split (sum of the eight partials; index = (column, token))
    // go to memory.  Called one page late, behind that page's barrier, and carried out by waves 4-7 alone, two
    // values per thread: they stream no pages, so waves 0-3 have nothing but page requests in flight and can count
    // them (loads and stores do not complete in one order).
    auto flush_scores = [&](int pg) {
      if constexpr (MODE == 1) {
        if (w >= 4) {
          constexpr int kW = 16 * kPart * 4;   // bytes between the partials of two waves
          const int i0 = tid - 256;            // columns 0 .. 7; the second value belongs to column + 8
          const unsigned at = lds_addr_of(&s_part[pg & 1][0][(i0 >> 5) * kPart + (i0 & 31)]);
          const float sum0 = lds_sum8_b32<kW>(at);
          const float sum1 = lds_sum8_b32<kW>(at + 8 * kPart * 4);
          float* dst = p.scores + ((int64_t)(grp * p.Hkv + h) * n_tiles + t_beg + pg) * 512 + i0;
          dst[0] = sum0;
          dst[256] = sum1;
        }
      }
    };

    // coefficient-domain part of the scores of a frame: C = sum over the cosine ksteps, S = over the sine ksteps.
    // Computed on the first (mirrored) page of the frame, whose rows are C - S; the second page's are C + S.
    float4v accC[2], accS[2];
    // one trip of the score pipeline: page `it` of the split (none on the trip after the last page)
    auto score_trip = [&](int it, auto mirrored_tag) {
      constexpr bool mirrored = decltype(mirrored_tag)::value;   // first page of its frame
      if (it < n_it) {
        const int t = t_beg_w + it;
        uint4v kraw[4];   // two ksteps of both token blocks at a time
        const unsigned kst = lds_addr_of(&s_stage[MODE == 0 ? w : stw][it % NST][0]) + lane * 16;
        uint4v rc[2][4];
        if (has_k) {
          // pages t+1 .. t+NST-2 may still be in flight; page t has landed: start its LDS reads now
          if (it + NST - 2 < n_it) wait_pages_in_flight<NST - 2, KMAX, 2>(nks);   // (two fragments per kstep)
          else wait_vmcnt<0>();
          // refills the stage read one page ago
          if (it + NST - 1 < n_it) issue_k(t + NST - 1, mirrored == (((NST - 1) & 1) == 0));
        }
        // The results of these reads arrive later (the wait is tied to them further down); until then no
        // instruction may touch their registers.  A read under a condition makes the compiler merge its result
        // with the other path, which it may do by copying the registers at once: where that happened the reads
        // are issued by every wave (a wave without pages reads its idle stage and drops the result).
        if (MODE != 0 || has_k) {
          // ksteps 0, 1: issued early, consumed after the coefficient-domain product
          kraw[0] = lds_read_b128_async_at<0>(kst);
          kraw[1] = lds_read_b128_async_at<1024>(kst);
          kraw[2] = lds_read_b128_async_at<KMAX * 1024>(kst);
          kraw[3] = lds_read_b128_async_at<(KMAX + 1) * 1024>(kst);
        }
        {
          // (the trip number goes through an empty asm statement: a condition the compiler can resolve for the
          // first trip makes it peel that trip, and the peeled copy of the loop body costs registers)
          int it_seen = it;
          asm volatile("" : "+s"(it_seen));
          if (it_seen > 0) flush_scores(it - 1);   // behind the page wait: the store has a whole page to complete
        }
        if constexpr (!mirrored) {
          rot_issue<0>(rot_lane, rc[0]);
          if (2 * KS > 4) rot_issue<1>(rot_lane, rc[1]);
        }
        float4v cd[2];   // coefficient-domain part of this page's scores, scaled, with the constant term
        if constexpr (mirrored) {
          accC[0] = accC[1] = accS[0] = accS[1] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int j = 0; j < KS / 2; ++j) {
            half8 wbc, wbs;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              wbc[e] = (_Float16)Wc[4 * j + (e >> 1)][e & 1];
              wbs[e] = (_Float16)Ws[4 * j + (e >> 1)][e & 1];
            }
            accC[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ea[0][2 * j], wbc, accC[0], 0, 0, 0);
            accC[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ea[1][2 * j], wbc, accC[1], 0, 0, 0);
            accS[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ea[0][2 * j + 1], wbs, accS[0], 0, 0, 0);
            accS[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ea[1][2 * j + 1], wbs, accS[1], 0, 0, 0);
          }
        }
        // offsets -(i + 1/2) on the mirrored page: the sines change sign
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
          cd[rb] = (mirrored ? accC[rb] - accS[rb] : accC[rb] + accS[rb]) * colscale + c0col;
        // behind the second page of a frame: W' moves on to the centre of the next frame
        if constexpr (!mirrored) rot_apply_in_place_from<2 * KS, 0>(rot_lane, rc, Wc, Ws);
        float4v accm[2] = {float4v{0.f, 0.f, 0.f, 0.f}, float4v{0.f, 0.f, 0.f, 0.f}};
        if (has_k) {
#pragma unroll
          for (int s0 = 0; s0 < KMAX; s0 += 2) {
            if (s0 > 0) {
              if (s0 >= nks) break;
              kraw[0] = lds_read_b128_async_at<0>(kst + s0 * 1024);
              kraw[1] = lds_read_b128_async_at<1024>(kst + s0 * 1024);
              kraw[2] = lds_read_b128_async_at<KMAX * 1024>(kst + s0 * 1024);
              kraw[3] = lds_read_b128_async_at<(KMAX + 1) * 1024>(kst + s0 * 1024);
            }
            lds_wait_for4<0>(kraw);
#pragma unroll
            for (int ss = 0; ss < 2; ++ss)
              if (s0 + ss < nks) {
                accm[0] = M::mma(__builtin_bit_cast(vec8, kraw[ss]), Qb[s0 + ss], accm[0]);
                accm[1] = M::mma(__builtin_bit_cast(vec8, kraw[2 + ss]), Qb[s0 + ss], accm[1]);
              }
          }
        }
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
          float4v o;
#pragma unroll
          for (int v = 0; v < 4; ++v) o[v] = cd[rb][v] + accm[rb][v] * p.sm_log2e;
          *(float4v*)&s_part[it & 1][sl][lc * kPart + rb * 16 + 4 * lg] = o;
        }
      } else if (n_it > 0) {   // (the trip after the last page)
        flush_scores(it - 1);
      }
      if (MODE == 0 || it < n_it) barrier_lds_only();
    };
    for (int it = 0; it <= n_it; it += 2) {
      score_trip(it, std::true_type{});
      if (it + 1 <= n_it) score_trip(it + 1, std::false_type{});
    }
  } else {
    // =============================== value waves ===============================
    const int vp0 = p.vpad_h[h], dpv = p.vpad_h[h + 1] - vp0;
    const int ndg = dpv >> 4;
    const E* vbase = p.v_mid + (int64_t)my_b * p.v_bs + (int64_t)vp0 * 32 * p.cap_pages;  // wave-uniform
    const bool streams_v = has_mn && ndg > 0;
    // (mirrored page: lane group lg takes the tokens of group 3 - lg; the probabilities follow, see below)
    auto issue_v = [&](int t, bool mir) {   // page t -> stage (t - t_beg_w) % NST
      const int tp = SUB ? min(t, n_tiles - 1) : t;
      const E* vp = vbase + (int64_t)tp * dpv * 32 + (mir ? lane_vrev : lane_nat);
      unsigned char* st = &s_stage[MODE == 0 ? w : stw][(t - t_beg_w) % NST][0];
#pragma unroll
      for (int f = 0; f < VMAX; ++f)
        if (f < ndg) load_frag_to_lds<2>(vp + f * 512, st + f * 1024);
    };
    rot_fetch();
    half8 ETa[2 * KS];   // tile 2j: cosines, tile 2j + 1: sines of the frequencies 16j .. 16j + 15 of the slice
#pragma unroll
    for (int rt = 0; rt < 2 * KS; ++rt) ETa[rt] = p.tabET[(sl * 2 * KS + rt) * 64 + lane];
    // value pass: the scores of frame fi of the split (pages 2 fi, 2 fi + 1) into the workgroup's stage of that frame;
    // wave 4 + j brings fragment j of the four (a split with an odd number of pages: the second page of its last
    // frame repeats the first and is never read)
    const int n_fr = (n_it + 1) >> 1;
    auto issue_sc = [&](int fi) {
      if constexpr (MODE == 2) {
        if (w >= 4) {
          const int j = w - 4;
          const int pgi = min(2 * fi + (j >> 1), n_it - 1);
          const float* src = p.scores + ((int64_t)(grp * p.Hkv + h) * n_tiles + t_beg + pgi) * 512 + lc * 32 + 8 * lg + 4 * (j & 1);
          load_frag_to_lds<0>(src, &s_sc[fi % kScoreFrames][j * 1024]);
        }
      }
    };
    // first pages requested behind the table (see the score waves); page by page, so that the requests of a page
    // sit together in the order of arrival
#pragma unroll
    for (int i = 0; i < NST - 1; ++i)
      if (i < n_it && streams_v) issue_v(t_beg_w + i, (i & 1) == 0);
    if constexpr (MODE == 2) {
#pragma unroll
      for (int i = 0; i < kScoreFrames - 1; ++i)
        if (i < n_fr) issue_sc(i);
    }
    rot_store();
    float4v hacc[2 * KS], oacc[VMAX];
#pragma unroll
    for (int rt = 0; rt < 2 * KS; ++rt) hacc[rt] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int f = 0; f < VMAX; ++f) oacc[f] = float4v{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, d_run = 0.f;
    const bool ragged_tail = (p.L_m & 31) != 0;
    // This wave's own operands may arrive while the score waves work on the first page.  They must have landed
    // before the loop starts: inside it the only waits on vector memory are the explicit page waits.
#pragma unroll
    for (int rt = 0; rt < 2 * KS; ++rt) asm volatile("" ::"v"(ETa[rt]));
    const unsigned rot_lane = lds_addr_of(&s_rotv[(MODE == 1 ? 0 : sl * 2 * KS) * 4 + lg]);

    // The probabilities of the first (mirrored) page of a frame wait here for the second page: the tokens at the
    // offsets -(i + 1/2) and +(i + 1/2) meet the same cosine and, with opposite signs, the same sine, so g of the frame
    // takes E_cos^T (P2 + P1) and E_sin^T (P2 - P1) in one product instead of one per page.
    half8 p_first;
#pragma unroll
    for (int e = 0; e < 8; ++e) p_first[e] = (_Float16)0.f;
    // one page of the value stage (page it - 1 of the split)
    // (whether this wave streams V is fixed for the whole loop: a parameter of the body, not a branch in it)
    auto value_page = [&](int it, auto first_tag, auto stream_tag) {
        constexpr bool has_v = decltype(stream_tag)::value;
        const int t = t_beg_w + it - 1, buf = (it - 1) & 1;
        const int pg = it - 1;   // page index within the split
        constexpr int RCB = VMAX > 4 ? 1 : 2;   // the wide variant has no registers to spare for a second batch
        constexpr bool first_of_frame = decltype(first_tag)::value;   // the mirrored page of a frame (rotates), or the second
        uint4v rc[RCB][4];
        if constexpr (first_of_frame) {
          rot_issue<0>(rot_lane, rc[0]);
          if (RCB == 2 && 2 * KS > 4) rot_issue<1>(rot_lane, rc[RCB - 1]);
        }
        float sc[8];
        // (value pass: the scores of the frame have landed before the workgroup's meeting at the top of the frame)
        if constexpr (has_v) {
          if (pg + NST - 2 < n_it) wait_pages_in_flight<NST - 2, VMAX, 1>(ndg);
          else wait_vmcnt<0>();
          // refills the stage read one page ago
          if (pg + NST - 1 < n_it) issue_v(t + NST - 1, first_of_frame == (((NST - 1) & 1) == 0));
        }
        // the g history moves into the frame of this pair of pages: unit u of the constants belongs to the rows
        // 2 (u % 2) + f2 of the cosine tile 2 (u / 2) and of the sine tile behind it
        if constexpr (first_of_frame)
        rot_apply<2 * KS, RCB>(rot_lane, rc, [&](int u, int f2, float c, float sn) {
          float x = hacc[2 * (u >> 1)][2 * (u & 1) + f2], y = hacc[2 * (u >> 1) + 1][2 * (u & 1) + f2];
          rot_pair(c, sn, x, y);
          hacc[2 * (u >> 1)][2 * (u & 1) + f2] = x;
          hacc[2 * (u >> 1) + 1][2 * (u & 1) + f2] = y;
          return y;
        }, [&](int b) {
          asm volatile("" : "+v"(hacc[4 * b]), "+v"(hacc[4 * b + 1]), "+v"(hacc[4 * b + 2]), "+v"(hacc[4 * b + 3]));
        });
        // scores of the page in B-operand layout (column lc, positions 8*lg + e; on a mirrored page position i is
        // token 31 - i): four partials to sum
        if constexpr (MODE == 0) {
          uint4v part[kFreqWaves][2];
          const unsigned pst = lds_addr_of(&s_part[buf][0][lc * kPart + 8 * lg]);
          constexpr int kW = 16 * kPart * 4;   // bytes between the partials of two score waves
          part[0][0] = lds_read_b128_async_at<0>(pst);
          part[0][1] = lds_read_b128_async_at<16>(pst);
          part[1][0] = lds_read_b128_async_at<kW>(pst);
          part[1][1] = lds_read_b128_async_at<kW + 16>(pst);
          part[2][0] = lds_read_b128_async_at<2 * kW>(pst);
          part[2][1] = lds_read_b128_async_at<2 * kW + 16>(pst);
          part[3][0] = lds_read_b128_async_at<3 * kW>(pst);
          part[3][1] = lds_read_b128_async_at<3 * kW + 16>(pst);
#pragma unroll
          for (int ww = 0; ww < kFreqWaves; ++ww) {
            lds_wait_for(part[ww][0]);
            lds_wait_for(part[ww][1]);
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const uint4v p0 = part[0][e >> 2], p1 = part[1][e >> 2], p2 = part[2][e >> 2], p3 = part[3][e >> 2];
            const unsigned u0 = p0[e & 3], u1 = p1[e & 3], u2 = p2[e & 3], u3 = p3[e & 3];
            sc[e] = (__builtin_bit_cast(float, u0) + __builtin_bit_cast(float, u1)) +
                    (__builtin_bit_cast(float, u2) + __builtin_bit_cast(float, u3));
          }
        }
        uint4v sraw[2];   // value pass: the scores of the page, column lc, positions 8*lg .. 8*lg + 7
        if constexpr (MODE == 2) {
          const unsigned sst = lds_addr_of(&s_sc[(pg >> 1) % kScoreFrames][(pg & 1) * 2048]) + lane * 16;
          sraw[0] = lds_read_b128_async_at<0>(sst);
          sraw[1] = lds_read_b128_async_at<1024>(sst);
        }
        uint4v vraw[4];   // four dim groups at a time
        const unsigned vst = lds_addr_of(&s_stage[MODE == 0 ? w : stw][pg % NST][0]) + lane * 16;
        if constexpr (has_v) {
          vraw[0] = lds_read_b128_async_at<0>(vst);
          vraw[1] = lds_read_b128_async_at<1024>(vst);
          vraw[2] = lds_read_b128_async_at<2048>(vst);
          vraw[3] = lds_read_b128_async_at<3072>(vst);
        }
        if constexpr (MODE == 2) {
          if constexpr (has_v) asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(sraw[0]), "+v"(sraw[1])::"memory");
          else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(sraw[0]), "+v"(sraw[1])::"memory");
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const uint4v r = sraw[e >> 2];
            const unsigned u = r[e & 3];
            sc[e] = __builtin_bit_cast(float, u);
          }
        }
        if constexpr (SUB) {
          // this lane's column belongs to a sub-split of its own: past its last page nothing counts
          const int tc = t_beg + c_beg + pg;
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int tok = tc * 32 + (first_of_frame ? 31 - 8 * lg - e : 8 * lg + e);
            if (pg >= c_n || tok >= p.L_m) sc[e] = -INFINITY;
          }
        } else if (ragged_tail && t == n_tiles - 1) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int tok = t * 32 + (first_of_frame ? 31 - 8 * lg - e : 8 * lg + e);
            if (tok >= p.L_m) sc[e] = -INFINITY;
          }
        }
        float tmax = fa_fmax8(sc);
        tmax = fa_rows_max(tmax);
        // The softmax reference of a column moves only when the page maximum exceeds it by more than kLazyLog2:
        // until then the probabilities are taken against the old reference (at most 2^kLazyLog2, exact in the
        // 16-bit operands and far from any overflow) and nothing accumulated so far has to be rescaled.  With a
        // reference that follows every new maximum, some column of the sixteen moves it on most pages, and each
        // time the whole g history and the outputs are multiplied through.
        const float m_new = tmax > m_run + kLazyLog2 ? tmax : m_run;   // first page: m_run = -inf, so tmax
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);  // 0 on the first page
        float psum = 0.f;
        half8 pf;
        vec8 pe;   // for the V fragments, whose lane group lg holds the tokens of positions 8 lg + 7 - e on a mirrored page
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float pv = __builtin_amdgcn_exp2f(sc[e] - m_new);
          psum += pv;
          pf[e] = (_Float16)pv;
          pe[first_of_frame ? 7 - e : e] = (typename M::elem)pv;
        }
        d_run = d_run * alpha + psum;
        m_run = m_new;
        const bool rescale = __any(alpha != 1.0f);
        if (rescale) {
#pragma unroll
          for (int rt = 0; rt < 2 * KS; ++rt) hacc[rt] *= alpha;
#pragma unroll
          for (int f = 0; f < VMAX; ++f) oacc[f] *= alpha;
          if constexpr (!first_of_frame) p_first *= (_Float16)alpha;   // taken against the reference of a page ago
        }
        if constexpr (first_of_frame) {
          p_first = pf;
        } else {
          // (the difference as a sum with the sign bits flipped: packed adds, where a subtraction of two vectors of
          // halves is taken apart into sixteen scalar ones)
          const uint4v flipped = __builtin_bit_cast(uint4v, p_first) ^ uint4v{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
          const half8 p_sum = pf + p_first, p_dif = pf + __builtin_bit_cast(half8, flipped);
#pragma unroll
          for (int j = 0; j < KS; ++j)
            hacc[2 * j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ETa[2 * j], p_sum, hacc[2 * j], 0, 0, 0);
#pragma unroll
          for (int j = 0; j < KS; ++j)
            hacc[2 * j + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ETa[2 * j + 1], p_dif, hacc[2 * j + 1], 0, 0, 0);
        }
        if constexpr (has_v) {
#pragma unroll
          for (int f0 = 0; f0 < VMAX; f0 += 4) {
            if (f0 > 0) {
              if (f0 >= ndg) break;
              vraw[0] = lds_read_b128_async_at<0>(vst + f0 * 1024);
              vraw[1] = lds_read_b128_async_at<1024>(vst + f0 * 1024);
              vraw[2] = lds_read_b128_async_at<2048>(vst + f0 * 1024);
              vraw[3] = lds_read_b128_async_at<3072>(vst + f0 * 1024);
            }
            lds_wait_for4<0>(vraw);
#pragma unroll
            for (int f = 0; f < 4; ++f)
              oacc[f0 + f] = M::mma(__builtin_bit_cast(vec8, vraw[f]), pe, oacc[f0 + f]);   // a fragment the head does not
              // have multiplies whatever its stage slot holds into an accumulator that is never stored
          }
        }
    };
    auto value_loop = [&](auto stream_tag) {
      if constexpr (MODE == 2) {
        // One meeting per frame.  It hands over the frame's scores (every loading wave has seen its fragment land) and
        // frees the stage of the frame before for the next request.  It also keeps the waves of a workgroup - and with
        // them the workgroups of the launch - in step: without any meeting the page streams drift apart, some
        // workgroups end a fifth later than the median one and the launch ends with them.
        for (int it = 1; it <= n_it; it += 2) {
          const int fr = (it - 1) >> 1;
          if (w >= 4) {
            if (fr + kScoreFrames - 2 < n_fr) wait_vmcnt<kScoreFrames - 2>();
            else wait_vmcnt<0>();
          }
          barrier_lds_only();
          if (fr + kScoreFrames - 1 < n_fr) issue_sc(fr + kScoreFrames - 1);
          value_page(it, std::true_type{}, stream_tag);
          if (it + 1 <= n_it) value_page(it + 1, std::false_type{}, stream_tag);
        }
      } else {
        barrier_lds_only();   // iteration 0: the score waves are one page ahead
        for (int it = 1; it <= n_it; it += 2) {
          value_page(it, std::true_type{}, stream_tag);
          barrier_lds_only();
          if (it + 1 <= n_it) {
            value_page(it + 1, std::false_type{}, stream_tag);
            barrier_lds_only();
          }
        }
      }
    };
    if (streams_v) value_loop(std::true_type{});
    else value_loop(std::false_type{});
    if (n_it & 1) {   // the last frame has a first page only: g takes E_cos^T P1 and -E_sin^T P1
      const uint4v flipped = __builtin_bit_cast(uint4v, p_first) ^ uint4v{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u};
      const half8 p_neg = __builtin_bit_cast(half8, flipped);
#pragma unroll
      for (int j = 0; j < KS; ++j)
        hacc[2 * j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ETa[2 * j], p_first, hacc[2 * j], 0, 0, 0);
#pragma unroll
      for (int j = 0; j < KS; ++j)
        hacc[2 * j + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ETa[2 * j + 1], p_neg, hacc[2 * j + 1], 0, 0, 0);
    }

    // ---- partials of this split ------------------------------------------------------
    const float dsum = fa_rows_sum(d_run);
    // SUB: a column whose sub-split has no page has seen masked scores only; what it accumulated is not a number
    const bool c_none = SUB && c_n == 0;
    if (valid_r) {
      const int64_t base = prow * p.n_split + split;
      if (sl == 0 && lg == 0) {
        p.pm[base] = c_none ? -INFINITY : m_run;
        p.pd[base] = c_none ? 0.f : dsum;
      }
    }
    {
      // g of this split, back from its last frame (rotation by +phi of the frame centre), in the layout the merge
      // reads: [batch group][KV head][split][slice][row tile rt][column][lane group lg'] x {cos f, sin f, cos f+1,
      // sin f+1} with f = 8 rt + 2 lg' (the layout of the weights W).  This lane holds the frequencies
      // 16 j + 4 lg + v, v = 0 .. 3, of tile pair j: rt = 2 j + lg / 2, lg' = 2 (lg % 2) + v / 2.  Lanes of columns
      // past the group store values that nobody reads.
      float4v* gl = (float4v*)p.pg + ((((int64_t)(grp * p.Hkv + h) * p.n_split + split) * NSL + sl) * 2 * KS) * 64 + lc * 4;
      // twice the centre of the last frame, in half tokens
      const int64_t c2 = (int64_t)64 * (t_beg + c_beg + (n_it > 0 ? ((n_it - 1) & ~1) : 0) + 1) - 1;
      float sn[4], co[4], s16, c16;   // stepped phases, as for the first frame of the score waves
      fast_sincos_phase(16, c2, 2 * p.T, &s16, &c16);
#pragma unroll
      for (int v = 0; v < 4; ++v) fast_sincos_phase(fbase + 4 * lg + v, c2, 2 * p.T, &sn[v], &co[v]);
#pragma unroll
      for (int j = 0; j < KS; ++j) {
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          float4v o;
#pragma unroll
          for (int f2 = 0; f2 < 2; ++f2) {
            const int v = 2 * h2 + f2;
            const float x = hacc[2 * j][v], y = hacc[2 * j + 1][v];
            o[2 * f2] = co[v] * x - sn[v] * y;
            o[2 * f2 + 1] = sn[v] * x + co[v] * y;
          }
          if (c_none) o = float4v{0.f, 0.f, 0.f, 0.f};
          gl[(2 * j + (lg >> 1)) * 64 + 2 * (lg & 1) + h2] = o;
        }
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float cn = co[v] * c16 - sn[v] * s16;
          sn[v] = sn[v] * c16 + co[v] * s16;
          co[v] = cn;
        }
      }
    }
    if (valid_r) {
      const int64_t base = prow * p.n_split + split;
      if (has_mn && bb_r == sl) {
        // rows of D floats: dims past the head's stored count are written too (zeros, never read)
        float* on = p.pon + base * p.D;
#pragma unroll
        for (int f = 0; f < VMAX; ++f)
          if (f < ndg) *(float4v*)&on[f * 16 + 4 * lg] = c_none ? float4v{0.f, 0.f, 0.f, 0.f} : oacc[f];
      }
    }
  }
  if constexpr (FUSE) {
    const FusedShare fs = fused_share<SUB>(p, fz_vc0, fz_vc_len, split, p.st.n[h], b0, nb_real, KS, tid);
    fused_merge_tail<E, SUB, UPD>(p, (float*)&s_stage[0][0][0], &s_part[0][0][0], &s_team_flag, fs, grp, h, split, p.st.n[h], b0, nb_real, KS);
  }
}

}  // namespace fa_mfma
