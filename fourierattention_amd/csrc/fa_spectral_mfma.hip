// Spectral compression of a long prefill on the matrix cores (gfx950, wave64):
//   c[b, n, m]     = sum_k cos(2 pi (k + k_start) n / T) a[b, k, cols[m]]
//   c[b, N + n, m] = sum_k sin(...)                       a[b, k, cols[m]]
// (mat_fourier_triton TRI:81-102 / the FFT branch of MultiDimHiPPO2.forward TRI:858-865).
//
// The token axis is cut into steps of 128 tokens.  Inside a step the basis depends on the token offset
// only, E[n, i] = e^{i theta n i}, a constant f16 MFMA operand that every wave keeps in registers for its
// frequencies; the position of the step enters as one complex rotation per step and frequency:
//   sum_k e^{i theta n (p0 + k)} a[k] = e^{i theta n p0} * Horner_s( e^{i theta n 128}, G_s[n] ),
//   G_s[n] = sum_{i<128} E[n, i] a[128 s + i]
// so the steps are walked from the last to the first, acc <- G_s + e^{i theta n 128} acc, with the
// accumulators (fp32) never leaving registers.  Three kernels:
//   pack    gathers the compressed columns of the token-major input, converts them to f16 and writes them
//           as ready-made MFMA B operands (column tile of 16, kstep of 32 tokens, 64 lanes x 8 tokens)
//   gemm    one workgroup = 128 frequencies x 64 columns x one chunk of steps; the operands of a step
//           travel HBM -> LDS with global_load_lds, one barrier per step
//   reduce  sums the chunks into c
#include "fa_mfma_util.h"

namespace fa_mfma {

constexpr int kStepTokens = 128;               // tokens per step (four MFMA ksteps)
constexpr int kStepK = kStepTokens / 32;
constexpr int kWgFreqs = 128;                  // frequencies per workgroup (four waves x four row tiles of 8)
constexpr int kWgCols = 64;                    // columns per workgroup (four column tiles of 16)

// ---- basis table: A operands E[row tile rt][kstep][lane] x half8, row r of a tile = frequency rt*8 + r/2,
// cos (r even) or sin (r odd); lane l holds row l % 16, tokens 8 * (l / 16) + e of the kstep ----------------
__global__ __launch_bounds__(256) void spectral_table_kernel(half8* __restrict__ tab, int N, int T) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  const int total = (N / 8) * kStepK * 64;
  if (idx >= total) return;
  const int lane = idx & 63, ks = (idx >> 6) % kStepK, rt = idx / (64 * kStepK);
  const int r = lane & 15, lg = lane >> 4;
  const int n = rt * 8 + (r >> 1);
  half8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    float sn, co;
    fa_sincos_phase(n, ks * 32 + 8 * lg + e, T, &sn, &co);
    v[e] = (_Float16)((r & 1) ? sn : co);
  }
  tab[idx] = v;
}

// ---- pack: block = 32 tokens x 256 columns; lanes run along the columns for the gather, the transposition to
// token-contiguous fragments goes through LDS ----------------------------------------------------------------
template <typename E>
__global__ __launch_bounds__(256) void spectral_pack_kernel(
    const E* __restrict__ a, int64_t a_bs, int64_t a_rs, const int32_t* __restrict__ cols,
    const float* __restrict__ col_inv_scale, half8* __restrict__ out, int K, int Mc, int CT, int KS32) {
  constexpr int kPitch = 256 + 4;   // f16 elements per LDS row: 8 rows apart = 16 banks apart
  __shared__ _Float16 tile[32][kPitch];
  const int tid = threadIdx.x;
  const int ks = blockIdx.x, m0 = blockIdx.y * 256, b = blockIdx.z;
  const int m = m0 + tid;
  const bool mok = m < Mc;
  const int col = mok ? (cols ? cols[m] : m) : 0;
  const E* ab = a + (int64_t)b * a_bs + col;
  const float mul = (col_inv_scale && mok) ? col_inv_scale[(int64_t)b * Mc + m] : 1.f;
  float v[32];
#pragma unroll
  for (int kk = 0; kk < 32; ++kk) {
    const int k = ks * 32 + kk;
    v[kk] = fa_to_float(ab[(int64_t)min(k, K - 1) * a_rs]);
  }
#pragma unroll
  for (int kk = 0; kk < 32; ++kk) {
    const int k = ks * 32 + kk;
    // f16 holds every bf16 / f16 value of magnitude below 65504 exactly (tiny ones as subnormals)
    const float x = (mok && k < K) ? fminf(fmaxf(v[kk] * mul, -65504.f), 65504.f) : 0.f;
    tile[kk][tid] = (_Float16)x;
  }
  __syncthreads();
  // 16 column tiles x 64 lanes of fragments, four per thread
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int f = i * 256 + tid;
    const int ctl = f >> 6, lane = f & 63;
    const int lc = lane & 15, lg = lane >> 4;
    const int ct = (m0 >> 4) + ctl;
    if (ct >= CT) continue;
    half8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = tile[8 * lg + e][ctl * 16 + lc];
    out[(((int64_t)b * CT + ct) * KS32 + ks) * 64 + lane] = o;
  }
}

// ---- one pass over the prompt's K (or V) rows for everything the cache's prefill needs from them -------------------
// block = (PPB consecutive pages of 32 tokens, KV head, batch element); the head's slice of the rows goes through LDS
// once and leaves as
//   pages      the stored dims in the page layout of the decode kernels (what fa_mid_pack writes),
//   fragments  the compressed dims as f16 B operands of the compression GEMM (what spectral_pack_kernel writes; a
//              column tile that two heads share is written by both, each its own 16-byte pieces),
//   partials   sum / max / min of every compressed column over the block's tokens (what col_stats_partial_kernel
//              leaves, finished by the same final launch).
constexpr int kPackPages = 4;   // pages per block

template <typename E>
struct PrefillPackParams {
  const E* src;
  int64_t src_bs, src_rs, row0;
  int L, K_fft;                 // mid rows; rows that enter the transform (K_fft <= L)
  E* store;                     // paged store of the stored dims
  int64_t st_bs;
  int cap_pages;
  const int32_t* n_list; const int32_t* n_h; const int32_t* pad_h;   // stored dims: flat h*D + d, per-head offsets
  const int32_t* c_list; const int32_t* c_h;                         // compressed dims, likewise
  half8* packed;                // [B][CT][KS32][64]
  float* psum; float* pmax; float* pmin;   // [B][n_blocks][Mc]
  int Mc, CT, KS32, n_pages, n_blocks, Hkv, D, is_v;
};

template <typename E>
__global__ __launch_bounds__(256) void prefill_pack_kernel(const PrefillPackParams<E> p) {
  constexpr int kMaxD = 256;
  constexpr int kPitch = kMaxD + 8;                 // elements; keeps rows 16-byte aligned
  struct alignas(sizeof(E) * 8) Piece { E v[8]; };
  __shared__ __attribute__((aligned(32))) E tile[32][kPitch];
  __shared__ int s_col[kMaxD];                      // dim within the head of every stored position
  __shared__ int s_ccol[kMaxD];                     // ... of every compressed position
  const int h = blockIdx.y, b = blockIdx.z, tid = threadIdx.x, D = p.D;
  const int n0 = p.n_h[h], n_len = p.n_h[h + 1] - n0;
  const int p0 = p.pad_h[h], dp = p.pad_h[h + 1] - p0;
  const int c0 = p.c_h[h], c_len = p.c_h[h + 1] - c0;
  for (int j = tid; j < dp; j += 256) s_col[j] = n_len > 0 ? min(max(p.n_list[n0 + min(j, n_len - 1)] - h * D, 0), D - 1) : 0;
  for (int j = tid; j < c_len; j += 256) s_ccol[j] = min(max(p.c_list[c0 + j] - h * D, 0), D - 1);
  const E* sb = p.src + (int64_t)b * p.src_bs + p.row0 * p.src_rs + (int64_t)h * D;
  const int ppr = D >> 3;                           // 16-byte pieces per row of the head
  const int pages_of_rows = (p.L + 31) >> 5;
  // columns past the last compressed dim in the last column tile belong to nobody: the last head clears them
  const int c_extra = h == p.Hkv - 1 ? p.CT * 16 - p.Mc : 0;
  float sum = 0.f, mx = -INFINITY, mn = INFINITY;   // thread j < c_len: statistics of its column
  for (int pp = 0; pp < kPackPages; ++pp) {
    const int page = blockIdx.x * kPackPages + pp;
    if (page >= p.n_pages) break;
    __syncthreads();                                // the tile of the page before has been read (and the lists stored)
    if (page < pages_of_rows) {
      const int64_t last = (int64_t)p.L - 1;
      for (int q = tid; q < 32 * ppr; q += 256) {
        const int t = q / ppr, c = q - t * ppr;
        const int64_t token = (int64_t)page * 32 + t;
        *(Piece*)&tile[t][c * 8] = *(const Piece*)(sb + (token < last ? token : last) * p.src_rs + c * 8);
      }
    }
    __syncthreads();
    // ---- pages of the stored dims
    if (page < pages_of_rows && n_len > 0) {
      Piece* out = (Piece*)(p.store + (int64_t)b * p.st_bs + (int64_t)p0 * 32 * p.cap_pages + (int64_t)page * dp * 32);
      const int n_pieces = dp * 32 / 8;
      for (int piece = tid; piece < n_pieces; piece += 256) {
        const int frag = piece >> 6, lane = piece & 63;
        Piece o;
        if (!p.is_v) {
          const int nks = dp >> 5;
          const int tb = frag / nks, s_ = frag - tb * nks;
          const int t = tb * 16 + (lane & 15), j0 = s_ * 32 + 8 * (lane >> 4);
          const bool row_ok = (int64_t)page * 32 + t < p.L;
#pragma unroll
          for (int e = 0; e < 8; ++e) o.v[e] = (row_ok && j0 + e < n_len) ? tile[t][s_col[j0 + e]] : E{};
        } else {
          const int j = frag * 16 + (lane & 15);
          const int col = s_col[j];
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            const int t = 8 * (lane >> 4) + i;
            o.v[i] = (j < n_len && (int64_t)page * 32 + t < p.L) ? tile[t][col] : E{};
          }
        }
        out[piece] = o;
      }
    }
    // ---- f16 fragments of the compressed dims (tokens past the transform's rows are zero)
    if (page < p.KS32) {
      for (int idx = tid; idx < (c_len + c_extra) * 4; idx += 256) {
        const int j = idx >> 2, lg = idx & 3;
        const int m = c0 + j;                       // column of the compressed matrix
        half8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int t = 8 * lg + e;
          float x = 0.f;
          if (j < c_len && (int64_t)page * 32 + t < p.K_fft) x = fminf(fmaxf(fa_to_float(tile[t][s_ccol[j]]), -65504.f), 65504.f);
          o[e] = (_Float16)x;
        }
        p.packed[(((int64_t)b * p.CT + (m >> 4)) * p.KS32 + page) * 64 + lg * 16 + (m & 15)] = o;
      }
    }
    // ---- column statistics over the mid rows
    if (tid < c_len && page < pages_of_rows) {
      const int col = s_ccol[tid];
      const int n_t = min(32, p.L - page * 32);
      for (int t = 0; t < n_t; ++t) {
        const float v = fa_to_float(tile[t][col]);
        sum += v;
        mx = fmaxf(mx, v);
        mn = fminf(mn, v);
      }
    }
  }
  if (tid < c_len) {
    const int64_t o = ((int64_t)b * p.n_blocks + blockIdx.x) * p.Mc + c0 + tid;
    p.psum[o] = sum;
    p.pmax[o] = mx;
    p.pmin[o] = mn;
  }
}

struct SpectralGemmParams {
  const half8* tab;      // basis table
  const half8* packed;   // [B][CT][KS32][64] fragments
  float* part;           // [S][B][2N][Mc]; with a single chunk: the result c itself (no reduction launch)
  int add_to_part;       // single chunk only: add to what part holds instead of overwriting it
  int B, N, Mc, CT, KS32, T;
  int n_steps, steps_per_chunk, n_chunks;
  int64_t k_start;
};

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void spectral_gemm_kernel(const SpectralGemmParams p) {
  constexpr int NST = 4;   // steps in LDS: the one in use and three on their way
  __shared__ __attribute__((aligned(16))) unsigned char s_stage[NST][4][kStepK][1024];
  const int tid = threadIdx.x, lane = tid & 63, lg = lane >> 4, lc = lane & 15;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int b = blockIdx.z / p.n_chunks, chunk = blockIdx.z - b * p.n_chunks;
  const int rt0 = (blockIdx.y * 4 + w) * 4;          // first of this wave's four row tiles
  const int ct0 = blockIdx.x * 4;                    // first of the workgroup's four column tiles
  const int n_rt = p.N / 8;
  const int s_beg = chunk * p.steps_per_chunk;
  const int s_end = min(p.n_steps, s_beg + p.steps_per_chunk);
  const int n_it = s_end - s_beg;

  // this wave stages column tile w of every step (clamped: a tile past the end repeats the last one)
  const int ct_mine = min(ct0 + w, p.CT - 1);
  const _Float16* src = (const _Float16*)(p.packed + (((int64_t)b * p.CT + ct_mine) * p.KS32) * 64) + lane * 8;
  auto issue = [&](int s, int stage) {
#pragma unroll
    for (int ks = 0; ks < kStepK; ++ks)
      load_frag_to_lds(src + (int64_t)(s * kStepK + ks) * 512, &s_stage[stage][w][ks][0]);
  };
#pragma unroll
  for (int i = 0; i < NST - 1; ++i)
    if (i < n_it) issue(s_end - 1 - i, i);

  half8 Ea[4][kStepK];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int ks = 0; ks < kStepK; ++ks) Ea[i][ks] = p.tab[((int64_t)min(rt0 + i, n_rt - 1) * kStepK + ks) * 64 + lane];
  // per frequency of this lane (row tile i, pair f2): rotation of one step
  float rc[4][2], rs[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int f2 = 0; f2 < 2; ++f2) fast_sincos_phase(min(rt0 + i, n_rt - 1) * 8 + lg * 2 + f2, kStepTokens, p.T, &rs[i][f2], &rc[i][f2]);
  float4v acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};
  // the table loads must have landed before the loop: inside it the only waits on vector memory are explicit
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int ks = 0; ks < kStepK; ++ks) asm volatile("" ::"v"(Ea[i][ks]));

  for (int it = 0; it < n_it; ++it) {
    const int s = s_end - 1 - it, stage = it % NST;
    if (it + NST - 2 < n_it) wait_vmcnt<(NST - 2) * kStepK>();   // the steps behind this one may still be in flight
    else wait_vmcnt<0>();
    barrier_lds_only();   // every wave's share of step s has landed; nobody still reads the stage refilled next
    if (it + NST - 1 < n_it) issue(s - (NST - 1), (it + NST - 1) % NST);
    if (it > 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int f2 = 0; f2 < 2; ++f2) {
            const float c = acc[i][j][2 * f2], sn = acc[i][j][2 * f2 + 1];
            acc[i][j][2 * f2] = rc[i][f2] * c - rs[i][f2] * sn;
            acc[i][j][2 * f2 + 1] = rs[i][f2] * c + rc[i][f2] * sn;
          }
    }
#pragma unroll
    for (int ks = 0; ks < kStepK; ++ks) {
      uint4v braw[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) braw[j] = lds_read_b128_async(&s_stage[stage][j][ks][lane * 16]);
      lds_wait_for4<0>(braw);
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ea[i][ks], __builtin_bit_cast(half8, braw[j]), acc[i][j], 0, 0, 0);
    }
  }

  // into the common frame (phase of the chunk's first token) and out
  const int64_t p0 = (int64_t)s_beg * kStepTokens + p.k_start;
  float* out = p.part + ((int64_t)chunk * p.B + b) * 2 * p.N * p.Mc;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (rt0 + i >= n_rt) continue;
#pragma unroll
    for (int f2 = 0; f2 < 2; ++f2) {
      const int n = (rt0 + i) * 8 + lg * 2 + f2;
      float sn, co;
      fast_sincos_phase(n, p0, p.T, &sn, &co);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int m = (ct0 + j) * 16 + lc;
        if (m < p.Mc) {
          const float c = acc[i][j][2 * f2], s_ = acc[i][j][2 * f2 + 1];
          float* oc = out + (int64_t)n * p.Mc + m;
          float* os = out + (int64_t)(p.N + n) * p.Mc + m;
          const float vc = co * c - sn * s_, vs = sn * c + co * s_;
          *oc = p.add_to_part ? *oc + vc : vc;
          *os = p.add_to_part ? *os + vs : vs;
        }
      }
    }
  }
}

__global__ __launch_bounds__(256) void spectral_reduce_kernel(const float* __restrict__ part, float* __restrict__ c,
                                                              int64_t total, int n_chunks, int accumulate) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= total) return;   // total is a multiple of 16 whatever Mc is: 2N is one
  float4 a = accumulate ? *(const float4*)(c + i) : make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s = 0; s < n_chunks; ++s) {
    const float4 v = *(const float4*)(part + (int64_t)s * total + i);
    a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
  }
  *(float4*)(c + i) = a;
}

// ---------------------------------------------------------------------------------------------------------
// Statistics of the reconstruction (mat_fourier_avg_std_triton, TRI:285-326) on the same machinery.
//   r[k, m] = (1/N) sum_n cos(theta k n) c[n, m] + sin(theta k n) c[N + n, m] = (1/N) Re sum_n e^{i theta k n} (c - i s)
// is the compression GEMM with the roles of position and frequency exchanged: the rows are the positions k,
// the "tokens" are the N coefficient indices.  A workgroup owns 128 positions, keeps their basis rows in
// registers, and walks over every block of 64 columns: one pass over the cos coefficients (keeps the real part A_k),
// one over the sin coefficients (keeps the imaginary part B_k), then folds its positions into sum / max / min.
// Position k gives r[k] = A_k + B_k and, because the period is a whole number of positions, also its mirror image
// r[T - k] = A_k - B_k: only the positions up to T / 2 are computed, each standing for two where the sequence
// reaches past T / 2.
// The coefficients travel as f16 scaled by a power of two per column (their range is not bounded).
// ---------------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void coef_colscale_kernel(const float* __restrict__ c, float* __restrict__ scale,
                                                             float* __restrict__ inv_scale, int N2, int Mc) {
  __shared__ float s_mx[16][64];
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;   // 64 columns x 16 row classes
  const int m = blockIdx.x * 64 + lane, b = blockIdx.y;
  float mx = 0.f;
  if (m < Mc) {
    const float* cp = c + (int64_t)b * N2 * Mc + m;
    for (int n0 = g; n0 < N2; n0 += 16 * 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = cp[(int64_t)min(n0 + 16 * u, N2 - 1) * Mc];
#pragma unroll
      for (int u = 0; u < 8; ++u) mx = fmaxf(mx, fabsf(v[u]));
    }
  }
  s_mx[g][lane] = mx;
  __syncthreads();
  if (g == 0 && m < Mc) {
#pragma unroll
    for (int i = 1; i < 16; ++i) mx = fmaxf(mx, s_mx[i][lane]);
    const float sc = mx > 0.f ? exp2f(ceilf(log2f(mx))) : 1.f;   // power of two: scaling is exact
    scale[(int64_t)b * Mc + m] = sc;
    inv_scale[(int64_t)b * Mc + m] = 1.0f / sc;
  }
}

struct ReconStatsParams {
  const half8* tab;        // basis rows of the positions: [ceil(K/8)][kStepK][64]
  const half8* packed[2];  // cos / sin coefficients, [B][CT][KS32][64] fragments
  const float* scale;      // [B][Mc]
  float* psum;
  float* pmax;
  float* pmin;             // [B][RB][Mc]
  int B, N, Mc, CT, KS32, K, T, n_steps, RB;
  int Kd;     // positions computed directly: min(K, T / 2 + 1)
  int half;   // T / 2: mirror images beyond it count as positions of their own (a value no position exceeds
              // when the sequence is longer than the period and every position is computed directly)
};

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void spectral_recon_stats_kernel(
    const ReconStatsParams p) {
  constexpr int NST = 4;
  __shared__ __attribute__((aligned(16))) unsigned char s_stage[NST][4][kStepK][1024];
  __shared__ float s_red[3][4][kWgCols];
  const int tid = threadIdx.x, lane = tid & 63, lg = lane >> 4, lc = lane & 15;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int rb = blockIdx.x, b = blockIdx.y;
  const int rt0 = (rb * 4 + w) * 4;
  const int n_rt = (p.Kd + 7) / 8;
  const int S = p.n_steps;
  const int n_cb = (p.Mc + kWgCols - 1) / kWgCols;
  const int Q = n_cb * 2 * S;   // steps of this workgroup: column block, pass (cos, sin), step (last to first)

  auto issue = [&](int q, int stage) {
    const int cb = q / (2 * S), rem = q - cb * 2 * S;
    const int pass = rem / S, s = S - 1 - (rem - pass * S);
    const int ct = min(cb * 4 + w, p.CT - 1);
    const _Float16* src = (const _Float16*)(p.packed[pass] + (((int64_t)b * p.CT + ct) * p.KS32) * 64) + lane * 8;
#pragma unroll
    for (int ks = 0; ks < kStepK; ++ks)
      load_frag_to_lds(src + (int64_t)(s * kStepK + ks) * 512, &s_stage[stage][w][ks][0]);
  };
#pragma unroll
  for (int i = 0; i < NST - 1; ++i)
    if (i < Q) issue(i, i);

  half8 Ea[4][kStepK];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int ks = 0; ks < kStepK; ++ks) Ea[i][ks] = p.tab[((int64_t)min(rt0 + i, n_rt - 1) * kStepK + ks) * 64 + lane];
  float rc[4][2], rs[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int f2 = 0; f2 < 2; ++f2) fast_sincos_phase(min(rt0 + i, n_rt - 1) * 8 + lg * 2 + f2, kStepTokens, p.T, &rs[i][f2], &rc[i][f2]);
  float4v acc[4][4];
  float re[4][4][2];   // real part left by the cos pass
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int ks = 0; ks < kStepK; ++ks) asm volatile("" ::"v"(Ea[i][ks]));

  const float inv_n = 1.0f / (float)p.N;
  for (int q = 0; q < Q; ++q) {
    const int cb = q / (2 * S), rem = q - cb * 2 * S;
    const int pass = rem / S, it = rem - pass * S;
    const int stage = q % NST;
    if (q + NST - 2 < Q) wait_vmcnt<(NST - 2) * kStepK>();
    else wait_vmcnt<0>();
    barrier_lds_only();
    if (q + NST - 1 < Q) issue(q + NST - 1, (q + NST - 1) % NST);
    if (it == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
          for (int f2 = 0; f2 < 2; ++f2) {
            const float c = acc[i][j][2 * f2], sn = acc[i][j][2 * f2 + 1];
            acc[i][j][2 * f2] = rc[i][f2] * c - rs[i][f2] * sn;
            acc[i][j][2 * f2 + 1] = rs[i][f2] * c + rc[i][f2] * sn;
          }
    }
#pragma unroll
    for (int ks = 0; ks < kStepK; ++ks) {
      uint4v braw[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) braw[j] = lds_read_b128_async(&s_stage[stage][j][ks][lane * 16]);
      lds_wait_for4<0>(braw);
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(Ea[i][ks], __builtin_bit_cast(half8, braw[j]), acc[i][j], 0, 0, 0);
    }
    if (it != S - 1) continue;
    if (pass == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          re[i][j][0] = acc[i][j][0];
          re[i][j][1] = acc[i][j][2];
        }
      continue;
    }
    // both passes done for this column block: r = (re +- im) * scale / N at this lane's 8 positions per column and
    // at their mirror images
    const int half = p.half;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int m = (cb * 4 + j) * 16 + lc;
      const float sc = m < p.Mc ? p.scale[(int64_t)b * p.Mc + m] * inv_n : 0.f;
      float sum = 0.f, mx = -INFINITY, mn = INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int f2 = 0; f2 < 2; ++f2) {
          const int k = (rt0 + i) * 8 + lg * 2 + f2;
          const float r = (re[i][j][f2] + acc[i][j][2 * f2 + 1]) * sc;
          if (k < p.Kd) {
            sum += r;
            mx = fmaxf(mx, r);
            mn = fminf(mn, r);
          }
          const int km = p.T - k;   // the mirror image counts where it is a position of its own beyond T / 2
          const float r2 = (re[i][j][f2] - acc[i][j][2 * f2 + 1]) * sc;
          if (k < p.Kd && km > half && km < p.K) {
            sum += r2;
            mx = fmaxf(mx, r2);
            mn = fminf(mn, r2);
          }
        }
      sum = fa_rows_sum(sum);
      mx = fa_rows_max(mx);
      mn = fa_rows_min(mn);
      if (lg == 0) {
        s_red[0][w][j * 16 + lc] = sum;
        s_red[1][w][j * 16 + lc] = mx;
        s_red[2][w][j * 16 + lc] = mn;
      }
    }
    __syncthreads();
    if (tid < kWgCols) {
      const int m = cb * kWgCols + tid;
      if (m < p.Mc) {
        const int64_t o = ((int64_t)b * p.RB + rb) * p.Mc + m;
        p.psum[o] = (s_red[0][0][tid] + s_red[0][1][tid]) + (s_red[0][2][tid] + s_red[0][3][tid]);
        p.pmax[o] = fmaxf(fmaxf(s_red[1][0][tid], s_red[1][1][tid]), fmaxf(s_red[1][2][tid], s_red[1][3][tid]));
        p.pmin[o] = fminf(fminf(s_red[2][0][tid], s_red[2][1][tid]), fminf(s_red[2][2][tid], s_red[2][3][tid]));
      }
    }
    // the next barrier (top of the loop) orders these reads before s_red is written again
  }
}

}  // namespace fa_mfma

namespace {
struct SpectralPlan {
  int CT, KS32, n_steps, n_chunks, steps_per_chunk;
  size_t off_tab, off_packed, off_part, total;
};
SpectralPlan spectral_plan(int B, int K, int Mc, int N) {
  using namespace fa_mfma;
  SpectralPlan p{};
  p.CT = fa_cdiv(Mc, 16);
  p.n_steps = fa_cdiv(K, kStepTokens);
  p.KS32 = p.n_steps * kStepK;
  const int64_t tiles = (int64_t)B * fa_cdiv(N, kWgFreqs) * fa_cdiv(Mc, kWgCols);
  int want = fa_cdiv(512, tiles);                  // two workgroups per CU
  if (want < 1) want = 1;
  const int max_chunks = p.n_steps / 4 > 0 ? p.n_steps / 4 : 1;   // at least four steps per chunk
  if (want > max_chunks) want = max_chunks;
  p.steps_per_chunk = fa_cdiv(p.n_steps, want);
  p.n_chunks = fa_cdiv(p.n_steps, p.steps_per_chunk);
  size_t o = 0;
  auto take = [&](size_t bytes) { size_t at = o; o += fa_align_up(bytes, 256); return at; };
  p.off_tab = take((size_t)(N / 8) * kStepK * 64 * 16);
  p.off_packed = take((size_t)B * p.CT * p.KS32 * 1024);
  p.off_part = take((size_t)p.n_chunks * B * 2 * N * Mc * 4);
  p.total = o;
  return p;
}
}  // namespace

bool fa_spectral_mfma_ok(int a_dtype, int K, int Mc, int N) {
  return (a_dtype == FA_BF16 || a_dtype == FA_FP16) && N % 8 == 0 && K >= 4 * fa_mfma::kStepTokens;
}

size_t fa_spectral_mfma_workspace(int B, int K, int Mc, int N) { return spectral_plan(B, K, Mc, N).total; }

namespace {
// table, GEMM and chunk reduction on fragments that are already in the workspace
int spectral_after_pack(const SpectralPlan& pl, float* c, int B, int Mc, int N, int T, int64_t k_start, int accumulate,
                        void* workspace, hipStream_t st);
}  // namespace

int fa_spectral_mfma_launch(const void* a, int a_dtype, int64_t a_bs, int64_t a_rs, const int32_t* cols, float* c, int B,
                            int K, int Mc, int N, int T, int64_t k_start, int accumulate, void* workspace,
                            hipStream_t st) {
  using namespace fa_mfma;
  const SpectralPlan pl = spectral_plan(B, K, Mc, N);
  half8* packed = (half8*)((char*)workspace + pl.off_packed);
  dim3 pgrid(pl.KS32, fa_cdiv(Mc, 256), B);
  if (a_dtype == FA_BF16)
    spectral_pack_kernel<bf16_t><<<pgrid, 256, 0, st>>>((const bf16_t*)a, a_bs, a_rs, cols, nullptr, packed, K, Mc, pl.CT, pl.KS32);
  else
    spectral_pack_kernel<f16_t><<<pgrid, 256, 0, st>>>((const f16_t*)a, a_bs, a_rs, cols, nullptr, packed, K, Mc, pl.CT, pl.KS32);
  return spectral_after_pack(pl, c, B, Mc, N, T, k_start, accumulate, workspace, st);
}

namespace {
int spectral_after_pack(const SpectralPlan& pl, float* c, int B, int Mc, int N, int T, int64_t k_start, int accumulate,
                        void* workspace, hipStream_t st) {
  using namespace fa_mfma;
  char* ws = (char*)workspace;
  half8* tab = (half8*)(ws + pl.off_tab);
  half8* packed = (half8*)(ws + pl.off_packed);
  float* part = (float*)(ws + pl.off_part);
  spectral_table_kernel<<<fa_cdiv((N / 8) * kStepK * 64, 256), 256, 0, st>>>(tab, N, T);
  SpectralGemmParams gp{};
  const bool direct = pl.n_chunks == 1;   // nothing to sum: the GEMM writes (or adds to) c itself
  gp.tab = tab; gp.packed = packed; gp.part = direct ? c : part;
  gp.add_to_part = direct && accumulate;
  gp.B = B; gp.N = N; gp.Mc = Mc; gp.CT = pl.CT; gp.KS32 = pl.KS32; gp.T = T;
  gp.n_steps = pl.n_steps; gp.steps_per_chunk = pl.steps_per_chunk; gp.n_chunks = pl.n_chunks;
  gp.k_start = k_start;
  dim3 ggrid(fa_cdiv(Mc, kWgCols), fa_cdiv(N, kWgFreqs), B * pl.n_chunks);
  spectral_gemm_kernel<<<ggrid, 256, 0, st>>>(gp);
  const int64_t total = (int64_t)B * 2 * N * Mc;
  if (!direct) spectral_reduce_kernel<<<fa_cdiv(total / 4, 256), 256, 0, st>>>(part, c, total, pl.n_chunks, accumulate);
  return fa_check_launch("fa_mat_fourier");
}

struct PrefillPlan {
  SpectralPlan sp;
  int n_pages, n_blocks;
  size_t off_sum, off_max, off_min, total;
};
PrefillPlan prefill_plan(int B, int L, int K_fft, int Mc, int N) {
  PrefillPlan p{};
  p.sp = spectral_plan(B, K_fft, Mc, N);
  const int pages_of_rows = fa_cdiv(L, 32);
  p.n_pages = pages_of_rows > p.sp.KS32 ? pages_of_rows : p.sp.KS32;
  p.n_blocks = fa_cdiv(p.n_pages, fa_mfma::kPackPages);
  size_t o = p.sp.total;
  auto take = [&](size_t bytes) { size_t at = o; o += fa_align_up(bytes, 256); return at; };
  p.off_sum = take((size_t)B * p.n_blocks * Mc * 4);
  p.off_max = take((size_t)B * p.n_blocks * Mc * 4);
  p.off_min = take((size_t)B * p.n_blocks * Mc * 4);
  p.total = o;
  return p;
}
}  // namespace

extern "C" int fa_prefill_compress_ok(int dtype, int L, int K_fft, int Mc, int N, int D) {
  return fa_spectral_mfma_ok(dtype, K_fft, Mc, N) && L >= K_fft && K_fft > 0 && D % 8 == 0 && D <= 256;
}

extern "C" size_t fa_prefill_compress_workspace_bytes(int B, int L, int K_fft, int Mc, int N) {
  if (B <= 0 || L <= 0 || K_fft <= 0 || Mc <= 0 || N <= 0) return 0;
  return prefill_plan(B, L, K_fft, Mc, N).total;
}

extern "C" int fa_prefill_compress(const void* src, int dtype, int64_t src_bs, int64_t src_rs, int64_t row0, int L, int K_fft,
                                   void* store, int64_t st_bs, int cap_pages, const int32_t* n_list, const int32_t* n_h,
                                   const int32_t* pad_h, const int32_t* c_list, const int32_t* c_h, int Mc, float* coef,
                                   float* avg, float* max_dev, int stats_round_dtype, int B, int Hkv, int D, int N, int T,
                                   int is_v, void* workspace, size_t workspace_bytes, fa_stream_t stream) {
  using namespace fa_mfma;
  FA_REQUIRE(src && store && n_h && pad_h && c_list && c_h && coef && avg && max_dev, FA_ERR_NULL_POINTER,
             "fa_prefill_compress: null pointer");
  FA_REQUIRE(B > 0 && Hkv > 0 && L > 0 && cap_pages > 0 && row0 >= 0 && T > 0, FA_ERR_BAD_SHAPE, "fa_prefill_compress: bad shape");
  FA_REQUIRE((int64_t)cap_pages * 32 >= L, FA_ERR_BAD_SHAPE, "fa_prefill_compress: %d rows do not fit %d pages", L, cap_pages);
  FA_REQUIRE(fa_prefill_compress_ok(dtype, L, K_fft, Mc, N, D), FA_ERR_UNSUPPORTED,
             "fa_prefill_compress: dtype=%d L=%d K=%d Mc=%d N=%d D=%d is for the separate calls", dtype, L, K_fft, Mc, N, D);
  FA_REQUIRE(src_rs >= (int64_t)Hkv * D && src_rs % 8 == 0 && src_bs % 8 == 0 && ((uintptr_t)src & 15) == 0,
             FA_ERR_MISALIGNED, "fa_prefill_compress: rows of %lld elements (need %d, 16-byte aligned)", (long long)src_rs, Hkv * D);
  const PrefillPlan pl = prefill_plan(B, L, K_fft, Mc, N);
  FA_REQUIRE(workspace && workspace_bytes >= pl.total, FA_ERR_WORKSPACE, "fa_prefill_compress: workspace %zu < %zu",
             workspace_bytes, pl.total);
  FA_REQUIRE(((uintptr_t)workspace & 255) == 0 && ((uintptr_t)coef & 15) == 0, FA_ERR_MISALIGNED,
             "fa_prefill_compress: workspace not 256-byte or coefficients not 16-byte aligned");
  hipStream_t st = fa_hip_stream(stream);
  char* ws = (char*)workspace;
  float* psum = (float*)(ws + pl.off_sum);
  float* pmax = (float*)(ws + pl.off_max);
  float* pmin = (float*)(ws + pl.off_min);
  auto launch = [&](auto tag) {
    using E = decltype(tag);
    PrefillPackParams<E> pp{};
    pp.src = (const E*)src; pp.src_bs = src_bs; pp.src_rs = src_rs; pp.row0 = row0; pp.L = L; pp.K_fft = K_fft;
    pp.store = (E*)store; pp.st_bs = st_bs; pp.cap_pages = cap_pages;
    pp.n_list = n_list; pp.n_h = n_h; pp.pad_h = pad_h; pp.c_list = c_list; pp.c_h = c_h;
    pp.packed = (half8*)(ws + pl.sp.off_packed);
    pp.psum = psum; pp.pmax = pmax; pp.pmin = pmin;
    pp.Mc = Mc; pp.CT = pl.sp.CT; pp.KS32 = pl.sp.KS32; pp.n_pages = pl.n_pages; pp.n_blocks = pl.n_blocks;
    pp.Hkv = Hkv; pp.D = D; pp.is_v = is_v;
    prefill_pack_kernel<E><<<dim3(pl.n_blocks, Hkv, B), 256, 0, st>>>(pp);
  };
  if (dtype == FA_BF16) launch(bf16_t{}); else launch(f16_t{});
  int rc = spectral_after_pack(pl.sp, coef, B, Mc, N, T, 0, 0, workspace, st);
  if (rc != FA_OK) return rc;
  fa_stats_finalize_launch(psum, pmax, pmin, avg, max_dev, B, L, Mc, pl.n_blocks, stats_round_dtype, st);
  return fa_check_launch("fa_prefill_compress");
}

namespace {
struct ReconPlan {
  int CT, KS32, n_steps, RB;
  size_t off_tab, off_pc, off_ps, off_scale, off_inv, off_sum, off_max, off_min, total;
};
ReconPlan recon_plan(int B, int N, int Mc, int K) {
  using namespace fa_mfma;
  ReconPlan p{};
  p.CT = fa_cdiv(Mc, 16);
  p.n_steps = fa_cdiv(N, kStepTokens);
  p.KS32 = p.n_steps * kStepK;
  p.RB = fa_cdiv(K, kWgFreqs);
  size_t o = 0;
  auto take = [&](size_t bytes) { size_t at = o; o += fa_align_up(bytes, 256); return at; };
  p.off_tab = take((size_t)fa_cdiv(K, 8) * kStepK * 64 * 16);
  p.off_pc = take((size_t)B * p.CT * p.KS32 * 1024);
  p.off_ps = take((size_t)B * p.CT * p.KS32 * 1024);
  p.off_scale = take((size_t)B * Mc * 4);
  p.off_inv = take((size_t)B * Mc * 4);
  p.off_sum = take((size_t)B * p.RB * Mc * 4);
  p.off_max = take((size_t)B * p.RB * Mc * 4);
  p.off_min = take((size_t)B * p.RB * Mc * 4);
  p.total = o;
  return p;
}
}  // namespace

bool fa_recon_stats_mfma_ok(int N, int Mc, int K) { return N >= 32 && Mc >= 16 && K >= 1024; }

size_t fa_recon_stats_mfma_workspace(int B, int N, int Mc, int K) { return recon_plan(B, N, Mc, K).total; }

int fa_recon_stats_mfma_launch(const float* c, int B, int N, int Mc, int K, int T, void* workspace, float** psum,
                               float** pmax, float** pmin, hipStream_t st) {
  using namespace fa_mfma;
  const ReconPlan pl = recon_plan(B, N, Mc, K);
  char* ws = (char*)workspace;
  half8* tab = (half8*)(ws + pl.off_tab);
  half8* pc = (half8*)(ws + pl.off_pc);
  half8* ps = (half8*)(ws + pl.off_ps);
  float* scale = (float*)(ws + pl.off_scale);
  float* inv = (float*)(ws + pl.off_inv);
  *psum = (float*)(ws + pl.off_sum);
  *pmax = (float*)(ws + pl.off_max);
  *pmin = (float*)(ws + pl.off_min);
  // positions 0 .. T / 2 stand for their mirror images as well (unless the sequence is longer than the period)
  const bool mirror = K <= T + 1;
  const int Kd = mirror && T / 2 + 1 < K ? T / 2 + 1 : K;
  const int RBd = fa_cdiv(Kd, kWgFreqs);
  const int kp8 = fa_cdiv(Kd, 8) * 8;
  spectral_table_kernel<<<fa_cdiv((kp8 / 8) * kStepK * 64, 256), 256, 0, st>>>(tab, kp8, T);
  coef_colscale_kernel<<<dim3(fa_cdiv(Mc, 64), B), 1024, 0, st>>>(c, scale, inv, 2 * N, Mc);
  dim3 pgrid(pl.KS32, fa_cdiv(Mc, 256), B);
  spectral_pack_kernel<float><<<pgrid, 256, 0, st>>>(c, (int64_t)2 * N * Mc, Mc, nullptr, inv, pc, N, Mc, pl.CT, pl.KS32);
  spectral_pack_kernel<float><<<pgrid, 256, 0, st>>>(c + (int64_t)N * Mc, (int64_t)2 * N * Mc, Mc, nullptr, inv, ps, N, Mc,
                                                     pl.CT, pl.KS32);
  ReconStatsParams rp{};
  rp.tab = tab; rp.packed[0] = pc; rp.packed[1] = ps; rp.scale = scale;
  rp.psum = *psum; rp.pmax = *pmax; rp.pmin = *pmin;
  rp.B = B; rp.N = N; rp.Mc = Mc; rp.CT = pl.CT; rp.KS32 = pl.KS32; rp.K = K; rp.T = T; rp.n_steps = pl.n_steps; rp.RB = RBd;
  rp.Kd = Kd;
  rp.half = mirror ? T / 2 : 0x7fffffff;
  spectral_recon_stats_kernel<<<dim3(RBd, B), 256, 0, st>>>(rp);
  return RBd;
}
