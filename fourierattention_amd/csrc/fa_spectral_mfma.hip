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
    half8* __restrict__ out, int K, int Mc, int CT, int KS32) {
  constexpr int kPitch = 256 + 4;   // f16 elements per LDS row: 8 rows apart = 16 banks apart
  __shared__ _Float16 tile[32][kPitch];
  const int tid = threadIdx.x;
  const int ks = blockIdx.x, m0 = blockIdx.y * 256, b = blockIdx.z;
  const int m = m0 + tid;
  const bool mok = m < Mc;
  const int col = mok ? (cols ? cols[m] : m) : 0;
  const E* ab = a + (int64_t)b * a_bs + col;
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
    const float x = (mok && k < K) ? fminf(fmaxf(v[kk], -65504.f), 65504.f) : 0.f;
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

struct SpectralGemmParams {
  const half8* tab;      // basis table
  const half8* packed;   // [B][CT][KS32][64] fragments
  float* part;           // [S][B][2N][Mc]
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
          out[(int64_t)n * p.Mc + m] = co * c - sn * s_;
          out[(int64_t)(p.N + n) * p.Mc + m] = sn * c + co * s_;
        }
      }
    }
  }
}

__global__ __launch_bounds__(256) void spectral_reduce_kernel(const float* __restrict__ part, float* __restrict__ c,
                                                              int64_t total, int n_chunks, int accumulate) {
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= total) return;   // total is a multiple of 4 (Mc is even and 2N a multiple of 16)
  float4 a = accumulate ? *(const float4*)(c + i) : make_float4(0.f, 0.f, 0.f, 0.f);
  for (int s = 0; s < n_chunks; ++s) {
    const float4 v = *(const float4*)(part + (int64_t)s * total + i);
    a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
  }
  *(float4*)(c + i) = a;
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
  return (a_dtype == FA_BF16 || a_dtype == FA_FP16) && N % 8 == 0 && Mc % 2 == 0 && K >= 4 * fa_mfma::kStepTokens;
}

size_t fa_spectral_mfma_workspace(int B, int K, int Mc, int N) { return spectral_plan(B, K, Mc, N).total; }

int fa_spectral_mfma_launch(const void* a, int a_dtype, int64_t a_bs, int64_t a_rs, const int32_t* cols, float* c, int B,
                            int K, int Mc, int N, int T, int64_t k_start, int accumulate, void* workspace,
                            hipStream_t st) {
  using namespace fa_mfma;
  const SpectralPlan pl = spectral_plan(B, K, Mc, N);
  char* ws = (char*)workspace;
  half8* tab = (half8*)(ws + pl.off_tab);
  half8* packed = (half8*)(ws + pl.off_packed);
  float* part = (float*)(ws + pl.off_part);
  spectral_table_kernel<<<fa_cdiv((N / 8) * kStepK * 64, 256), 256, 0, st>>>(tab, N, T);
  dim3 pgrid(pl.KS32, fa_cdiv(Mc, 256), B);
  if (a_dtype == FA_BF16)
    spectral_pack_kernel<bf16_t><<<pgrid, 256, 0, st>>>((const bf16_t*)a, a_bs, a_rs, cols, packed, K, Mc, pl.CT, pl.KS32);
  else
    spectral_pack_kernel<f16_t><<<pgrid, 256, 0, st>>>((const f16_t*)a, a_bs, a_rs, cols, packed, K, Mc, pl.CT, pl.KS32);
  SpectralGemmParams gp{};
  gp.tab = tab; gp.packed = packed; gp.part = part;
  gp.B = B; gp.N = N; gp.Mc = Mc; gp.CT = pl.CT; gp.KS32 = pl.KS32; gp.T = T;
  gp.n_steps = pl.n_steps; gp.steps_per_chunk = pl.steps_per_chunk; gp.n_chunks = pl.n_chunks;
  gp.k_start = k_start;
  dim3 ggrid(fa_cdiv(Mc, kWgCols), fa_cdiv(N, kWgFreqs), B * pl.n_chunks);
  spectral_gemm_kernel<<<ggrid, 256, 0, st>>>(gp);
  const int64_t total = (int64_t)B * 2 * N * Mc;
  spectral_reduce_kernel<<<fa_cdiv(total / 4, 256), 256, 0, st>>>(part, c, total, pl.n_chunks, accumulate);
  return fa_check_launch("fa_mat_fourier");
}
