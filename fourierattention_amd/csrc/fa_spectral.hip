// Spectral compression, its statistics, reconstruction and the rank-1 update:
// straightforward wave64 VALU kernels that accept any shape.  The basis is never
// read from memory: each thread carries e^{i*theta} factors forward with a complex
// rotation and re-seeds them from an exactly reduced integer phase every 64 steps.
#include "fa_common.h"

namespace {

constexpr int kReseed = 64;

// ---------------------------------------------------------------------------
// c[b, n, m] (+)= sum_k cos(2 pi (k + k_start) n / T) a[b, k, m]   (sin rows at N + n)
// block = 64 column lanes x 4 frequency groups; thread owns MT columns x NT frequencies
// ---------------------------------------------------------------------------
template <typename E, int MT, int NT>
__global__ __launch_bounds__(256) void mat_fourier_kernel(
    const E* __restrict__ a, int64_t a_bs, int64_t a_rs, const int32_t* __restrict__ cols,
    float* __restrict__ c, int K, int Mc, int N, int T, int64_t k_start, int accumulate) {
  const int lane = threadIdx.x & 63;
  const int ng = threadIdx.x >> 6;
  const int b = blockIdx.z;
  const int m_base = blockIdx.x * (64 * MT) + lane;
  const int n_base = blockIdx.y * (4 * NT) + ng * NT;

  int col[MT];
  bool mok[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    int m = m_base + 64 * i;
    mok[i] = m < Mc;
    col[i] = mok[i] ? (cols ? cols[m] : m) : 0;
  }
  float acc_c[NT][MT], acc_s[NT][MT], zr[NT], zi[NT], sr[NT], si[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    int n = n_base + j;
    fa_sincos_phase(n, 1, T, &si[j], &sr[j]);
    zr[j] = 1.f;
    zi[j] = 0.f;
#pragma unroll
    for (int i = 0; i < MT; ++i) acc_c[j][i] = acc_s[j][i] = 0.f;
  }
  const E* ab = a + (int64_t)b * a_bs;
  for (int k = 0; k < K; ++k) {
    if ((k % kReseed) == 0) {
#pragma unroll
      for (int j = 0; j < NT; ++j) fa_sincos_phase(n_base + j, k + k_start, T, &zi[j], &zr[j]);
    }
    float av[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) av[i] = mok[i] ? fa_to_float(ab[(int64_t)k * a_rs + col[i]]) : 0.f;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        acc_c[j][i] = fmaf(zr[j], av[i], acc_c[j][i]);
        acc_s[j][i] = fmaf(zi[j], av[i], acc_s[j][i]);
      }
      float nr = zr[j] * sr[j] - zi[j] * si[j];
      float ni = zr[j] * si[j] + zi[j] * sr[j];
      zr[j] = nr;
      zi[j] = ni;
    }
  }
  float* cb = c + (int64_t)b * 2 * N * Mc;
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    int n = n_base + j;
    if (n >= N) continue;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      if (!mok[i]) continue;
      int m = m_base + 64 * i;
      float* pc = cb + (int64_t)n * Mc + m;
      float* ps = cb + (int64_t)(N + n) * Mc + m;
      if (accumulate) {
        *pc += acc_c[j][i];
        *ps += acc_s[j][i];
      } else {
        *pc = acc_c[j][i];
        *ps = acc_s[j][i];
      }
    }
  }
}

// ---------------------------------------------------------------------------
// column statistics of the original signal: partial sum / max / min per k-split
// ---------------------------------------------------------------------------
template <typename E>
__global__ __launch_bounds__(256) void col_stats_partial_kernel(
    const E* __restrict__ a, int64_t a_bs, int64_t a_rs, const int32_t* __restrict__ cols,
    float* __restrict__ psum, float* __restrict__ pmax, float* __restrict__ pmin, int K, int Mc,
    int rows_per_split, int nsplit) {
  __shared__ float s_sum[4][64], s_max[4][64], s_min[4][64];
  const int lane = threadIdx.x & 63, kg = threadIdx.x >> 6;
  const int m = blockIdx.x * 64 + lane;
  const int split = blockIdx.y, b = blockIdx.z;
  const int k0 = split * rows_per_split;
  const int k1 = min(K, k0 + rows_per_split);
  float sum = 0.f, mx = -INFINITY, mn = INFINITY;
  if (m < Mc) {
    const int col = cols ? cols[m] : m;
    const E* p = a + (int64_t)b * a_bs + col;
    // eight rows in flight per thread (clamped, so that none of the loads is conditional)
    for (int k = k0 + kg; k < k1; k += 4 * 8) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = fa_to_float(p[(int64_t)min(k + 4 * u, k1 - 1) * a_rs]);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (k + 4 * u < k1) {
          sum += v[u];
          mx = fmaxf(mx, v[u]);
          mn = fminf(mn, v[u]);
        }
    }
  }
  s_sum[kg][lane] = sum;
  s_max[kg][lane] = mx;
  s_min[kg][lane] = mn;
  __syncthreads();
  if (kg == 0 && m < Mc) {
    for (int g = 1; g < 4; ++g) {
      sum += s_sum[g][lane];
      mx = fmaxf(mx, s_max[g][lane]);
      mn = fminf(mn, s_min[g][lane]);
    }
    int64_t o = ((int64_t)b * nsplit + split) * Mc + m;
    psum[o] = sum;
    pmax[o] = mx;
    pmin[o] = mn;
  }
}

__global__ __launch_bounds__(256) void stats_finalize_kernel(
    const float* __restrict__ psum, const float* __restrict__ pmax, const float* __restrict__ pmin,
    float* __restrict__ avg, float* __restrict__ dev, int K, int Mc, int nsplit, int round_dtype) {
  // block = 64 columns x 4 classes of splits, eight splits in flight per thread
  __shared__ float s_red[3][4][64];
  const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int m = blockIdx.x * 64 + lane, b = blockIdx.y;
  float sum = 0.f, mx = -INFINITY, mn = INFINITY;
  if (m < Mc) {
    for (int s0 = g; s0 < nsplit; s0 += 4 * 8) {
      float a[8], x[8], n[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int64_t o = ((int64_t)b * nsplit + min(s0 + 4 * u, nsplit - 1)) * Mc + m;
        a[u] = psum[o];
        x[u] = pmax[o];
        n[u] = pmin[o];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + 4 * u < nsplit) {
          sum += a[u];
          mx = fmaxf(mx, x[u]);
          mn = fminf(mn, n[u]);
        }
    }
  }
  s_red[0][g][lane] = sum;
  s_red[1][g][lane] = mx;
  s_red[2][g][lane] = mn;
  __syncthreads();
  if (g != 0 || m >= Mc) return;
  for (int i = 1; i < 4; ++i) {
    sum += s_red[0][i][lane];
    mx = fmaxf(mx, s_red[1][i][lane]);
    mn = fminf(mn, s_red[2][i][lane]);
  }
  float av = sum / (float)K;
  float dv = fmaxf(mx - av, av - mn);
  avg[(int64_t)b * Mc + m] = fa_round_through(av, round_dtype);
  dev[(int64_t)b * Mc + m] = fa_round_through(dv, round_dtype);
}

// ---------------------------------------------------------------------------
// reconstruction r[b,k,m] = (1/N) sum_n cos(2 pi k n/T) c[b,n,m] + sin(..) c[b,N+n,m]
// thread = one position k, MB columns in registers; coefficient chunks staged in LDS.
// STATS: reduce over the block's 256 positions to partial sum/max/min; else store r
// (optionally through the affine (r - avg_d) * scale + avg_u).
// ---------------------------------------------------------------------------
template <bool STATS, int MB>
__global__ __launch_bounds__(256) void reconstruct_kernel(
    const float* __restrict__ c, int N, int Mc, int K, int T,
    float* __restrict__ psum, float* __restrict__ pmax, float* __restrict__ pmin, int nsplit,
    float* __restrict__ r_out, const float* __restrict__ avg_u, const float* __restrict__ avg_d,
    const float* __restrict__ scale) {
  constexpr int NC = 64;
  __shared__ float s_c[NC][MB], s_s[NC][MB];
  __shared__ float s_red[3][4][MB];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.x * MB;
  const int kb = blockIdx.y, b = blockIdx.z;
  const int k = kb * 256 + tid;
  const bool kok = k < K;
  const float* cb = c + (int64_t)b * 2 * N * Mc;

  float acc[MB];
#pragma unroll
  for (int i = 0; i < MB; ++i) acc[i] = 0.f;
  float sr, si;
  fa_sincos_phase(k, 1, T, &si, &sr);

  for (int n0 = 0; n0 < N; n0 += NC) {
    __syncthreads();
    for (int e = tid; e < NC * MB; e += 256) {
      int nn = e / MB, mm = e % MB;
      int n = n0 + nn, m = m0 + mm;
      bool ok = (n < N) && (m < Mc);
      s_c[nn][mm] = ok ? cb[(int64_t)n * Mc + m] : 0.f;
      s_s[nn][mm] = ok ? cb[(int64_t)(N + n) * Mc + m] : 0.f;
    }
    __syncthreads();
    float zr, zi;
    fa_sincos_phase(k, n0, T, &zi, &zr);
    for (int nn = 0; nn < NC; ++nn) {
#pragma unroll
      for (int i = 0; i < MB; ++i) acc[i] = fmaf(zr, s_c[nn][i], fmaf(zi, s_s[nn][i], acc[i]));
      float nr = zr * sr - zi * si;
      float ni = zr * si + zi * sr;
      zr = nr;
      zi = ni;
    }
  }
  const float inv_n = 1.0f / (float)N;
  if (!STATS) {
    if (kok) {
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        int m = m0 + i;
        if (m >= Mc) break;
        float v = acc[i] * inv_n;
        if (scale) {
          int64_t o = (int64_t)b * Mc + m;
          v = (v - avg_d[o]) * scale[o] + avg_u[o];
        }
        r_out[((int64_t)b * K + k) * Mc + m] = v;
      }
    }
    return;
  }
  const int lane = tid & 63, w = tid >> 6;
#pragma unroll
  for (int i = 0; i < MB; ++i) {
    float v = acc[i] * inv_n;
    float s = fa_wave_sum(kok ? v : 0.f);
    float mx = fa_wave_max(kok ? v : -INFINITY);
    float mn = fa_wave_min(kok ? v : INFINITY);
    if (lane == 0) {
      s_red[0][w][i] = s;
      s_red[1][w][i] = mx;
      s_red[2][w][i] = mn;
    }
  }
  __syncthreads();
  if (tid < MB && m0 + tid < Mc) {
    float s = 0.f, mx = -INFINITY, mn = INFINITY;
    for (int g = 0; g < 4; ++g) {
      s += s_red[0][g][tid];
      mx = fmaxf(mx, s_red[1][g][tid]);
      mn = fminf(mn, s_red[2][g][tid]);
    }
    int64_t o = ((int64_t)b * nsplit + kb) * Mc + m0 + tid;
    psum[o] = s;
    pmax[o] = mx;
    pmin[o] = mn;
  }
}

// ---------------------------------------------------------------------------
// rank-1 update: c[b,n,m] += cos(2 pi p n/T) row[b, cols[m]]
// ---------------------------------------------------------------------------
template <typename E>
__global__ __launch_bounds__(256) void coeff_update_kernel(
    float* __restrict__ c, const E* __restrict__ row, int64_t row_bs, const int32_t* __restrict__ cols,
    int N, int Mc, int64_t p, int T) {
  // block = 64 columns x 64 frequencies, thread = (column, 16 frequencies).  The phase factors depend on the
  // frequency only: 64 threads evaluate one each while the coefficient loads are on their way.
  __shared__ float2 s_cs[64];
  const int tid = threadIdx.x, lane = tid & 63, ng = tid >> 6;
  const int m = blockIdx.x * 64 + lane, b = blockIdx.z;
  const bool live = m < Mc;
  const int n_beg = blockIdx.y * 64;
  const int n_end = min(N, n_beg + 64);
  float e = 0.f;
  float* cb = c + (int64_t)b * 2 * N * Mc + (live ? m : 0);
  float cv[16], sv[16];
  if (live) {
    e = fa_to_float(row[(int64_t)b * row_bs + (cols ? cols[m] : m)]);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int n = min(n_beg + ng + 4 * i, N - 1);
      cv[i] = cb[(int64_t)n * Mc];
      sv[i] = cb[(int64_t)(N + n) * Mc];
    }
  }
  if (tid < 64) {
    float sn, co;
    fa_sincos_phase(min(n_beg + tid, N - 1), p, T, &sn, &co);
    s_cs[tid] = make_float2(co, sn);
  }
  __syncthreads();
  if (live) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int n = n_beg + ng + 4 * i;
      if (n < n_end) {
        const float2 cs = s_cs[ng + 4 * i];
        cb[(int64_t)n * Mc] = cv[i] + cs.x * e;
        cb[(int64_t)(N + n) * Mc] = sv[i] + cs.y * e;
      }
    }
  }
}

int stats_splits(int K) { return K <= 0 ? 1 : fa_cdiv(K, 256); }

}  // namespace

void fa_stats_finalize_launch(const float* psum, const float* pmax, const float* pmin, float* avg, float* dev, int B, int K,
                              int Mc, int nsplit, int round_dtype, hipStream_t st) {
  stats_finalize_kernel<<<dim3(fa_cdiv(Mc, 64), B), 256, 0, st>>>(psum, pmax, pmin, avg, dev, K, Mc, nsplit, round_dtype);
}

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------
extern "C" size_t fa_stats_workspace_bytes(int B, int Mc, int K) {
  if (B <= 0 || Mc <= 0 || K <= 0) return 0;
  return (size_t)3 * B * stats_splits(K) * Mc * sizeof(float);
}

extern "C" int fa_mat_fourier(const void* a, int a_dtype, int64_t a_bs, int64_t a_rs, const int32_t* cols,
                              float* c, int B, int K, int Mc, int N, int T, int64_t k_start, int accumulate,
                              void* workspace, size_t workspace_bytes, fa_stream_t stream) {
  FA_REQUIRE(a && c, FA_ERR_NULL_POINTER, "fa_mat_fourier: null pointer");
  FA_REQUIRE(B > 0 && K >= 0 && Mc > 0 && N > 0 && T > 0, FA_ERR_BAD_SHAPE,
             "fa_mat_fourier: bad shape B=%d K=%d Mc=%d N=%d T=%d", B, K, Mc, N, T);
  FA_REQUIRE(a_dtype == FA_BF16 || a_dtype == FA_FP16 || a_dtype == FA_FP32, FA_ERR_BAD_DTYPE, "fa_mat_fourier: dtype %d",
             a_dtype);
  if (workspace && ((uintptr_t)c & 15) == 0 && fa_spectral_mfma_ok(a_dtype, K, Mc, N) &&
      workspace_bytes >= fa_spectral_mfma_workspace(B, K, Mc, N)) {
    FA_REQUIRE(((uintptr_t)workspace & 255) == 0, FA_ERR_MISALIGNED, "fa_mat_fourier: workspace not 256-byte aligned");
    return fa_spectral_mfma_launch(a, a_dtype, a_bs, a_rs, cols, c, B, K, Mc, N, T, k_start, accumulate, workspace,
                                   fa_hip_stream(stream));
  }
  constexpr int MT = 4, NT = 8;
  dim3 grid(fa_cdiv(Mc, 64 * MT), fa_cdiv(N, 4 * NT), B), block(256);
  hipStream_t s = fa_hip_stream(stream);
  switch (a_dtype) {
    case FA_BF16:
      mat_fourier_kernel<bf16_t, MT, NT><<<grid, block, 0, s>>>((const bf16_t*)a, a_bs, a_rs, cols, c, K, Mc, N, T, k_start, accumulate);
      break;
    case FA_FP16:
      mat_fourier_kernel<f16_t, MT, NT><<<grid, block, 0, s>>>((const f16_t*)a, a_bs, a_rs, cols, c, K, Mc, N, T, k_start, accumulate);
      break;
    case FA_FP32:
      mat_fourier_kernel<float, MT, NT><<<grid, block, 0, s>>>((const float*)a, a_bs, a_rs, cols, c, K, Mc, N, T, k_start, accumulate);
      break;
    default:
      FA_REQUIRE(false, FA_ERR_BAD_DTYPE, "fa_mat_fourier: dtype %d", a_dtype);
  }
  return fa_check_launch("fa_mat_fourier");
}

extern "C" size_t fa_mat_fourier_workspace_bytes(int a_dtype, int B, int K, int Mc, int N) {
  if (B <= 0 || K <= 0 || Mc <= 0 || N <= 0 || !fa_spectral_mfma_ok(a_dtype, K, Mc, N)) return 0;
  return fa_spectral_mfma_workspace(B, K, Mc, N);
}

extern "C" int fa_mat_avg_std(const void* a, int a_dtype, int64_t a_bs, int64_t a_rs, const int32_t* cols,
                              float* avg, float* max_dev, int B, int K, int Mc, int round_dtype,
                              void* workspace, size_t workspace_bytes, fa_stream_t stream) {
  FA_REQUIRE(a && avg && max_dev, FA_ERR_NULL_POINTER, "fa_mat_avg_std: null pointer");
  FA_REQUIRE(B > 0 && K > 0 && Mc > 0, FA_ERR_BAD_SHAPE, "fa_mat_avg_std: bad shape B=%d K=%d Mc=%d", B, K, Mc);
  FA_REQUIRE(workspace && workspace_bytes >= fa_stats_workspace_bytes(B, Mc, K), FA_ERR_WORKSPACE,
             "fa_mat_avg_std: workspace %zu < %zu", workspace_bytes, fa_stats_workspace_bytes(B, Mc, K));
  const int nsplit = stats_splits(K);
  float* psum = (float*)workspace;
  float* pmax = psum + (size_t)B * nsplit * Mc;
  float* pmin = pmax + (size_t)B * nsplit * Mc;
  dim3 grid(fa_cdiv(Mc, 64), nsplit, B), block(256);
  hipStream_t s = fa_hip_stream(stream);
  switch (a_dtype) {
    case FA_BF16:
      col_stats_partial_kernel<bf16_t><<<grid, block, 0, s>>>((const bf16_t*)a, a_bs, a_rs, cols, psum, pmax, pmin, K, Mc, 256, nsplit);
      break;
    case FA_FP16:
      col_stats_partial_kernel<f16_t><<<grid, block, 0, s>>>((const f16_t*)a, a_bs, a_rs, cols, psum, pmax, pmin, K, Mc, 256, nsplit);
      break;
    case FA_FP32:
      col_stats_partial_kernel<float><<<grid, block, 0, s>>>((const float*)a, a_bs, a_rs, cols, psum, pmax, pmin, K, Mc, 256, nsplit);
      break;
    default:
      FA_REQUIRE(false, FA_ERR_BAD_DTYPE, "fa_mat_avg_std: dtype %d", a_dtype);
  }
  stats_finalize_kernel<<<dim3(fa_cdiv(Mc, 64), B), 256, 0, s>>>(psum, pmax, pmin, avg, max_dev, K, Mc, nsplit, round_dtype);
  return fa_check_launch("fa_mat_avg_std");
}

extern "C" size_t fa_mat_fourier_avg_std_workspace_bytes(int B, int N, int Mc, int K) {
  if (B <= 0 || N <= 0 || Mc <= 0 || K <= 0) return 0;
  size_t a = fa_stats_workspace_bytes(B, Mc, K);
  if (fa_recon_stats_mfma_ok(N, Mc, K)) {
    const size_t m = fa_recon_stats_mfma_workspace(B, N, Mc, K);
    if (m > a) a = m;
  }
  return a;
}

extern "C" int fa_mat_fourier_avg_std(const float* c, float* avg, float* max_dev, int B, int N, int Mc, int K,
                                      int T, int round_dtype, void* workspace, size_t workspace_bytes,
                                      fa_stream_t stream) {
  FA_REQUIRE(c && avg && max_dev, FA_ERR_NULL_POINTER, "fa_mat_fourier_avg_std: null pointer");
  FA_REQUIRE(B > 0 && N > 0 && Mc > 0 && K > 0 && T > 0, FA_ERR_BAD_SHAPE,
             "fa_mat_fourier_avg_std: bad shape B=%d N=%d Mc=%d K=%d T=%d", B, N, Mc, K, T);
  FA_REQUIRE(workspace && workspace_bytes >= fa_stats_workspace_bytes(B, Mc, K), FA_ERR_WORKSPACE,
             "fa_mat_fourier_avg_std: workspace %zu < %zu", workspace_bytes, fa_stats_workspace_bytes(B, Mc, K));
  hipStream_t s = fa_hip_stream(stream);
  if (fa_recon_stats_mfma_ok(N, Mc, K) && workspace_bytes >= fa_recon_stats_mfma_workspace(B, N, Mc, K)) {
    FA_REQUIRE(((uintptr_t)workspace & 255) == 0, FA_ERR_MISALIGNED, "fa_mat_fourier_avg_std: workspace not 256-byte aligned");
    float *ps, *px, *pn;
    const int rb = fa_recon_stats_mfma_launch(c, B, N, Mc, K, T, workspace, &ps, &px, &pn, s);
    stats_finalize_kernel<<<dim3(fa_cdiv(Mc, 64), B), 256, 0, s>>>(ps, px, pn, avg, max_dev, K, Mc, rb, round_dtype);
    return fa_check_launch("fa_mat_fourier_avg_std");
  }
  const int nsplit = stats_splits(K);
  float* psum = (float*)workspace;
  float* pmax = psum + (size_t)B * nsplit * Mc;
  float* pmin = pmax + (size_t)B * nsplit * Mc;
  constexpr int MB = 32;
  reconstruct_kernel<true, MB><<<dim3(fa_cdiv(Mc, MB), nsplit, B), 256, 0, s>>>(
      c, N, Mc, K, T, psum, pmax, pmin, nsplit, nullptr, nullptr, nullptr, nullptr);
  stats_finalize_kernel<<<dim3(fa_cdiv(Mc, 64), B), 256, 0, s>>>(psum, pmax, pmin, avg, max_dev, K, Mc, nsplit, round_dtype);
  return fa_check_launch("fa_mat_fourier_avg_std");
}

extern "C" int fa_reconstruct(const float* c, const float* avg_u, const float* avg_d, const float* scale, float* r,
                              int B, int N, int Mc, int K, int T, fa_stream_t stream) {
  FA_REQUIRE(c && r, FA_ERR_NULL_POINTER, "fa_reconstruct: null pointer");
  FA_REQUIRE(B > 0 && N > 0 && Mc > 0 && K > 0 && T > 0, FA_ERR_BAD_SHAPE,
             "fa_reconstruct: bad shape B=%d N=%d Mc=%d K=%d T=%d", B, N, Mc, K, T);
  const bool affine = avg_u || avg_d || scale;
  FA_REQUIRE(!affine || (avg_u && avg_d && scale), FA_ERR_NULL_POINTER,
             "fa_reconstruct: avg_u, avg_d and scale must be given together");
  constexpr int MB = 32;
  reconstruct_kernel<false, MB><<<dim3(fa_cdiv(Mc, MB), fa_cdiv(K, 256), B), 256, 0, fa_hip_stream(stream)>>>(
      c, N, Mc, K, T, nullptr, nullptr, nullptr, 0, r, avg_u, avg_d, scale);
  return fa_check_launch("fa_reconstruct");
}

extern "C" int fa_coeff_update(float* c, const void* row, int row_dtype, int64_t row_bs, const int32_t* cols, int B,
                               int N, int Mc, int64_t p, int T, fa_stream_t stream) {
  FA_REQUIRE(c && row, FA_ERR_NULL_POINTER, "fa_coeff_update: null pointer");
  FA_REQUIRE(B > 0 && N > 0 && Mc >= 0 && T > 0, FA_ERR_BAD_SHAPE, "fa_coeff_update: bad shape B=%d N=%d Mc=%d T=%d", B, N, Mc, T);
  if (Mc == 0) return FA_OK;
  dim3 grid(fa_cdiv(Mc, 64), fa_cdiv(N, 64), B), block(256);
  hipStream_t s = fa_hip_stream(stream);
  switch (row_dtype) {
    case FA_BF16:
      coeff_update_kernel<bf16_t><<<grid, block, 0, s>>>(c, (const bf16_t*)row, row_bs, cols, N, Mc, p, T);
      break;
    case FA_FP16:
      coeff_update_kernel<f16_t><<<grid, block, 0, s>>>(c, (const f16_t*)row, row_bs, cols, N, Mc, p, T);
      break;
    case FA_FP32:
      coeff_update_kernel<float><<<grid, block, 0, s>>>(c, (const float*)row, row_bs, cols, N, Mc, p, T);
      break;
    default:
      FA_REQUIRE(false, FA_ERR_BAD_DTYPE, "fa_coeff_update: dtype %d", row_dtype);
  }
  return fa_check_launch("fa_coeff_update");
}
