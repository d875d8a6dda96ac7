// The elementwise steps of one decoder layer around the attention path, each as one launch: residual add +
// RMSNorm (modeling_llama_fourier.py:87-92, 735-750), rotary embedding of q and k (213-244), SwiGLU gate
// (277).  Every value is rounded where the reference's chain of tensor operations rounds it (each tensor op
// of a 16-bit model rounds its result to that type), so the results agree with that chain to the last bit
// except where a reduction order or an exponential differs in the last place.
#include "fa_common.h"
#include "fa_mfma_util.h"

namespace {

template <typename E> struct Rounder;
template <> struct Rounder<bf16_t> {
  static __device__ __forceinline__ bf16_t put(float v) { return bf16_t{fa_f32_to_bf16_bits(v)}; }
};
template <> struct Rounder<f16_t> {
  static __device__ __forceinline__ f16_t put(float v) { return f16_t{(_Float16)v}; }
};
template <> struct Rounder<float> {
  static __device__ __forceinline__ float put(float v) { return v; }
};
// through the storage type and back: what a tensor op leaves for the next one.  The value passes through an empty
// asm: the compiler otherwise contracts a product and the sum that follows into one multiply-add (fp32), or folds
// a conversion to half and back into a mixed-precision multiply-add (fp16) -- both skip exactly the rounding this
// function is for.
template <typename E>
__device__ __forceinline__ float rnd(float v) {
  float r = fa_to_float(Rounder<E>::put(v));
  asm("" : "+v"(r));
  return r;
}
template <>
__device__ __forceinline__ float rnd<f16_t>(float v) {
  _Float16 h = (_Float16)v;
  asm("" : "+v"(h));
  return (float)h;
}

// one block per row: h += delta (optional), y = weight * (h * rsqrt(mean(h^2) + eps)).to(dtype)
// W = elements per access: 16 bytes when the row length allows (rows then start 16-byte aligned), else one element
template <typename E, int W>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(E* __restrict__ h, const E* __restrict__ delta,
                                                           const E* __restrict__ weight, E* __restrict__ y, int hidden,
                                                           float eps) {
  struct alignas(sizeof(E) * W) Pack { E e[W]; };
  __shared__ float s_red[4];
  const int64_t row = blockIdx.x;
  Pack* hr = reinterpret_cast<Pack*>(h + row * hidden);
  const Pack* dr = delta ? reinterpret_cast<const Pack*>(delta + row * hidden) : nullptr;
  const Pack* wr = reinterpret_cast<const Pack*>(weight);
  Pack* yr = reinterpret_cast<Pack*>(y + row * hidden);
  constexpr int kIter = 8192 / (256 * W);   // hidden <= 8192; all indexing below is static (registers, no scratch)
  const int packs = hidden / W;
  float v[kIter][W];
  float ss = 0.f;
#pragma unroll
  for (int n = 0; n < kIter; ++n) {
    const int i = n * 256 + threadIdx.x;
    if (i < packs) {
      Pack a = hr[i];
      if (dr) {
        const Pack d = dr[i];
#pragma unroll
        for (int e = 0; e < W; ++e) a.e[e] = Rounder<E>::put(fa_to_float(a.e[e]) + fa_to_float(d.e[e]));
        hr[i] = a;
      }
#pragma unroll
      for (int e = 0; e < W; ++e) {
        v[n][e] = fa_to_float(a.e[e]);
        ss += v[n][e] * v[n][e];
      }
    }
  }
  ss = fa_wave_sum(ss);
  if ((threadIdx.x & 63) == 0) s_red[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float inv = rsqrtf((s_red[0] + s_red[1] + s_red[2] + s_red[3]) / (float)hidden + eps);
#pragma unroll
  for (int n = 0; n < kIter; ++n) {
    const int i = n * 256 + threadIdx.x;
    if (i < packs) {
      const Pack wv = wr[i];
      Pack o;
#pragma unroll
      for (int e = 0; e < W; ++e) o.e[e] = Rounder<E>::put(fa_to_float(wv.e[e]) * rnd<E>(v[n][e] * inv));
      yr[i] = o;
    }
  }
}

// grid (rows, Hq + Hkv), block D / 2: x <- x * cos + rotate_half(x) * sin on one head of q or k.  The rows of
// q_in and k may be slices of wider rows (a fused projection output); q goes out densely packed (q_out may be
// q_in when that is dense), k in place.
template <typename E>
__global__ void rope_qk_kernel(const E* q_in, int64_t q_stride, E* q_out, E* k, int64_t k_stride,
                               const E* __restrict__ cs, const E* __restrict__ sn, int Hq, int Hkv, int D) {
  const int64_t row = blockIdx.x;
  const int head = blockIdx.y, i = threadIdx.x, half = D >> 1;
  const E* src = head < Hq ? q_in + row * q_stride + head * D : k + row * k_stride + (head - Hq) * D;
  E* x = head < Hq ? q_out + (row * Hq + head) * D : k + row * k_stride + (head - Hq) * D;
  const float x1 = fa_to_float(src[i]), x2 = fa_to_float(src[i + half]);
  const float c1 = fa_to_float(cs[row * D + i]), c2 = fa_to_float(cs[row * D + i + half]);
  const float s1 = fa_to_float(sn[row * D + i]), s2 = fa_to_float(sn[row * D + i + half]);
  // rotate_half(x) = (-x2, x1)
  x[i] = Rounder<E>::put(rnd<E>(x1 * c1) + rnd<E>(-x2 * s1));
  x[i + half] = Rounder<E>::put(rnd<E>(x2 * c2) + rnd<E>(x1 * s2));
}

// The same on 16 bytes per thread (16-bit storage, D a multiple of 16, rows and pointers 16-byte aligned): one block
// per row walks over every (head, pair of 8-element pieces i / i + D/2); long prompts are bound by memory here.
template <typename E>
__global__ __launch_bounds__(256) void rope_qk_vec_kernel(const E* q_in, int64_t q_stride, E* q_out, E* k, int64_t k_stride,
                                                          const E* __restrict__ cs, const E* __restrict__ sn, int Hq, int Hkv,
                                                          int D) {
  struct alignas(16) Pack { E e[8]; };
  const int64_t row = blockIdx.x;
  const int half = D >> 1, per_head = half >> 3;
  for (int item = threadIdx.x; item < (Hq + Hkv) * per_head; item += 256) {
    const int head = item / per_head, i = (item - head * per_head) * 8;
    const E* src = head < Hq ? q_in + row * q_stride + head * D : k + row * k_stride + (head - Hq) * D;
    E* x = head < Hq ? q_out + (row * Hq + head) * D : k + row * k_stride + (head - Hq) * D;
    const Pack a1 = *(const Pack*)(src + i), a2 = *(const Pack*)(src + i + half);
    const Pack c1 = *(const Pack*)(cs + row * D + i), c2 = *(const Pack*)(cs + row * D + i + half);
    const Pack s1 = *(const Pack*)(sn + row * D + i), s2 = *(const Pack*)(sn + row * D + i + half);
    Pack o1, o2;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float x1 = fa_to_float(a1.e[e]), x2 = fa_to_float(a2.e[e]);
      o1.e[e] = Rounder<E>::put(rnd<E>(x1 * fa_to_float(c1.e[e])) + rnd<E>(-x2 * fa_to_float(s1.e[e])));
      o2.e[e] = Rounder<E>::put(rnd<E>(x2 * fa_to_float(c2.e[e])) + rnd<E>(x1 * fa_to_float(s2.e[e])));
    }
    *(Pack*)(x + i) = o1;
    *(Pack*)(x + i + half) = o2;
  }
}

// grid (column blocks, rows): gate and up rows may be slices of wider rows (a fused projection output)
template <typename E>
__global__ __launch_bounds__(256) void silu_mul_vec_kernel(const E* __restrict__ gate, const E* __restrict__ up,
                                                            E* __restrict__ out, int cols, int64_t in_stride) {
  struct alignas(16) Pack { E e[8]; };   // (16-bit storage: 16 bytes per thread)
  const int i = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (i >= cols) return;
  const int64_t row = blockIdx.y;
  const Pack g8 = *(const Pack*)(gate + row * in_stride + i), u8 = *(const Pack*)(up + row * in_stride + i);
  Pack o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float g = fa_to_float(g8.e[e]);
    o.e[e] = Rounder<E>::put(rnd<E>(g / (1.0f + expf(-g))) * fa_to_float(u8.e[e]));
  }
  *(Pack*)(out + row * cols + i) = o;
}

template <typename E>
__global__ __launch_bounds__(256) void silu_mul_kernel(const E* __restrict__ gate, const E* __restrict__ up,
                                                        E* __restrict__ out, int cols, int64_t in_stride) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= cols) return;
  const int64_t row = blockIdx.y;
  const float g = fa_to_float(gate[row * in_stride + i]);
  out[row * cols + i] = Rounder<E>::put(rnd<E>(g / (1.0f + expf(-g))) * fa_to_float(up[row * in_stride + i]));
}

// ---------------------------------------------------------------------------------------------------------
// Projections of a decode step: out[rows <= 16][n_out] = x[rows][K] . W[n_out][K]^T (nn.Linear without bias,
// modeling_llama_fourier.py:283, 597-599, 665).  With a handful of rows the product is a stream over the weights,
// so they are kept in the order the matrix cores take them: fragment (tile of 16 output features, step of 32 input
// features) = 64 lanes x 8 elements, lane (lg, lc) holding W[16 tile + lc][32 step + 8 lg ..] - every load is one
// contiguous KiB and goes straight into an MFMA as the A operand.  A workgroup owns one tile of 16 output features;
// its eight waves share the input features, keep two groups of four fragments in flight each, and meet in LDS.
// ---------------------------------------------------------------------------------------------------------
constexpr int kLinWaves = 8, kLinGroup = 4;

template <typename E>
__global__ __launch_bounds__(256) void linear_pack_kernel(const E* __restrict__ w, E* __restrict__ packed, int n_out, int K) {
  struct alignas(16) Pack { E e[8]; };
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;   // one 16-byte piece: (tile, step, lane)
  const int KS = K >> 5;
  if (idx >= (int64_t)(n_out >> 4) * KS * 64) return;
  const int lane = (int)(idx & 63), lg = lane >> 4, lc = lane & 15;
  const int64_t frag = idx >> 6;
  const int ks = (int)(frag % KS);
  const int64_t tile = frag / KS;
  *(Pack*)(packed + idx * 8) = *(const Pack*)(w + (tile * 16 + lc) * K + ks * 32 + 8 * lg);
}

template <typename E>
__global__ __launch_bounds__(64 * kLinWaves) void linear_packed_kernel(const E* __restrict__ x, int64_t x_rs,
                                                                        const E* __restrict__ wp, E* __restrict__ out,
                                                                        int rows, int K, int n_out) {
  using M = fa_mfma::Mma<E>;
  using vec8 = typename M::vec8;
  using fa_mfma::float4v;
  using fa_mfma::uint4v;
  __shared__ float4v s_part[kLinWaves][64];
  const int tid = threadIdx.x, lane = tid & 63, lg = lane >> 4, lc = lane & 15;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int tile = blockIdx.x;
  const int KS = K >> 5, per_wave = KS / kLinWaves, n_groups = per_wave / kLinGroup;
  const bool row_ok = lc < rows;
  const uint4v* a_ptr = (const uint4v*)wp + ((int64_t)tile * KS + w * per_wave) * 64 + lane;
  const E* b_row = x + (int64_t)(row_ok ? lc : 0) * x_rs + w * per_wave * 32 + 8 * lg;
  float4v acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
  uint4v A0[kLinGroup], B0[kLinGroup], A1[kLinGroup], B1[kLinGroup];
  auto load = [&](int g, uint4v (&A)[kLinGroup], uint4v (&B)[kLinGroup]) {
#pragma unroll
    for (int i = 0; i < kLinGroup; ++i) {
      A[i] = __builtin_nontemporal_load(a_ptr + (int64_t)(g * kLinGroup + i) * 64);   // read once: keep it out of the caches
      B[i] = *(const uint4v*)(b_row + (g * kLinGroup + i) * 32);
    }
  };
  auto compute = [&](uint4v (&A)[kLinGroup], uint4v (&B)[kLinGroup]) {
#pragma unroll
    for (int i = 0; i < kLinGroup; ++i) {
      uint4v b = B[i];
      if (!row_ok) b = uint4v{0u, 0u, 0u, 0u};   // columns past the rows: the clamped row must not reach the result
      if (i & 1) acc1 = M::mma(__builtin_bit_cast(vec8, A[i]), __builtin_bit_cast(vec8, b), acc1);
      else acc0 = M::mma(__builtin_bit_cast(vec8, A[i]), __builtin_bit_cast(vec8, b), acc0);
    }
  };
  load(0, A0, B0);
  for (int g = 0; g < n_groups; g += 2) {
    if (g + 1 < n_groups) load(g + 1, A1, B1);
    compute(A0, B0);
    if (g + 2 < n_groups) load(g + 2, A0, B0);
    if (g + 1 < n_groups) compute(A1, B1);
  }
  s_part[w][lane] = acc0 + acc1;
  __syncthreads();
  if (w == 0 && row_ok) {
    float4v s = s_part[0][lane];
#pragma unroll
    for (int i = 1; i < kLinWaves; ++i) s += s_part[i][lane];
    // lane (lg, lc) holds the output features 4 lg .. 4 lg + 3 of the tile for row lc
    struct alignas(sizeof(E) * 4) Quad { E e[4]; } o;
    o.e[0] = Rounder<E>::put(s.x); o.e[1] = Rounder<E>::put(s.y);
    o.e[2] = Rounder<E>::put(s.z); o.e[3] = Rounder<E>::put(s.w);
    *(Quad*)(out + (int64_t)lc * n_out + tile * 16 + 4 * lg) = o;
  }
}

template <typename F>
int by_dtype(int dtype, const char* what, F&& f) {
  switch (dtype) {
    case FA_BF16: f(bf16_t{}); return FA_OK;
    case FA_FP16: f(f16_t{}); return FA_OK;
    case FA_FP32: f(float{}); return FA_OK;
    default: fa_set_error("%s: dtype %d", what, dtype); return FA_ERR_BAD_DTYPE;
  }
}

}  // namespace

extern "C" int fa_add_rmsnorm(void* h, const void* delta, const void* weight, void* y, int rows, int hidden, float eps,
                              int dtype, fa_stream_t stream) {
  FA_REQUIRE(h && weight && y, FA_ERR_NULL_POINTER, "fa_add_rmsnorm: null pointer");
  FA_REQUIRE(rows >= 0 && hidden > 0 && hidden <= 8192, FA_ERR_BAD_SHAPE, "fa_add_rmsnorm: rows=%d hidden=%d (at most 8192)",
             rows, hidden);
  if (rows == 0) return FA_OK;
  hipStream_t st = fa_hip_stream(stream);
  int rc = by_dtype(dtype, "fa_add_rmsnorm", [&](auto tag) {
    using E = decltype(tag);
    constexpr int kVec = 16 / (int)sizeof(E);
    const bool vec = hidden % kVec == 0 && (((uintptr_t)h | (uintptr_t)delta | (uintptr_t)weight | (uintptr_t)y) & 15) == 0;
    if (vec) add_rmsnorm_kernel<E, kVec><<<rows, 256, 0, st>>>((E*)h, (const E*)delta, (const E*)weight, (E*)y, hidden, eps);
    else add_rmsnorm_kernel<E, 1><<<rows, 256, 0, st>>>((E*)h, (const E*)delta, (const E*)weight, (E*)y, hidden, eps);
  });
  return rc != FA_OK ? rc : fa_check_launch("fa_add_rmsnorm");
}

extern "C" int fa_rope_qk(const void* q_in, int64_t q_in_stride, void* q_out, void* k, int64_t k_stride, const void* cos,
                          const void* sin, int rows, int Hq, int Hkv, int D, int dtype, fa_stream_t stream) {
  FA_REQUIRE(q_in && q_out && k && cos && sin, FA_ERR_NULL_POINTER, "fa_rope_qk: null pointer");
  FA_REQUIRE(rows >= 0 && Hq > 0 && Hkv > 0 && D > 0 && D % 2 == 0 && D <= 2048, FA_ERR_BAD_SHAPE,
             "fa_rope_qk: rows=%d Hq=%d Hkv=%d D=%d", rows, Hq, Hkv, D);
  FA_REQUIRE(q_in_stride >= (int64_t)Hq * D && k_stride >= (int64_t)Hkv * D, FA_ERR_BAD_SHAPE,
             "fa_rope_qk: row strides %lld, %lld shorter than the rows", (long long)q_in_stride, (long long)k_stride);
  // (a single row is dense whatever stride its view reports: the q slice of one token's fused q/k/v projection)
  FA_REQUIRE(q_out != q_in || rows <= 1 || q_in_stride == (int64_t)Hq * D, FA_ERR_BAD_SHAPE,
             "fa_rope_qk: in place needs densely packed q rows");
  if (rows == 0) return FA_OK;
  hipStream_t st = fa_hip_stream(stream);
  int rc = by_dtype(dtype, "fa_rope_qk", [&](auto tag) {
    using E = decltype(tag);
    if constexpr (sizeof(E) == 2) {
      const uintptr_t ptrs = (uintptr_t)q_in | (uintptr_t)q_out | (uintptr_t)k | (uintptr_t)cos | (uintptr_t)sin;
      // (a decode step has too few rows to fill the device with one block per row: those keep one block per head)
      if (rows >= 64 && D % 16 == 0 && (ptrs & 15) == 0 && q_in_stride % 8 == 0 && k_stride % 8 == 0) {
        rope_qk_vec_kernel<E><<<rows, 256, 0, st>>>((const E*)q_in, q_in_stride, (E*)q_out, (E*)k, k_stride, (const E*)cos,
                                                    (const E*)sin, Hq, Hkv, D);
        return;
      }
    }
    rope_qk_kernel<E><<<dim3(rows, Hq + Hkv), D / 2, 0, st>>>((const E*)q_in, q_in_stride, (E*)q_out, (E*)k, k_stride,
                                                              (const E*)cos, (const E*)sin, Hq, Hkv, D);
  });
  return rc != FA_OK ? rc : fa_check_launch("fa_rope_qk");
}

extern "C" int fa_silu_mul(const void* gate, const void* up, void* out, int rows, int cols, int64_t in_stride, int dtype,
                           fa_stream_t stream) {
  FA_REQUIRE(gate && up && out, FA_ERR_NULL_POINTER, "fa_silu_mul: null pointer");
  FA_REQUIRE(rows >= 0 && cols >= 0 && rows <= 65535 && in_stride >= cols, FA_ERR_BAD_SHAPE,
             "fa_silu_mul: rows=%d cols=%d stride=%lld", rows, cols, (long long)in_stride);
  if (rows == 0 || cols == 0) return FA_OK;
  hipStream_t st = fa_hip_stream(stream);
  int rc = by_dtype(dtype, "fa_silu_mul", [&](auto tag) {
    using E = decltype(tag);
    if constexpr (sizeof(E) == 2) {
      if (cols % 8 == 0 && in_stride % 8 == 0 && (((uintptr_t)gate | (uintptr_t)up | (uintptr_t)out) & 15) == 0) {
        silu_mul_vec_kernel<E><<<dim3(fa_cdiv(cols / 8, 256), rows), 256, 0, st>>>((const E*)gate, (const E*)up, (E*)out,
                                                                                cols, in_stride);
        return;
      }
    }
    silu_mul_kernel<E><<<dim3(fa_cdiv(cols, 256), rows), 256, 0, st>>>((const E*)gate, (const E*)up, (E*)out, cols, in_stride);
  });
  return rc != FA_OK ? rc : fa_check_launch("fa_silu_mul");
}

extern "C" int fa_linear_pack(const void* w, void* packed, int n_out, int K, int dtype, fa_stream_t stream) {
  FA_REQUIRE(w && packed, FA_ERR_NULL_POINTER, "fa_linear_pack: null pointer");
  FA_REQUIRE(n_out > 0 && K > 0 && n_out % 16 == 0 && K % 32 == 0, FA_ERR_BAD_SHAPE,
             "fa_linear_pack: n_out=%d (multiple of 16) K=%d (multiple of 32)", n_out, K);
  FA_REQUIRE(dtype == FA_BF16 || dtype == FA_FP16, FA_ERR_BAD_DTYPE, "fa_linear_pack: dtype %d (16-bit storage only)", dtype);
  FA_REQUIRE((((uintptr_t)w | (uintptr_t)packed) & 15) == 0, FA_ERR_MISALIGNED, "fa_linear_pack: pointers not 16-byte aligned");
  hipStream_t st = fa_hip_stream(stream);
  const int64_t pieces = (int64_t)(n_out / 16) * (K / 32) * 64;
  by_dtype(dtype, "fa_linear_pack", [&](auto tag) {
    using E = decltype(tag);
    if constexpr (sizeof(E) == 2)
      linear_pack_kernel<E><<<(unsigned)fa_cdiv(pieces, (int64_t)256), 256, 0, st>>>((const E*)w, (E*)packed, n_out, K);
  });
  return fa_check_launch("fa_linear_pack");
}

extern "C" int fa_linear_packed_ok(int rows, int K, int n_out) {
  return rows >= 1 && rows <= 16 && n_out > 0 && n_out % 16 == 0 && K > 0 && K % (32 * kLinWaves * kLinGroup) == 0;
}

extern "C" int fa_linear_packed(const void* x, int64_t x_row_stride, const void* w_packed, void* out, int rows, int K,
                                int n_out, int dtype, fa_stream_t stream) {
  FA_REQUIRE(x && w_packed && out, FA_ERR_NULL_POINTER, "fa_linear_packed: null pointer");
  FA_REQUIRE(fa_linear_packed_ok(rows, K, n_out), FA_ERR_UNSUPPORTED,
             "fa_linear_packed: rows=%d (1..16) K=%d (multiple of %d) n_out=%d (multiple of 16)", rows, K,
             32 * kLinWaves * kLinGroup, n_out);
  FA_REQUIRE(dtype == FA_BF16 || dtype == FA_FP16, FA_ERR_BAD_DTYPE, "fa_linear_packed: dtype %d (16-bit storage only)", dtype);
  FA_REQUIRE(x_row_stride >= K && x_row_stride % 8 == 0 && (((uintptr_t)x | (uintptr_t)w_packed | (uintptr_t)out) & 15) == 0,
             FA_ERR_MISALIGNED, "fa_linear_packed: rows of x / pointers not 16-byte aligned");
  hipStream_t st = fa_hip_stream(stream);
  by_dtype(dtype, "fa_linear_packed", [&](auto tag) {
    using E = decltype(tag);
    if constexpr (sizeof(E) == 2)
      linear_packed_kernel<E><<<n_out / 16, 64 * kLinWaves, 0, st>>>((const E*)x, x_row_stride, (const E*)w_packed, (E*)out,
                                                                    rows, K, n_out);
  });
  return fa_check_launch("fa_linear_packed");
}
