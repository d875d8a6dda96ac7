/*
 * fourier_attn_hip.h - C ABI of the MI355X (gfx950) Fourier KV-cache hot path.
 *
 * Every entry point takes plain device pointers and sizes, enqueues its work on
 * the given HIP stream and returns without synchronising.  Return value: 0 on
 * success, a negative FA_ERR_* code otherwise (fa_last_error_string() gives the
 * text of the last failure on the calling thread).  Nothing here allocates
 * device memory: scratch space is passed in by the caller and sized with the
 * matching *_workspace_bytes() function.
 *
 * Citations name the reference interface each entry point stands in for
 * (paths relative to the reference repository root):
 *   TRI   = fourier_attn_triton/fourier_triton_valid4_v2.py
 *   CACHE = fourier_attn_triton/cache_utils_fourier.py
 *   MODEL = fourier_attn_triton/modeling_llama_fourier.py
 */
#ifndef FOURIER_ATTN_HIP_H
#define FOURIER_ATTN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* opaque stream handle: a hipStream_t passed as void* (NULL = default stream) */
typedef void* fa_stream_t;

enum fa_status {
  FA_OK = 0,
  FA_ERR_NULL_POINTER = -1,   /* a required pointer is NULL                          */
  FA_ERR_BAD_SHAPE = -2,      /* a size is non-positive / inconsistent / q_len != 1  */
  FA_ERR_BAD_DTYPE = -3,      /* dtype code not one of fa_dtype                      */
  FA_ERR_WORKSPACE = -4,      /* workspace missing or too small                      */
  FA_ERR_UNSUPPORTED = -5,    /* shape outside what the kernels were built for       */
  FA_ERR_LAUNCH = -6,         /* HIP reported a launch error                         */
  FA_ERR_MISALIGNED = -7      /* pointer or stride not aligned as the kernel needs   */
};

enum fa_dtype { FA_BF16 = 0, FA_FP16 = 1, FA_FP32 = 2 };

const char* fa_last_error_string(void);
int fa_abi_version(void);

/* ---------------------------------------------------------------------------
 * Spectral compression and its statistics
 * ------------------------------------------------------------------------- */

/* mat_fourier_triton(a, N, T, K_start) (TRI:81-102) and the FFT branch of
 * MultiDimHiPPO2.forward (TRI:858-865, K_start = 0, K = min(L, T)):
 *   c[b, n, m]     (+)= sum_{k<K} cos(2 pi (k + k_start) n / T) a[b, k, m]
 *   c[b, N + n, m] (+)= sum_{k<K} sin(...)                      a[b, k, m]
 * a: (B, K, Mc) elements of `a_dtype`, row stride a_row_stride, batch stride
 * a_batch_stride (elements); if `cols` is non-NULL it holds Mc int32 column
 * indices into the row (the gather `x[:, :, idx]` of CACHE:561 fused in),
 * otherwise columns 0..Mc-1 are read.  c: (B, 2N, Mc) fp32 contiguous.
 * accumulate != 0 adds into c (the `base_input + ...` of TRI:856). */
int fa_mat_fourier(const void* a, int a_dtype, int64_t a_batch_stride, int64_t a_row_stride,
                   const int32_t* cols, float* c, int B, int K, int Mc, int N, int T,
                   int64_t k_start, int accumulate, fa_stream_t stream);

/* mat_avg_std_triton(a) (TRI:433-461): per (b, m) mean over k and
 * max(max - mean, mean - min).  Outputs fp32 (B, Mc); when round_dtype is
 * FA_BF16 / FA_FP16 each result is rounded through that type first (the
 * reference casts back to a.dtype, TRI:461).  Gather as in fa_mat_fourier.
 * workspace: fa_stats_workspace_bytes(B, Mc, K). */
int fa_mat_avg_std(const void* a, int a_dtype, int64_t a_batch_stride, int64_t a_row_stride,
                   const int32_t* cols, float* avg, float* max_dev, int B, int K, int Mc,
                   int round_dtype, void* workspace, size_t workspace_bytes, fa_stream_t stream);

/* mat_fourier_avg_std_triton(c, K, T) (TRI:285-326): statistics of the signal
 * reconstructed from c (B, 2N, Mc) fp32 at positions 0..K-1 with period T:
 *   r[b,k,m] = (1/N) sum_n cos(2 pi k n / T) c[b,n,m] + sin(...) c[b,N+n,m].
 * Outputs fp32 (B, Mc) rounded through round_dtype (the reference returns
 * fp16, TRI:326).  workspace: fa_stats_workspace_bytes(B, Mc, K). */
int fa_mat_fourier_avg_std(const float* c, float* avg, float* max_dev, int B, int N, int Mc,
                           int K, int T, int round_dtype, void* workspace, size_t workspace_bytes,
                           fa_stream_t stream);

size_t fa_stats_workspace_bytes(int B, int Mc, int K);

/* Reconstruction r (B, K, Mc) fp32 from coefficients (mat_fourier_inv_torch,
 * TRI:782-791); with stats pointers non-NULL also applies
 * (r - avg_d) * scale + avg_u (TRI:813).  Used for validation and for
 * materialising a dense view; decode attention never calls it. */
int fa_reconstruct(const float* c, const float* avg_u, const float* avg_d, const float* scale,
                   float* r, int B, int N, int Mc, int K, int T, fa_stream_t stream);

/* ---------------------------------------------------------------------------
 * Streaming update of one layer (CACHE:731-748)
 * ------------------------------------------------------------------------- */

/* Rank-1 coefficient update for the evicted token (CACHE:733, 739 ->
 * TRI:853-856 -> mat_fourier_kernel with K = 1, K_start = p):
 *   c[b, n, j] += cos(2 pi p n / T) * row[b, cols[j]],  sin rows likewise.
 * row: B rows of `row_dtype`, row_batch_stride elements apart. */
int fa_coeff_update(float* c, const void* row, int row_dtype, int64_t row_batch_stride,
                    const int32_t* cols, int B, int N, int Mc, int64_t p, int T, fa_stream_t stream);

/* ---------------------------------------------------------------------------
 * Decode attention (triton_fourier_attn, TRI:684-779; kernel TRI:464-681)
 * ------------------------------------------------------------------------- */

typedef struct fa_decode_args {
  /* query (B, 1, Hq*D) of `dtype`, contiguous */
  const void* q;
  /* full-width sink and local-window rows: two segments so that a ring-buffered
   * window needs no concatenation (MODEL:642-643 builds cat(k_init, k_local)).
   * Segment i holds il_rows[i] rows of Hkv*D elements; batch stride and row
   * stride in elements.  Either segment may be empty. */
  const void* k_il[2];
  const void* v_il[2];
  int32_t il_rows[2];
  int64_t il_batch_stride[2];
  int64_t il_row_stride[2];
  /* coefficients (B, 2N, Ck) / (B, 2N, Cv) fp32 contiguous (k_mc, v_mc) */
  const float* k_mc;
  const float* v_mc;
  /* stored ("critical") dims of the mid rows, token-major (B, >=L_m, Cn):
   * k_mn, v_mn with batch and row strides in elements */
  const void* k_mn;
  const void* v_mn;
  int64_t k_mn_batch_stride, k_mn_row_stride;
  int64_t v_mn_batch_stride, v_mn_row_stride;
  /* affine statistics, fp32 (B, Ck) / (B, Cv): avg_*_u, avg_*_d, scale_* */
  const float* avg_k_u; const float* avg_k_d; const float* scale_k;
  const float* avg_v_u; const float* avg_v_d; const float* scale_v;
  /* index lists, int32: flat dims (h*D + d) ascending, and cumulative per-head
   * offsets with the leading 0 (Hkv + 1 entries), as the cache holds them
   * (CACHE:444-452) */
  const int32_t* kc_list; const int32_t* kc_h_list;
  const int32_t* kn_list; const int32_t* kn_h_list;
  const int32_t* vc_list; const int32_t* vc_h_list;
  const int32_t* vn_list; const int32_t* vn_h_list;
  int32_t Ck, Cnk, Cv, Cnv;
  /* output (B, Hq, 1, D) fp32 contiguous (TRI:779) */
  float* out;
  int32_t B, Hq, Hkv, D;
  int32_t q_len;      /* must be 1 (TRI:692) */
  int32_t N;          /* frequencies = coefficient rows / 2 */
  int32_t L_m;        /* mid rows in use (seq_len_m) */
  int32_t T;          /* reconstruction period (MODEL:660) */
  float sm_scale;     /* <= 0 selects 1/sqrt(D) (TRI:696) */
  int32_t dtype;      /* fa_dtype of q, k_il, v_il, k_mn, v_mn */
  void* workspace;
  size_t workspace_bytes;
} fa_decode_args;

/* sizeof(fa_decode_args) as this library was built: lets a foreign-language binding
 * check its mirror of the struct. */
size_t fa_decode_args_size(void);

size_t fa_decode_attn_workspace_bytes(int B, int Hq, int Hkv, int D, int N, int il_rows_total, int L_m);

/* One decode step of Fourier attention over
 * [sink ; local window ; mid rows (stored dims + dims rebuilt from coefficients)]. */
int fa_decode_attn(const fa_decode_args* args, fa_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FOURIER_ATTN_HIP_H */
