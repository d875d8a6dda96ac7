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
 * accumulate != 0 adds into c (the `base_input + ...` of TRI:856).
 * workspace (optional): with at least fa_mat_fourier_workspace_bytes(B, K, Mc, N)
 * bytes (256-byte aligned), 16-bit inputs of K >= 512 rows with N % 8 == 0 (any
 * number of columns Mc) run on the matrix cores (basis rounded to fp16, fp32 accumulation);
 * without it, and for every other shape, an fp32 vector kernel is used. */
int fa_mat_fourier(const void* a, int a_dtype, int64_t a_batch_stride, int64_t a_row_stride,
                   const int32_t* cols, float* c, int B, int K, int Mc, int N, int T,
                   int64_t k_start, int accumulate, void* workspace, size_t workspace_bytes,
                   fa_stream_t stream);

/* 0 when the matrix-core path does not apply to the shape. */
size_t fa_mat_fourier_workspace_bytes(int a_dtype, int B, int K, int Mc, int N);

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
 * fp16, TRI:326).  workspace: at least fa_stats_workspace_bytes(B, Mc, K);
 * with fa_mat_fourier_avg_std_workspace_bytes(B, N, Mc, K) bytes (256-byte
 * aligned) long reconstructions (K >= 1024) run on the matrix cores (basis and
 * per-column scaled coefficients in fp16, fp32 accumulation). */
int fa_mat_fourier_avg_std(const float* c, float* avg, float* max_dev, int B, int N, int Mc,
                           int K, int T, int round_dtype, void* workspace, size_t workspace_bytes,
                           fa_stream_t stream);

size_t fa_stats_workspace_bytes(int B, int Mc, int K);
size_t fa_mat_fourier_avg_std_workspace_bytes(int B, int N, int Mc, int K);

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

/* One streaming step of one layer in a single launch (the body of CACHE:731-748 for
 * K and V): the row in window slot evict_slot leaves the window -- rank-1
 * coefficient update at `phase` over its compressed columns (fa_coeff_update),
 * its stored columns appended at token position mid_pos of the page store
 * (fa_mid_append) -- and the new token is written to window slot write_slot.
 * The window buffers are (B, slots, width) with batch / row strides in elements;
 * evict_slot != write_slot (keep one slot more than the window is long), so
 * the three pieces of work are independent.  Pointers of a tensor whose column
 * count is 0 may be NULL. */
typedef struct fa_stream_args {
  const void* k_new; const void* v_new;      /* (B, width) new token rows, batch stride new_batch_stride */
  int64_t new_batch_stride;
  void* k_ring; void* v_ring;                /* window buffers */
  int64_t ring_batch_stride, ring_row_stride;
  int32_t evict_slot, write_slot;
  float* k_coef; float* v_coef;              /* (B, 2N, Ck) / (B, 2N, Cv) fp32 */
  const int32_t* kc_list; const int32_t* vc_list;
  int32_t Ck, Cv, N, T;
  int64_t phase;
  void* k_mid; void* v_mid;                  /* page stores (see below) */
  int64_t k_mid_batch_stride, v_mid_batch_stride;
  int32_t cap_pages;
  int64_t mid_pos;
  const int32_t* kn_list; const int32_t* kn_h_list; const int32_t* k_pad_h_list;
  const int32_t* vn_list; const int32_t* vn_h_list; const int32_t* v_pad_h_list;
  int32_t Cnk, Cnv;
  int32_t B, Hkv, width, dtype;
  /* != 0: leave the coefficients alone (page stores and window are updated as always).  The caller owes them the
   * rank-1 update of the row in `evict_slot` at `phase`: fa_coeff_update, or the next fa_decode_attn of the layer
   * through its upd_* arguments, which applies it while it streams the coefficients anyway.  The row stays in its
   * window slot until the next fa_stream_update of the layer writes there. */
  int32_t skip_coef;
} fa_stream_args;

int fa_stream_update(const fa_stream_args* args, fa_stream_t stream);
size_t fa_stream_args_size(void);

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
  /* stored ("critical") dims of the mid rows (k_mn, v_mn).
   * mid_layout == FA_MID_TOKEN_MAJOR: (B, >=L_m, Cn) with batch and row strides
   * in elements, as the reference holds k_uncompressed (CACHE:560, 735).
   * mid_layout == FA_MID_PAGED: the library's own page layout written by
   * fa_mid_pack / fa_mid_append (see there); row strides are ignored and
   * mid_cap_pages, k_pad_h_list, v_pad_h_list describe the store. */
  const void* k_mn;
  const void* v_mn;
  int64_t k_mn_batch_stride, k_mn_row_stride;
  int64_t v_mn_batch_stride, v_mn_row_stride;
  int32_t mid_layout;
  int32_t mid_cap_pages;
  const int32_t* k_pad_h_list;
  const int32_t* v_pad_h_list;
  int32_t mid_max_k_pad;   /* largest per-head padded dim count of K / V (host copies of */
  int32_t mid_max_v_pad;   /* max_h(pad_h[h+1] - pad_h[h]); select the kernel instance)   */
  /* optional HOST copies of k_pad_h_list / v_pad_h_list (Hkv + 1 entries each), or NULL: with them the mid rows
   * of a head that stores more dims are cut into more splits than those of a head that stores few (the
   * reference's masks differ head by head), so that all workgroups finish together */
  const int32_t* k_pad_h_host;
  const int32_t* v_pad_h_host;
  /* optional constant operand tables built by fa_decode_tables_build for this (N, T);
   * NULL lets the call build them in its workspace */
  const void* tables;
  int32_t force_generic;   /* != 0: never take the MFMA path (testing) */
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
  /* output (B, Hq, 1, D) contiguous: fp32 in `out` (TRI:779) and / or rounded to `dtype`
   * in `out_cast` (what the caller's `.to(query_states.dtype)` of MODEL:663 would make of
   * it); either may be NULL, not both */
  float* out;
  void* out_cast;
  int32_t B, Hq, Hkv, D;
  int32_t q_len;      /* must be 1 (TRI:692) */
  int32_t N;          /* frequencies = coefficient rows / 2 */
  int32_t L_m;        /* mid rows in use (seq_len_m) */
  int32_t T;          /* reconstruction period (MODEL:660) */
  float sm_scale;     /* <= 0 selects 1/sqrt(D) (TRI:696) */
  int32_t dtype;      /* fa_dtype of q, k_il, v_il, k_mn, v_mn */
  void* workspace;
  size_t workspace_bytes;
  /* bit 0: never run the merge inside the mid-row launch (see fa_decode_attn); the mid rows and the merge then run as
   * launches of their own.  bit 1: with a batch of one sequence, keep one page stream per workgroup instead of four
   * sub-splits.  (Both for testing and comparison.) */
  int32_t no_fuse;
  /* A rank-1 update that the coefficients are still owed (fa_stream_update with skip_coef), applied by this call
   * before it uses them: k_mc[b, n, j] += cos(2 pi n p / upd_T) x_k[b, kc_list[j]] and k_mc[b, N + n, j] += sin(...),
   * likewise v_mc with x_v and vc_list (CACHE:731-748 with TRI:853-856, K = 1).  upd_k_row / upd_v_row: the rows
   * x_k, x_v (B, Hkv*D) of `dtype` that left the window, batch stride upd_batch_stride elements; p = upd_phase.
   * Both NULL: nothing pending.  k_mc and v_mc are WRITTEN then, once: a second call with the same upd_* arguments
   * would apply the update again.  No counterpart in the reference, which updates in `update` (a launch of its
   * own) what the attention that follows reads again. */
  const void* upd_k_row;
  const void* upd_v_row;
  int64_t upd_batch_stride;
  int64_t upd_phase;
  int32_t upd_T;
} fa_decode_args;

/* sizeof(fa_decode_args) as this library was built: lets a foreign-language binding
 * check its mirror of the struct. */
size_t fa_decode_args_size(void);

size_t fa_decode_attn_workspace_bytes(int B, int Hq, int Hkv, int D, int N, int il_rows_total, int L_m);

/* ---------------------------------------------------------------------------
 * Page layout of the stored mid dims (the cache's HBM layout; no counterpart in
 * the reference, which keeps k_uncompressed token-major and grows it with
 * torch.cat, CACHE:735, 741)
 * ------------------------------------------------------------------------- */
enum fa_mid_layout { FA_MID_TOKEN_MAJOR = 0, FA_MID_PAGED = 1 };
#define FA_PAGE_TOKENS 32
#define FA_K_DIM_PAD 32 /* per-head stored K dims are padded to a multiple of this */
#define FA_V_DIM_PAD 16 /* per-head stored V dims are padded to a multiple of this */

/* One tensor (K or V) of one layer is stored per (batch, KV head) as a run of
 * pages of FA_PAGE_TOKENS tokens.  With pad_h_list the cumulative padded dim
 * counts (Hkv + 1 int32, leading 0; head h owns dp = pad_h[h+1] - pad_h[h]
 * padded dims), the page p of head h of batch b starts at element
 *     b * batch_stride + pad_h[h] * 32 * cap_pages + p * dp * 32
 * and holds dp * 32 elements in fragments of 512 elements (64 lanes x 8):
 *   K: fragment (tb, s), tb in {0,1}, s < dp/32, at index tb * (dp/32) + s;
 *      lane l, element e = token p*32 + tb*16 + l%16, stored dim s*32 + 8*(l/16) + e
 *   V: fragment dg < dp/16;
 *      lane l, element e = stored dim dg*16 + l%16, token p*32 + 8*(l/16) + e
 * i.e. exactly the register image of a 16x16x32 MFMA A operand, so a wave
 * loads a fragment with one 16-byte load per lane.  Padded dims and unused
 * token slots must be zero: allocate the store zero-filled.
 * batch_stride >= pad_h[Hkv] * 32 * cap_pages. */

/* What the entries of an index list handed to fa_mid_pack mean. */
#define FA_COLS_ANY 0       /* plain column numbers of the source rows, in any order and range */
#define FA_COLS_HEAD_DIMS 1 /* the source rows are full K/V rows of Hkv*D elements and the entries of head h
                               lie in [h*D, (h+1)*D): the reference's kn_list / vn_list (CACHE:445-447) */

/* Scatter rows [row0, row0 + L) of src (B, S, width), taking for each head the
 * columns n_list[n_h[h] .. n_h[h+1]) (the gather x[:, :, kn] of CACHE:560, 578),
 * into pages starting at token 0.  is_v selects the V fragment order.  With
 * cols_kind == FA_COLS_HEAD_DIMS (and 16-bit, 16-byte aligned rows) the head's
 * slice of every row is read whole and the stored dims are picked from it, which
 * is faster; entries outside the head's range then read a clamped dim.  With
 * FA_COLS_ANY (e.g. an identity list over rows that are gathered already) every
 * element is fetched by its own column number. */
int fa_mid_pack(const void* src, int dtype, int64_t src_batch_stride, int64_t src_row_stride, int64_t row0,
                int L, void* store, int64_t store_batch_stride, int cap_pages, const int32_t* n_list,
                const int32_t* n_h_list, const int32_t* pad_h_list, int B, int Hkv, int D, int is_v,
                int cols_kind, fa_stream_t stream);

/* The prompt's mid rows of K (or V) in one pass: what the cache's prefill does with them in CACHE:560-565 (K) and
 * CACHE:578-587 (V) -- keep the stored dims (fa_mid_pack with FA_COLS_HEAD_DIMS), transform the first K_fft rows of
 * the compressed dims (fa_mat_fourier with k_start 0) and take the compressed dims' column statistics over all L rows
 * (fa_mat_avg_std).  The rows [row0, row0 + L) of src (B, S, Hkv*D) are read once.  pages and coefficients equal
 * those of the separate calls bit for bit; the statistics sum in another order (equal to rounding).
 * c_list / c_h_list: the compressed dims as flat h*D + d entries, head by head, and their per-head offsets
 * (Hkv + 1 entries), Mc = c_h_list[Hkv]; coef (B, 2N, Mc), avg and max_dev (B, Mc) fp32.
 * Supported (fa_prefill_compress_ok) for 16-bit rows whose transform runs on the matrix cores, K_fft <= L, D a
 * multiple of 8 up to 256; FA_ERR_UNSUPPORTED otherwise, and the caller makes the three calls. */
int fa_prefill_compress_ok(int dtype, int L, int K_fft, int Mc, int N, int D);
size_t fa_prefill_compress_workspace_bytes(int B, int L, int K_fft, int Mc, int N);
int fa_prefill_compress(const void* src, int dtype, int64_t src_batch_stride, int64_t src_row_stride, int64_t row0,
                        int L, int K_fft, void* store, int64_t store_batch_stride, int cap_pages,
                        const int32_t* n_list, const int32_t* n_h_list, const int32_t* pad_h_list,
                        const int32_t* c_list, const int32_t* c_h_list, int Mc, float* coef, float* avg,
                        float* max_dev, int stats_round_dtype, int B, int Hkv, int D, int N, int T, int is_v,
                        void* workspace, size_t workspace_bytes, fa_stream_t stream);

/* Write one row (the evicted window row, CACHE:735, 741) at token position pos. */
int fa_mid_append(const void* row, int dtype, int64_t row_batch_stride, int64_t pos, void* store,
                  int64_t store_batch_stride, int cap_pages, const int32_t* n_list, const int32_t* n_h_list,
                  const int32_t* pad_h_list, int B, int Hkv, int Cn, int is_v, fa_stream_t stream);

/* Inverse of fa_mid_pack: dst (B, L, Cn) token-major contiguous, the reference's
 * k_uncompressed / v_uncompressed. */
int fa_mid_unpack(const void* store, int dtype, int64_t store_batch_stride, int cap_pages, int L, void* dst,
                  const int32_t* n_h_list, const int32_t* pad_h_list, int B, int Hkv, int D, int Cn, int is_v,
                  fa_stream_t stream);

/* Constant MFMA operand tables of decode attention (cos/sin of in-page token offsets and
 * the per-page rotation); they depend on N and T only, so a cache builds them once. */
size_t fa_decode_tables_bytes(int N);
int fa_decode_tables_build(void* tables, size_t tables_bytes, int N, int T, fa_stream_t stream);

/* One decode step of Fourier attention over
 * [sink ; local window ; mid rows (stored dims + dims rebuilt from coefficients)].
 * Launches: query preparation + sink/window tiles, mid rows (two passes with 1024 frequencies), merge.  On the
 * matrix-core path with 16-bit storage, head_dim 128 and at most four query heads per KV head the workgroups of the
 * last mid-row launch merge their own partials and write the output rows (one launch fewer); args->no_fuse bit 0
 * keeps the merge launch.  With a batch of one sequence and up to 512 frequencies every workgroup of that launch then
 * runs four sub-splits of its pages side by side (in the matrix-core columns and page streams that further batch
 * elements would use).
 * That needs the device to deal the workgroups of a launch out to its dies in turn, which the first call on a device
 * checks with a tiny launch and ONE synchronisation of `stream` (skipped, and asked again by the next call, while
 * the stream is being captured). */
int fa_decode_attn(const fa_decode_args* args, fa_stream_t stream);

/* How fa_decode_attn would cut the mid rows of each KV head into splits on the matrix-core kernels (host-side
 * arithmetic only, no GPU work; no counterpart in the reference): splits_out[h] for h < Hkv, given the host copies of
 * the per-head padded dim counts (or NULL for both: every head the same), and in *room_out (optional) the number of
 * splits per head that fa_decode_attn_workspace_bytes leaves room for.  FA_ERR_UNSUPPORTED for shapes that take the
 * generic kernels. */
int fa_decode_split_plan(int B, int Hq, int Hkv, int D, int N, int il_rows_total, int L_m,
                         const int32_t* k_pad_h_host, const int32_t* v_pad_h_host, int32_t* splits_out,
                         int32_t* room_out);

/* fa_decode_attn for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): no counterpart in the reference.  `args->workspace` and
 * `args->workspace_bytes` are ignored; the partial results live in a buffer of FA_DECODE_NOALLOC_SCRATCH_BYTES
 * that is part of the library image on every GPU it runs on (held until the process ends).  Nothing is allocated
 * or freed, by this call or by anything it calls.  k_pad_h_host / v_pad_h_host are ignored as well: every KV head
 * gets the same number of splits, and shapes whose partial results then exceed that size (at most what
 * fa_decode_attn_workspace_bytes(...) reports, which leaves room for uneven shares) are refused with
 * FA_ERR_WORKSPACE.  Every call on one GPU shares that GPU's buffer: calls that may
 * overlap on one GPU (two streams, two threads) race and must be serialised by the caller; consecutive calls on
 * one stream are fine (every kernel writes what it later reads, nothing needs clearing).  The first call on a
 * device looks the buffer's address up (hipGetSymbolAddress): make it outside any stream capture.  This entry
 * point never runs fa_decode_attn's one-off check of the device's workgroup placement (its copy to the host could
 * make the runtime set up a staging buffer): until a fa_decode_attn call has run that check on the device, the merge
 * stays a launch of its own here. */
#define FA_DECODE_NOALLOC_SCRATCH_BYTES (32u << 20)
int fa_decode_attn_noalloc(const fa_decode_args* args, fa_stream_t stream);

/* Whether the last fa_decode_attn / _noalloc / _timed call of the calling thread ran the merge inside the mid-row
 * launch (1; 2: with the four sub-splits per workgroup of a batch of one) or as a launch of its own (0).  A
 * measurement aid (the reference has no counterpart). */
int fa_decode_attn_last_fused(void);

/* Same call, bracketed by HIP events on `stream`; synchronises and returns in ms_out[0..3] the
 * milliseconds spent in (0) the coefficient-domain query kernel (plus the operand tables when
 * they are built in the workspace), (1) the mid-row kernel, (2) the sink/window kernel and
 * (3) the merge kernel.  A measurement aid for benchmarks (the reference has no timers). */
int fa_decode_attn_timed(const fa_decode_args* args, fa_stream_t stream, float* ms_out);

/* ---------------------------------------------------------------------------
 * Exact attention of the prompt pass
 * ------------------------------------------------------------------------- */

/* The other arm of the attention forward (MODEL:623-633): while the cache holds a layer's keys in full
 * (`update` returned only `*_local`), attention is exact and causal - flash_attn_func(q, k, v, causal=True)
 * in the reference.  q: (B, Hq, q_len, D) given by batch / head / row strides in elements with D contiguous
 * (the transposed view of the projection output works as it is); k, v: token-major (B, S, Hkv*D) as `update`
 * returns them, sharing their strides; out: (B, q_len, Hq, D) contiguous, of `dtype` (what the reference reshapes
 * to (B, q_len, Hq*D), MODEL:663).  Query row i sees keys 0 .. i + (S - q_len) (bottom-right aligned, as
 * flash-attn does when q_len < S).  16-bit dtypes, D in {64, 128}, rows 16-byte aligned; sm_scale <= 0 means
 * 1/sqrt(D).  workspace: fa_prefill_attn_workspace_bytes(B, Hkv, D, S) bytes (a transposed copy of V in
 * matrix-core operand order, written by a first launch). */
size_t fa_prefill_attn_workspace_bytes(int B, int Hkv, int D, int S);
int fa_prefill_attn(const void* q, int64_t q_batch_stride, int64_t q_head_stride, int64_t q_row_stride,
                    const void* k, const void* v, int64_t kv_batch_stride, int64_t kv_row_stride, void* out,
                    int dtype, int B, int Hq, int Hkv, int D, int S, int q_len, float sm_scale, void* workspace,
                    size_t workspace_bytes, fa_stream_t stream);

/* ---------------------------------------------------------------------------
 * Elementwise steps of the decoder layer around the attention (one launch each)
 * ------------------------------------------------------------------------- */

/* The residual add of LlamaDecoderLayer.forward followed by LlamaRMSNorm.forward
 * (MODEL:735-750, 87-92): if delta is non-NULL, h <- h + delta (rounded to
 * `dtype`, in place); y = weight * (h * rsqrt(mean(h^2) + eps)).to(dtype).
 * h, delta, y: (rows, hidden) contiguous; weight: (hidden); hidden <= 8192. */
int fa_add_rmsnorm(void* h, const void* delta, const void* weight, void* y, int rows, int hidden,
                   float eps, int dtype, fa_stream_t stream);

/* apply_rotary_pos_emb (MODEL:213-244): x <- x * cos + rotate_half(x) * sin on every
 * head of q and k; cos, sin: (rows, D) in `dtype`.  Products and sum are rounded to
 * `dtype` one by one like the tensor ops.  Row r of q is read at q_in + r * q_in_stride
 * (Hq * D elements; the rows may be slices of a wider fused projection output) and
 * written to q_out as (rows, Hq * D) densely packed; q_out may be q_in when q_in is
 * densely packed itself (a single row always is, whatever q_in_stride says).  k: row r
 * at k + r * k_stride, Hkv * D elements, in place.
 * Strides in elements. */
int fa_rope_qk(const void* q_in, int64_t q_in_stride, void* q_out, void* k, int64_t k_stride,
               const void* cos, const void* sin, int rows, int Hq, int Hkv, int D, int dtype,
               fa_stream_t stream);

/* act_fn(gate_proj(x)) * up_proj(x) of LlamaMLP.forward (MODEL:277) with
 * act_fn = silu: out[r][i] = silu(gate[r][i]).to(dtype) * up[r][i]; gate and up rows
 * in_stride elements apart (slices of a fused projection output, or in_stride = cols),
 * out (rows, cols) densely packed; rows <= 65535. */
int fa_silu_mul(const void* gate, const void* up, void* out, int rows, int cols, int64_t in_stride,
                int dtype, fa_stream_t stream);

/* The projections of a decode step, nn.Linear without bias (q/k/v_proj MODEL:597-599, o_proj MODEL:665, the MLP
 * MODEL:283): out[r][n] = sum_k x[r][k] * w[n][k] for a handful of rows, where the product is one pass over the
 * weights.  fa_linear_pack re-lays a row-major weight (n_out, K) once, in the order the matrix cores take it
 * (tile of 16 output features x step of 32 input features = 64 lanes x 8 elements, lane 16 g + c holding
 * w[16 tile + c][32 step + 8 g ..]); fa_linear_packed multiplies: x (rows, K) with rows x_row_stride elements apart,
 * out (rows, n_out) densely packed, fp32 accumulation, result rounded to `dtype`.  16-bit storage only;
 * fa_linear_packed_ok says whether a shape is covered (1 <= rows <= 16, n_out a multiple of 16, K of 1024): other
 * shapes belong to a GEMM library. */
int fa_linear_pack(const void* w, void* packed, int n_out, int K, int dtype, fa_stream_t stream);
int fa_linear_packed_ok(int rows, int K, int n_out);
int fa_linear_packed(const void* x, int64_t x_row_stride, const void* w_packed, void* out, int rows, int K,
                     int n_out, int dtype, fa_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* FOURIER_ATTN_HIP_H */
