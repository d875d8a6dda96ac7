// Page layout of the stored mid dims: pack (prefill), append (eviction) and unpack.
#include "fa_common.h"

namespace {

// element offset inside one (batch, head) run of pages
__device__ __forceinline__ int64_t page_elem_offset(bool is_v, int dp, int64_t token, int j) {
  const int64_t page = token >> 5;
  const int t = (int)(token & 31);
  int frag, lane, e;
  if (!is_v) {
    frag = (t >> 4) * (dp >> 5) + (j >> 5);
    lane = ((j & 31) >> 3) * 16 + (t & 15);
    e = j & 7;
  } else {
    frag = j >> 4;
    lane = (t >> 3) * 16 + (j & 15);
    e = t & 7;
  }
  return page * dp * 32 + (int64_t)frag * 512 + lane * 8 + e;
}

// one block per page (32 tokens) of one (b, h): the gather reads run along the stored dims of a token row,
// the page is assembled in LDS and leaves as whole fragments (16 bytes per lane); grid (pages, Hkv, B)
template <typename E>
__global__ __launch_bounds__(256) void mid_pack_kernel(
    const E* __restrict__ src, int64_t src_bs, int64_t src_rs, int64_t row0, int L, E* __restrict__ store,
    int64_t st_bs, int cap_pages, const int32_t* __restrict__ n_list, const int32_t* __restrict__ n_h,
    const int32_t* __restrict__ pad_h, int is_v) {
  constexpr int kMaxDp = 256;                       // padded stored dims of a head
  constexpr int kPitch = kMaxDp + 8;                // elements; keeps rows 16-byte aligned
  struct alignas(sizeof(E) * 8) Piece { E v[8]; };  // what one lane of a fragment holds
  __shared__ __attribute__((aligned(32))) E tile[32][kPitch];
  const int page = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int n0 = n_h[h], n_len = n_h[h + 1] - n0;
  const int p0 = pad_h[h], dp = pad_h[h + 1] - p0;
  if (n_len == 0) return;
  const int tid = threadIdx.x;
  __shared__ int s_col[kMaxDp];
  for (int j = tid; j < dp; j += 256) s_col[j] = n_list[n0 + min(j, n_len - 1)];
  __syncthreads();
  // gather: consecutive threads take consecutive stored dims of one token; eight loads in flight per thread,
  // all unconditional (clamped to the last real dim / row, masked afterwards)
  const E* sb = src + (int64_t)b * src_bs + row0 * src_rs;
  const int64_t last = (int64_t)L - 1;
  for (int base = tid; base < 32 * dp; base += 256 * 8) {
    E v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int idx = min(base + 256 * u, 32 * dp - 1);
      const int t = idx / dp, j = idx - t * dp;
      const int64_t token = (int64_t)page * 32 + t;
      v[u] = sb[(token < last ? token : last) * src_rs + s_col[j]];
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int idx = base + 256 * u;
      if (idx < 32 * dp) {
        const int t = idx / dp, j = idx - t * dp;
        const bool ok = j < n_len && (int64_t)page * 32 + t < L;
        tile[t][j] = ok ? v[u] : E{};
      }
    }
  }
  __syncthreads();
  Piece* out = (Piece*)(store + (int64_t)b * st_bs + (int64_t)p0 * 32 * cap_pages + (int64_t)page * dp * 32);
  const int n_pieces = dp * 32 / 8;
  for (int piece = tid; piece < n_pieces; piece += 256) {
    const int frag = piece >> 6, lane = piece & 63;
    Piece o;
    if (!is_v) {
      const int nks = dp >> 5;
      const int tb = frag / nks, s_ = frag - tb * nks;
      o = *(const Piece*)&tile[tb * 16 + (lane & 15)][s_ * 32 + 8 * (lane >> 4)];
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) o.v[i] = tile[8 * (lane >> 4) + i][frag * 16 + (lane & 15)];
    }
    out[piece] = o;
  }
}

// The same for 16-bit rows that are 16-byte aligned: the head's whole slice of the 32 token rows is read with
// 16-byte loads into LDS (every line of the source is needed anyway: stored and compressed dims interleave), and
// the gather along the stored dims happens on the way out of LDS.
template <typename E>
__global__ __launch_bounds__(256) void mid_pack_rows_kernel(
    const E* __restrict__ src, int64_t src_bs, int64_t src_rs, int64_t row0, int L, E* __restrict__ store,
    int64_t st_bs, int cap_pages, const int32_t* __restrict__ n_list, const int32_t* __restrict__ n_h,
    const int32_t* __restrict__ pad_h, int D, int is_v) {
  constexpr int kMaxD = 256;                        // head dim, and padded stored dims of a head
  constexpr int kPitch = kMaxD + 8;                 // elements; keeps rows 16-byte aligned
  struct alignas(sizeof(E) * 8) Piece { E v[8]; };
  __shared__ __attribute__((aligned(32))) E tile[32][kPitch];
  __shared__ int s_col[kMaxD];
  const int page = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
  const int n0 = n_h[h], n_len = n_h[h + 1] - n0;
  const int p0 = pad_h[h], dp = pad_h[h + 1] - p0;
  if (n_len == 0) return;
  const int tid = threadIdx.x;
  // dim within the head of every stored position (clamped into the head: the reads below stay inside the tile)
  for (int j = tid; j < dp; j += 256) s_col[j] = min(max(n_list[n0 + min(j, n_len - 1)] - h * D, 0), D - 1);
  const E* sb = src + (int64_t)b * src_bs + row0 * src_rs + (int64_t)h * D;
  const int ppr = D >> 3;                           // 16-byte pieces per row of the head
  const int64_t last = (int64_t)L - 1;
  for (int p = tid; p < 32 * ppr; p += 256) {
    const int t = p / ppr, c = p - t * ppr;
    const int64_t token = (int64_t)page * 32 + t;
    *(Piece*)&tile[t][c * 8] = *(const Piece*)(sb + (token < last ? token : last) * src_rs + c * 8);
  }
  __syncthreads();
  Piece* out = (Piece*)(store + (int64_t)b * st_bs + (int64_t)p0 * 32 * cap_pages + (int64_t)page * dp * 32);
  const int n_pieces = dp * 32 / 8;
  for (int piece = tid; piece < n_pieces; piece += 256) {
    const int frag = piece >> 6, lane = piece & 63;
    Piece o;
    if (!is_v) {
      const int nks = dp >> 5;
      const int tb = frag / nks, s_ = frag - tb * nks;
      const int t = tb * 16 + (lane & 15), j0 = s_ * 32 + 8 * (lane >> 4);
      const bool row_ok = (int64_t)page * 32 + t < L;
#pragma unroll
      for (int e = 0; e < 8; ++e) o.v[e] = (row_ok && j0 + e < n_len) ? tile[t][s_col[j0 + e]] : E{};
    } else {
      const int j = frag * 16 + (lane & 15);
      const int col = s_col[j];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int t = 8 * (lane >> 4) + i;
        o.v[i] = (j < n_len && (int64_t)page * 32 + t < L) ? tile[t][col] : E{};
      }
    }
    out[piece] = o;
  }
}

template <typename E>
__global__ __launch_bounds__(256) void mid_append_kernel(
    const E* __restrict__ row, int64_t row_bs, int64_t pos, E* __restrict__ store, int64_t st_bs, int cap_pages,
    const int32_t* __restrict__ n_list, const int32_t* __restrict__ n_h, const int32_t* __restrict__ pad_h, int Hkv,
    int Cn, int is_v) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= Cn) return;
  int h = 0;
  while (h + 1 < Hkv && n_h[h + 1] <= c) ++h;
  const int j = c - n_h[h];
  const int p0 = pad_h[h], dp = pad_h[h + 1] - p0;
  store[(int64_t)b * st_bs + (int64_t)p0 * 32 * cap_pages + page_elem_offset(is_v, dp, pos, j)] =
      row[(int64_t)b * row_bs + n_list[c]];
}

template <typename E>
__global__ __launch_bounds__(256) void mid_unpack_kernel(
    const E* __restrict__ store, int64_t st_bs, int cap_pages, int L, E* __restrict__ dst,
    const int32_t* __restrict__ n_h, const int32_t* __restrict__ pad_h, int Cn, int is_v) {
  const int h = blockIdx.y, b = blockIdx.z;
  const int n0 = n_h[h], n_len = n_h[h + 1] - n0;
  const int p0 = pad_h[h], dp = pad_h[h + 1] - p0;
  if (n_len == 0) return;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)L * n_len) return;
  const int64_t token = idx / n_len;
  const int j = (int)(idx % n_len);
  dst[((int64_t)b * L + token) * Cn + n0 + j] =
      store[(int64_t)b * st_bs + (int64_t)p0 * 32 * cap_pages + page_elem_offset(is_v, dp, token, j)];
}

template <typename F>
int dispatch16(int dtype, const char* what, F&& f) {
  switch (dtype) {
    case FA_BF16: f(bf16_t{}); return FA_OK;
    case FA_FP16: f(f16_t{}); return FA_OK;
    case FA_FP32: f(float{}); return FA_OK;
    default: fa_set_error("%s: dtype %d", what, dtype); return FA_ERR_BAD_DTYPE;
  }
}

}  // namespace

extern "C" int fa_mid_pack(const void* src, int dtype, int64_t src_bs, int64_t src_rs, int64_t row0, int L,
                           void* store, int64_t st_bs, int cap_pages, const int32_t* n_list, const int32_t* n_h,
                           const int32_t* pad_h, int B, int Hkv, int D, int is_v, int cols_kind, fa_stream_t stream) {
  FA_REQUIRE(src && store && n_h && pad_h, FA_ERR_NULL_POINTER, "fa_mid_pack: null pointer");
  FA_REQUIRE(cols_kind == FA_COLS_ANY || cols_kind == FA_COLS_HEAD_DIMS, FA_ERR_BAD_SHAPE, "fa_mid_pack: cols_kind %d",
             cols_kind);
  FA_REQUIRE(B > 0 && Hkv > 0 && L >= 0 && cap_pages > 0 && row0 >= 0, FA_ERR_BAD_SHAPE, "fa_mid_pack: bad shape");
  FA_REQUIRE((int64_t)cap_pages * 32 >= L, FA_ERR_BAD_SHAPE, "fa_mid_pack: %d rows do not fit %d pages", L, cap_pages);
  if (L == 0) return FA_OK;
  hipStream_t st = fa_hip_stream(stream);
  FA_REQUIRE(D > 0, FA_ERR_BAD_SHAPE, "fa_mid_pack: head_dim %d", D);
  FA_REQUIRE(D <= 256, FA_ERR_UNSUPPORTED, "fa_mid_pack: head_dim %d above 256", D);
  dim3 grid(fa_cdiv(L, 32), Hkv, B);
  // the row kernel reads head h's slice [h*D, (h+1)*D) of every source row and picks the stored dims out of it:
  // only the caller knows whether the index list means that (it cannot be told from the strides)
  const bool rows16 = cols_kind == FA_COLS_HEAD_DIMS && ((uintptr_t)src & 15) == 0 && src_bs % 8 == 0 &&
                      src_rs % 8 == 0 && D % 8 == 0;
  FA_REQUIRE(cols_kind != FA_COLS_HEAD_DIMS || src_rs >= (int64_t)Hkv * D, FA_ERR_BAD_SHAPE,
             "fa_mid_pack: rows of %lld elements cannot hold %d heads of %d dims", (long long)src_rs, Hkv, D);
  int rc = dispatch16(dtype, "fa_mid_pack", [&](auto tag) {
    using E = decltype(tag);
    if constexpr (sizeof(E) == 2) {
      if (rows16) {
        mid_pack_rows_kernel<E><<<grid, 256, 0, st>>>((const E*)src, src_bs, src_rs, row0, L, (E*)store, st_bs, cap_pages,
                                                     n_list, n_h, pad_h, D, is_v);
        return;
      }
    }
    mid_pack_kernel<E><<<grid, 256, 0, st>>>((const E*)src, src_bs, src_rs, row0, L, (E*)store, st_bs, cap_pages, n_list,
                                            n_h, pad_h, is_v);
  });
  return rc != FA_OK ? rc : fa_check_launch("fa_mid_pack");
}

extern "C" int fa_mid_append(const void* row, int dtype, int64_t row_bs, int64_t pos, void* store, int64_t st_bs,
                             int cap_pages, const int32_t* n_list, const int32_t* n_h, const int32_t* pad_h, int B,
                             int Hkv, int Cn, int is_v, fa_stream_t stream) {
  FA_REQUIRE(row && store && n_h && pad_h, FA_ERR_NULL_POINTER, "fa_mid_append: null pointer");
  FA_REQUIRE(B > 0 && Hkv > 0 && Cn >= 0 && pos >= 0 && cap_pages > 0, FA_ERR_BAD_SHAPE, "fa_mid_append: bad shape");
  FA_REQUIRE(pos < (int64_t)cap_pages * 32, FA_ERR_BAD_SHAPE, "fa_mid_append: position %lld beyond %d pages",
             (long long)pos, cap_pages);
  if (Cn == 0) return FA_OK;
  FA_REQUIRE(n_list, FA_ERR_NULL_POINTER, "fa_mid_append: index list null");
  hipStream_t st = fa_hip_stream(stream);
  dim3 grid(fa_cdiv(Cn, 256), B);
  int rc = dispatch16(dtype, "fa_mid_append", [&](auto tag) {
    using E = decltype(tag);
    mid_append_kernel<E><<<grid, 256, 0, st>>>((const E*)row, row_bs, pos, (E*)store, st_bs, cap_pages, n_list, n_h, pad_h,
                                              Hkv, Cn, is_v);
  });
  return rc != FA_OK ? rc : fa_check_launch("fa_mid_append");
}

extern "C" int fa_mid_unpack(const void* store, int dtype, int64_t st_bs, int cap_pages, int L, void* dst,
                             const int32_t* n_h, const int32_t* pad_h, int B, int Hkv, int D, int Cn, int is_v,
                             fa_stream_t stream) {
  FA_REQUIRE(store && n_h && pad_h, FA_ERR_NULL_POINTER, "fa_mid_unpack: null pointer");
  FA_REQUIRE(B > 0 && Hkv > 0 && L >= 0 && Cn >= 0 && cap_pages > 0, FA_ERR_BAD_SHAPE, "fa_mid_unpack: bad shape");
  FA_REQUIRE((int64_t)cap_pages * 32 >= L, FA_ERR_BAD_SHAPE, "fa_mid_unpack: %d rows beyond %d pages", L, cap_pages);
  if (L == 0 || Cn == 0) return FA_OK;
  FA_REQUIRE(dst, FA_ERR_NULL_POINTER, "fa_mid_unpack: dst null");
  FA_REQUIRE(D > 0, FA_ERR_BAD_SHAPE, "fa_mid_unpack: head_dim %d", D);
  hipStream_t st = fa_hip_stream(stream);
  dim3 grid(fa_cdiv((int64_t)L * D, 256), Hkv, B);
  int rc = dispatch16(dtype, "fa_mid_unpack", [&](auto tag) {
    using E = decltype(tag);
    mid_unpack_kernel<E><<<grid, 256, 0, st>>>((const E*)store, st_bs, cap_pages, L, (E*)dst, n_h, pad_h, Cn, is_v);
  });
  return rc != FA_OK ? rc : fa_check_launch("fa_mid_unpack");
}
