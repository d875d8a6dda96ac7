// One decode step of the cache for one layer in one launch (CACHE:731-748): the oldest window row of K and of V
// leaves the window -- its compressed dims enter the coefficients as a rank-1 update (TRI:853-856 with K = 1,
// K_start = p), its stored dims are appended to the page store -- and the new token takes a free window slot.
// The window buffer keeps one slot more than the window is long, so the slot that is written is never the slot
// that is read in the same step, and the three pieces of work need no order among themselves: the blocks of
// one grid take one of them each.
#include "fa_common.h"

namespace {

struct StreamTensor {
  const void* new_row;      // (B, width) new token, batch stride new_bs
  void* ring;               // window buffer (B, slots, width)
  float* coef;              // (B, 2N, C) fp32
  const int32_t* c_list;    // compressed columns (C)
  void* mid;                // page store of the stored dims
  int64_t mid_bs;
  const int32_t* n_list;    // stored columns (Cn)
  const int32_t* n_h;
  const int32_t* pad_h;
  int C, Cn, is_v;
};

struct StreamParams {
  StreamTensor t[2];        // K, V
  int64_t new_bs, ring_bs, ring_rs;
  int evict_slot, write_slot;
  int N, T, Hkv, width, cap_pages;
  int64_t phase, mid_pos;
  // block ranges along x: [0, c_end[0]) K coefficients, [c_end[0], c_end[1]) V coefficients,
  // [c_end[1], a_end[0]) K append, [a_end[0], a_end[1]) V append, the rest: window write
  int c_end[2], a_end[2], cblk_n;   // cblk_n: frequency blocks per column block
};

// element offset inside one (batch, head) run of pages (the page layout of the public header)
__device__ __forceinline__ int64_t stream_page_offset(bool is_v, int dp, int64_t token, int j) {
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

template <typename E>
__global__ __launch_bounds__(256) void stream_update_kernel(const StreamParams p) {
  const int bx = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  if (bx < p.c_end[1]) {
    // ---- rank-1 coefficient update: block = 64 columns x 64 frequencies, thread = (column, 16 frequencies)
    // The phase factors depend on the frequency only: 64 threads evaluate one each (exactly reduced phase, as
    // fa_coeff_update) while the coefficient loads of all threads are on their way, and hand them over in LDS.
    __shared__ float2 s_cs[64];
    const int which = bx >= p.c_end[0];
    const StreamTensor& t = p.t[which];
    const int rel = bx - (which ? p.c_end[0] : 0);
    const int cb = rel / p.cblk_n, nb = rel - cb * p.cblk_n;
    const int lane = tid & 63, ng = tid >> 6;
    const int m = cb * 64 + lane;
    const bool live = m < t.C;
    const int n_beg = nb * 64;
    const int n_end = min(p.N, n_beg + 64);
    float e = 0.f;
    float* cbase = t.coef + (int64_t)b * 2 * p.N * t.C + (live ? m : 0);
    float cv[16], sv[16];
    if (live) {
      const E* old_row = (const E*)t.ring + (int64_t)b * p.ring_bs + (int64_t)p.evict_slot * p.ring_rs;
      e = fa_to_float(old_row[t.c_list[m]]);
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int n = min(n_beg + ng + 4 * i, p.N - 1);
        cv[i] = cbase[(int64_t)n * t.C];
        sv[i] = cbase[(int64_t)(p.N + n) * t.C];
      }
    }
    if (tid < 64) {
      float sn, co;
      fa_sincos_phase(min(n_beg + tid, p.N - 1), p.phase, p.T, &sn, &co);
      s_cs[tid] = make_float2(co, sn);
    }
    __syncthreads();
    if (live) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int n = n_beg + ng + 4 * i;
        if (n < n_end) {
          const float2 cs = s_cs[ng + 4 * i];
          cbase[(int64_t)n * t.C] = cv[i] + cs.x * e;
          cbase[(int64_t)(p.N + n) * t.C] = sv[i] + cs.y * e;
        }
      }
    }
    return;
  }
  if (bx < p.a_end[1]) {
    // ---- stored dims of the evicted row into the page store
    const int which = bx >= p.a_end[0];
    const StreamTensor& t = p.t[which];
    const int rel = bx - (which ? p.a_end[0] : p.c_end[1]);
    const int c = rel * 256 + tid;
    if (c >= t.Cn) return;
    int h = 0;
    while (h + 1 < p.Hkv && t.n_h[h + 1] <= c) ++h;
    const int j = c - t.n_h[h];
    const int p0 = t.pad_h[h], dp = t.pad_h[h + 1] - p0;
    const E* old_row = (const E*)t.ring + (int64_t)b * p.ring_bs + (int64_t)p.evict_slot * p.ring_rs;
    ((E*)t.mid)[(int64_t)b * t.mid_bs + (int64_t)p0 * 32 * p.cap_pages + stream_page_offset(t.is_v, dp, p.mid_pos, j)] =
        old_row[t.n_list[c]];
    return;
  }
  // ---- the new token into its window slot (K and V)
  const int rel = bx - p.a_end[1];
  for (int which = 0; which < 2; ++which) {
    const StreamTensor& t = p.t[which];
    const E* src = (const E*)t.new_row + (int64_t)b * p.new_bs;
    E* dst = (E*)t.ring + (int64_t)b * p.ring_bs + (int64_t)p.write_slot * p.ring_rs;
    const int i = rel * 256 + tid;
    if (i < p.width) dst[i] = src[i];
  }
}

}  // namespace

extern "C" int fa_stream_update(const fa_stream_args* a, fa_stream_t stream) {
  FA_REQUIRE(a, FA_ERR_NULL_POINTER, "fa_stream_update: args null");
  FA_REQUIRE(a->B > 0 && a->Hkv > 0 && a->width > 0 && a->N > 0 && a->T > 0 && a->cap_pages > 0, FA_ERR_BAD_SHAPE,
             "fa_stream_update: bad shape B=%d Hkv=%d width=%d N=%d T=%d cap_pages=%d", a->B, a->Hkv, a->width, a->N, a->T,
             a->cap_pages);
  FA_REQUIRE(a->evict_slot >= 0 && a->write_slot >= 0 && a->evict_slot != a->write_slot, FA_ERR_BAD_SHAPE,
             "fa_stream_update: the slot read (%d) and the slot written (%d) must differ", a->evict_slot, a->write_slot);
  FA_REQUIRE(a->phase >= 0 && a->mid_pos >= 0 && a->mid_pos < (int64_t)a->cap_pages * 32, FA_ERR_BAD_SHAPE,
             "fa_stream_update: phase %lld / position %lld outside the store", (long long)a->phase, (long long)a->mid_pos);
  FA_REQUIRE(a->dtype == FA_BF16 || a->dtype == FA_FP16 || a->dtype == FA_FP32, FA_ERR_BAD_DTYPE, "fa_stream_update: dtype %d",
             a->dtype);
  StreamParams p{};
  const void* news[2] = {a->k_new, a->v_new};
  void* rings[2] = {a->k_ring, a->v_ring};
  float* coefs[2] = {a->k_coef, a->v_coef};
  const int32_t* cl[2] = {a->kc_list, a->vc_list};
  void* mids[2] = {a->k_mid, a->v_mid};
  const int64_t mbs[2] = {a->k_mid_batch_stride, a->v_mid_batch_stride};
  const int32_t* nl[2] = {a->kn_list, a->vn_list};
  const int32_t* nh[2] = {a->kn_h_list, a->vn_h_list};
  const int32_t* ph[2] = {a->k_pad_h_list, a->v_pad_h_list};
  const int C[2] = {a->Ck, a->Cv}, Cn[2] = {a->Cnk, a->Cnv};
  for (int i = 0; i < 2; ++i) {
    FA_REQUIRE(news[i] && rings[i], FA_ERR_NULL_POINTER, "fa_stream_update: new row / window null");
    FA_REQUIRE(C[i] >= 0 && Cn[i] >= 0, FA_ERR_BAD_SHAPE, "fa_stream_update: negative column count");
    FA_REQUIRE(C[i] == 0 || (coefs[i] && cl[i]), FA_ERR_NULL_POINTER, "fa_stream_update: coefficients / column list null");
    FA_REQUIRE(Cn[i] == 0 || (mids[i] && nl[i] && nh[i] && ph[i]), FA_ERR_NULL_POINTER,
               "fa_stream_update: page store / index lists null");
    p.t[i] = StreamTensor{news[i], rings[i], coefs[i], cl[i], mids[i], mbs[i], nl[i], nh[i], ph[i], C[i], Cn[i], i};
  }
  p.new_bs = a->new_batch_stride; p.ring_bs = a->ring_batch_stride; p.ring_rs = a->ring_row_stride;
  p.evict_slot = a->evict_slot; p.write_slot = a->write_slot;
  p.N = a->N; p.T = a->T; p.Hkv = a->Hkv; p.width = a->width; p.cap_pages = a->cap_pages;
  p.phase = a->phase; p.mid_pos = a->mid_pos;
  p.cblk_n = fa_cdiv(a->N, 64);
  // (skip_coef: the launch has no coefficient blocks; the caller applies the rank-1 update elsewhere)
  p.c_end[0] = a->skip_coef ? 0 : fa_cdiv(C[0], 64) * p.cblk_n;
  p.c_end[1] = p.c_end[0] + (a->skip_coef ? 0 : fa_cdiv(C[1], 64) * p.cblk_n);
  p.a_end[0] = p.c_end[1] + fa_cdiv(Cn[0], 256);
  p.a_end[1] = p.a_end[0] + fa_cdiv(Cn[1], 256);
  const int total = p.a_end[1] + fa_cdiv(a->width, 256);
  dim3 grid(total, a->B);
  hipStream_t st = fa_hip_stream(stream);
  switch (a->dtype) {
    case FA_BF16: stream_update_kernel<bf16_t><<<grid, 256, 0, st>>>(p); break;
    case FA_FP16: stream_update_kernel<f16_t><<<grid, 256, 0, st>>>(p); break;
    default: stream_update_kernel<float><<<grid, 256, 0, st>>>(p); break;
  }
  return fa_check_launch("fa_stream_update");
}

extern "C" size_t fa_stream_args_size(void) { return sizeof(fa_stream_args); }
