// Exact causal attention over full-width keys: the prompt pass of the attention forward
// (fourier_attn_triton/modeling_llama_fourier.py:623-633, flash_attn_func(q, k, v, causal=True)).
//
// Everything is computed transposed, so that no operand ever has to change lanes between the two products:
//   S^T[keys x rows] = K[keys x D] . Q^T[D x rows]        A = K rows as they lie in memory (a lane takes 16 bytes
//                                                          of one key), B = query rows (16 bytes of one row)
//   P^T = exp2(S^T - m)                                    per row = per lane column: running reference, base 2
//   O^T[D x rows] += V^T[D x keys] . P^T[keys x rows]      B = the lane's own eight probabilities of a 32-key tile
// The accumulator layout gives a lane the keys 4 lg .. 4 lg + 3 of each 16-key block; taking the two blocks of a
// 32-key tile as ONE contraction step whose slots are ordered {4 lg .. 4 lg + 3 of block 0, the same of block 1}
// makes those eight values the B operand as they are.  The A operand of that step, V^T with the keys in the same
// slot order, is prepared once per call by a transposing pass over V (prefill_vt_kernel): 1 KiB fragments that
// the main kernel streams into LDS unchanged.
//
// Workgroup: one KV head, HW query heads of it (all that share its keys, up to four) times RW blocks of 32 query
// rows, one wave each.  The key tiles travel HBM -> LDS once per workgroup (global_load_lds, two stages, one
// meeting per tile) in fragment order, so every LDS read of a wave is one conflict-free 16 bytes per lane.
#include "fa_common.h"
#include "fa_mfma_util.h"

namespace {
using namespace fa_mfma;

constexpr int kTileKeys = 32;

template <typename E>
struct PrefillParams {
  const E* q;          // (B, Hq, q_len, D) through strides, D contiguous
  int64_t q_bs, q_hs, q_rs;
  const E* k;          // (B, S, Hkv * D) token-major
  int64_t k_bs, k_rs;
  const f16_t* vt;     // [B][Hkv][tiles][D / 16][64 lanes][8]: V^T fragments, always f16 (see prefill_vt_kernel)
  E* out;              // (B, q_len, Hq, D) contiguous
  int B, Hq, Hkv, S, q_len, n_tiles, HW, RW;
  float sm_log2e;
};

// slot e of lane group lg in a 32-key tile
__device__ __forceinline__ int slot_key(int lg, int e) { return e < 4 ? 4 * lg + e : 16 + 4 * lg + (e - 4); }

template <typename E, int D>
__global__ __launch_bounds__(256) void prefill_vt_kernel(const E* __restrict__ v, int64_t v_bs, int64_t v_rs,
                                                         f16_t* __restrict__ vt, int S, int Hkv, int n_tiles) {
  // The second product runs in f16 whatever the storage type: the reference computes this attention as
  // flash_attn_func(q.half(), k.half(), v.half()) (MODEL:633), with probabilities of 11 significant bits; a bf16
  // operand would keep 8.  bf16 -> f16 is exact between 2^-14 and 65504 (larger magnitudes are clamped there).
  struct alignas(sizeof(E) * 8) Piece { E e[8]; };
  struct alignas(16) PieceOut { f16_t e[8]; };
  __shared__ __attribute__((aligned(16))) E tile[kTileKeys][D + 8];
  const int t = blockIdx.x, h = blockIdx.y, b = blockIdx.z, tid = threadIdx.x;
  const E* src = v + (int64_t)b * v_bs + (int64_t)h * D;
  constexpr int PPR = D / 8;
  for (int pidx = tid; pidx < kTileKeys * PPR; pidx += 256) {
    const int r = pidx / PPR, c = pidx - r * PPR;
    const int key = t * kTileKeys + r;
    Piece pc{};
    if (key < S) pc = *(const Piece*)(src + (int64_t)key * v_rs + c * 8);
    *(Piece*)&tile[r][c * 8] = pc;
  }
  __syncthreads();
  PieceOut* dst = (PieceOut*)(vt + (((int64_t)b * Hkv + h) * n_tiles + t) * (int64_t)(kTileKeys * D));
  for (int pidx = tid; pidx < (D / 16) * 64; pidx += 256) {
    const int dg = pidx >> 6, lane = pidx & 63, lg = lane >> 4, ld = lane & 15;
    PieceOut o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float x = fa_to_float(tile[slot_key(lg, e)][16 * dg + ld]);
      o.e[e] = f16_t{(_Float16)fminf(fmaxf(x, -65504.f), 65504.f)};
    }
    dst[pidx] = o;
  }
}

template <typename E, int D, int WAVES>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(3, 3))) void prefill_attn_kernel(const PrefillParams<E> p) {
  using M = Mma<E>;
  using vec8 = typename M::vec8;
  constexpr int KS = D / 32, DG = D / 16;
  constexpr int NF = 2 * KS + DG;                 // fragments (1 KiB) of one key tile: K (block, kstep), then V^T
  constexpr int OPS = (NF + WAVES - 1) / WAVES;   // fragments a wave brings in per tile
  __shared__ __attribute__((aligned(16))) unsigned char s_tile[2][NF * 1024];

  const int tid = threadIdx.x, lane = tid & 63, lg = lane >> 4, lc = lane & 15;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int G = p.Hq / p.Hkv;
  const int groups = G / p.HW;                    // workgroups per KV head along the heads
  const int kvh = blockIdx.y / groups, hg = blockIdx.y - kvh * groups;
  const int b = blockIdx.z;
  const int head = kvh * G + hg * p.HW + (w % p.HW);
  const int rblk = ((int)gridDim.x - 1 - (int)blockIdx.x) * p.RW + w / p.HW;   // long rows first
  const int r0 = rblk * 32;
  const int offset = p.S - p.q_len;               // row i sees keys 0 .. i + offset
  const int wg_last_row = min(p.q_len, ((int)gridDim.x - (int)blockIdx.x) * p.RW * 32) - 1;
  const int n_t = min(p.n_tiles, (wg_last_row + offset) / kTileKeys + 1);

  // this wave's share of a tile: fragments w, w + WAVES, ... (clamped to the last one: every wave issues OPS loads)
  const E* kb_base = p.k + (int64_t)b * p.k_bs + (int64_t)kvh * D + 8 * lg;
  const f16_t* vt_base = p.vt + ((int64_t)b * p.Hkv + kvh) * p.n_tiles * (int64_t)(kTileKeys * D) + lane * 8;
  // The tiles are requested in order, so every load keeps a running pointer that moves on by one tile; only a last
  // tile that reaches past the keys computes its (clamped) rows afresh.
  const E* run[OPS];
#pragma unroll
  for (int i = 0; i < OPS; ++i) {
    const int f = min(w + i * WAVES, NF - 1);
    if (f < 2 * KS) run[i] = kb_base + (int64_t)(16 * (f / KS) + lc) * p.k_rs + 32 * (f % KS);
    else run[i] = (const E*)(vt_base + (int64_t)(f - 2 * KS) * 512);   // (both 16-bit: the pointer only counts elements)
  }
  const int64_t k_step = (int64_t)kTileKeys * p.k_rs;
  const bool ragged_keys = (p.S % kTileKeys) != 0;
  auto issue = [&](int t, int buf) {
    const bool clamp = ragged_keys && t == p.n_tiles - 1;   // wave-uniform
#pragma unroll
    for (int i = 0; i < OPS; ++i) {
      const int f = min(w + i * WAVES, NF - 1);
      const E* src = run[i];
      if (f < 2 * KS) {
        if (clamp) {
          const int key = min(t * kTileKeys + 16 * (f / KS) + lc, p.S - 1);
          src = kb_base + (int64_t)key * p.k_rs + 32 * (f % KS);
        }
        run[i] += k_step;
      } else {
        run[i] += DG * 512;
      }
      load_frag_to_lds(src, &s_tile[buf][f * 1024]);
    }
  };
  if (n_t > 0) issue(0, 0);

  // query rows of this wave as B operands: row 16 rb + lc, dims 32 ks + 8 lg ..
  vec8 Qf[2][KS];
  {
    const E* qb = p.q + (int64_t)b * p.q_bs + (int64_t)head * p.q_hs + 8 * lg;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      const int row = min(r0 + 16 * rb + lc, p.q_len - 1);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        Qf[rb][ks] = __builtin_bit_cast(vec8, *(const uint4v*)(qb + (int64_t)row * p.q_rs + 32 * ks));
    }
  }
  float4v oacc[DG][2];
#pragma unroll
  for (int dg = 0; dg < DG; ++dg) oacc[dg][0] = oacc[dg][1] = float4v{0.f, 0.f, 0.f, 0.f};
  float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.f, 0.f};
  // the query loads above must not be confused with the tile loads by the counted waits below
#pragma unroll
  for (int rb = 0; rb < 2; ++rb)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) asm volatile("" ::"v"(Qf[rb][ks]));

  for (int t = 0; t < n_t; ++t) {
    const int buf = t & 1;
    wait_vmcnt<0>();        // this wave's fragments of tile t have landed (nothing else is outstanding)
    barrier_lds_only();     // everybody's have, and everybody is done with the other stage
    if (t + 1 < n_t) issue(t + 1, buf ^ 1);
    if (t * kTileKeys > r0 + 31 + offset) continue;   // this wave's rows end before the tile (a lower row block)
    const unsigned base = lds_addr_of(&s_tile[buf][0]) + lane * 16;
    // ---- S^T = K . Q^T
    float4v sacc[2][2] = {{float4v{0.f, 0.f, 0.f, 0.f}, float4v{0.f, 0.f, 0.f, 0.f}},
                          {float4v{0.f, 0.f, 0.f, 0.f}, float4v{0.f, 0.f, 0.f, 0.f}}};
    // K fragments f = block * KS + kstep, two at a time into alternating halves of kf: the reads of a pair are on
    // their way while the matrix unit works on the pair before
    uint4v kf[4];
    constexpr int NFK = 2 * KS;
    auto s_pair = [&](uint4v& f0, uint4v& f1, int f) {   // fragments f, f + 1 (f is a constant after unrolling)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        sacc[f / KS][rb] = M::mma(__builtin_bit_cast(vec8, f0), Qf[rb][f % KS], sacc[f / KS][rb]);
        sacc[(f + 1) / KS][rb] = M::mma(__builtin_bit_cast(vec8, f1), Qf[rb][(f + 1) % KS], sacc[(f + 1) / KS][rb]);
      }
    };
    kf[0] = lds_read_b128_async_at<0 * 1024>(base);
    kf[1] = lds_read_b128_async_at<1 * 1024>(base);
    kf[2] = lds_read_b128_async_at<2 * 1024>(base);
    kf[3] = lds_read_b128_async_at<3 * 1024>(base);
    if constexpr (NFK == 8) {
      lds_wait_for2<2>(kf[0], kf[1]);
      s_pair(kf[0], kf[1], 0);
      kf[0] = lds_read_b128_async_at<4 * 1024>(base);
      kf[1] = lds_read_b128_async_at<5 * 1024>(base);
      lds_wait_for2<2>(kf[2], kf[3]);
      s_pair(kf[2], kf[3], 2);
      kf[2] = lds_read_b128_async_at<6 * 1024>(base);
      kf[3] = lds_read_b128_async_at<7 * 1024>(base);
      lds_wait_for2<2>(kf[0], kf[1]);
      s_pair(kf[0], kf[1], 4);
      lds_wait_for2<0>(kf[2], kf[3]);
      s_pair(kf[2], kf[3], 6);
    } else {   // heads of 64 dims: four fragments
      static_assert(NFK == 4, "head dims of 64 or 128");
      lds_wait_for2<2>(kf[0], kf[1]);
      s_pair(kf[0], kf[1], 0);
      lds_wait_for2<0>(kf[2], kf[3]);
      s_pair(kf[2], kf[3], 2);
    }
    // V^T fragments of the first half of the dims are requested now and used after the softmax
    uint4v vf[4];
    const unsigned vbase = base + 2 * KS * 1024;
    vf[0] = lds_read_b128_async_at<0>(vbase);
    vf[1] = lds_read_b128_async_at<1024>(vbase);
    vf[2] = lds_read_b128_async_at<2048>(vbase);
    vf[3] = lds_read_b128_async_at<3072>(vbase);
    // ---- softmax of the tile (base 2), per row = per lane column
    const bool edge = t * kTileKeys + 31 > r0 + offset || t * kTileKeys + 31 >= p.S;   // wave-uniform
    half8 pb[2];   // probabilities as f16 operands
    float alpha[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
      float s[8];   // raw products: the softmax scale rides in the instruction that subtracts the reference
#pragma unroll
      for (int e = 0; e < 8; ++e) s[e] = sacc[e >> 2][rb][e & 3];
      if (edge) {
        asm volatile("");   // a real branch: as selects these masks would run on every tile
        const int row_lim = r0 + 16 * rb + lc + offset;   // last key this row may see
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int key = t * kTileKeys + slot_key(lg, e);
          if (key > row_lim || key >= p.S) s[e] = -INFINITY;
        }
      }
      float tmax = fa_fmax8(s);
      tmax = fa_rows_max(tmax) * p.sm_log2e;   // (the scale is positive)
      const float m_new = fa_fmax(m_run[rb], tmax);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;   // a row that has seen no key yet
      alpha[rb] = __builtin_amdgcn_exp2f(m_run[rb] - m_use);   // 0 on the row's first tile
      float psum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s[e], p.sm_log2e, -m_use));
        psum += pv;
        pb[rb][e] = (_Float16)pv;
      }
      l_run[rb] = l_run[rb] * alpha[rb] + psum;
      m_run[rb] = m_new;
    }
    if (__any(alpha[0] != 1.0f || alpha[1] != 1.0f)) {
#pragma unroll
      for (int dg = 0; dg < DG; ++dg) {
        oacc[dg][0] *= alpha[0];
        oacc[dg][1] *= alpha[1];
      }
    }
    // ---- O^T += V^T . P^T (the fragments in pairs, like the K fragments above)
    auto o_pair = [&](uint4v& f0, uint4v& f1, int dg) {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        oacc[dg][rb] = Mma<f16_t>::mma(__builtin_bit_cast(half8, f0), pb[rb], oacc[dg][rb]);
        oacc[dg + 1][rb] = Mma<f16_t>::mma(__builtin_bit_cast(half8, f1), pb[rb], oacc[dg + 1][rb]);
      }
    };
    if constexpr (DG == 8) {
      lds_wait_for2<2>(vf[0], vf[1]);
      o_pair(vf[0], vf[1], 0);
      vf[0] = lds_read_b128_async_at<4 * 1024>(vbase);
      vf[1] = lds_read_b128_async_at<5 * 1024>(vbase);
      lds_wait_for2<2>(vf[2], vf[3]);
      o_pair(vf[2], vf[3], 2);
      vf[2] = lds_read_b128_async_at<6 * 1024>(vbase);
      vf[3] = lds_read_b128_async_at<7 * 1024>(vbase);
      lds_wait_for2<2>(vf[0], vf[1]);
      o_pair(vf[0], vf[1], 4);
      lds_wait_for2<0>(vf[2], vf[3]);
      o_pair(vf[2], vf[3], 6);
    } else {
      static_assert(DG == 4, "head dims of 64 or 128");
      lds_wait_for2<2>(vf[0], vf[1]);
      o_pair(vf[0], vf[1], 0);
      lds_wait_for2<0>(vf[2], vf[3]);
      o_pair(vf[2], vf[3], 2);
    }
  }

  // ---- out[b, row, head, :] = O / l
  typedef typename M::elem elem4 __attribute__((ext_vector_type(4)));
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    const float l = fa_rows_sum(l_run[rb]);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    const int row = r0 + 16 * rb + lc;
    if (row < p.q_len) {
      E* o = p.out + (((int64_t)b * p.q_len + row) * p.Hq + head) * D + 4 * lg;
#pragma unroll
      for (int dg = 0; dg < DG; ++dg) {
        elem4 e4;
#pragma unroll
        for (int v = 0; v < 4; ++v) e4[v] = (typename M::elem)(oacc[dg][rb][v] * inv);
        *(elem4*)(o + 16 * dg) = e4;
      }
    }
  }
}

template <typename E, int D>
int launch_prefill(const void* q, int64_t q_bs, int64_t q_hs, int64_t q_rs, const void* k, int64_t k_bs, int64_t k_rs,
                   const void* v, int64_t v_bs, int64_t v_rs, void* out, void* workspace, int B, int Hq, int Hkv, int S,
                   int q_len, float sm_scale, hipStream_t st) {
  const int n_tiles = fa_cdiv(S, kTileKeys);
  f16_t* vt = (f16_t*)workspace;
  prefill_vt_kernel<E, D><<<dim3(n_tiles, Hkv, B), 256, 0, st>>>((const E*)v, v_bs, v_rs, vt, S, Hkv, n_tiles);
  const int G = Hq / Hkv;
  PrefillParams<E> p{};
  p.q = (const E*)q; p.q_bs = q_bs; p.q_hs = q_hs; p.q_rs = q_rs;
  p.k = (const E*)k; p.k_bs = k_bs; p.k_rs = k_rs;
  p.vt = vt; p.out = (E*)out;
  p.B = B; p.Hq = Hq; p.Hkv = Hkv; p.S = S; p.q_len = q_len; p.n_tiles = n_tiles;
  p.HW = G % 4 == 0 ? 4 : G % 3 == 0 ? 3 : G % 2 == 0 ? 2 : 1;   // query heads of one KV head per workgroup
  p.RW = 4 / p.HW;                                                // blocks of 32 query rows per workgroup
  p.sm_log2e = sm_scale * 1.4426950408889634f;
  const int waves = p.HW * p.RW;
  dim3 grid(fa_cdiv(q_len, 32 * p.RW), Hkv * (G / p.HW), B);
  if (waves == 3) prefill_attn_kernel<E, D, 3><<<grid, 192, 0, st>>>(p);
  else prefill_attn_kernel<E, D, 4><<<grid, 256, 0, st>>>(p);
  return fa_check_launch("fa_prefill_attn");
}

}  // namespace

extern "C" size_t fa_prefill_attn_workspace_bytes(int B, int Hkv, int D, int S) {
  if (B <= 0 || Hkv <= 0 || D <= 0 || S <= 0) return 0;
  return (size_t)B * Hkv * fa_cdiv(S, kTileKeys) * kTileKeys * D * 2;
}

extern "C" int fa_prefill_attn(const void* q, int64_t q_batch_stride, int64_t q_head_stride, int64_t q_row_stride,
                               const void* k, const void* v, int64_t kv_batch_stride, int64_t kv_row_stride, void* out,
                               int dtype, int B, int Hq, int Hkv, int D, int S, int q_len, float sm_scale,
                               void* workspace, size_t workspace_bytes, fa_stream_t stream) {
  FA_REQUIRE(q && k && v && out, FA_ERR_NULL_POINTER, "fa_prefill_attn: null pointer");
  FA_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && S > 0 && q_len > 0 && q_len <= S && Hq % Hkv == 0, FA_ERR_BAD_SHAPE,
             "fa_prefill_attn: B=%d Hq=%d Hkv=%d S=%d q_len=%d", B, Hq, Hkv, S, q_len);
  FA_REQUIRE(dtype == FA_BF16 || dtype == FA_FP16, FA_ERR_BAD_DTYPE,
             "fa_prefill_attn: dtype %d (the matrix cores take 16-bit operands)", dtype);
  FA_REQUIRE(D == 64 || D == 128, FA_ERR_UNSUPPORTED, "fa_prefill_attn: head_dim %d (64 or 128)", D);
  const size_t need = fa_prefill_attn_workspace_bytes(B, Hkv, D, S);
  FA_REQUIRE(workspace && workspace_bytes >= need, FA_ERR_WORKSPACE, "fa_prefill_attn: workspace %zu < %zu",
             workspace_bytes, need);
  FA_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out | (uintptr_t)workspace) & 15) == 0 &&
                 ((q_batch_stride | q_head_stride | q_row_stride | kv_batch_stride | kv_row_stride) & 7) == 0,
             FA_ERR_MISALIGNED, "fa_prefill_attn: rows must be 16-byte aligned");
  FA_REQUIRE(B <= 65535 && Hq <= 65535, FA_ERR_UNSUPPORTED, "fa_prefill_attn: batch or head count above 65535");
  const float sm = sm_scale > 0.f ? sm_scale : 1.0f / sqrtf((float)D);
  hipStream_t st = fa_hip_stream(stream);
#define FA_PREFILL(E, DD)                                                                                              \
  return launch_prefill<E, DD>(q, q_batch_stride, q_head_stride, q_row_stride, k, kv_batch_stride, kv_row_stride, v,   \
                               kv_batch_stride, kv_row_stride, out, workspace, B, Hq, Hkv, S, q_len, sm, st)
  if (dtype == FA_BF16) {
    if (D == 128) FA_PREFILL(bf16_t, 128);
    FA_PREFILL(bf16_t, 64);
  }
  if (D == 128) FA_PREFILL(f16_t, 128);
  FA_PREFILL(f16_t, 64);
#undef FA_PREFILL
}
