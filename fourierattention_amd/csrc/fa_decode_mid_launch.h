// Launches of the matrix-core mid-row kernel (fa_decode_mfma.h).  Its instances are many and each takes seconds to
// compile, so they live in translation units of their own, one per storage type (fa_decode_mid_bf16.hip,
// fa_decode_mid_f16.hip), which the build compiles side by side with fa_decode.hip; everybody else sees the
// declaration of launch_mid_rows only.
#pragma once

#include "fa_decode_mfma.h"

namespace fa_mfma {

struct MidLaunch {
  int n_wg, n_groups;   // workgroups per batch group, batch groups
  int ks;               // ksteps per frequency slice (2, 4 or 8)
  bool wide;            // a head stores more than 64 K or V dims
  bool two_pass;        // 1024 frequencies: a score pass, then a value pass over the same pages
  bool fused;           // the (last) launch merges its own partials; its workgroups are numbered through mp.fz.wg_map
  bool sub;             // ... and runs four sub-splits per workgroup (a batch of one sequence)
};

template <typename E>
void launch_mid_rows(const MidParams<E>& mp, const MidLaunch& ml, hipStream_t st);

#ifdef FA_DECODE_MID_INSTANTIATE
// eight frequency slices: a score pass, then a value pass over the same pages
// (fused: the value pass merges its own partials; its workgroups are then numbered through wg_map, those of the score
// pass, which hands over whole pages of scores, keep the plain numbering)
template <typename E>
void launch_mid_mfma_two_pass(const MidParams<E>& mp, const MidLaunch& ml, hipStream_t st) {
  dim3 grid(ml.n_wg, ml.n_groups), flat(ml.n_wg * ml.n_groups);
  if (ml.wide) {
    decode_mid_mfma_kernel<E, 8, 4, 8, 3, 1><<<grid, 512, 0, st>>>(mp);
    if (ml.fused) decode_mid_mfma_kernel<E, 8, 4, 8, 3, 2, true><<<flat, 512, 0, st>>>(mp);
    else decode_mid_mfma_kernel<E, 8, 4, 8, 3, 2><<<grid, 512, 0, st>>>(mp);
  } else {
    decode_mid_mfma_kernel<E, 8, 2, 4, 4, 1><<<grid, 512, 0, st>>>(mp);
    if (ml.fused) decode_mid_mfma_kernel<E, 8, 2, 4, 4, 2, true><<<flat, 512, 0, st>>>(mp);
    else decode_mid_mfma_kernel<E, 8, 2, 4, 4, 2><<<grid, 512, 0, st>>>(mp);
  }
}

template <typename E, int KS>
void launch_mid_mfma_ks(const MidParams<E>& mp, const MidLaunch& ml, hipStream_t st) {
  dim3 grid(ml.n_wg, ml.n_groups);
  if (ml.fused) {
    grid = dim3(ml.n_wg * ml.n_groups);   // numbered through wg_map
    const bool upd = mp.fz.upd_row != nullptr;   // (instances of their own, like the query preparation's)
    auto go = [&](auto sub_tag, auto upd_tag) {
      constexpr bool S = decltype(sub_tag)::value, U = decltype(upd_tag)::value;
      if (ml.wide)
        decode_mid_mfma_kernel<E, KS, 4, 8, 2, 0, true, S, U><<<grid, 512, 0, st>>>(mp);
      else
        decode_mid_mfma_kernel<E, KS, 2, 4, 2, 0, true, S, U><<<grid, 512, 0, st>>>(mp);
    };
    if (ml.sub && upd) go(std::true_type{}, std::true_type{});
    else if (ml.sub) go(std::true_type{}, std::false_type{});
    else if (upd) go(std::false_type{}, std::true_type{});
    else go(std::false_type{}, std::false_type{});
  } else if (ml.wide) {
    decode_mid_mfma_kernel<E, KS, 4, 8, 2><<<grid, 512, 0, st>>>(mp);
  } else {
    decode_mid_mfma_kernel<E, KS, 2, 4, 2><<<grid, 512, 0, st>>>(mp);
  }
}

template <typename E>
void launch_mid_rows(const MidParams<E>& mp, const MidLaunch& ml, hipStream_t st) {
  if (ml.two_pass) launch_mid_mfma_two_pass<E>(mp, ml, st);
  else switch (ml.ks) {
    case 2: launch_mid_mfma_ks<E, 2>(mp, ml, st); break;
    case 4: launch_mid_mfma_ks<E, 4>(mp, ml, st); break;
    default: launch_mid_mfma_ks<E, 8>(mp, ml, st); break;
  }
}
#else
extern template void launch_mid_rows<bf16_t>(const MidParams<bf16_t>&, const MidLaunch&, hipStream_t);
extern template void launch_mid_rows<f16_t>(const MidParams<f16_t>&, const MidLaunch&, hipStream_t);
#endif

}  // namespace fa_mfma
