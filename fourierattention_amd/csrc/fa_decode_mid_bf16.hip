// The matrix-core mid-row kernels of decode attention for bf16 storage (see fa_decode_mid_launch.h).
#define FA_DECODE_MID_INSTANTIATE
#include "fa_decode_mid_launch.h"

namespace fa_mfma {
template void launch_mid_rows<bf16_t>(const MidParams<bf16_t>&, const MidLaunch&, hipStream_t);
}  // namespace fa_mfma
