// The matrix-core mid-row kernels of decode attention for f16 storage (see fa_decode_mid_launch.h).
#define FA_DECODE_MID_INSTANTIATE
#include "fa_decode_mid_launch.h"

namespace fa_mfma {
template void launch_mid_rows<f16_t>(const MidParams<f16_t>&, const MidLaunch&, hipStream_t);
}  // namespace fa_mfma
