// conv_mfma_kernel for tiles of 128 output channels x 128 pixels, 128 K-bytes per step, 4 wavefronts.
#include "conv_mfma_kernel.h"

namespace chx {

int launch_conv_mfma_2_2_128_2(const ConvMfmaArgs& a, bool x_unsigned, bool out_int32, bool rne, int max_wgs_per_cu, hipStream_t s) {
    return launch_config<2, 2, 128, 2>(a, x_unsigned, out_int32, rne, max_wgs_per_cu, s);
}

}  // namespace chx
