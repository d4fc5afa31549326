// Backward kernels for the strided layout: lengths as in the reference's layout (S a multiple of 128, as many
// keys), any row, head and batch strides, grouped K/V heads; in a translation unit of their own.
#include "fa_bwd_kernel_impl.h"

hipError_t fa_launch_backward_strided(const FaBwdArgs &a, int bf16, int D, int masked, int compute_units, hipStream_t stream,
                                      bool configure_only)
{
#define FA_BWD_CASE(BF, DD, MK) \
    if (bf16 == BF && D == DD && masked == MK) return launch_bwd<BF != 0, DD, MK != 0, 1, false, false>(a, compute_units, stream, configure_only);
    FA_BWD_CASE(0, 64, 0) FA_BWD_CASE(0, 64, 1) FA_BWD_CASE(0, 128, 0) FA_BWD_CASE(0, 128, 1)
    FA_BWD_CASE(1, 64, 0) FA_BWD_CASE(1, 64, 1) FA_BWD_CASE(1, 128, 0) FA_BWD_CASE(1, 128, 1)
#undef FA_BWD_CASE
    return hipErrorInvalidValue;
}

// the LDS opt-in of every instantiation above for the current device, without a launch (fa_init)
hipError_t fa_configure_backward_strided()
{
    const FaBwdArgs a = {};
    for (int bf16 = 0; bf16 < 2; ++bf16)
        for (int D = 64; D <= 128; D += 64)
            for (int masked = 0; masked < 2; ++masked) {
                const hipError_t e = fa_launch_backward_strided(a, bf16, D, masked, 0, nullptr, true);
                if (e != hipSuccess) return e;
            }
    return hipSuccess;
}
