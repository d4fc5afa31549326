// Backward kernels without dropout: the instantiations for the reference's layout and the general ones.
#include "fa_bwd_kernel_impl.h"

// layout 0: the reference's; 2 (general): strides, any lengths, grouped K/V heads (always with the mask code);
// alibi needs general.  (Layout 1, strided, is instantiated in a translation unit of its own.)
hipError_t fa_launch_backward(const FaBwdArgs &a, int bf16, int D, int masked, int general, int alibi, int compute_units,
                              hipStream_t stream, bool configure_only)
{
#define FA_BWD_CASE(BF, DD, MK, GN, AL) \
    if (bf16 == BF && D == DD && masked == MK && general == GN && alibi == AL) \
        return launch_bwd<BF != 0, DD, MK != 0, GN != 0 ? 2 : 0, AL != 0, false>(a, compute_units, stream, configure_only);
    FA_BWD_CASE(0, 64, 0, 0, 0) FA_BWD_CASE(0, 64, 1, 0, 0) FA_BWD_CASE(0, 128, 0, 0, 0) FA_BWD_CASE(0, 128, 1, 0, 0)
    FA_BWD_CASE(1, 64, 0, 0, 0) FA_BWD_CASE(1, 64, 1, 0, 0) FA_BWD_CASE(1, 128, 0, 0, 0) FA_BWD_CASE(1, 128, 1, 0, 0)
    FA_BWD_CASE(0, 64, 1, 1, 0) FA_BWD_CASE(0, 128, 1, 1, 0) FA_BWD_CASE(1, 64, 1, 1, 0) FA_BWD_CASE(1, 128, 1, 1, 0)
    FA_BWD_CASE(0, 64, 1, 1, 1) FA_BWD_CASE(0, 128, 1, 1, 1) FA_BWD_CASE(1, 64, 1, 1, 1) FA_BWD_CASE(1, 128, 1, 1, 1)
#undef FA_BWD_CASE
    return hipErrorInvalidValue;
}

// the LDS opt-in of every instantiation above for the current device, without a launch (fa_init)
hipError_t fa_configure_backward()
{
    const FaBwdArgs a = {};
    for (int bf16 = 0; bf16 < 2; ++bf16)
        for (int D = 64; D <= 128; D += 64)
            for (int combo = 0; combo < 4; ++combo) {
                // (not masked, masked) in the reference's layout; general; general with ALiBi
                const int masked = combo != 0, general = combo >= 2, alibi = combo == 3;
                const hipError_t e = fa_launch_backward(a, bf16, D, masked, general, alibi, 0, nullptr, true);
                if (e != hipSuccess) return e;
            }
    return hipSuccess;
}
