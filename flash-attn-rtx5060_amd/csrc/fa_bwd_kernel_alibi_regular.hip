// Backward kernels with ALiBi for regular lengths (S a multiple of 128, as many keys, no dropout), in the
// reference's layout and in strided ones; in a translation unit of their own.  The bias enters the recomputed
// score in the key-owning kernel only; the five-product form's dQ kernel works on finished dS blocks.
#include "fa_bwd_kernel_impl.h"

hipError_t fa_launch_backward_alibi_regular(const FaBwdArgs &a, int bf16, int D, int masked, int strided, int compute_units,
                                            hipStream_t stream, bool configure_only)
{
#define FA_BWD_CASE(BF, DD, MK, ST) \
    if (bf16 == BF && D == DD && masked == MK && strided == ST) \
        return launch_bwd<BF != 0, DD, MK != 0, ST, true, false>(a, compute_units, stream, configure_only);
    FA_BWD_CASE(0, 64, 0, 0) FA_BWD_CASE(0, 64, 1, 0) FA_BWD_CASE(0, 128, 0, 0) FA_BWD_CASE(0, 128, 1, 0)
    FA_BWD_CASE(1, 64, 0, 0) FA_BWD_CASE(1, 64, 1, 0) FA_BWD_CASE(1, 128, 0, 0) FA_BWD_CASE(1, 128, 1, 0)
    FA_BWD_CASE(0, 64, 0, 1) FA_BWD_CASE(0, 64, 1, 1) FA_BWD_CASE(0, 128, 0, 1) FA_BWD_CASE(0, 128, 1, 1)
    FA_BWD_CASE(1, 64, 0, 1) FA_BWD_CASE(1, 64, 1, 1) FA_BWD_CASE(1, 128, 0, 1) FA_BWD_CASE(1, 128, 1, 1)
#undef FA_BWD_CASE
    return hipErrorInvalidValue;
}

// the LDS opt-in of every instantiation above for the current device, without a launch (fa_init)
hipError_t fa_configure_backward_alibi_regular()
{
    const FaBwdArgs a = {};
    for (int bf16 = 0; bf16 < 2; ++bf16)
        for (int D = 64; D <= 128; D += 64)
            for (int masked = 0; masked < 2; ++masked)
                for (int strided = 0; strided < 2; ++strided) {
                    const hipError_t e = fa_launch_backward_alibi_regular(a, bf16, D, masked, strided, 0, nullptr, true);
                    if (e != hipSuccess) return e;
                }
    return hipSuccess;
}
