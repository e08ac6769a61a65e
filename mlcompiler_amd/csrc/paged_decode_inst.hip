// One translation unit per (head_dim, heads-per-wave) pair of the fast decode kernel:
// compiled with -DMLC_D=<64|128> -DMLC_HPW=<1|2|4|8>, so the variants build in parallel.
#include "paged_decode_kernels.h"

#ifndef MLC_D
#error "compile with -DMLC_D=64|128 -DMLC_HPW=1|2|4|8"
#endif

#define MLC_CAT_(a, b, c) launch_decode_fast_##a##_##b
#define MLC_CAT(a, b) MLC_CAT_(a, b, 0)

namespace mlc_hip {

namespace {
template <int NW, int NS>
void launch_one(bool pv16, const DecodeArgs& a, hipStream_t stream) {
    const dim3 grid(a.n_items), block(64 * NW * NS);
    if (pv16)
        hipLaunchKernelGGL((paged_decode_fast_kernel<MLC_D, MLC_HPW, NW, NS, true>), grid, block, 0, stream, a);
    else
        hipLaunchKernelGGL((paged_decode_fast_kernel<MLC_D, MLC_HPW, NW, NS, false>), grid, block, 0, stream, a);
}
}  // namespace

// nw = waves over the GQA group, ns = tile rows; returns false for an unbuilt combination.
bool MLC_CAT(MLC_D, MLC_HPW)(int nw, int ns, bool pv16, const DecodeArgs& a, hipStream_t stream) {
    const int key = nw * 10 + ns;
    switch (key) {
        case 11: launch_one<1, 1>(pv16, a, stream); return true;
        case 12: launch_one<1, 2>(pv16, a, stream); return true;
        case 14: launch_one<1, 4>(pv16, a, stream); return true;
        case 21: launch_one<2, 1>(pv16, a, stream); return true;
        case 22: launch_one<2, 2>(pv16, a, stream); return true;
        case 24: launch_one<2, 4>(pv16, a, stream); return true;
        case 41: launch_one<4, 1>(pv16, a, stream); return true;
        case 42: launch_one<4, 2>(pv16, a, stream); return true;
        default: return false;
    }
}

}  // namespace mlc_hip
