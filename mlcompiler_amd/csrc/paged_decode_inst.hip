// One translation unit per (head_dim, heads-per-wave) pair of the fast decode kernel:
// compiled with -DMLC_D=<64|128> -DMLC_HPW=<1|2|4|8>, so the variants build in parallel.
#include "paged_decode_kernels.h"
#include "paged_decode_stream.h"

#ifndef MLC_D
#error "compile with -DMLC_D=64|128 -DMLC_HPW=1|2|4|8"
#endif

#define MLC_CAT_(a, b, c) launch_decode_fast_##a##_##b
#define MLC_CAT(a, b) MLC_CAT_(a, b, 0)
#define MLC_SCAT_(a, b, c) launch_decode_stream_##a##_##b
#define MLC_SCAT(a, b) MLC_SCAT_(a, b, 0)

namespace mlc_hip {

namespace {
template <int NW, int NS, int NBUF>
bool launch_buf(bool pv16, const DecodeArgs& a, hipStream_t stream) {
    if constexpr (decode_lds_bytes(MLC_D, MLC_HPW, NW, NS, NBUF) <= kMaxStaticLds) {
        const dim3 grid(a.n_items), block(64 * NW * NS);
        if (pv16)
            hipLaunchKernelGGL((paged_decode_fast_kernel<MLC_D, MLC_HPW, NW, NS, NBUF, true>), grid, block, 0, stream, a);
        else
            hipLaunchKernelGGL((paged_decode_fast_kernel<MLC_D, MLC_HPW, NW, NS, NBUF, false>), grid, block, 0, stream, a);
        return true;
    } else {
        return false;
    }
}

template <int NW, int NS>
bool launch_one(int nbuf, bool pv16, const DecodeArgs& a, hipStream_t stream) {
    return nbuf == 1 ? launch_buf<NW, NS, 1>(pv16, a, stream) : launch_buf<NW, NS, 2>(pv16, a, stream);
}
}  // namespace

// nw = waves over the GQA group, ns = tile rows; returns false for an unbuilt combination.
bool MLC_CAT(MLC_D, MLC_HPW)(int nw, int ns, int nbuf, bool pv16, const DecodeArgs& a, hipStream_t stream) {
    const int key = nw * 10 + ns;
    switch (key) {
        case 11: return launch_one<1, 1>(nbuf, pv16, a, stream);
        case 12: return launch_one<1, 2>(nbuf, pv16, a, stream);
        case 21: return launch_one<2, 1>(nbuf, pv16, a, stream);
        case 22: return launch_one<2, 2>(nbuf, pv16, a, stream);
        case 41: return launch_one<4, 1>(nbuf, pv16, a, stream);
        case 42: return launch_one<4, 2>(nbuf, pv16, a, stream);
        default: return false;
    }
}

namespace {
template <int NW>
bool launch_stream(bool pv16, const StreamArgs& a, unsigned n_wg, size_t dyn_lds, hipStream_t stream) {
    if constexpr (stream_static_lds_bytes(MLC_D, MLC_HPW * NW) <= 60 * 1024) {
        const dim3 grid(n_wg), block(64 * NW);
        if (pv16)
            hipLaunchKernelGGL((paged_decode_stream_kernel<MLC_D, MLC_HPW, NW, true>), grid, block, dyn_lds, stream, a);
        else
            hipLaunchKernelGGL((paged_decode_stream_kernel<MLC_D, MLC_HPW, NW, false>), grid, block, dyn_lds, stream, a);
        return true;
    } else {
        return false;
    }
}
}  // namespace

// Tile-balanced kernel: nw = waves over the GQA group, n_wg = grid size; false for an unbuilt combination.
bool MLC_SCAT(MLC_D, MLC_HPW)(int nw, bool pv16, const StreamArgs& a, unsigned n_wg, size_t dyn_lds, hipStream_t stream) {
    switch (nw) {
        case 1: return launch_stream<1>(pv16, a, n_wg, dyn_lds, stream);
        case 2: return launch_stream<2>(pv16, a, n_wg, dyn_lds, stream);
        case 4: return launch_stream<4>(pv16, a, n_wg, dyn_lds, stream);
        default: return false;
    }
}

}  // namespace mlc_hip
