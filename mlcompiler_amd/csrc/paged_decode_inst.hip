// One translation unit per (head_dim, heads-per-wave) pair of the tile-balanced decode kernel:
// compiled with -DMLC_D=<64|128> -DMLC_HPW=<1|2|4|8>, so the variants build in parallel.
#include "paged_decode_kernels.h"
#include "paged_decode_stream.h"

#ifndef MLC_D
#error "compile with -DMLC_D=64|128 -DMLC_HPW=1|2|4|8"
#endif

#define MLC_SCAT_(a, b, c) launch_decode_stream_##a##_##b
#define MLC_SCAT(a, b) MLC_SCAT_(a, b, 0)

namespace mlc_hip {

namespace {
template <int NW, bool SMALL, int NBUF, bool SPLIT>
void launch_stream_pv(int pvm, const StreamArgs& a, unsigned n_wg, size_t dyn_lds, hipStream_t stream) {
    const dim3 grid(n_wg), block(64 * NW);
    if constexpr (NW == 4 && MLC_HPW * NW <= 16) {
        if (pvm == 2) {
            hipLaunchKernelGGL((paged_decode_stream_kernel<MLC_D, MLC_HPW, NW, 2, SMALL, NBUF, SPLIT>), grid, block, dyn_lds, stream, a);
            return;
        }
        if (pvm == 3) {
            hipLaunchKernelGGL((paged_decode_stream_kernel<MLC_D, MLC_HPW, NW, 3, SMALL, NBUF, SPLIT>), grid, block, dyn_lds, stream, a);
            return;
        }
    }
    if (pvm == 1 || pvm == 2)
        hipLaunchKernelGGL((paged_decode_stream_kernel<MLC_D, MLC_HPW, NW, 1, SMALL, NBUF, SPLIT>), grid, block, dyn_lds, stream, a);
    else
        hipLaunchKernelGGL((paged_decode_stream_kernel<MLC_D, MLC_HPW, NW, 0, SMALL, NBUF, SPLIT>), grid, block, dyn_lds, stream, a);
}
template <int NW>
bool launch_stream(int nbuf, int pvm, const StreamArgs& a, unsigned n_wg, size_t dyn_lds, hipStream_t stream) {
    // at most 64 requests: the variant that keeps the per-request figures in registers; larger
    // batches keep them in dynamic LDS, next to two or three stages
    // (the form that also splits its output for the matmul behind it: built for the default of
    // small batches only, two stages)
    if (a.split_frag) {
        if (a.batch > 64 || nbuf != 2) return false;
        launch_stream_pv<NW, true, 2, true>(pvm, a, n_wg, 0, stream);
        return true;
    }
    if (a.batch <= 64) {
        if (nbuf == 2) launch_stream_pv<NW, true, 2, false>(pvm, a, n_wg, 0, stream);
        else if (nbuf == 3) launch_stream_pv<NW, true, 3, false>(pvm, a, n_wg, 0, stream);
        else launch_stream_pv<NW, true, 4, false>(pvm, a, n_wg, 0, stream);
    } else {
        if (nbuf == 2) launch_stream_pv<NW, false, 2, false>(pvm, a, n_wg, dyn_lds, stream);
        else launch_stream_pv<NW, false, 3, false>(pvm, a, n_wg, dyn_lds, stream);
    }
    return true;
}
}  // namespace

// Tile-balanced kernel: nw = waves over the GQA group, nbuf = LDS stages (large batches: at most 3),
// pvm = arithmetic mode (0 fp32 weights, 1 fp16 weights on the vector pipe, 2 / 3 matrix pipe with
// fp16 / split weights where built: 4 waves and at most 16 heads per KV head; the caller falls
// back to 1 / 0 elsewhere), n_wg = grid size; false for an unbuilt combination.
bool MLC_SCAT(MLC_D, MLC_HPW)(int nw, int nbuf, int pvm, const StreamArgs& a, unsigned n_wg, size_t dyn_lds, hipStream_t stream) {
    switch (nw) {
        case 1: return launch_stream<1>(nbuf, pvm, a, n_wg, dyn_lds, stream);
        case 2: return launch_stream<2>(nbuf, pvm, a, n_wg, dyn_lds, stream);
        case 4: return launch_stream<4>(nbuf, pvm, a, n_wg, dyn_lds, stream);
        default: return false;
    }
}

}  // namespace mlc_hip
