// C ABI (include/mlc_hip.h) of the MI355X paged-attention hot path: device
// buffers, the single in-order stream that stands in for the reference's
// command buffer, argument checks, and the kernel launches.  One translation
// unit (the entry points share the library's state), written as sections:
// the abi_*.h files included at the end of this file.
//
// Host-side behaviour follows the reference's MetalExecutor entry points
// (compiler/runtime/metal_runtime.mm): see the citation at each function.
#include "../../include/mlc_hip.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <tuple>
#include <string>
#include <unordered_map>
#include <vector>

#include "paged_copy_kernels.h"
#include "paged_decode_generic.h"
#include "paged_decode_kernels.h"
#include "paged_decode_stream.h"
#include "paged_prefill_kernels.h"
#include "paged_rope_kernels.h"
#include "walker_kernels.h"
#include "q4_matmul_kernels.h"
#include "q6k_matmul_kernels.h"

namespace mlc_hip {
// Defined in paged_decode_inst.hip, one object per (head_dim, heads-per-wave).
#define MLC_DECL(d, h) bool launch_decode_stream_##d##_##h(int, int, int, const StreamArgs&, unsigned, size_t, hipStream_t);
MLC_DECL(64, 1) MLC_DECL(64, 2) MLC_DECL(64, 4) MLC_DECL(64, 8)
MLC_DECL(128, 1) MLC_DECL(128, 2) MLC_DECL(128, 4) MLC_DECL(128, 8)
#undef MLC_DECL
}  // namespace mlc_hip

// The sections of this translation unit, in the order they build on one another.
#include "abi_context.h"
#include "abi_decode_tables.h"
#include "abi_buffers.h"
#include "abi_decode.h"
#include "abi_kv_copy.h"
#include "abi_rope.h"
#include "abi_row_ops.h"
#include "abi_matmul.h"
#include "abi_prefill.h"
#include "abi_capture.h"
#include "abi_misc.h"
