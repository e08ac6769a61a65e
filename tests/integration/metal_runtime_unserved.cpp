// The rest of mlc::runtime::MetalExecutor (compiler/runtime/metal_runtime.hpp:23-711) that the
// reference's single-stream path links against (operator_backend.cpp, execution_executor.cpp,
// execution_context.cpp): the per-operator run* / encode*From* entry points of the Metal build.
// The HIP build serves the batched paged path (metal_runtime_hip.cpp) and leaves these operators
// to the reference's own CPU implementations: shouldUseFor() says no for every node, and each
// entry point reports "not done here" exactly like the reference's non-Apple fall-throughs
// (metal_runtime.mm:7161-7165), so DecodeRunner / ExecutionExecutor run on the CPU unchanged.
// Compiled against the reference's header where that lies; nothing of the reference is in this file.
#include "runtime/metal_runtime.hpp"

namespace mlc {
namespace runtime {

using FloatVec = std::vector<float>;
using ByteVec = std::vector<uint8_t>;

bool MetalExecutor::shouldUseFor(const ExecutionNode&) const { return false; }

// ---- single-request operators (dense and quantised matmuls, norms, attention, feed-forward)
bool MetalExecutor::runMatMul(const std::string&, const FloatVec&, const FloatVec&, size_t, size_t, bool, FloatVec&,
                              const FloatVec*) const { return false; }
#define MLC_UNSERVED_QMATMUL(name)                                                                              \
    bool MetalExecutor::name(const std::string&, const ByteVec&, const FloatVec&, size_t, size_t, size_t, FloatVec&, \
                             const FloatVec*) const { return false; }
MLC_UNSERVED_QMATMUL(runMatMulQ3K)
MLC_UNSERVED_QMATMUL(runMatMulQ4K)
MLC_UNSERVED_QMATMUL(runMatMulQ4_1)
MLC_UNSERVED_QMATMUL(runMatMulQ5K)
MLC_UNSERVED_QMATMUL(runMatMulQ5_0)
MLC_UNSERVED_QMATMUL(runMatMulQ5_1)
MLC_UNSERVED_QMATMUL(runMatMulQ6KTransposed)
MLC_UNSERVED_QMATMUL(runMatMulQ8K)
MLC_UNSERVED_QMATMUL(runMatMulQ8_0)
MLC_UNSERVED_QMATMUL(runMatMulQ8_1)
#undef MLC_UNSERVED_QMATMUL
bool MetalExecutor::runMatMulQ4_0Transposed(const std::string&, const ByteVec&, const FloatVec&, size_t, size_t, size_t,
                                            uint32_t, FloatVec&, const FloatVec*) const { return false; }
bool MetalExecutor::runAdd(const FloatVec&, const FloatVec&, FloatVec&, const FloatVec*) const { return false; }
bool MetalExecutor::runRmsNorm(const FloatVec&, const FloatVec&, float, FloatVec&) const { return false; }
bool MetalExecutor::runLayerNorm(const FloatVec&, const FloatVec&, const FloatVec*, float, FloatVec&) const { return false; }
bool MetalExecutor::runSoftmax(const FloatVec&, FloatVec&) const { return false; }
bool MetalExecutor::runFeedForward(const FloatVec&, const FloatVec&, FloatVec&, const std::string&) const { return false; }
bool MetalExecutor::runAttention(const FloatVec&, const FloatVec&, const FloatVec&, size_t, size_t, size_t, size_t,
                                 const FloatVec&, const FloatVec*, size_t, size_t, float, float, const CacheDescriptor&,
                                 const CacheDescriptor&, FloatVec&, const std::string&) const { return false; }

// ---- the single-stream fusion window (deferred read-back, pooled buffers)
bool MetalExecutor::encodeAddMixed(const FloatVec*, void*, const FloatVec*, void*, size_t, void*, FloatVec*, bool) const { return false; }
bool MetalExecutor::encodeMatMulQ4_0FromBuffer(const std::string&, const ByteVec&, void*, size_t, size_t, size_t, size_t,
                                               uint32_t, void*, FloatVec*, bool) const { return false; }
bool MetalExecutor::encodeMatMulQ4_0FromHost(const std::string&, const ByteVec&, const FloatVec&, size_t, size_t, size_t,
                                             uint32_t, void*, FloatVec*, bool) const { return false; }
bool MetalExecutor::encodeRmsNormFromBuffer(void*, size_t, const FloatVec&, float, void*, FloatVec*, bool,
                                            const std::string&) const { return false; }
bool MetalExecutor::encodeRmsNormFromHost(const FloatVec&, const FloatVec&, float, void*, FloatVec*, bool,
                                          const std::string&) const { return false; }
bool MetalExecutor::encodeSliceFromBuffer(void*, size_t, size_t, size_t, void*, const std::string&, FloatVec*, bool) const { return false; }
bool MetalExecutor::encodeSliceFromHost(const FloatVec&, size_t, size_t, void*, const std::string&, FloatVec*, bool) const { return false; }
bool MetalExecutor::flushForwardPassCB(const std::function<FloatVec*(const std::string&)>&) const { return false; }
void MetalExecutor::discardForwardPassCB() const {}
bool MetalExecutor::hasDeferredReadback(const std::string&) const { return false; }
void* MetalExecutor::lastDeferredOutputBuffer() const { return nullptr; }
size_t MetalExecutor::lastDeferredOutputElementCount() const { return 0; }
void MetalExecutor::clearLastDeferredOutput() const {}
void* MetalExecutor::checkoutPoolBuffer(size_t) const { return nullptr; }
void MetalExecutor::trackWindowBuffer(void*) const {}

}  // namespace runtime
}  // namespace mlc
