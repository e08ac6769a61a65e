// Runs the reference's own PagedKVStorage (compiler/runtime/paged_kv.cpp, compiled where it
// lies) and its paged-path calls on top of libmlc_hip.so through MetalExecutor::Instance(), i.e.
// through the binding of metal_runtime_hip.cpp.  The cases follow tests/test_paged_kv.cpp:
//   1. PagedKVStorage::initialize allocates one zero-filled K and V pool per layer (:99-120 of
//      paged_kv.cpp) -- read back and checked;
//   2. scatterKVPaged(start_slot = 3, 11 tokens, pages {5, 1}) followed by gatherKVPages of both
//      pages, fp32 and fp16, element by element (tests/test_paged_kv.cpp:404-474, 476-560);
//   3. a decode step on the storage's layer-0 pools: PagePool / RequestKVState hand out the
//      (page, slot) of each request's new row, scatterKVPagedBatched writes K and V rows,
//      runPagedFlashAttention attends; every request holds one token, so the output must be
//      that token's V row exactly (softmax over one score).
// Prints one "ok" line per case; exit status 0 only if all pass.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <optional>
#include <vector>

#include "runtime/metal_runtime.hpp"
#include "runtime/paged_kv.hpp"

using mlc::runtime::MetalExecutor;
using mlc::runtime::PagedKVStorage;
using mlc::runtime::PagePool;
using mlc::runtime::RequestKVState;

namespace {

int failures = 0;
#define CHECK(cond, what)                                              \
    do {                                                               \
        if (!(cond)) {                                                 \
            std::printf("FAILED: %s (%s:%d)\n", what, __FILE__, __LINE__); \
            ++failures;                                                \
            return;                                                    \
        }                                                              \
    } while (0)

// fp32 -> fp16 bits, round to nearest even (values here are small integers, exactly representable)
uint16_t half_bits(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    int32_t e = (int32_t)((x >> 23) & 0xFF) - 127 + 15;
    uint32_t m = x & 0x7FFFFFu;
    if (e <= 0) return (uint16_t)sign;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);
    uint32_t h = sign | ((uint32_t)e << 10) | (m >> 13);
    const uint32_t rem = m & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;
    return (uint16_t)h;
}
float half_value(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    if (e == 0 && m == 0) { float z; uint32_t b = sign; std::memcpy(&z, &b, 4); return z; }
    if (e == 0) return (sign ? -1.f : 1.f) * std::ldexp((float)m, -24);
    uint32_t bits = sign | ((e - 15 + 127) << 23) | (m << 13);
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

void storage_is_zero_filled() {
    auto& exec = MetalExecutor::Instance();
    PagedKVStorage storage(/*capacity_pages=*/6, /*n_layers=*/3, /*page_size_tokens=*/8, /*n_kv_heads=*/2,
                           /*head_dim=*/16, /*dtype_bytes=*/2);
    CHECK(storage.initialize(), "PagedKVStorage::initialize");
    const size_t bytes = (size_t)storage.capacity_pages() * storage.page_bytes();
    for (size_t layer = 0; layer < 3; ++layer) {
        CHECK(storage.k_buffer(layer) && storage.v_buffer(layer), "layer buffers");
        std::vector<uint8_t> got(bytes, 0xAB);
        exec.downloadFromBuffer(storage.k_buffer(layer), got.data(), bytes);
        for (uint8_t b : got) CHECK(b == 0, "K pool zero-filled");
        exec.downloadFromBuffer(storage.v_buffer(layer), got.data(), bytes);
        for (uint8_t b : got) CHECK(b == 0, "V pool zero-filled");
    }
    std::printf("storage_is_zero_filled ok\n");
}

template <typename T>
void scatter_gather_round_trip(const char* name) {
    auto& exec = MetalExecutor::Instance();
    const uint32_t capacity_pages = 8, P = 8, Hkv = 4, D = 16, tokens = 11, start_slot = 3;
    const size_t storage_bytes = (size_t)capacity_pages * P * Hkv * D * sizeof(T);
    void* storage = exec.allocateScratchBuffer(storage_bytes);
    CHECK(storage, "allocate storage");
    std::vector<uint8_t> zeros(storage_bytes, 0);
    exec.uploadToBuffer(storage, zeros.data(), storage_bytes);
    // projection output [Hkv][tokens][D] with the pattern h*1000 + t*10 + d
    std::vector<T> src((size_t)Hkv * tokens * D);
    std::vector<float> src_f(src.size());
    for (uint32_t h = 0; h < Hkv; ++h)
        for (uint32_t t = 0; t < tokens; ++t)
            for (uint32_t d = 0; d < D; ++d) {
                const float val = (float)h * 1000.f + (float)t * 10.f + (float)d;
                const size_t i = ((size_t)h * tokens + t) * D + d;
                src_f[i] = val;
                if (sizeof(T) == 4) std::memcpy(&src[i], &val, 4);
                else { const uint16_t hb = half_bits(val); std::memcpy(&src[i], &hb, 2); }
            }
    void* src_buf = exec.allocateScratchBuffer(src.size() * sizeof(T));
    CHECK(src_buf, "allocate source");
    exec.uploadToBuffer(src_buf, src.data(), src.size() * sizeof(T));
    const std::vector<uint32_t> page_table = {5, 1};
    CHECK(exec.scatterKVPaged(storage, page_table, P, Hkv, D, tokens, start_slot, src_buf, sizeof(T)), "scatterKVPaged");
    const uint32_t gather_tokens = 2 * P;
    std::vector<T> dst((size_t)Hkv * gather_tokens * D);
    void* dst_buf = exec.allocateScratchBuffer(dst.size() * sizeof(T));
    CHECK(dst_buf, "allocate destination");
    CHECK(exec.gatherKVPages(storage, page_table, P, Hkv, D, gather_tokens, dst_buf, sizeof(T)), "gatherKVPages");
    exec.downloadFromBuffer(dst_buf, dst.data(), dst.size() * sizeof(T));
    for (uint32_t h = 0; h < Hkv; ++h)
        for (uint32_t t = 0; t < gather_tokens; ++t)
            for (uint32_t d = 0; d < D; ++d) {
                float want = 0.f;
                if (t >= start_slot && t < start_slot + tokens) want = src_f[((size_t)h * tokens + (t - start_slot)) * D + d];
                const size_t i = ((size_t)h * gather_tokens + t) * D + d;
                float got;
                if (sizeof(T) == 4) std::memcpy(&got, &dst[i], 4);
                else { uint16_t hb; std::memcpy(&hb, &dst[i], 2); got = half_value(hb); want = half_value(half_bits(want)); }
                CHECK(got == want, "round trip element");
            }
    exec.releaseScratchBuffer(storage);
    exec.releaseScratchBuffer(src_buf);
    exec.releaseScratchBuffer(dst_buf);
    std::printf("scatter_gather_round_trip_%s ok\n", name);
}

void decode_step_on_storage() {
    auto& exec = MetalExecutor::Instance();
    const uint32_t capacity = 8, P = 64, Hkv = 4, D = 64, H = 32, B = 3;
    PagePool pool(capacity);
    PagedKVStorage storage(capacity, /*n_layers=*/1, P, Hkv, D, /*dtype_bytes=*/2);
    CHECK(storage.initialize(), "PagedKVStorage::initialize");
    std::vector<RequestKVState> reqs(B);
    for (uint32_t r = 0; r < B; ++r) {
        reqs[r].request_id = r;
        reqs[r].page_size_tokens = P;
    }
    std::vector<uint32_t> ids(B), slots(B), flat, off(B + 1, 0), seq(B), qpos(B);
    for (uint32_t r = 0; r < B; ++r) {
        const auto where = reqs[r].extend_one_token(pool);
        CHECK(where.has_value(), "extend_one_token");
        ids[r] = where->first;
        slots[r] = where->second;
        for (uint32_t id : reqs[r].page_table) flat.push_back(id);
        off[r + 1] = (uint32_t)flat.size();
        seq[r] = (uint32_t)reqs[r].total_tokens();
        qpos[r] = seq[r] - 1;
    }
    // new rows [B][Hkv][D]: K anything, V = r + h/8 + d/1024 (exact in fp16)
    std::vector<uint16_t> k_rows((size_t)B * Hkv * D), v_rows(k_rows.size());
    for (uint32_t r = 0; r < B; ++r)
        for (uint32_t h = 0; h < Hkv; ++h)
            for (uint32_t d = 0; d < D; ++d) {
                const size_t i = ((size_t)r * Hkv + h) * D + d;
                k_rows[i] = half_bits(0.25f * (float)((r + h + d) % 7) - 0.5f);
                v_rows[i] = half_bits((float)r + (float)h / 8.f + (float)d / 1024.f);
            }
    void* k_src = exec.allocateScratchBuffer(k_rows.size() * 2);
    void* v_src = exec.allocateScratchBuffer(v_rows.size() * 2);
    void* q_buf = exec.allocateScratchBuffer((size_t)B * H * D * 4);
    void* o_buf = exec.allocateScratchBuffer((size_t)B * H * D * 4);
    CHECK(k_src && v_src && q_buf && o_buf, "allocate step buffers");
    exec.uploadToBuffer(k_src, k_rows.data(), k_rows.size() * 2);
    exec.uploadToBuffer(v_src, v_rows.data(), v_rows.size() * 2);
    std::vector<float> q((size_t)B * H * D);
    for (size_t i = 0; i < q.size(); ++i) q[i] = 0.01f * (float)(i % 97) - 0.3f;
    exec.uploadToBuffer(q_buf, q.data(), q.size() * 4);
    CHECK(exec.scatterKVPagedBatched(storage.k_buffer(0), ids, slots, P, Hkv, D, B, k_src), "scatterKVPagedBatched K");
    CHECK(exec.scatterKVPagedBatched(storage.v_buffer(0), ids, slots, P, Hkv, D, B, v_src), "scatterKVPagedBatched V");
    CHECK(exec.runPagedFlashAttention(q_buf, storage.k_buffer(0), storage.v_buffer(0), o_buf, flat, off, seq, qpos, B, H,
                                      Hkv, D, P, true), "runPagedFlashAttention");
    std::vector<float> o(q.size());
    exec.downloadFromBuffer(o_buf, o.data(), o.size() * 4);
    for (uint32_t r = 0; r < B; ++r)
        for (uint32_t h = 0; h < H; ++h)
            for (uint32_t d = 0; d < D; ++d) {
                const uint32_t kvh = h * Hkv / H;
                const float want = half_value(v_rows[((size_t)r * Hkv + kvh) * D + d]);
                CHECK(o[((size_t)r * H + h) * D + d] == want, "one-token attention returns the V row");
            }
    // the same step through the encode variants inside one open pass
    std::vector<float> nan_fill(o.size(), NAN);
    exec.uploadToBuffer(o_buf, nan_fill.data(), o.size() * 4);
    CHECK(exec.beginForwardPassCB(), "beginForwardPassCB");
    CHECK(exec.hasForwardPassCB(), "hasForwardPassCB");
    CHECK(exec.encodeScatterKVPagedBatched(storage.k_buffer(0), ids, slots, P, Hkv, D, B, k_src), "encode scatter K");
    CHECK(exec.encodeScatterKVPagedBatched(storage.v_buffer(0), ids, slots, P, Hkv, D, B, v_src), "encode scatter V");
    CHECK(exec.encodePagedFlashAttention(q_buf, storage.k_buffer(0), storage.v_buffer(0), o_buf, flat, off, seq, qpos, B,
                                         H, Hkv, D, P, true), "encodePagedFlashAttention");
    CHECK(exec.flushForwardPassCB(), "flushForwardPassCB");
    std::vector<float> o2(o.size());
    exec.downloadFromBuffer(o_buf, o2.data(), o2.size() * 4);
    CHECK(std::memcmp(o.data(), o2.data(), o.size() * 4) == 0, "encode variants give the same output");
    for (auto& r : reqs) r.release_all(pool);
    for (void* b : {k_src, v_src, q_buf, o_buf}) exec.releaseScratchBuffer(b);
    std::printf("decode_step_on_storage ok\n");
}

}  // namespace

int main() {
    auto& exec = MetalExecutor::Instance();
    if (!exec.isAvailable()) {
        std::printf("FAILED: executor unavailable (no gfx950 device)\n");
        return 2;
    }
    storage_is_zero_filled();
    scatter_gather_round_trip<float>("f32");
    scatter_gather_round_trip<uint16_t>("f16");
    decode_step_on_storage();
    return failures ? 1 : 0;
}
