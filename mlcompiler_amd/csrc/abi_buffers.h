// Entry points for device buffers and the pass: availability, errors, alloc / free / cached / upload /
// download / zero, begin / flush / has_open_pass.
//
// A section of the one translation unit mlc_hip.hip, which includes it once, in order, after the
// sections before it; not a header for anybody else.

extern "C" {

int mlc_hip_available(void) { return init_once() ? 1 : 0; }

const char* mlc_hip_last_error(void) { return g_err.c_str(); }

void* mlc_hip_alloc(size_t bytes) {
    if (!init_once()) return nullptr;
    if (g_capturing) { fail("alloc: not possible while a pass is being captured"); return nullptr; }
    void* p = nullptr;
    if (hipMalloc(&p, bytes ? bytes : 1) != hipSuccess) {
        g_err = "hipMalloc failed";
        (void)hipGetLastError();
        return nullptr;
    }
    g.allocs[p] = bytes;
    return p;
}

void mlc_hip_free(void* buffer) {
    if (!buffer || !init_once()) return;
    if (g_capturing) { fail("free: not possible while a pass is being captured"); return; }
    (void)settle();
    (void)hipStreamSynchronize(g.stream);
    g.allocs.erase(buffer);
    (void)hipFree(buffer);
}

namespace {
// Named grow-only device buffer; does not touch the pending row chain.
void* cached_buffer(const char* name, size_t bytes) {
    if (!init_once() || !name) return nullptr;
    auto it = g.cached.find(name);
    if (it != g.cached.end() && it->second.second >= bytes) return it->second.first;
    if (g_capturing) { fail("cached buffer: allocation is not possible while a pass is being captured"); return nullptr; }
    if (it != g.cached.end()) {  // grow-only reallocation, metal_runtime.mm:8222-8241
        (void)hipStreamSynchronize(g.stream);
        g.allocs.erase(it->second.first);
        (void)hipFree(it->second.first);
        ++g.buffer_generation;
        g.cached.erase(it);
    }
    void* p = nullptr;
    if (hipMalloc(&p, bytes ? bytes : 1) != hipSuccess) {
        g_err = "hipMalloc failed";
        (void)hipGetLastError();
        return nullptr;
    }
    g.cached[name] = {p, bytes};
    g.allocs[p] = bytes;
    return p;
}
}  // namespace

void* mlc_hip_cached(const char* name, size_t bytes) {
    if (!init_once() || !settle()) return nullptr;
    return cached_buffer(name, bytes);
}

int mlc_hip_upload(void* buffer, const void* src, size_t bytes, size_t dst_offset) {
    if (!init_once()) return fail("GPU unavailable");
    NOT_WHILE_CAPTURING("upload");
    if (!settle()) return 0;
    if (!buffer || (!src && bytes)) return fail("upload: null pointer");
    if (!bytes) return 1;
    const size_t known = known_bytes(buffer);
    if (known && dst_offset + bytes > known) return fail("upload: beyond the buffer");
    HIP_OK(hipMemcpyAsync(static_cast<char*>(buffer) + dst_offset, src, bytes,
                          hipMemcpyHostToDevice, g.stream));
    HIP_OK(hipStreamSynchronize(g.stream));
    return 1;
}

int mlc_hip_download(const void* buffer, void* dst, size_t bytes, size_t src_offset) {
    if (!init_once()) return fail("GPU unavailable");
    NOT_WHILE_CAPTURING("download");
    if (!settle()) return 0;
    if (!buffer || (!dst && bytes)) return fail("download: null pointer");
    if (!bytes) return 1;
    const size_t known = known_bytes(buffer);
    if (known && src_offset + bytes > known) return fail("download: beyond the buffer");
    HIP_OK(hipMemcpyAsync(dst, static_cast<const char*>(buffer) + src_offset, bytes,
                          hipMemcpyDeviceToHost, g.stream));
    HIP_OK(hipStreamSynchronize(g.stream));
    return 1;
}

int mlc_hip_zero(void* buffer, size_t bytes) {
    if (!init_once()) return fail("GPU unavailable");
    NOT_WHILE_CAPTURING("zero fill (a memset node in a replayed graph is not reliable on this platform)");
    if (!settle()) return 0;
    if (!buffer) return fail("zero: null pointer");
    const size_t known = known_bytes(buffer);
    if (known && bytes > known) return fail("zero: beyond the buffer");
    if (bytes) HIP_OK(hipMemsetAsync(buffer, 0, bytes, g.stream));
    return 1;
}

int mlc_hip_begin(void) {
    if (!init_once()) return fail("GPU unavailable");
    g.pass_open = true;  // idempotent, metal_runtime.mm:6003
    return 1;
}

int mlc_hip_flush(void) {
    if (!init_once()) return fail("GPU unavailable");
    NOT_WHILE_CAPTURING("flush");
    if (!settle()) return 0;
    if (!g.pass_open) return 1;
    g.pass_open = false;
    HIP_OK(hipStreamSynchronize(g.stream));
    return check_fault();
}

int mlc_hip_has_open_pass(void) { return (g.inited && g.pass_open) ? 1 : 0; }

}  // extern "C"
