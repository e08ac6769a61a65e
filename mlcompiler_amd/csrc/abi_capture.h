// Entry points that record a pass into a HIP graph and replay it.
//
// A section of the one translation unit mlc_hip.hip, which includes it once, in order, after the
// sections before it; not a header for anybody else.

extern "C" {

// ---------------------------------------------------------------- captured passes (HIP graph)

int mlc_hip_capture_begin(void) {
    if (!init_once()) return fail("GPU unavailable");
    if (g_capturing) return fail("capture: a pass is already being captured");
    if (!g.pass_open) return fail("capture: no open forward pass");
    if (!settle()) return 0;  // what was encoded before belongs to the uncaptured part
    // The per-request arrays of the last decode call travelled inside its kernel arguments; a
    // captured launch reads them from the device copy, which is brought up to date now.
    if (!g.tables.last_meta.empty()) {
        const uint32_t* d_flat = nullptr;
        const uint32_t* d_meta = nullptr;
        if (!tables_upload(g.tables.last_meta.data(), g.tables.last_meta.size() / 3, &d_flat, &d_meta)) return 0;
    }
    g.cap = Ctx::Captured{};
    g_capture_failed = false;
    HIP_OK(hipStreamBeginCapture(g.stream, hipStreamCaptureModeThreadLocal));
    g_capturing = true;
    hipLaunchKernelGGL(replay_word_kernel, dim3(1), dim3(1), 0, g.stream,
                       reinterpret_cast<uint32_t*>(g.scratch_ptr + kScratchReplayWordOffset), kReplayTagStep);
    return 1;
}

int mlc_hip_capture_end(void) {
    if (!g.inited || !g_capturing) return fail("capture: no pass is being captured");
    const int settled = settle();  // the operators still held back are launches of the captured pass
    g_capturing = false;
    hipGraph_t graph = nullptr;
    const hipError_t e = hipStreamEndCapture(g.stream, &graph);
    if (e != hipSuccess || !graph) {
        (void)hipGetLastError();
        if (graph) (void)hipGraphDestroy(graph);
        return fail(std::string("capture: hipStreamEndCapture: ") + hipGetErrorString(e));
    }
    if (!settled || g_capture_failed) {
        (void)hipGraphDestroy(graph);
        if (g_capture_failed) return 0;  // the failing call's message stands
        return fail("capture: the held-back operators could not be launched");
    }
    // kernel launches only: anything else (a copy, a memset) means some call did more than encode
    size_t count = 0;
    std::vector<hipGraphNode_t> nodes;
    bool ok = hipGraphGetNodes(graph, nullptr, &count) == hipSuccess;
    if (ok && count) {
        nodes.resize(count);
        ok = hipGraphGetNodes(graph, nodes.data(), &count) == hipSuccess;
    }
    for (size_t i = 0; ok && i < count; ++i) {
        hipGraphNodeType type;
        ok = hipGraphNodeGetType(nodes[i], &type) == hipSuccess && type == hipGraphNodeTypeKernel;
    }
    if (!ok || count <= 1) {
        (void)hipGraphDestroy(graph);
        return fail(count <= 1 ? "capture: nothing was encoded" : "capture: the pass holds something other than kernel launches");
    }
    hipGraphExec_t exec = nullptr;
    if (hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0) != hipSuccess || !exec) {
        (void)hipGetLastError();
        (void)hipGraphDestroy(graph);
        return fail("capture: hipGraphInstantiate failed");
    }
    Ctx::Captured c = g.cap;
    c.buffer_generation = g.buffer_generation;
    c.graph = graph;
    c.exec = exec;
    c.n_nodes = count - 1;   // (not counted: the library's own first launch, which moves the replay word on)
    const int handle = g.next_capture++;
    g.captures[handle] = c;
    return handle;
}

size_t mlc_hip_captured_launches(int handle) {
    auto it = g.captures.find(handle);
    return it == g.captures.end() ? 0 : it->second.n_nodes;
}

int mlc_hip_replay_update(int handle, const uint32_t* page_tables_flat, size_t n_flat,
                          const uint32_t* page_table_offsets, const uint32_t* seq_lens,
                          const uint32_t* q_positions, const uint32_t* page_ids, const uint32_t* slots_in_page,
                          size_t batch) {
    if (!init_once()) return fail("GPU unavailable");
    NOT_WHILE_CAPTURING("replay update");
    auto it = g.captures.find(handle);
    if (it == g.captures.end()) return fail("replay: unknown handle");
    const Ctx::Captured& c = it->second;
    if (c.buffer_generation != g.buffer_generation)
        return fail("replay: a device buffer of the library was freed or moved since the capture (capture again)");
    if (!settle()) return 0;
    if (c.used_tables) {
        if (!page_table_offsets || !seq_lens || !q_positions || (n_flat && !page_tables_flat))
            return fail("replay: null metadata");
        if (batch != c.B) return fail("replay: the batch size differs from the captured pass (capture again)");
        if (n_flat < page_table_offsets[batch]) return fail("replay: page table shorter than offsets");
        const size_t tile = c.D == 64 ? 64 : 32;
        uint64_t total_tiles = 0;
        for (size_t r = 0; r < batch; ++r) {
            const size_t pages = ((size_t)seq_lens[r] + c.P - 1) / c.P;
            if ((size_t)page_table_offsets[r] + pages > n_flat) return fail("replay: page table does not cover seq_len");
            uint64_t lim = seq_lens[r];
            if (c.causal && (uint64_t)q_positions[r] + 1 < lim) lim = (uint64_t)q_positions[r] + 1;
            total_tiles += (lim + tile - 1) / tile;
        }
        // (the same bound as the encode path: the kernel counts in units, tiles plus at most 64 per pair)
        if (total_tiles * c.Hkv + 64ull * batch * c.Hkv >= 0x7FFFFFFFull)
            return fail("replay: too many KV tiles for the captured kernel");
        tables_refresh(page_tables_flat, n_flat, page_table_offsets, batch);
        static thread_local std::vector<uint32_t> meta3;
        meta3.resize(3 * batch);
        std::memcpy(meta3.data(), seq_lens, batch * 4);
        std::memcpy(meta3.data() + batch, q_positions, batch * 4);
        std::memcpy(meta3.data() + 2 * batch, page_table_offsets, batch * 4);
        const uint32_t* d_flat = nullptr;
        const uint32_t* d_meta = nullptr;
        if (!tables_upload(meta3.data(), batch, &d_flat, &d_meta)) return 0;
        if (d_flat != c.tables_flat || d_meta != c.tables_meta)
            return fail("replay: the device copy of the tables had to move (capture again)");
        if (c.carried_kv) {
            // the captured attention launch writes the step's K / V rows itself: they must still be
            // every request's newest visible position, on pages no two requests share
            if (!page_ids || !slots_in_page) return fail("replay: the captured pass writes K / V rows, page ids needed");
            bool ok = g.tables.shared_pages == 0;
            for (size_t r = 0; ok && r < batch; ++r) {
                const uint64_t S = seq_lens[r];
                const bool visible = !c.causal || (uint64_t)q_positions[r] + 1 >= S;
                ok = S > 0 && visible && slots_in_page[r] == (S - 1) % c.P &&
                     page_ids[r] == page_tables_flat[page_table_offsets[r] + (S - 1) / c.P];
            }
            if (!ok) return fail("replay: the rows to write are not every request's newest position (run this step uncaptured)");
        }
    }
    if (c.ids_dev) {
        if (!page_ids || !slots_in_page) return fail("replay: the captured pass writes K / V rows, page ids needed");
        if (batch != c.ids_batch) return fail("replay: the batch size differs from the captured pass (capture again)");
        for (size_t r = 0; r < batch; ++r)
            if (c.P && slots_in_page[r] >= c.P) return fail("replay: slot >= page size");
        const void* dev = resident_ids(page_ids, slots_in_page, batch, align_up(batch * 4, 16));
        if (!dev) return 0;
        if (dev != c.ids_dev) return fail("replay: the device copy of the page ids had to move (capture again)");
    }
    return 1;
}

int mlc_hip_replay(int handle) {
    if (!init_once()) return fail("GPU unavailable");
    NOT_WHILE_CAPTURING("replay");
    auto it = g.captures.find(handle);
    if (it == g.captures.end()) return fail("replay: unknown handle");
    if (it->second.buffer_generation != g.buffer_generation)
        return fail("replay: a device buffer of the library was freed or moved since the capture (capture again)");
    if (!settle()) return 0;
    if (it->second.n_decode && !scratch_follow(g.stream)) return 0;
    HIP_OK(hipGraphLaunch(it->second.exec, g.stream));
    if (it->second.n_decode && !scratch_launched(g.stream)) return 0;
    return 1;
}

void mlc_hip_capture_release(int handle) {
    auto it = g.captures.find(handle);
    if (it == g.captures.end()) return;
    (void)hipStreamSynchronize(g.stream);
    if (it->second.exec) (void)hipGraphExecDestroy(it->second.exec);
    if (it->second.graph) (void)hipGraphDestroy(it->second.graph);
    g.captures.erase(it);
}

}  // extern "C"
