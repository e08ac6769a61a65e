// Entry points of the paged decode attention: mlc_hip_paged_attn_decode and its variant that allocates nothing.
//
// A section of the one translation unit mlc_hip.hip, which includes it once, in order, after the
// sections before it; not a header for anybody else.

extern "C" {

int mlc_hip_paged_attn_decode(const void* q, const void* k_pages, const void* v_pages, void* o,
                              const uint32_t* page_tables_flat, size_t n_flat,
                              const uint32_t* page_table_offsets, const uint32_t* seq_lens,
                              const uint32_t* q_positions, size_t batch, size_t num_heads,
                              size_t kv_heads, size_t head_dim, size_t page_size_tokens,
                              int apply_causal, int sync) {
    if (!init_once()) return fail("GPU unavailable");
    // A pending pair of batched K / V scatters into these pools may be this step's KV write
    // (batched_walker.cpp:304-331): then the attention launch does it (decided below, once the
    // tables are known to be valid); anything else pending is launched now.
    bool carries_kv = g.opt_fuse_rows && g.kv.active && !g.kv.rope && g.kv.n == 2 && g.kv.wide && !g.rows.active &&
                      !g.gemm.active && !g.dec.active && g.kv.pages[0] == k_pages && g.kv.pages[1] == v_pages && g.kv.batch == batch &&
                      g.kv.row_elems == kv_heads * head_dim && g.kv.page_size == page_size_tokens;
    if (!carries_kv && !settle()) return 0;
    if (!sync && !g.pass_open) return fail("encode: no open forward pass");  // :7090
    // metal_runtime.mm:7742-7750
    if (!q || !k_pages || !v_pages || !o) return fail("decode: null buffer");
    if (batch == 0 || num_heads == 0 || head_dim == 0 || page_size_tokens == 0)
        return fail("decode: zero dimension");
    if (kv_heads == 0 || (num_heads % kv_heads) != 0) return fail("decode: heads % kv_heads != 0");
    if (!page_table_offsets || !seq_lens || !q_positions) return fail("decode: null metadata");
    if (n_flat && !page_tables_flat) return fail("decode: null page table");
    if (n_flat < page_table_offsets[batch]) return fail("decode: page table shorter than offsets");
    if (head_dim > 256) return fail("decode: head_dim > 256");
    if (batch > 0x7FFFFFFFull / num_heads) return fail("decode: batch*heads too large");
    // Beyond the reference: every request's table must cover its sequence, or the
    // kernel would read page ids past the end of the metadata.
    for (size_t r = 0; r < batch; ++r) {
        const size_t pages = ((size_t)seq_lens[r] + page_size_tokens - 1) / page_size_tokens;
        if ((size_t)page_table_offsets[r] + pages > n_flat)
            return fail("decode: page table does not cover seq_len");
    }
    {
        const size_t qo_bytes = batch * num_heads * head_dim * 4;
        const size_t kq = known_bytes(q), ko = known_bytes(o);
        if ((kq && qo_bytes > kq) || (ko && qo_bytes > ko)) return fail("decode: q / o buffer too small");
    }
    const size_t row_bytes = kv_heads * head_dim * 2;
    // What is remembered about the tables (content, largest page id, repeated page ids) is
    // refreshed only when they changed; the walker passes the same tables for every layer of a
    // step (compiler/runtime/batched_walker.cpp:316-325).
    tables_refresh(page_tables_flat, n_flat, page_table_offsets, batch);
    {
        // pools this library allocated: no page id of the table may lie beyond them.  The largest
        // id of the whole table decides at once; only if that one is too large (it may sit in a
        // part of the table no request uses) the pages in use are checked one by one.
        const size_t page_bytes = page_size_tokens * row_bytes;
        const size_t kk = known_bytes(k_pages), kv = known_bytes(v_pages);
        const size_t need = n_flat ? ((size_t)g.tables.max_page + 1) * page_bytes : 0;
        if (((kk && need > kk) || (kv && need > kv)) &&
            (!check_pool_bounds(k_pages, page_tables_flat, page_table_offsets, seq_lens, batch,
                                page_size_tokens, row_bytes, "decode K") ||
             !check_pool_bounds(v_pages, page_tables_flat, page_table_offsets, seq_lens, batch,
                                page_size_tokens, row_bytes, "decode V")))
            return 0;
    }
    const bool aligned = aligned16(q) && aligned16(k_pages) && aligned16(v_pages) && aligned16(o);
    const size_t G = num_heads / kv_heads;
    const size_t tile = (head_dim == 64) ? 64 : 32;

    // ---- which kernel: the tile-balanced one wherever it applies
    int s_hpw = 0, s_nw = 0;
    bool use_stream = !g.opt_force_generic && aligned &&
                      (page_size_tokens % tile) == 0 && batch <= kStreamMaxBatch &&
                      stream_variant(G, head_dim, &s_hpw, &s_nw);
    uint64_t total_tiles = 0;
    if (use_stream) {
        for (size_t r = 0; r < batch; ++r) {
            uint64_t lim = seq_lens[r];
            if (apply_causal && (uint64_t)q_positions[r] + 1 < lim) lim = (uint64_t)q_positions[r] + 1;  // :2286
            total_tiles += (lim + tile - 1) / tile;
        }
        total_tiles *= kv_heads;
        // (the kernel counts in units: tiles plus at most 64 per (request, KV head) pair)
        if (total_tiles + 64ull * batch * kv_heads >= 0x7FFFFFFFull) use_stream = false;
    }
    const DecodePlan* plan = nullptr;
    if (!use_stream) {
        if (!build_plan(page_tables_flat, n_flat, page_table_offsets, seq_lens, q_positions, batch,
                        apply_causal ? 1 : 0))
            return 0;
        plan = &g.plan;
    }

    if (carries_kv) {
        // Only the tile-balanced kernel writes rows, and only rows that are every request's newest
        // visible position: then exactly one workgroup reads each of them, after writing it.
        // That also needs every page to belong to one request (and to appear once in its
        // table): with a repeated page id another workgroup could read the row while it is
        // being written, and the separate launches are the ones that give the order of the calls.
        carries_kv = use_stream && g.tables.shared_pages == 0;
        for (size_t r = 0; carries_kv && r < batch; ++r) {
            const uint64_t S = seq_lens[r];
            const bool visible = !apply_causal || (uint64_t)q_positions[r] + 1 >= S;
            carries_kv = S > 0 && visible && g.kv.slots[r] == (S - 1) % page_size_tokens &&
                         g.kv.ids[r] == page_tables_flat[page_table_offsets[r] + (S - 1) / page_size_tokens];
        }
        if (!carries_kv && !settle()) return 0;
    }

    g.last_launches = 0;
    if (use_stream) {
        // per-request arrays: inside the kernel arguments when they fit, else uploaded with the table
        // (a captured pass reads them from the device copy, which mlc_hip_replay_update refreshes)
        const bool embed = batch <= kStreamEmbBatch && !g_capturing;
        // (kept on the host in any case: mlc_hip_capture_begin sends them to the device, so that a
        // pass captured right after this call finds them there)
        std::vector<uint32_t>& meta3 = g.tables.last_meta;
        meta3.resize(3 * batch);
        std::memcpy(meta3.data(), seq_lens, batch * 4);
        std::memcpy(meta3.data() + batch, q_positions, batch * 4);
        std::memcpy(meta3.data() + 2 * batch, page_table_offsets, batch * 4);
        // ... and the flat table with them when it fits behind them: then nothing is copied to the
        // device, however often the tables change
        // (up to 64 requests: the arrays sit at a fixed stride, see the kernel)
        const size_t emb_stride = batch <= 64 ? kStreamSmallStride : batch;
        const bool embed_table = embed && 3 * emb_stride + n_flat <= kStreamEmbWords;
        const uint32_t* d_flat = nullptr;
        const uint32_t* d_meta = nullptr;
        if (!embed_table && !tables_upload(embed ? nullptr : meta3.data(), batch, &d_flat, &d_meta)) return 0;
        const size_t dyn_lds = batch <= 64 ? 0 : stream_dynamic_lds_bytes(batch);
        const int nbuf = stream_stages(batch);
        const unsigned n_wg = stream_grid(G, head_dim, nbuf, dyn_lds);
        StreamArgs a;
        stream_fill_common(a, q, k_pages, v_pages, o, batch, num_heads, kv_heads, head_dim, page_size_tokens,
                           apply_causal);
        a.pair_cost = stream_pair_cost(s_nw, G, head_dim);
        a.pt_flat = d_flat;
        {
            // pools this library allocated: the kernel clamps page ids below their size (the host
            // checks above already refuse such tables; the clamp keeps a stale or overwritten
            // table from turning into a stray access)
            const size_t page_bytes = page_size_tokens * row_bytes;
            const size_t kk = known_bytes(k_pages), kv = known_bytes(v_pages);
            size_t pages = std::min(kk ? kk / page_bytes : SIZE_MAX, kv ? kv / page_bytes : SIZE_MAX);
            if (pages != SIZE_MAX) a.capacity_pages = (uint32_t)std::min<size_t>(pages, 0xFFFFFFFFu);
        }
        a.meta_stride = (uint32_t)batch;
        if (embed) {
            for (int i = 0; i < 3; ++i) std::memcpy(a.emb + i * emb_stride, meta3.data() + i * batch, batch * 4);
            if (embed_table && n_flat) std::memcpy(a.emb + 3 * emb_stride, page_tables_flat, n_flat * 4);
        } else {
            a.meta = d_meta;
        }
        if (carries_kv) {
            a.new_k = static_cast<const uint4*>(g.kv.src[0]);
            a.new_v = static_cast<const uint4*>(g.kv.src[1]);
            a.new_ids = g.kv.d_ids;
            a.new_slots = g.kv.d_slots;
        }
        if (g_capturing && g.cap.n_decode > kReplayTagStep)
            return fail("capture: more decode launches in one pass than its tags can tell apart");
        // Held back for one call where a Q4_0 matmul reading o could take its activations from
        // this launch (see Ctx::DecodePending); launched now otherwise.
        const size_t o_cols = num_heads * head_dim;
        if (g.opt_fuse_rows && g.opt_q4_int_operand && !g.opt_q4_force_generic && !sync && batch <= 64 &&
            nbuf == 2 && o_cols % 32 == 0 && o_cols >= 64) {
            Ctx::DecodePending& d = g.dec;
            if (d.active && !settle_decode()) return 0;   // (never the case: whatever led here has launched it)
            d.active = true;
            d.a = a;
            d.head_dim = head_dim; d.dyn_lds = dyn_lds;
            d.hpw = s_hpw; d.nw = s_nw; d.nbuf = nbuf;
            d.n_wg = n_wg;
            d.o = o;
            d.batch = batch;
            d.cols = o_cols;
        } else if (!launch_stream_variant(head_dim, s_hpw, s_nw, nbuf, a, n_wg, dyn_lds, g.stream)) {
            return fail("decode: kernel variant not built");
        }
        if (g_capturing) {
            Ctx::Captured& c = g.cap;
            if (c.used_tables && (c.B != batch || c.tables_flat != d_flat || c.tables_meta != d_meta))
                return fail("capture: every decode call of a captured pass must use the same tables");
            c.used_tables = true;
            c.tables_flat = d_flat;
            c.tables_meta = d_meta;
            c.B = batch; c.H = num_heads; c.Hkv = kv_heads; c.D = head_dim; c.P = page_size_tokens;
            c.causal = apply_causal ? 1 : 0;
            c.carried_kv = c.carried_kv || carries_kv;
        }
        g.last_items = (int)std::min<uint64_t>(n_wg, total_tiles);
        std::snprintf(g.last_kernel, sizeof g.last_kernel, "stream<%zu,%d,%d,%s,%s,%d>", head_dim, s_hpw, s_nw,
                      stream_pv_name(s_hpw, s_nw), batch <= 64 ? "regs" : "lds", nbuf);
        if (carries_kv) {
            g.kv.active = false;
            ++g.kv_fused;
            ++g.kv_in_decode;
        }
        ++g.last_launches;
        return finish(sync);
    }

    const DecodePlan& p = *plan;
    MetaSlot& slot = g.plan_slots[p.slot];
    const char* dev = static_cast<const char*>(slot.dev);
    const float scale_log2e = (1.0f / std::sqrt(static_cast<float>(head_dim))) * 1.44269504088896340736f;
    g.last_items = (int)(batch * num_heads);
    {
        GenericArgs a;
        a.q = static_cast<const float*>(q);
        a.k_pages = static_cast<const _Float16*>(k_pages);
        a.v_pages = static_cast<const _Float16*>(v_pages);
        a.o = static_cast<float*>(o);
        a.pt_flat = reinterpret_cast<const uint32_t*>(dev);
        a.pt_off = reinterpret_cast<const uint32_t*>(dev + p.off_ptoff);
        a.limits = reinterpret_cast<const uint32_t*>(dev + p.off_limits);
        a.num_heads = (uint32_t)num_heads;
        a.kv_heads = (uint32_t)kv_heads;
        a.head_dim = (uint32_t)head_dim;
        a.page_size = (uint32_t)page_size_tokens;
        a.scale_log2e = scale_log2e;
        hipLaunchKernelGGL(paged_decode_generic_kernel, dim3((unsigned)(batch * num_heads)),
                           dim3(64), 0, g.stream, a);
        std::snprintf(g.last_kernel, sizeof g.last_kernel, "generic");
        ++g.last_launches;
    }
    if (!slot_mark(slot)) return 0;
    return finish(sync);
}

int mlc_hip_paged_attn_decode_noalloc(const void* q, const void* k_pages, const void* v_pages, void* o,
                                      const uint32_t* page_tables_flat_device, size_t n_flat,
                                      const uint32_t* page_table_offsets, const uint32_t* seq_lens,
                                      const uint32_t* q_positions, size_t batch, size_t num_heads,
                                      size_t kv_heads, size_t head_dim, size_t page_size_tokens,
                                      int apply_causal, void* stream) {
    // Nothing here allocates device or pinned memory: no hipMalloc / hipFree / hipHostMalloc, no
    // event or stream creation (only the text of an error message, on a refusal, takes host heap).
    // The kernel's scratch memory (split-K partials, arrival counters) is
    // the file-scope device array whose address init_once() looked up; the per-request arrays travel
    // inside the kernel arguments and the page table stays where the caller keeps it.
    if (!g.inited || !g.available) return fail("decode (no allocation): call mlc_hip_available() once at set-up");
    if (g_capturing) return fail("decode (no allocation): not while a pass is being captured (the captured launch would keep this call's lengths)");
    hipStream_t st = stream ? static_cast<hipStream_t>(stream) : g.stream;
    {
        // operators held back by earlier encode calls are launched now, on the library's stream
        // (kernel launches only); a caller's stream of its own is put behind them
        const bool pending = g.rows.active || g.kv.active || g.gemm.active || g.dec.active;
        if (!settle()) return 0;
        if (pending && st != g.stream) {
            HIP_OK(hipEventRecord(g.scratch_ev, g.stream));
            HIP_OK(hipStreamWaitEvent(st, g.scratch_ev, 0));
        }
    }
    if (!q || !k_pages || !v_pages || !o) return fail("decode: null buffer");  // metal_runtime.mm:7742-7750
    if (batch == 0 || num_heads == 0 || head_dim == 0 || page_size_tokens == 0) return fail("decode: zero dimension");
    if (kv_heads == 0 || (num_heads % kv_heads) != 0) return fail("decode: heads % kv_heads != 0");
    if (!page_table_offsets || !seq_lens || !q_positions) return fail("decode: null metadata");
    if (n_flat && !page_tables_flat_device) return fail("decode: null page table");
    if (n_flat < page_table_offsets[batch]) return fail("decode: page table shorter than offsets");
    if (batch > kStreamEmbBatch) return fail("decode (no allocation): more than 256 requests");
    const size_t G = num_heads / kv_heads;
    const size_t tile = (head_dim == 64) ? 64 : 32;
    int hpw = 0, nw = 0;
    if (!stream_variant(G, head_dim, &hpw, &nw) || (page_size_tokens % tile) != 0)
        return fail("decode (no allocation): head_dim must be 64 or 128, the GQA ratio 1, 2, 4, 8, 16 or 32, "
                    "the page size a multiple of 64 (head_dim 64) or 32 (head_dim 128) tokens");
    if (!aligned16(q) || !aligned16(k_pages) || !aligned16(v_pages) || !aligned16(o) ||
        (reinterpret_cast<uintptr_t>(page_tables_flat_device) & 3u))
        return fail("decode (no allocation): buffers must be 16-byte aligned");
    uint64_t total_tiles = 0;
    for (size_t r = 0; r < batch; ++r) {
        const size_t pages = ((size_t)seq_lens[r] + page_size_tokens - 1) / page_size_tokens;
        if ((size_t)page_table_offsets[r] + pages > n_flat) return fail("decode: page table does not cover seq_len");
        uint64_t lim = seq_lens[r];
        if (apply_causal && (uint64_t)q_positions[r] + 1 < lim) lim = (uint64_t)q_positions[r] + 1;  // :2286
        total_tiles += (lim + tile - 1) / tile;
    }
    total_tiles *= kv_heads;
    if (total_tiles + 64ull * batch * kv_heads >= 0x7FFFFFFFull) return fail("decode (no allocation): too many KV tiles");
    {
        const size_t qo_bytes = batch * num_heads * head_dim * 4;
        const size_t kq = known_bytes(q), ko = known_bytes(o), kt = known_bytes(page_tables_flat_device);
        if ((kq && qo_bytes > kq) || (ko && qo_bytes > ko)) return fail("decode: q / o buffer too small");
        if (kt && n_flat * 4 > kt) return fail("decode: page table buffer too small");
    }
    const int nbuf = stream_stages(batch);
    const size_t dyn_lds = batch <= 64 ? 0 : stream_dynamic_lds_bytes(batch);
    const unsigned n_wg = stream_grid(G, head_dim, nbuf, dyn_lds);
    StreamArgs a;
    stream_fill_common(a, q, k_pages, v_pages, o, batch, num_heads, kv_heads, head_dim, page_size_tokens, apply_causal);
    a.pair_cost = stream_pair_cost(nw, G, head_dim);
    a.pt_flat = page_tables_flat_device;
    {
        // the page ids are on the device and cannot be checked here: pools this library allocated
        // are protected by the kernel's clamp of the ids to their size
        const size_t page_bytes = page_size_tokens * kv_heads * head_dim * 2;
        const size_t kk = known_bytes(k_pages), kv = known_bytes(v_pages);
        const size_t pages = std::min(kk ? kk / page_bytes : SIZE_MAX, kv ? kv / page_bytes : SIZE_MAX);
        if (pages != SIZE_MAX) a.capacity_pages = (uint32_t)std::min<size_t>(pages, 0xFFFFFFFFu);
    }
    a.meta_stride = (uint32_t)batch;
    const size_t emb_stride = batch <= 64 ? kStreamSmallStride : batch;
    std::memcpy(a.emb, seq_lens, batch * 4);
    std::memcpy(a.emb + emb_stride, q_positions, batch * 4);
    std::memcpy(a.emb + 2 * emb_stride, page_table_offsets, batch * 4);
    if (!launch_stream_variant(head_dim, hpw, nw, nbuf, a, n_wg, dyn_lds, st))
        return fail("decode: kernel variant not built");
    HIP_OK(hipGetLastError());
    g.last_items = (int)std::min<uint64_t>(n_wg, total_tiles);
    std::snprintf(g.last_kernel, sizeof g.last_kernel, "stream<%zu,%d,%d,%s,%s,%d>", head_dim, hpw, nw,
                  stream_pv_name(hpw, nw), batch <= 64 ? "regs" : "lds", nbuf);
    g.last_launches = 1;
    return 1;
}

}  // extern "C"
