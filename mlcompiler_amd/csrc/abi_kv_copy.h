// Entry points that move K/V rows between the caller's buffers and the paged pools: batched scatter,
// multi-token scatter, gather.
//
// A section of the one translation unit mlc_hip.hip, which includes it once, in order, after the
// sections before it; not a header for anybody else.

extern "C" {

int mlc_hip_scatter_kv_paged_batched_f16(void* page_storage, const uint32_t* page_ids,
                                         const uint32_t* slots_in_page, size_t page_size_tokens,
                                         size_t n_kv_heads, size_t head_dim, size_t batch,
                                         const void* src, int sync) {
    if (!init_once()) return fail("GPU unavailable");
    if (!sync && !g.pass_open) return fail("encode: no open forward pass");  // :7178
    // metal_runtime.mm:7241-7243
    if (!page_storage || !src) return fail("scatter: null buffer");
    if (batch == 0 || n_kv_heads == 0 || head_dim == 0 || page_size_tokens == 0)
        return fail("scatter: zero dimension");
    if (!page_ids || !slots_in_page) return fail("scatter: null metadata");
    const size_t row_bytes = n_kv_heads * head_dim * 2;
    if (batch * row_bytes / 2 > 0x7FFFFFFFull) return fail("scatter: too many elements");
    // Beyond the reference: a slot outside the page would land in the next page.
    for (size_t r = 0; r < batch; ++r)
        if (slots_in_page[r] >= page_size_tokens) return fail("scatter: slot >= page size");
    const size_t known = known_bytes(page_storage);
    if (known) {
        for (size_t r = 0; r < batch; ++r)
            if (((size_t)page_ids[r] + 1) * page_size_tokens * row_bytes > known)
                return fail("scatter: page id beyond the pool");
    }
    const size_t known_src = known_bytes(src);
    if (known_src && batch * row_bytes > known_src) return fail("scatter: src too small");

    const bool wide = (row_bytes % 16) == 0 && aligned16(page_storage) && aligned16(src);
    Ctx::KvPending& kv = g.kv;
    // ---- does this scatter complete a pending KV write?  (only while nothing younger is pending)
    if (g.opt_fuse_rows && kv.active && !g.rows.active && kv.batch == batch && kv.row_elems == row_bytes / 2 &&
        (kv.ids.empty() || (kv.page_size == page_size_tokens &&
                            std::memcmp(kv.ids.data(), page_ids, batch * 4) == 0 &&
                            std::memcmp(kv.slots.data(), slots_in_page, batch * 4) == 0))) {
        bool joined = false;
        if (kv.rope) {
            const bool as_k = src == kv.a.k_f16 && !kv.a.k_pages && kv.a.k_rows == row_bytes / 2;
            const bool as_v = !as_k && src == kv.a.v_f16 && !kv.a.v_pages && kv.a.v_rows == row_bytes / 2;
            if ((as_k || as_v) && (reinterpret_cast<uintptr_t>(page_storage) & 3u) == 0) {
                if (kv.ids.empty()) {
                    const size_t ids_bytes = align_up(batch * 4, 16);
                    const char* blob = static_cast<const char*>(resident_ids(page_ids, slots_in_page, batch, ids_bytes));
                    if (!blob) return 0;
                    kv.a.page_ids = reinterpret_cast<const uint32_t*>(blob);
                    kv.a.slots = reinterpret_cast<const uint32_t*>(blob + ids_bytes);
                    kv.a.page_size = (uint32_t)page_size_tokens;
                    kv.page_size = page_size_tokens;
                    kv.ids.assign(page_ids, page_ids + batch);
                    kv.slots.assign(slots_in_page, slots_in_page + batch);
                }
                (as_k ? kv.a.k_pages : kv.a.v_pages) = static_cast<_Float16*>(page_storage);
                joined = true;
            }
        } else if (kv.n == 1 && kv.wide == wide && page_storage != kv.pages[0]) {
            kv.src[1] = src;
            kv.pages[1] = page_storage;
            kv.n = 2;
            joined = true;
        }
        if (joined) return finish(sync);
    }
    if (!settle()) return 0;

    const size_t ids_bytes = align_up(batch * 4, 16);
    const char* d_blob = static_cast<const char*>(resident_ids(page_ids, slots_in_page, batch, ids_bytes));
    if (!d_blob) return 0;
    kv = Ctx::KvPending{};
    kv.active = true;
    kv.src[0] = src;
    kv.pages[0] = page_storage;
    kv.n = 1;
    kv.wide = wide;
    kv.ids.assign(page_ids, page_ids + batch);
    kv.slots.assign(slots_in_page, slots_in_page + batch);
    kv.d_ids = reinterpret_cast<const uint32_t*>(d_blob);
    kv.d_slots = reinterpret_cast<const uint32_t*>(d_blob + ids_bytes);
    kv.batch = batch;
    kv.row_elems = row_bytes / 2;
    kv.page_size = page_size_tokens;
    if (!g.opt_fuse_rows && !settle_kv()) return 0;  // no deferral: launched as encoded
    return finish(sync);
}

int mlc_hip_scatter_kv_paged(void* page_storage, const uint32_t* page_table, size_t n_page_table,
                             size_t page_size_tokens, size_t n_kv_heads, size_t head_dim,
                             size_t tokens, size_t start_slot, const void* src,
                             size_t dtype_bytes) {
    if (!init_once()) return fail("GPU unavailable");
    if (!settle()) return 0;
    // metal_runtime.mm:7839-7845
    if (!page_storage || !src) return fail("scatter_paged: null buffer");
    if (page_size_tokens == 0 || n_kv_heads == 0 || head_dim == 0 || tokens == 0)
        return fail("scatter_paged: zero dimension");
    if (dtype_bytes != 2 && dtype_bytes != 4) return fail("scatter_paged: dtype_bytes");
    if (start_slot >= page_size_tokens) return fail("scatter_paged: start_slot >= page size");
    const size_t needed = (start_slot + tokens + page_size_tokens - 1) / page_size_tokens;
    if (n_page_table < needed || !page_table) return fail("scatter_paged: page table too short");
    const size_t row_bytes = n_kv_heads * head_dim * dtype_bytes;
    const size_t known = known_bytes(page_storage);
    if (known)
        for (size_t i = 0; i < needed; ++i)
            if (((size_t)page_table[i] + 1) * page_size_tokens * row_bytes > known)
                return fail("scatter_paged: page id beyond the pool");
    const size_t known_src = known_bytes(src);
    if (known_src && tokens * row_bytes > known_src) return fail("scatter_paged: src too small");

    MetaSlot& s = g.ring[g.ring_next];
    g.ring_next = (g.ring_next + 1) % 8;
    if (!slot_reserve(s, needed * 4)) return 0;
    std::memcpy(s.host, page_table, needed * 4);
    if (!slot_upload(s, needed * 4)) return 0;
    const uint32_t* d_pt = static_cast<const uint32_t*>(s.dev);
    const size_t head_bytes = head_dim * dtype_bytes;
    const unsigned block = 256;
    if ((head_bytes % 16) == 0 && aligned16(page_storage) && aligned16(src)) {
        const uint32_t hu = (uint32_t)(head_bytes / 16);
        const size_t total = n_kv_heads * tokens * hu;
        hipLaunchKernelGGL(scatter_kv_paged_kernel<uint4>, dim3((unsigned)((total + block - 1) / block)),
                           dim3(block), 0, g.stream, static_cast<const uint4*>(src),
                           static_cast<uint4*>(page_storage), d_pt, (uint32_t)n_kv_heads,
                           (uint32_t)tokens, hu, (uint32_t)page_size_tokens, (uint32_t)start_slot);
    } else if (dtype_bytes == 4) {
        const size_t total = n_kv_heads * tokens * head_dim;
        hipLaunchKernelGGL(scatter_kv_paged_kernel<uint32_t>, dim3((unsigned)((total + block - 1) / block)),
                           dim3(block), 0, g.stream, static_cast<const uint32_t*>(src),
                           static_cast<uint32_t*>(page_storage), d_pt, (uint32_t)n_kv_heads,
                           (uint32_t)tokens, (uint32_t)head_dim, (uint32_t)page_size_tokens,
                           (uint32_t)start_slot);
    } else {
        const size_t total = n_kv_heads * tokens * head_dim;
        hipLaunchKernelGGL(scatter_kv_paged_kernel<uint16_t>, dim3((unsigned)((total + block - 1) / block)),
                           dim3(block), 0, g.stream, static_cast<const uint16_t*>(src),
                           static_cast<uint16_t*>(page_storage), d_pt, (uint32_t)n_kv_heads,
                           (uint32_t)tokens, (uint32_t)head_dim, (uint32_t)page_size_tokens,
                           (uint32_t)start_slot);
    }
    if (!slot_mark(s)) return 0;
    return finish(1);
}

int mlc_hip_gather_kv_pages(const void* page_storage, const uint32_t* page_table,
                            size_t n_page_table, size_t page_size_tokens, size_t n_kv_heads,
                            size_t head_dim, size_t num_tokens, void* dst, size_t dtype_bytes) {
    if (!init_once()) return fail("GPU unavailable");
    if (!settle()) return 0;
    // metal_runtime.mm:7657-7662
    if (!page_storage || !dst) return fail("gather: null buffer");
    if (page_size_tokens == 0 || n_kv_heads == 0 || head_dim == 0 || num_tokens == 0)
        return fail("gather: zero dimension");
    if (dtype_bytes != 2 && dtype_bytes != 4) return fail("gather: dtype_bytes");
    const size_t needed = (num_tokens + page_size_tokens - 1) / page_size_tokens;
    if (n_page_table < needed || !page_table) return fail("gather: page table too short");
    const size_t row_bytes = n_kv_heads * head_dim * dtype_bytes;
    const size_t known = known_bytes(page_storage);
    if (known)
        for (size_t i = 0; i < needed; ++i)
            if (((size_t)page_table[i] + 1) * page_size_tokens * row_bytes > known)
                return fail("gather: page id beyond the pool");
    const size_t known_dst = known_bytes(dst);
    if (known_dst && num_tokens * row_bytes > known_dst) return fail("gather: dst too small");

    MetaSlot& s = g.ring[g.ring_next];
    g.ring_next = (g.ring_next + 1) % 8;
    if (!slot_reserve(s, needed * 4)) return 0;
    std::memcpy(s.host, page_table, needed * 4);
    if (!slot_upload(s, needed * 4)) return 0;
    const uint32_t* d_pt = static_cast<const uint32_t*>(s.dev);
    const size_t head_bytes = head_dim * dtype_bytes;
    const unsigned block = 256;
    if ((head_bytes % 16) == 0 && aligned16(page_storage) && aligned16(dst)) {
        const uint32_t hu = (uint32_t)(head_bytes / 16);
        const size_t total = n_kv_heads * num_tokens * hu;
        hipLaunchKernelGGL(gather_kv_pages_kernel<uint4>, dim3((unsigned)((total + block - 1) / block)),
                           dim3(block), 0, g.stream, static_cast<const uint4*>(page_storage),
                           static_cast<uint4*>(dst), d_pt, (uint32_t)n_kv_heads,
                           (uint32_t)num_tokens, hu, (uint32_t)page_size_tokens);
    } else if (dtype_bytes == 4) {
        const size_t total = n_kv_heads * num_tokens * head_dim;
        hipLaunchKernelGGL(gather_kv_pages_kernel<uint32_t>, dim3((unsigned)((total + block - 1) / block)),
                           dim3(block), 0, g.stream, static_cast<const uint32_t*>(page_storage),
                           static_cast<uint32_t*>(dst), d_pt, (uint32_t)n_kv_heads,
                           (uint32_t)num_tokens, (uint32_t)head_dim, (uint32_t)page_size_tokens);
    } else {
        const size_t total = n_kv_heads * num_tokens * head_dim;
        hipLaunchKernelGGL(gather_kv_pages_kernel<uint16_t>, dim3((unsigned)((total + block - 1) / block)),
                           dim3(block), 0, g.stream, static_cast<const uint16_t*>(page_storage),
                           static_cast<uint16_t*>(dst), d_pt, (uint32_t)n_kv_heads,
                           (uint32_t)num_tokens, (uint32_t)head_dim, (uint32_t)page_size_tokens);
    }
    if (!slot_mark(s)) return 0;
    return finish(1);
}

}  // extern "C"
