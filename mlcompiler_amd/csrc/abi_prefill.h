// Entry point of the chunked prefill attention over paged KV.
//
// A section of the one translation unit mlc_hip.hip, which includes it once, in order, after the
// sections before it; not a header for anybody else.

extern "C" {

int mlc_hip_paged_attn_prefill(const void* q_f16, const void* k_pages, const void* v_pages,
                               void* o, const uint32_t* page_tables_flat, size_t n_flat,
                               const uint32_t* page_table_offsets, const uint32_t* seq_lens,
                               const uint32_t* q_start, size_t batch, size_t chunk,
                               size_t num_heads, size_t kv_heads, size_t head_dim,
                               size_t page_size_tokens, int sync) {
    if (!init_once()) return fail("GPU unavailable");
    if (!settle()) return 0;
    if (!sync && !g.pass_open) return fail("encode: no open forward pass");
    if (!q_f16 || !k_pages || !v_pages || !o) return fail("prefill: null buffer");
    if (batch == 0 || chunk == 0 || num_heads == 0 || head_dim == 0 || page_size_tokens == 0)
        return fail("prefill: zero dimension");
    if (kv_heads == 0 || (num_heads % kv_heads) != 0) return fail("prefill: heads % kv_heads != 0");
    if (!page_table_offsets || !seq_lens || !q_start) return fail("prefill: null metadata");
    if (n_flat && !page_tables_flat) return fail("prefill: null page table");
    if (n_flat < page_table_offsets[batch]) return fail("prefill: page table shorter than offsets");
    for (size_t r = 0; r < batch; ++r) {
        const size_t pages = ((size_t)seq_lens[r] + page_size_tokens - 1) / page_size_tokens;
        if ((size_t)page_table_offsets[r] + pages > n_flat)
            return fail("prefill: page table does not cover seq_len");
    }
    {
        const size_t rows = batch * chunk * num_heads * head_dim;
        const size_t kq = known_bytes(q_f16), ko = known_bytes(o);
        if ((kq && rows * 2 > kq) || (ko && rows * 4 > ko)) return fail("prefill: q / o buffer too small");
    }
    const size_t row_bytes = kv_heads * head_dim * 2;
    if (!check_pool_bounds(k_pages, page_tables_flat, page_table_offsets, seq_lens, batch,
                           page_size_tokens, row_bytes, "prefill K") ||
        !check_pool_bounds(v_pages, page_tables_flat, page_table_offsets, seq_lens, batch,
                           page_size_tokens, row_bytes, "prefill V"))
        return 0;
    if (!prefill_shape_supported(head_dim, page_size_tokens, num_heads, kv_heads) || !aligned16(q_f16) ||
        !aligned16(k_pages) || !aligned16(v_pages) || !aligned16(o))
        return fail("prefill: unsupported shape (head_dim 64 or 128, page size a multiple of 32, heads/kv_heads in {1,2,4,8}, 16-byte aligned buffers)");

    MetaSlot& s = g.ring[g.ring_next];
    g.ring_next = (g.ring_next + 1) % 8;
    const size_t flat_bytes = align_up(std::max<size_t>(n_flat, 1) * 4, 16);
    const size_t vec_bytes = align_up(batch * 4, 16);
    const size_t total = flat_bytes + 3 * vec_bytes;
    if (!slot_reserve(s, total)) return 0;
    char* h = static_cast<char*>(s.host);
    if (n_flat) std::memcpy(h, page_tables_flat, n_flat * 4);
    std::memcpy(h + flat_bytes, page_table_offsets, batch * 4);
    std::memcpy(h + flat_bytes + vec_bytes, seq_lens, batch * 4);
    std::memcpy(h + flat_bytes + 2 * vec_bytes, q_start, batch * 4);
    if (!slot_upload(s, total)) return 0;
    const char* dev = static_cast<const char*>(s.dev);
    PrefillArgs a;
    a.q = static_cast<const _Float16*>(q_f16);
    a.k_pages = static_cast<const _Float16*>(k_pages);
    a.v_pages = static_cast<const _Float16*>(v_pages);
    a.o = static_cast<float*>(o);
    a.pt_flat = reinterpret_cast<const uint32_t*>(dev);
    a.pt_off = reinterpret_cast<const uint32_t*>(dev + flat_bytes);
    a.seq_lens = reinterpret_cast<const uint32_t*>(dev + flat_bytes + vec_bytes);
    a.q_start = reinterpret_cast<const uint32_t*>(dev + flat_bytes + 2 * vec_bytes);
    a.batch = (uint32_t)batch;
    a.chunk = (uint32_t)chunk;
    a.num_heads = (uint32_t)num_heads;
    a.kv_heads = (uint32_t)kv_heads;
    a.page_size = (uint32_t)page_size_tokens;
    a.scale_log2e = (1.0f / std::sqrt(static_cast<float>(head_dim))) * 1.44269504088896340736f;
    a.row_blocks = 0;  // set by the launcher
    launch_prefill(a, head_dim, (int)g.opt_prefill_stages, g.opt_prefill_rows64 != 0, g.stream);
    if (!slot_mark(s)) return 0;
    return finish(sync);
}

}  // extern "C"
