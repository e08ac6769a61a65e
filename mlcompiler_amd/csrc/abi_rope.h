// Entry points of the fused split + RoPE + cast of a qkv row, with or without the paged KV write.
//
// A section of the one translation unit mlc_hip.hip, which includes it once, in order, after the
// sections before it; not a header for anybody else.

extern "C" {

namespace {

// Shared argument checks of the two qkv-split entry points.  The reference validates
// nothing here (metal_runtime.mm:7932-7936 only checks availability and the open pass);
// these checks keep the kernel inside the buffers the arguments describe.
const char* rope_args_problem(const void* qkv, const void* q, const void* cos_buf, const void* sin_buf,
                              size_t batch, size_t num_heads, size_t kv_heads, size_t head_dim,
                              size_t qkv_rows, size_t q_rows, size_t k_rows, size_t v_rows,
                              size_t rotary_dim) {
    if (!qkv || !q) return "qkv split: null buffer";
    if (batch == 0 || num_heads == 0 || kv_heads == 0 || head_dim == 0) return "qkv split: zero dimension";
    if (q_rows + k_rows + v_rows > qkv_rows) return "qkv split: q_rows + k_rows + v_rows > qkv_rows";
    if (q_rows != num_heads * head_dim || k_rows != kv_heads * head_dim)
        return "qkv split: q_rows / k_rows do not match heads * head_dim";
    if (rotary_dim > head_dim) return "qkv split: rotary_dim > head_dim";
    if (rotary_dim > 0 && (!cos_buf || !sin_buf)) return "qkv split: null cos/sin table";
    if ((head_dim | rotary_dim | qkv_rows | q_rows | k_rows | v_rows) & 1)
        return "qkv split: odd head_dim / rotary_dim / row counts are not supported";
    if (batch * qkv_rows > 0x7FFFFFFFull) return "qkv split: too many elements";
    if ((reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(q)) & 7u)
        return "qkv split: buffers must be 8-byte aligned";
    const size_t kq = known_bytes(qkv), ko = known_bytes(q);
    if (kq && batch * qkv_rows * 4 > kq) return "qkv split: qkv buffer too small";
    if (ko && batch * q_rows * 4 > ko) return "qkv split: q buffer too small";
    const size_t kc = known_bytes(cos_buf), ks = known_bytes(sin_buf);
    if (rotary_dim && ((kc && batch * (rotary_dim / 2) * 4 > kc) || (ks && batch * (rotary_dim / 2) * 4 > ks)))
        return "qkv split: cos/sin table too small";
    return nullptr;
}

}  // namespace

int mlc_hip_qkv_split_rope_cast(const void* qkv, void* q, void* k, void* v, void* k_f16, void* v_f16,
                                const void* cos_buf, const void* sin_buf, size_t batch,
                                size_t num_heads, size_t kv_heads, size_t head_dim, size_t qkv_rows,
                                size_t q_rows, size_t k_rows, size_t v_rows, size_t rotary_dim,
                                int sync) {
    if (!init_once()) return fail("GPU unavailable");
    const bool from_gemm = gemm_feeds_rope(qkv, batch, qkv_rows, q_rows, k_rows, v_rows);
    if (!from_gemm && !settle()) return 0;
    if (!sync && !g.pass_open) return fail("encode: no open forward pass");  // :7936
    if (const char* why = rope_args_problem(qkv, q, cos_buf, sin_buf, batch, num_heads, kv_heads,
                                            head_dim, qkv_rows, q_rows, k_rows, v_rows, rotary_dim))
        return fail(why);
    if (!k || !v || !k_f16 || !v_f16) return fail("qkv split: null buffer");
    if ((reinterpret_cast<uintptr_t>(k) | reinterpret_cast<uintptr_t>(v)) & 7u ||
        (reinterpret_cast<uintptr_t>(k_f16) | reinterpret_cast<uintptr_t>(v_f16)) & 3u)
        return fail("qkv split: buffers must be 8-byte (fp32) / 4-byte (fp16) aligned");
    const struct { const void* p; size_t need; } outs[] = {
        {k, batch * k_rows * 4}, {v, batch * v_rows * 4}, {k_f16, batch * k_rows * 2}, {v_f16, batch * v_rows * 2}};
    for (const auto& o : outs) {
        const size_t kb = known_bytes(o.p);
        if (kb && o.need > kb) return fail("qkv split: output buffer too small");
    }
    RopeArgs a{};
    a.qkv = static_cast<const float*>(qkv);
    a.q = static_cast<float*>(q);
    a.k = static_cast<float*>(k);
    a.v = static_cast<float*>(v);
    a.k_f16 = static_cast<_Float16*>(k_f16);
    a.v_f16 = static_cast<_Float16*>(v_f16);
    a.cos_table = static_cast<const float*>(cos_buf);
    a.sin_table = static_cast<const float*>(sin_buf);
    a.batch = (uint32_t)batch; a.head_dim = (uint32_t)head_dim; a.qkv_rows = (uint32_t)qkv_rows;
    a.q_rows = (uint32_t)q_rows; a.k_rows = (uint32_t)k_rows; a.v_rows = (uint32_t)v_rows;
    a.rotary_dim = (uint32_t)rotary_dim; a.page_size = 0;
    // held back: the batched scatters of k_f16 / v_f16 that usually follow join this launch
    Ctx::KvPending& kv = g.kv;
    kv = Ctx::KvPending{};
    kv.active = true;
    kv.rope = true;
    kv.from_gemm = from_gemm;
    kv.a = a;
    kv.batch = batch;
    kv.row_elems = k_rows;
    if (!g.opt_fuse_rows && !settle_kv()) return 0;
    return finish(sync);
}

int mlc_hip_qkv_split_rope_scatter(const void* qkv, void* q, void* k_pages, void* v_pages,
                                   void* k_f32, void* v_f32, const void* cos_buf, const void* sin_buf,
                                   const uint32_t* page_ids, const uint32_t* slots_in_page,
                                   size_t page_size_tokens, size_t batch, size_t num_heads,
                                   size_t kv_heads, size_t head_dim, size_t qkv_rows, size_t q_rows,
                                   size_t k_rows, size_t v_rows, size_t rotary_dim, int sync) {
    if (!init_once()) return fail("GPU unavailable");
    const bool from_gemm = gemm_feeds_rope(qkv, batch, qkv_rows, q_rows, k_rows, v_rows);
    if (!from_gemm && !settle()) return 0;
    if (!sync && !g.pass_open) return fail("encode: no open forward pass");
    if (const char* why = rope_args_problem(qkv, q, cos_buf, sin_buf, batch, num_heads, kv_heads,
                                            head_dim, qkv_rows, q_rows, k_rows, v_rows, rotary_dim))
        return fail(why);
    if (!k_pages || !v_pages) return fail("qkv split: null page storage");
    if (!page_ids || !slots_in_page) return fail("qkv split: null metadata");
    if (page_size_tokens == 0) return fail("qkv split: zero page size");
    if (v_rows != k_rows) return fail("qkv split: K and V rows differ, pages hold kv_heads * head_dim each");
    if ((reinterpret_cast<uintptr_t>(k_pages) | reinterpret_cast<uintptr_t>(v_pages)) & 3u ||
        (reinterpret_cast<uintptr_t>(k_f32) | reinterpret_cast<uintptr_t>(v_f32)) & 7u)
        return fail("qkv split: buffers must be 8-byte (fp32) / 4-byte (fp16) aligned");
    const size_t row_bytes = k_rows * 2;
    const size_t known_k = known_bytes(k_pages), known_v = known_bytes(v_pages);
    for (size_t r = 0; r < batch; ++r) {
        if (slots_in_page[r] >= page_size_tokens) return fail("qkv split: slot >= page size");
        const size_t end = ((size_t)page_ids[r] + 1) * page_size_tokens * row_bytes;
        if ((known_k && end > known_k) || (known_v && end > known_v))
            return fail("qkv split: page id beyond the pool");
    }
    const size_t ids_bytes = align_up(batch * 4, 16);
    const char* d_blob = static_cast<const char*>(resident_ids(page_ids, slots_in_page, batch, ids_bytes));
    if (!d_blob) return 0;
    RopeArgs a{};
    a.qkv = static_cast<const float*>(qkv);
    a.q = static_cast<float*>(q);
    a.k = static_cast<float*>(k_f32);
    a.v = static_cast<float*>(v_f32);
    a.k_pages = static_cast<_Float16*>(k_pages);
    a.v_pages = static_cast<_Float16*>(v_pages);
    a.cos_table = static_cast<const float*>(cos_buf);
    a.sin_table = static_cast<const float*>(sin_buf);
    a.page_ids = reinterpret_cast<const uint32_t*>(d_blob);
    a.slots = reinterpret_cast<const uint32_t*>(d_blob + ids_bytes);
    a.batch = (uint32_t)batch; a.head_dim = (uint32_t)head_dim; a.qkv_rows = (uint32_t)qkv_rows;
    a.q_rows = (uint32_t)q_rows; a.k_rows = (uint32_t)k_rows; a.v_rows = (uint32_t)v_rows;
    a.rotary_dim = (uint32_t)rotary_dim; a.page_size = (uint32_t)page_size_tokens;
    if (from_gemm && g.gemm.active) {  // (still held back: the id upload above launches nothing)
        if (!settle_gemm(&a)) return 0;
    } else {
        launch_qkv_split_rope_cast(a, g.stream);
    }
    return finish(sync);
}

}  // extern "C"
