// Host side of the two decode kernels: the tables of the shape-agnostic kernel, what is remembered about the
// caller's page tables (content, largest page id, shared pages), their device copy, and the launch shape of the
// tile-balanced kernel (variant, stages, grid, pair cost, arithmetic mode, scratch ordering across streams).
//
// A section of the one translation unit mlc_hip.hip, which includes it once, in order, after the
// sections before it; not a header for anybody else.

namespace {

// ---------------------------------------------------------------- tables of the shape-agnostic decode kernel

bool plan_matches(const DecodePlan& p, const uint32_t* flat, size_t n_flat, const uint32_t* off,
                  const uint32_t* seq, const uint32_t* qpos, size_t B, int causal) {
    if (!p.valid || p.B != B || p.causal != causal) return false;
    if (p.pt_flat.size() != n_flat) return false;
    if (n_flat && std::memcmp(p.pt_flat.data(), flat, n_flat * 4) != 0) return false;
    if (std::memcmp(p.pt_off.data(), off, (B + 1) * 4) != 0) return false;
    if (std::memcmp(p.seq_lens.data(), seq, B * 4) != 0) return false;
    if (std::memcmp(p.q_pos.data(), qpos, B * 4) != 0) return false;
    return true;
}

// Brings the tables of the shape-agnostic kernel onto the device (cached, see DecodePlan).
int build_plan(const uint32_t* flat, size_t n_flat, const uint32_t* off, const uint32_t* seq,
               const uint32_t* qpos, size_t B, int causal) {
    DecodePlan& p = g.plan;
    if (plan_matches(p, flat, n_flat, off, seq, qpos, B, causal)) return 1;
    p.valid = false;
    p.pt_flat.assign(flat, flat + n_flat);
    p.pt_off.assign(off, off + B + 1);
    p.seq_lens.assign(seq, seq + B);
    p.q_pos.assign(qpos, qpos + B);
    p.B = B;
    p.causal = causal;
    std::vector<uint32_t> limits(B);
    for (size_t r = 0; r < B; ++r) {
        uint64_t lim = seq[r];
        if (causal && (uint64_t)qpos[r] + 1 < lim) lim = (uint64_t)qpos[r] + 1;  // :2286
        limits[r] = (uint32_t)lim;
    }
    p.off_ptoff = align_up(n_flat * 4, 16);
    p.off_limits = p.off_ptoff + align_up(B * 4, 16);
    const size_t total = p.off_limits + align_up(B * 4, 16);
    MetaSlot& s = g.plan_slots[g.plan_next];
    if (!slot_reserve(s, total)) return 0;
    char* h = static_cast<char*>(s.host);
    if (n_flat) std::memcpy(h, flat, n_flat * 4);
    std::memcpy(h + p.off_ptoff, off, B * 4);
    std::memcpy(h + p.off_limits, limits.data(), B * 4);
    if (!slot_upload(s, total)) return 0;
    p.slot = g.plan_next;
    g.plan_next = (g.plan_next + 1) % 4;
    p.valid = true;
    return 1;
}

// Largest page id a request actually dereferences, for bounds checks against
// pools this library allocated itself.
int check_pool_bounds(const void* pool, const uint32_t* flat, const uint32_t* off,
                      const uint32_t* seq, size_t B, size_t P, size_t row_bytes,
                      const char* what) {
    const size_t bytes = known_bytes(pool);
    if (!bytes) return 1;
    for (size_t r = 0; r < B; ++r) {
        const size_t pages = (seq[r] + P - 1) / P;
        for (size_t i = 0; i < pages; ++i) {
            const size_t end = ((size_t)flat[off[r] + i] + 1) * P * row_bytes;
            if (end > bytes) return fail(std::string(what) + ": page id beyond the pool");
        }
    }
    return 1;
}

// ---------------------------------------------------------------- tile-balanced decode

// Refreshes what is remembered about the caller's page tables: their content, the largest
// page id and whether any page id occurs twice (in one table or in two requests' tables).
// The device copy is brought up to date by tables_upload.
void tables_refresh(const uint32_t* flat, size_t n_flat, const uint32_t* off, size_t B) {
    StreamTables& t = g.tables;
    const bool same_flat = t.flat.size() == n_flat && (n_flat == 0 || std::memcmp(t.flat.data(), flat, n_flat * 4) == 0);
    const bool same_off = t.off.size() == B + 1 && std::memcmp(t.off.data(), off, (B + 1) * 4) == 0;
    if (same_flat && same_off && t.shared_pages >= 0) return;
    if (!same_flat) {
        ++t.version;
        t.flat.assign(flat, flat + n_flat);
        t.max_page = 0;
        for (size_t i = 0; i < n_flat; ++i) t.max_page = std::max(t.max_page, flat[i]);
    }
    t.off.assign(off, off + B + 1);
    // duplicates among the entries the requests own ([off[r], off[r+1]), a superset of what a
    // call dereferences): the owned ids, sorted.  (No table indexed by page id: an id may be any
    // 32-bit number -- padding, or a corrupt entry that the bounds checks refuse afterwards.)
    static thread_local std::vector<uint32_t> owned;
    owned.clear();
    for (size_t r = 0; r < B; ++r) {
        const size_t b0 = std::min<size_t>(off[r], n_flat), e = std::min<size_t>(off[r + 1], n_flat);
        if (e > b0) owned.insert(owned.end(), flat + b0, flat + e);
    }
    std::sort(owned.begin(), owned.end());
    t.shared_pages = std::adjacent_find(owned.begin(), owned.end()) != owned.end() ? 1 : 0;
}

// Makes the device copy of the flat table (and of the per-request arrays when `meta3` is
// given: seq_lens | q_positions | offsets, B each) current.  Returns the device pointer of the
// table in *d_flat and of the arrays in *d_meta.  The arrays sit behind room for twice the
// table's entries (at least 16 Ki), so that a table that grows by a page now and then keeps both
// addresses.
int tables_upload(const uint32_t* meta3, size_t B, const uint32_t** d_flat, const uint32_t** d_meta) {
    StreamTables& t = g.tables;
    const size_t n_flat = t.flat.size();
    const size_t meta_bytes = meta3 ? 3 * B * 4 : 0;
    size_t flat_room = t.meta_off;
    if (n_flat * 4 > flat_room) flat_room = align_up(std::max<size_t>(2 * n_flat, 16384) * 4, 256);
    const size_t total = flat_room + std::max<size_t>(meta_bytes, 3 * 4096 * 4);
    bool upload = t.uploaded != t.version || !t.filled || flat_room != t.meta_off;
    if (meta3) {
        if (t.meta.size() != 3 * B || std::memcmp(t.meta.data(), meta3, meta_bytes) != 0) upload = true;
    }
    if (upload) {
        NOT_WHILE_CAPTURING("copying the decode tables to the device (run the pass once uncaptured first)");
        if (total > t.cap) {
            HIP_OK(hipStreamSynchronize(g.stream));
            if (t.dev) HIP_OK(hipFree(t.dev));
            if (t.dev) ++g.buffer_generation;
            t.dev = nullptr;
            t.cap = 0;
            HIP_OK(hipMalloc(&t.dev, total));
            t.cap = total;
        }
        MetaSlot& s = g.ring[g.ring_next];
        g.ring_next = (g.ring_next + 1) % 8;
        const size_t flat_stage = align_up(n_flat * 4, 16);   // the staging slot holds the two side by side
        if (!slot_reserve(s, flat_stage + meta_bytes)) return 0;
        char* h = static_cast<char*>(s.host);
        if (n_flat) std::memcpy(h, t.flat.data(), n_flat * 4);
        if (meta3) {
            std::memcpy(h + flat_stage, meta3, meta_bytes);
            t.meta.assign(meta3, meta3 + 3 * B);
            // table and arrays in two copies: what lies between them on the device is not sent
            if (n_flat) HIP_OK(hipMemcpyAsync(t.dev, h, n_flat * 4, hipMemcpyHostToDevice, g.stream));
            HIP_OK(hipMemcpyAsync(static_cast<char*>(t.dev) + flat_room, h + flat_stage, meta_bytes,
                                  hipMemcpyHostToDevice, g.stream));
        } else {
            t.meta.clear();
            if (n_flat) HIP_OK(hipMemcpyAsync(t.dev, h, n_flat * 4, hipMemcpyHostToDevice, g.stream));
        }
        if (!slot_mark(s)) return 0;
        t.filled = true;
        t.uploaded = t.version;
        t.meta_off = flat_room;
        ++g.table_uploads;
    }
    const char* dev = static_cast<const char*>(t.dev);
    *d_flat = reinterpret_cast<const uint32_t*>(dev);
    *d_meta = meta3 ? reinterpret_cast<const uint32_t*>(dev + t.meta_off) : nullptr;
    return 1;
}

// Shape of the tile-balanced launch for (G, D): query heads per wave, waves per workgroup;
// false when the kernel does not cover the shape.
bool stream_variant(size_t G, size_t D, int* hpw_out, int* nw_out) {
    if (D != 64 && D != 128) return false;
    const long hpw_cap = g.opt_hpw_max > 0 ? g.opt_hpw_max : std::max<long>(1, (long)G / 4);
    int hpw = 8;
    while (hpw > 1 && (hpw > hpw_cap || (G % (size_t)hpw) != 0)) hpw >>= 1;
    size_t nw = G / (size_t)hpw;
    if (nw > 4 || nw == 3) {
        hpw = 8;
        while (hpw > 1 && (G % (size_t)hpw) != 0) hpw >>= 1;
        nw = G / (size_t)hpw;
    }
    if (nw > 4 || nw == 3) return false;
    *hpw_out = hpw;
    *nw_out = (int)nw;
    return true;
}

// LDS stages of the tile-balanced kernel.  Two by default: swept over 2..4 stages and 1..5
// workgroups per CU on MI355X, in both arithmetic modes, two stages and two workgroups per CU
// were fastest at 38 MB and at 1.2 GB of KV per launch (deeper stages only delay the first tile
// of every workgroup).  Batches above 64 requests keep their per-request figures in LDS as well
// and take three stages at most.
int stream_stages(size_t batch) {
    const int most = batch <= 64 ? 4 : 3;
    int nbuf = 2;
    if (g.opt_stream_stages > 0) nbuf = (int)std::min<long>(g.opt_stream_stages, most);
    return nbuf;
}

// Grid of the tile-balanced kernel: as many workgroups as stay resident (LDS decides), within
// what the scratch array holds.
unsigned stream_grid(size_t G, size_t D, int nbuf, size_t dyn_lds) {
    const bool matrix_pipe = g.opt_decode_mfma && G >= 4 && G <= 16;
    const size_t lds = stream_static_lds_bytes(nbuf, G, D, matrix_pipe) + dyn_lds;
    size_t per_cu = std::max<size_t>(1, std::min<size_t>(160 * 1024 / lds, 2));
    if (g.opt_wgs_per_cu > 0) per_cu = (size_t)g.opt_wgs_per_cu;
    size_t W = (size_t)g.n_cu * per_cu;
    if (g.opt_grid_wgs > 0) W = (size_t)g.opt_grid_wgs;
    W = std::min<size_t>(W, kStreamMaxWgs);
    int hpw = 1, nw = 1;
    if (stream_variant(G, D, &hpw, &nw)) W = std::min<size_t>(W, kStreamPartBytes / stream_partial_bytes(G, D, (size_t)nw));
    return (unsigned)std::max<size_t>(W, 1);
}

uint32_t stream_pair_cost(int nw, size_t G, size_t D) {
    if (g.opt_pair_cost >= 0) return (uint32_t)g.opt_pair_cost;
    (void)G;
    (void)D;
    return nw == 4 ? 2u : 0u;
}

// Arithmetic mode of the tile-balanced kernel: 0 fp32 softmax weights, 1 fp16 weights on the vector
// pipe, 2 matrix pipe (4 waves per workgroup, at most 16 heads per KV head).
int stream_pv_mode(int hpw, int nw) {
    const bool matrix_pipe = g.opt_decode_mfma && nw == 4 && hpw * nw <= 16;
    if (!g.opt_pv_fp16) return matrix_pipe ? 3 : 0;
    return matrix_pipe ? 2 : 1;
}
const char* stream_pv_name(int hpw, int nw) {
    const int m = stream_pv_mode(hpw, nw);
    return m == 3 ? "mfma-p32" : m == 2 ? "mfma" : m == 1 ? "pv16" : "pv32";
}

// Orders a launch that uses the scratch array on `stream` behind the last one that did (see
// Ctx::scratch_stream).  The library's own stream lives as long as the library, so the event that
// marks its last launch is recorded only when another stream shows up; a caller's stream may be
// gone by then, so the event is recorded right behind a launch on one.  A captured pass runs on
// the library's stream, where its replays are ordered like any other launch there.
int scratch_follow(hipStream_t stream) {
    if (g_capturing) return 1;
    if (g.scratch_in_use && g.scratch_stream != stream) {
        if (g.scratch_stream == g.stream) HIP_OK(hipEventRecord(g.scratch_ev, g.stream));
        HIP_OK(hipStreamWaitEvent(stream, g.scratch_ev, 0));
    }
    return 1;
}
int scratch_launched(hipStream_t stream) {
    if (g_capturing) return 1;
    g.scratch_stream = stream;
    g.scratch_in_use = true;
    if (stream != g.stream) HIP_OK(hipEventRecord(g.scratch_ev, stream));
    return 1;
}

bool launch_stream_variant(size_t D, int hpw, int nw, int nbuf, const StreamArgs& a, unsigned n_wg, size_t dyn_lds,
                           hipStream_t stream) {
    if (!scratch_follow(stream)) return false;
    const int pvm = stream_pv_mode(hpw, nw);
    bool launched = false;
#define MLC_CASE(d, h) \
    if (D == d && hpw == h) launched = launch_decode_stream_##d##_##h(nw, nbuf, pvm, a, n_wg, dyn_lds, stream);
    MLC_CASE(64, 1) MLC_CASE(64, 2) MLC_CASE(64, 4) MLC_CASE(64, 8)
    MLC_CASE(128, 1) MLC_CASE(128, 2) MLC_CASE(128, 4) MLC_CASE(128, 8)
#undef MLC_CASE
    return launched && scratch_launched(stream);
}

void stream_fill_common(StreamArgs& a, const void* q, const void* k_pages, const void* v_pages, void* o,
                        size_t B, size_t H, size_t Hkv, size_t D, size_t P, int causal) {
    a.q = static_cast<const float*>(q);
    a.k_pages = static_cast<const uint4*>(k_pages);
    a.v_pages = static_cast<const uint4*>(v_pages);
    a.o = static_cast<float*>(o);
    a.part = reinterpret_cast<uint64_t*>(g.scratch_ptr);
    a.fault = g.fault_dev;
    a.spin_limit = (uint32_t)g.opt_spin_limit;
    a.test_flags = (uint32_t)g.opt_test_flags;
    if (g_capturing) {
        // the arguments of a captured launch are the same at every replay: its tag is its number in
        // the pass plus the replay word, which the pass's first launch moves on by kReplayTagStep
        a.tag = 0x80000000u | (uint32_t)g.cap.n_decode++;
        a.tag_dev = reinterpret_cast<const uint32_t*>(g.scratch_ptr + kScratchReplayWordOffset);
    } else {
        if (++g.next_tag == 0) ++g.next_tag;   // (zero is what untouched memory holds)
        a.tag = g.next_tag;
        a.tag_dev = nullptr;
    }
    a.batch = (uint32_t)B;
    a.num_heads = (uint32_t)H;
    a.kv_heads = (uint32_t)Hkv;
    a.page_size = (uint32_t)P;
    a.causal = causal ? 1u : 0u;
    a.capacity_pages = 0;
    a.meta = nullptr;
    a.meta_stride = 0;
    a.scale_log2e = (1.0f / std::sqrt(static_cast<float>(D))) * 1.44269504088896340736f;
    a.pair_cost = 0;  // (set by the caller once the workgroup shape is known: stream_pair_cost)
    a.new_k = a.new_v = nullptr;
    a.new_ids = a.new_slots = nullptr;
    a.split_frag = nullptr;
    a.split_exp = nullptr;
    a.split_rows = 0;
}

}  // namespace
