// Library state and the helpers every entry point shares: error reporting, the context (Ctx) with its
// options, set-up, pinned metadata slots, device-resident copies of small host arrays, the operators that are
// held back to be fused with their neighbours (row chains, the KV write, the matmul with an epilogue) and the
// calls that launch them, the end of a call (finish).
//
// A section of the one translation unit mlc_hip.hip, which includes it once, in order, after the
// sections before it; not a header for anybody else.

namespace {

using namespace mlc_hip;

thread_local std::string g_err;
bool g_capture_failed = false;   // a call failed while a pass was being captured
bool g_capturing = false;        // between mlc_hip_capture_begin and mlc_hip_capture_end

int fail(const std::string& msg) {
    g_err = msg;
    if (g_capturing) g_capture_failed = true;
    return 0;
}

// For calls that allocate, copy or wait: none of that can be part of a captured pass.
#define NOT_WHILE_CAPTURING(what)                                                                   \
    do {                                                                                            \
        if (g_capturing) return fail(what ": not possible while a pass is being captured");         \
    } while (0)

#define HIP_OK(expr)                                                                  \
    do {                                                                              \
        hipError_t e_ = (expr);                                                       \
        if (e_ != hipSuccess)                                                         \
            return fail(std::string(#expr) + ": " + hipGetErrorString(e_));           \
    } while (0)

// A host-pinned + device pair used to hand small metadata to kernels with one
// stream-ordered copy.  `done` is recorded after the kernel that reads the
// device copy, so waiting on it makes both halves safe to overwrite or grow.
struct MetaSlot {
    void* host = nullptr;
    void* dev = nullptr;
    size_t cap = 0;
    hipEvent_t done = nullptr;
    bool pending = false;
};

// Scratch memory of the tile-balanced decode kernel: the split-K partials (one slot per
// workgroup, tagged words that say by themselves whether they were written in the current
// launch, so nothing has to be cleared between launches), the replay word of captured passes,
// and, in probe builds, the time stamps.  A file-scope device array, so that no entry point
// that uses it has to allocate; every GPU the library runs on holds its own copy at its own
// address, which host code learns from hipGetSymbolAddress (the array's name is not a device
// address in host code).  Launches on one GPU share the array: they must not overlap.
constexpr size_t kScratchProbeBytes = (size_t)kStreamMaxWgs * 256;
constexpr size_t kScratchReplayWordOffset = kStreamPartBytes + kScratchProbeBytes;
constexpr size_t kScratchBytes = kScratchReplayWordOffset + 256;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// First launch of every captured pass: moves the replay word on, so that the decode launches of
// this replay (whose arguments, tag included, are the same at every replay) use tags that the
// replay before did not.
__global__ void replay_word_kernel(uint32_t* word, uint32_t step) { *word += step; }
constexpr uint32_t kReplayTagStep = 4096;   // decode launches of one captured pass, at most

// Device copy of the flat page table (and, where the per-request arrays do not travel inside the
// kernel arguments, of those arrays) as the tile-balanced decode kernel reads it; uploaded only
// when the content changes.  One grow-only device buffer: its address stays the same from call to
// call (a captured pass keeps reading it), and a new content is copied over the old one in
// stream order, behind every launch that read the old one, from a slot of the pinned ring.
struct StreamTables {
    void* dev = nullptr;
    size_t cap = 0;
    bool filled = false;          // dev holds `flat` (version `uploaded`) and `meta`
    std::vector<uint32_t> flat;   // the caller's flat table as last seen
    uint64_t version = 0;         // counts the changes of `flat`
    uint64_t uploaded = ~0ull;    // version of `flat` that dev holds
    std::vector<uint32_t> meta;   // seq_lens | q_positions | offsets when they are uploaded too
    size_t meta_off = 0;          // byte offset of the arrays in dev
    uint32_t max_page = 0;        // largest page id in flat
    // does some page id occur in two requests' tables (then a row written for one request may be
    // read for another)?  -1: not computed for this content
    int shared_pages = -1;
    std::vector<uint32_t> off;    // page_table_offsets the shared_pages answer was computed for
    std::vector<uint32_t> last_meta;  // seq_lens | q_positions | offsets of the last decode call (host copy)
};

// What the shape-agnostic decode kernel reads: the flat page table, the page-table offsets and the
// visible length of every request, in one device blob that is re-uploaded only when the tables
// change (the walker passes the same tables for every layer of a step).
struct DecodePlan {
    bool valid = false;
    // key
    std::vector<uint32_t> pt_flat, pt_off, seq_lens, q_pos;
    size_t B = 0;
    int causal = 0;
    // result
    size_t off_ptoff = 0, off_limits = 0;  // byte offsets in blob
    int slot = -1;
};

struct Ctx {
    bool inited = false;
    bool available = false;
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    bool pass_open = false;
    std::unordered_map<std::string, std::pair<void*, size_t>> cached;
    std::unordered_map<const void*, size_t> allocs;  // base pointer -> bytes (ours only)
    // Quantised weights, uploaded once per name (getOrCacheWeight, metal_runtime.mm:2434-2437):
    // the raw rows and, for shapes the MFMA path takes, the repacked nibbles and scales.
    struct Q4Weight {
        size_t bytes = 0, rows = 0, cols = 0, stride = 0;
        void* raw = nullptr;
        void* qs = nullptr;
        void* d = nullptr;
    };
    std::unordered_map<std::string, Q4Weight> q4_weights;
    struct Q6KWeight {
        size_t bytes = 0, rows = 0, cols = 0, stride = 0;
        void* raw = nullptr;
        void* qa = nullptr;
        void* sc = nullptr;
        void* d = nullptr;
    };
    std::unordered_map<std::string, Q6KWeight> q6k_weights;
    long opt_q4_force_generic = 0;
    long opt_q4_int_operand = 1;  // Q4_0 matrix-core kernel: integer weights as operand, d applied per block
    long opt_q4_ksplit = 0;  // 0 = automatic
    MetaSlot ring[8];
    int ring_next = 0;
    // Small host arrays that callers pass again and again with the same content (norm weights,
    // the page ids of a decode step across its layers): kept on the device, uploaded only when
    // the content changes.
    struct Resident {
        std::vector<unsigned char> content;
        void* dev = nullptr;
        size_t cap = 0;
    };
    std::map<std::tuple<int, const void*, size_t>, Resident> resident;
    // Row-local operators of the open pass that have been encoded but not launched yet: a chain
    // that one row_program_kernel launch can run (walker_kernels.h).  Everything else that
    // touches the stream or device memory calls settle() first.
    struct RowPending {
        bool active = false;
        RowProgram p{};
        size_t batch = 0;            // 0 while only the flat element count is known (a lone add)
        size_t n_flat = 0;
        size_t len = 0;              // current row length
        const void* cur = nullptr;   // buffer that will hold the chain's current values
        size_t grid_rows = 0;        // rows launched (padded to a multiple of 32 for the split stage)
    } rows;
    // The KV write of a decode step that has been encoded but not launched: either the split +
    // RoPE + cast (whose fp16 K / V rows the batched scatters that follow it consume: they join
    // it, and the three become one launch), or a batched scatter waiting for its twin.
    struct KvPending {
        bool active = false;
        bool rope = false;
        bool from_gemm = false;             // rope form: runs as the epilogue of the pending matmul
        RopeArgs a{};                       // rope form
        const void* src[2] = {nullptr, nullptr};   // plain form: fp16 rows of the first / second scatter
        void* pages[2] = {nullptr, nullptr};
        int n = 0;
        bool wide = false;                  // plain form: 16-byte units
        std::vector<uint32_t> ids, slots;   // of the scatter(s) that joined so far
        const uint32_t* d_ids = nullptr;
        const uint32_t* d_slots = nullptr;
        size_t batch = 0, row_elems = 0, page_size = 0;
    } kv;
    // A Q4_0 matmul of the open pass whose launch is held back for one call: when that call is
    // the split + RoPE + cast of the matmul's output (the qkv projection of a layer), the
    // matmul's epilogue does it and the two -- with the KV scatters that join -- are one launch.
    // When that call is the gate/up split + SiLU * up of the matmul's output (the gate/up
    // projection), the epilogue does that instead and the matmul is held back for one call more:
    // a Q4_0 matmul that reads the products (the down-projection) lets the epilogue also write
    // its activation fragments.  And while a residual add and an RMSNorm of the matmul's output
    // build their chain (RowPending) the matmul stays held back, too: a Q4_0 matmul that reads the
    // norm takes the chain's work over together with this one (mlc_hip_matmul_q4_0_batched).
    struct GemmPending {
        bool active = false;
        Q4Args a{};
        unsigned grid_x = 0, grid_z = 1;
        int nbt = 1, rt = 1;
        const void* out = nullptr;
        size_t batch = 0, rows = 0;
        bool block_scales = false;       // the activations carry one scale per (request, block)
        bool silu = false;               // the gate/up split + SiLU * up has joined
        const void* silu_out = nullptr;
        size_t ffn_inner = 0;
    } gemm;
    // The tile-balanced decode attention launch of the open pass, held back for one call: when that
    // call is a Q4_0 matmul that reads the attention's output (the out-projection), the kernel
    // that writes a row of the output also writes it as that matmul's split-fp16 activations, one
    // scale exponent per (request, block of 32 columns), and the split kernel's launch goes away.
    // Everything about the call (tables, tags, the KV write it carries) was settled when it was
    // encoded; only the launch waits.
    struct DecodePending {
        bool active = false;
        StreamArgs a{};
        size_t head_dim = 0, dyn_lds = 0;
        int hpw = 0, nw = 0, nbuf = 0;
        unsigned n_wg = 0;
        const void* o = nullptr;
        size_t batch = 0, cols = 0;
    } dec;
    long decode_split_fused = 0;     // decode launches that also wrote the next matmul's activation fragments (for tests)
    long gemm_rope_fused = 0;        // matmuls launched with the RoPE epilogue (for tests)
    long gemm_silu_fused = 0;        // ... with the gate/up split + SiLU * up as epilogue
    long gemm_rms_fused = 0;         // ... with the residual add, the RMSNorm's sums and the next matmul's fragments as epilogue
    long gemm_silu_split_fused = 0;  // ... of which also wrote the next matmul's activation fragments
    long kv_fused = 0;               // KV writes that went out fused with a neighbour (for tests)
    long kv_in_decode = 0;           // ... of which inside the attention launch
    long opt_fuse_rows = 1;          // 0 = every operator is launched when it is encoded
    long row_launches = 0;           // row_program_kernel launches (for tests)
    MetaSlot plan_slots[4];
    int plan_next = 0;
    DecodePlan plan;
    long opt_force_generic = 0;
    long opt_hpw_max = 0;                                      // query heads per wave, at most (0 = automatic)
    long opt_prefill_stages = 0;                               // LDS pipeline depth of the prefill kernel (0 = automatic)
    long opt_decode_mfma = 1;                                  // tile-balanced decode kernel: tile arithmetic on the matrix pipe
    long opt_prefill_rows64 = 1;                               // prefill: 64 chunk rows per wave where the GQA ratio allows it
    long opt_pv_fp16 = 0;                                      // 1 = softmax weights rounded to fp16 for P.V (default: fp32-grade)
    int last_launches = 0;
    int last_items = 0;
    char last_kernel[96] = "";   // kernel variant of the last decode launch (for benchmarks)
    int n_cu = 256;
    unsigned char* scratch_ptr = nullptr;   // device address of `scratch` on g.device
    uint32_t next_tag = 0;                  // tag of the last tile-balanced decode launch (never zero)
    // Every decode launch on this GPU uses the one scratch array, so launches on different
    // streams must follow each other: the stream of the last launch is remembered, and a launch
    // on another stream first waits for that one (one event, created at set-up; launches that
    // stay on the library's stream cost nothing).
    hipStream_t scratch_stream = nullptr;
    bool scratch_in_use = false;
    hipEvent_t scratch_ev = nullptr;
    // One word of pinned host memory that the decode kernel sets (through its device address) when a
    // merge gives up waiting for another workgroup's partial; looked at wherever the host has
    // waited for the stream.
    volatile uint32_t* fault_host = nullptr;
    uint32_t* fault_dev = nullptr;
    long opt_spin_limit = 200000;           // rounds a merge polls before it gives up (about 0.1 s)
    long opt_test_flags = 0;                // bit 0: workgroups do not publish their partials (tests of the give-up path)
    StreamTables tables;
    long opt_wgs_per_cu = 0;        // tile-balanced kernel: workgroups per CU (0 = automatic)
    long opt_stream_stages = 0;     // tile-balanced kernel: LDS stages per workgroup (0 = automatic)
    long opt_grid_wgs = 0;          // tile-balanced kernel: exact grid size (0 = from workgroups per CU)
    // tile-balanced kernel: units the end of a (request, KV head) pair counts for when the ranges are
    // cut (a tile is one unit).  -1 = automatic: 2 for workgroups of four waves (swept 0..4 on
    // MI355X at the TinyLlama shape: batch 32 14.3 / 13.5 / 13.4 / 13.5 / 14.1 us, with the step's
    // KV write carried 15.5 / 14.8 / 13.9 / 14.1 / 14.6 us), 0 for the one- and two-wave workgroups
    // of GQA ratios 1 and 2, whose pair ends are cheap (there any cost was 1 to 5 % slower than 0).
    long opt_pair_cost = -1;
    long table_uploads = 0;         // page-table uploads of the tile-balanced path (for tests)
    // A captured pass: the kernel launches of the encode calls between mlc_hip_capture_begin and
    // mlc_hip_capture_end as an executable HIP graph, and what the launches read that changes from
    // decode step to decode step (device copies at fixed addresses, refreshed in place).
    struct Captured {
        hipGraph_t graph = nullptr;
        hipGraphExec_t exec = nullptr;
        size_t n_nodes = 0;
        bool used_tables = false;            // a decode launch reads the device page table and arrays
        const void* tables_flat = nullptr;
        const void* tables_meta = nullptr;
        size_t B = 0, H = 0, Hkv = 0, D = 0, P = 0;
        int causal = 0;
        bool carried_kv = false;             // ... and does the step's KV write
        size_t n_decode = 0;                 // tile-balanced decode launches of the pass
        uint64_t buffer_generation = 0;      // Ctx::buffer_generation when the pass was captured
        const void* ids_dev = nullptr;       // device copy of the KV write's page ids and slots
        size_t ids_batch = 0;
    };
    std::map<int, Captured> captures;
    // Counts the times a device buffer that the library owns (and a captured launch may have its
    // address baked in) was freed or moved: a capture taken at another count is stale.
    uint64_t buffer_generation = 0;
    int next_capture = 1;
    Captured cap;                            // the pass being captured
};

Ctx g;

bool init_once() {
    if (g.inited) return g.available;
    g.inited = true;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) {
        g_err = "no HIP device";
        return false;
    }
    if (hipGetDevice(&g.device) != hipSuccess) return false;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, g.device) != hipSuccess) return false;
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        g_err = std::string("device is ") + prop.gcnArchName + ", library is built for gfx950";
        return false;
    }
    g.n_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    // the device address of the scratch array on this device (see its definition)
    void* sp = nullptr;
    if (hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch)) != hipSuccess || !sp) {
        g_err = "hipGetSymbolAddress(scratch) failed";
        return false;
    }
    g.scratch_ptr = static_cast<unsigned char*>(sp);
    {
        void* fh = nullptr;
        void* fd = nullptr;
        if (hipHostMalloc(&fh, 64, hipHostMallocMapped) != hipSuccess || !fh ||
            hipHostGetDevicePointer(&fd, fh, 0) != hipSuccess || !fd) {
            g_err = "hipHostMalloc(fault word) failed";
            return false;
        }
        g.fault_host = static_cast<volatile uint32_t*>(fh);
        *g.fault_host = 0;
        g.fault_dev = static_cast<uint32_t*>(fd);
    }
    if (hipStreamCreateWithFlags(&g.stream, hipStreamNonBlocking) != hipSuccess) return false;
    if (hipEventCreate(&g.ev0) != hipSuccess || hipEventCreate(&g.ev1) != hipSuccess) return false;
    if (hipEventCreateWithFlags(&g.scratch_ev, hipEventDisableTiming) != hipSuccess) return false;
    g.available = true;
    return true;
}

int slot_reserve(MetaSlot& s, size_t bytes) {
    // (every copy of metadata to the device comes through here)
    NOT_WHILE_CAPTURING("copying metadata to the device (run the pass once uncaptured first; the planned and "
                        "generic decode kernels, one-request scatter / gather and prefill copy on every call)");
    if (s.pending) {
        HIP_OK(hipEventSynchronize(s.done));
        s.pending = false;
    }
    if (!s.done) HIP_OK(hipEventCreateWithFlags(&s.done, hipEventDisableTiming));
    if (bytes > s.cap) {
        size_t cap = std::max<size_t>(4096, bytes * 2);
        if (s.host) HIP_OK(hipHostFree(s.host));
        if (s.dev) HIP_OK(hipFree(s.dev));
        s.host = s.dev = nullptr;
        s.cap = 0;
        HIP_OK(hipHostMalloc(&s.host, cap, hipHostMallocDefault));
        HIP_OK(hipMalloc(&s.dev, cap));
        s.cap = cap;
    }
    return 1;
}

int slot_upload(MetaSlot& s, size_t bytes) {
    HIP_OK(hipMemcpyAsync(s.dev, s.host, bytes, hipMemcpyHostToDevice, g.stream));
    return 1;
}

int slot_mark(MetaSlot& s) {
    HIP_OK(hipEventRecord(s.done, g.stream));
    s.pending = true;
    return 1;
}

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Device copy of a small host blob, uploaded only when (kind, key, bytes) has not been seen
// with this content.  The copy is ordered on the library stream, so kernels already enqueued
// that read the previous content are not disturbed.  nullptr on failure (error recorded).
const void* resident_blob(int kind, const void* key, const void* blob, size_t bytes) {
    // A caller that never repeats itself: start over -- but only while no held-back operator
    // refers to one of the copies (their launches come later).
    if (g.resident.size() > 1024 && !g.rows.active && !g.kv.active && !g.gemm.active && !g.dec.active && !g_capturing &&
        g.captures.empty()) {   // (a captured pass keeps the addresses of the copies it read)
        if (hipStreamSynchronize(g.stream) != hipSuccess) { fail("resident: synchronize failed"); return nullptr; }
        for (auto& kv : g.resident)
            if (kv.second.dev) (void)hipFree(kv.second.dev);
        g.resident.clear();
    }
    Ctx::Resident& r = g.resident[std::make_tuple(kind, key, bytes)];
    if (r.dev && r.content.size() == bytes && std::memcmp(r.content.data(), blob, bytes) == 0) return r.dev;
    if (bytes > r.cap) {
        if (g_capturing) { fail("capture: a small host array is not on the device yet (run the pass once uncaptured first)"); return nullptr; }
        if (r.dev && hipFree(r.dev) != hipSuccess) { fail("resident: hipFree failed"); return nullptr; }
        if (r.dev) ++g.buffer_generation;
        r.dev = nullptr;
        r.cap = 0;
        const size_t cap = std::max<size_t>(256, align_up(bytes, 256));
        if (hipMalloc(&r.dev, cap) != hipSuccess) { r.dev = nullptr; fail("resident: hipMalloc failed"); return nullptr; }
        r.cap = cap;
    }
    r.content.clear();  // not valid until the copy has been enqueued
    MetaSlot& s = g.ring[g.ring_next];
    g.ring_next = (g.ring_next + 1) % 8;
    if (!slot_reserve(s, bytes)) return nullptr;
    std::memcpy(s.host, blob, bytes);
    if (hipMemcpyAsync(r.dev, s.host, bytes, hipMemcpyHostToDevice, g.stream) != hipSuccess) {
        fail("resident: upload failed");
        return nullptr;
    }
    if (!slot_mark(s)) return nullptr;
    r.content.assign(static_cast<const unsigned char*>(blob), static_cast<const unsigned char*>(blob) + bytes);
    return r.dev;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

size_t known_bytes(const void* p) {
    auto it = g.allocs.find(p);
    return it == g.allocs.end() ? 0 : it->second;
}

constexpr size_t kRowMaxLen = 16384;  // row_program_kernel: 8 groups of 8 elements per thread

bool row_len_ok(size_t len) { return len > 0 && len % 8 == 0 && len <= kRowMaxLen; }

// The matrix-core Q4_0 kernel for nbt batch tiles of 32 and rt row tiles per workgroup; option
// q4_int_operand picks the arithmetic (see q4_matmul_kernels.h).
void launch_q4_mfma(int nbt, int rt, dim3 grid, const Q4Args& a) {
#define MLC_Q4(NBT, RT, WAVES)                                                                              \
    if (g.opt_q4_int_operand)                                                                               \
        hipLaunchKernelGGL((q4_0_matmul_mfma_kernel<NBT, RT, WAVES, true>), grid, dim3(WAVES * 64), 0, g.stream, a); \
    else                                                                                                    \
        hipLaunchKernelGGL((q4_0_matmul_mfma_kernel<NBT, RT, WAVES, false>), grid, dim3(WAVES * 64), 0, g.stream, a)
    if (nbt == 1) {
        if (rt == 1) { MLC_Q4(1, 1, 16); } else { MLC_Q4(1, 2, 16); }
    } else {
        if (rt == 1) { MLC_Q4(2, 1, 8); } else { MLC_Q4(2, 2, 8); }
    }
#undef MLC_Q4
}

// The same with activations that were split with one scale per (request, block): a.blk_exp.
// Integer-operand arithmetic only.  Two row tiles per workgroup run with 8 waves (the 128 registers
// a wave of 16 has do not hold the exponents as well), and not with two batch tiles (256 do not
// either): q4_block_scales_fit() is what callers ask first.
bool q4_block_scales_fit(size_t bpad, int row_tiles) { return !(bpad > 32 && row_tiles == 2); }
void launch_q4_mfma_block_scales(int nbt, int rt, dim3 grid, const Q4Args& a) {
#define MLC_Q4(NBT, RT, WAVES) \
    hipLaunchKernelGGL((q4_0_matmul_mfma_kernel<NBT, RT, WAVES, true, true>), grid, dim3(WAVES * 64), 0, g.stream, a)
    if (nbt == 1) {
        if (rt == 1) { MLC_Q4(1, 1, 16); } else { MLC_Q4(1, 2, 8); }
    } else {
        MLC_Q4(2, 1, 8);
    }
#undef MLC_Q4
}

// The gate/up projection with the gate/up split + SiLU * up (and, when a.split_frag is set, the
// split of the products for the matmul that reads them) as epilogue: two row tiles per workgroup.
// (with block-wise activation scales: one batch tile only, see launch_q4_mfma_block_scales; its 16
// waves fit their 128 registers because the epilogue's kernel schedules the scaling in groups of four)
void launch_q4_mfma_silu(int nbt, bool block_scales, dim3 grid, const Q4Args& a) {
    if (nbt == 1 && block_scales)
        hipLaunchKernelGGL((q4_0_matmul_mfma_kernel<1, 2, 16, true, true, true>), grid, dim3(16 * 64), 0, g.stream, a);
    else if (nbt == 1)
        hipLaunchKernelGGL((q4_0_matmul_mfma_kernel<1, 2, 16, true, false, true>), grid, dim3(16 * 64), 0, g.stream, a);
    else
        hipLaunchKernelGGL((q4_0_matmul_mfma_kernel<2, 2, 8, true, false, true>), grid, dim3(8 * 64), 0, g.stream, a);
}

// Launches the held-back matmul, with the split + RoPE + cast of its output as epilogue when
// `rope` is given.
int settle_gemm(const RopeArgs* rope = nullptr) {
    Ctx::GemmPending& m = g.gemm;
    if (!m.active) return 1;
    m.active = false;
    Q4Args a = m.a;
    if (rope) {
        a.rope_on = 1;
        a.rope = *rope;
        ++g.gemm_rope_fused;
    }
    const dim3 grid(m.grid_x, 1, m.grid_z);
    if (m.silu) {
        m.silu = false;
        ++g.gemm_silu_fused;
        if (a.split_frag) ++g.gemm_silu_split_fused;
        launch_q4_mfma_silu(m.nbt, m.block_scales, grid, a);
        HIP_OK(hipGetLastError());
        return 1;
    }
    if (m.block_scales)
        launch_q4_mfma_block_scales(m.nbt, m.rt, grid, a);
    else
        launch_q4_mfma(m.nbt, m.rt, grid, a);
    HIP_OK(hipGetLastError());
    return 1;
}

// True when the held-back matmul's output is exactly the fused qkv rows a split + RoPE + cast
// call describes, so that the matmul's epilogue can do that call's work.
bool gemm_feeds_rope(const void* qkv, size_t batch, size_t qkv_rows, size_t q_rows, size_t k_rows, size_t v_rows) {
    const Ctx::GemmPending& m = g.gemm;
    return g.opt_fuse_rows && m.active && !m.silu && !g.kv.active && !g.rows.active && m.out == qkv && m.batch == batch &&
           m.rows == qkv_rows && q_rows + k_rows + v_rows == qkv_rows;
}

bool launch_stream_variant(size_t D, int hpw, int nw, int nbuf, const StreamArgs& a, unsigned n_wg, size_t dyn_lds,
                           hipStream_t stream);

// Launches the held-back decode attention.
int settle_decode() {
    Ctx::DecodePending& d = g.dec;
    if (!d.active) return 1;
    d.active = false;
    if (d.a.split_frag) ++g.decode_split_fused;
    if (!launch_stream_variant(d.head_dim, d.hpw, d.nw, d.nbuf, d.a, d.n_wg, d.dyn_lds, g.stream))
        return fail("decode: kernel variant not built");
    HIP_OK(hipGetLastError());
    return 1;
}

// Launches the pending KV write.
int settle_kv() {
    Ctx::KvPending& kv = g.kv;
    if (!kv.active) return 1;
    kv.active = false;
    if (kv.rope) {
        if (kv.a.k_pages || kv.a.v_pages) ++g.kv_fused;
        if (kv.from_gemm) return settle_gemm(&kv.a);
        launch_qkv_split_rope_cast(kv.a, g.stream);
        HIP_OK(hipGetLastError());
        return 1;
    }
    const unsigned block = 256;
    const uint32_t row_units = (uint32_t)(kv.row_elems * 2 / (kv.wide ? 16 : 2));
    const unsigned total = (unsigned)(kv.batch * row_units) * (unsigned)kv.n;
    const dim3 grid((total + block - 1) / block);
    if (kv.n == 2) ++g.kv_fused;
    if (kv.wide)
        hipLaunchKernelGGL(scatter_kv_pair_kernel<uint4>, grid, dim3(block), 0, g.stream,
                           static_cast<const uint4*>(kv.src[0]), static_cast<uint4*>(kv.pages[0]),
                           static_cast<const uint4*>(kv.src[1]), static_cast<uint4*>(kv.pages[1]), kv.d_ids,
                           kv.d_slots, (uint32_t)kv.batch, row_units, (uint32_t)kv.page_size, (uint32_t)kv.n);
    else
        hipLaunchKernelGGL(scatter_kv_pair_kernel<uint16_t>, grid, dim3(block), 0, g.stream,
                           static_cast<const uint16_t*>(kv.src[0]), static_cast<uint16_t*>(kv.pages[0]),
                           static_cast<const uint16_t*>(kv.src[1]), static_cast<uint16_t*>(kv.pages[1]), kv.d_ids,
                           kv.d_slots, (uint32_t)kv.batch, row_units, (uint32_t)kv.page_size, (uint32_t)kv.n);
    HIP_OK(hipGetLastError());
    return 1;
}

// Launches what is pending, in the order it was encoded: a pending KV write is always older
// than a pending chain (whatever starts the KV write launches the chain first, and a scatter
// only joins while no chain is pending).
int settle() {
    // a held-back attention launch is older than anything else: whatever was pending when it was
    // encoded has been launched, and nothing joins a chain behind it before it is launched
    if (!settle_decode()) return 0;
    // a held-back matmul is older than anything else pending, unless the pending KV write is
    // its own epilogue
    if (g.gemm.active && !(g.kv.active && g.kv.rope && g.kv.from_gemm) && !settle_gemm()) return 0;
    if (!settle_kv()) return 0;
    Ctx::RowPending& r = g.rows;
    if (!r.active) return 1;
    r.active = false;
    const RowProgram& p = r.p;
    if (r.batch == 0) {  // a lone add over a flat range
        hipLaunchKernelGGL(add_kernel, dim3((unsigned)((r.n_flat + 255) / 256)), dim3(256), 0, g.stream, p.src,
                           p.addend, p.add_out, (uint32_t)r.n_flat);
        HIP_OK(hipGetLastError());
        return 1;
    }
    if (r.len > kRowMaxLen) {  // only a sum over K slices can be this long (nothing joined it)
        const uint32_t n = (uint32_t)(r.batch * r.len);
        hipLaunchKernelGGL(q4_sum_slices_kernel, dim3((n + 255) / 256), dim3(256), 0, g.stream, p.src, p.src_store, n,
                           p.n_slices);
        HIP_OK(hipGetLastError());
        return 1;
    }
    const dim3 grid((unsigned)(p.frag ? r.grid_rows : r.batch));
    if (r.len <= 8 * (size_t)kRowThreads) hipLaunchKernelGGL((row_program_kernel<1>), grid, dim3(kRowThreads), 0, g.stream, p);
    else hipLaunchKernelGGL((row_program_kernel<2>), grid, dim3(kRowThreads), 0, g.stream, p);
    ++g.row_launches;
    HIP_OK(hipGetLastError());
    return 1;
}

// True when the pending chain's current values are those of `buf` as rows of `len` floats; fixes
// the row shape of a chain that so far only knew its element count.
bool rows_continue(const void* buf, size_t batch, size_t len) {
    Ctx::RowPending& r = g.rows;
    if (!g.opt_fuse_rows || !r.active || r.cur != buf || r.p.frag) return false;
    if (r.batch == 0) {
        if (r.n_flat != batch * len || !row_len_ok(len)) return false;
        r.batch = batch;
        r.len = len;
        r.p.len_src = (uint32_t)len;
        r.p.batch = (uint32_t)batch;
        return true;
    }
    return r.batch == batch && r.len == len;  // callers check that the length they go on with fits
}

// Starts a chain whose source is a plain buffer of rows.
void rows_begin(const void* src, size_t batch, size_t len) {
    Ctx::RowPending& r = g.rows;
    r = Ctx::RowPending{};
    r.active = true;
    r.p.src = static_cast<const float*>(src);
    r.p.n_slices = 1;
    r.p.len_src = (uint32_t)len;
    r.p.batch = (uint32_t)batch;
    r.batch = batch;
    r.len = len;
    r.n_flat = batch * len;
    r.cur = src;
}

// After a wait for the stream: did a decode launch give up on a partial?
int check_fault() {
    if (g.fault_host && *g.fault_host) {
        *g.fault_host = 0;
        return fail("decode: a workgroup gave up waiting for another workgroup's partial result; the outputs of this "
                    "pass are not valid (launches that share the library's scratch memory must not overlap)");
    }
    return 1;
}

int finish(int sync) {
    HIP_OK(hipGetLastError());
    if (sync) {
        NOT_WHILE_CAPTURING("a call with sync = 1");
        if (!settle()) return 0;
        HIP_OK(hipStreamSynchronize(g.stream));
        return check_fault();
    }
    return 1;
}

// Page ids and slots of one batched KV write, side by side in one resident blob: the layers of
// a decode step all write to the same (page, slot) per request, so only the first of them uploads.
const void* resident_ids(const uint32_t* page_ids, const uint32_t* slots, size_t batch, size_t ids_bytes) {
    static thread_local std::vector<unsigned char> blob;
    blob.assign(ids_bytes * 2, 0);
    std::memcpy(blob.data(), page_ids, batch * 4);
    std::memcpy(blob.data() + ids_bytes, slots, batch * 4);
    const void* dev = resident_blob(1, nullptr, blob.data(), blob.size());
    if (dev && g_capturing) {
        g.cap.ids_dev = dev;
        g.cap.ids_batch = batch;
    }
    return dev;
}

}  // namespace
