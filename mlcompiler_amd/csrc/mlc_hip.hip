// C ABI (include/mlc_hip.h) of the MI355X paged-attention hot path: device
// buffers, the single in-order stream that stands in for the reference's
// command buffer, the host-side split-K planner, and the kernel launches.
//
// Host-side behaviour follows the reference's MetalExecutor entry points
// (compiler/runtime/metal_runtime.mm): see the citation at each function.
#include "../../include/mlc_hip.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <map>
#include <tuple>
#include <string>
#include <unordered_map>
#include <vector>

#include "paged_copy_kernels.h"
#include "paged_decode_generic.h"
#include "paged_decode_kernels.h"
#include "paged_decode_stream.h"
#include "paged_prefill_kernels.h"
#include "paged_rope_kernels.h"
#include "walker_kernels.h"
#include "q4_matmul_kernels.h"
#include "q6k_matmul_kernels.h"

namespace mlc_hip {
// Defined in paged_decode_inst.hip, one object per (head_dim, heads-per-wave).
#define MLC_DECL(d, h) bool launch_decode_stream_##d##_##h(int, int, int, const StreamArgs&, unsigned, size_t, hipStream_t);
MLC_DECL(64, 1) MLC_DECL(64, 2) MLC_DECL(64, 4) MLC_DECL(64, 8)
MLC_DECL(128, 1) MLC_DECL(128, 2) MLC_DECL(128, 4) MLC_DECL(128, 8)
#undef MLC_DECL
}  // namespace mlc_hip

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
    struct GemmPending {
        bool active = false;
        Q4Args a{};
        unsigned grid_x = 0;
        int nbt = 1, rt = 1;
        const void* out = nullptr;
        size_t batch = 0, rows = 0;
    } gemm;
    long gemm_rope_fused = 0;        // matmuls launched with the RoPE epilogue (for tests)
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
    if (g.resident.size() > 1024 && !g.rows.active && !g.kv.active && !g.gemm.active && !g_capturing &&
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
    const dim3 grid(m.grid_x, 1);
    launch_q4_mfma(m.nbt, m.rt, grid, a);
    HIP_OK(hipGetLastError());
    return 1;
}

// True when the held-back matmul's output is exactly the fused qkv rows a split + RoPE + cast
// call describes, so that the matmul's epilogue can do that call's work.
bool gemm_feeds_rope(const void* qkv, size_t batch, size_t qkv_rows, size_t q_rows, size_t k_rows, size_t v_rows) {
    const Ctx::GemmPending& m = g.gemm;
    return g.opt_fuse_rows && m.active && !g.kv.active && !g.rows.active && m.out == qkv && m.batch == batch &&
           m.rows == qkv_rows && q_rows + k_rows + v_rows == qkv_rows;
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
}

}  // namespace

// ============================================================== C ABI

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
                      !g.gemm.active && g.kv.pages[0] == k_pages && g.kv.pages[1] == v_pages && g.kv.batch == batch &&
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
        if (!launch_stream_variant(head_dim, s_hpw, s_nw, nbuf, a, n_wg, dyn_lds, g.stream))
            return fail("decode: kernel variant not built");
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
        const bool pending = g.rows.active || g.kv.active || g.gemm.active;
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

// ---- the walker's small per-layer operators ----------------------------------------------

int mlc_hip_rms_norm_batched(const void* in, const float* weight, size_t n_weight, float epsilon,
                             size_t batch, size_t length, void* out, int sync) {
    if (!init_once()) return fail("GPU unavailable");
    if (!sync && !g.pass_open) return fail("encode: no open forward pass");
    if (!in || !out || batch == 0 || length == 0) return fail("rms norm: null buffer or zero size");  // :6895
    if (n_weight && !weight) return fail("rms norm: null weight");
    if (batch * length > 0x7FFFFFFFull) return fail("rms norm: too many elements");
    const size_t ki = known_bytes(in), ko = known_bytes(out);
    if ((ki && batch * length * 4 > ki) || (ko && batch * length * 4 > ko))
        return fail("rms norm: buffer too small");
    const bool fusable = row_len_ok(length) && aligned16(in) && aligned16(out);
    const bool joins = fusable && !g.rows.p.rms && rows_continue(in, batch, length);
    if (!joins && !settle()) return 0;  // before the weight's device copy may be replaced
    // the weight vector is borrowed for the call; its device copy is kept between calls
    const float one = 1.0f;
    const void* d_weight = resident_blob(0, weight, n_weight ? (const void*)weight : (const void*)&one,
                                         n_weight ? n_weight * 4 : 4);
    if (!d_weight) return 0;
    if (fusable && g.opt_fuse_rows) {
        if (!joins) rows_begin(in, batch, length);
        RowProgram& p = g.rows.p;
        p.rms = 1;
        p.rms_weight = static_cast<const float*>(d_weight);
        p.n_weight = (uint32_t)n_weight;
        p.epsilon = epsilon;
        p.rms_out = static_cast<float*>(out);
        g.rows.cur = out;
        return finish(sync);
    }
    hipLaunchKernelGGL(rms_norm_batched_kernel, dim3((unsigned)batch), dim3(256), 0, g.stream,
                       static_cast<const float*>(in), static_cast<const float*>(d_weight),
                       (uint32_t)n_weight, epsilon, (uint32_t)length, static_cast<float*>(out));
    return finish(sync);
}

namespace {
const char* flat3_problem(const void* a, const void* b, const void* out, size_t n, const char* what) {
    static thread_local std::string msg;
    if (!a || !b || !out || n == 0) { msg = std::string(what) + ": null buffer or zero size"; return msg.c_str(); }
    if (n > 0x7FFFFFFFull) { msg = std::string(what) + ": too many elements"; return msg.c_str(); }
    for (const void* p : {a, b, out}) {
        const size_t k = known_bytes(p);
        if (k && n * 4 > k) { msg = std::string(what) + ": buffer too small"; return msg.c_str(); }
    }
    return nullptr;
}
}  // namespace

int mlc_hip_add_batched(const void* a, const void* b, void* out, size_t total_elements, int sync) {
    if (!init_once()) return fail("GPU unavailable");
    if (!sync && !g.pass_open) return fail("encode: no open forward pass");
    if (const char* why = flat3_problem(a, b, out, total_elements, "add")) return fail(why);  // :7018
    const bool fusable = g.opt_fuse_rows && total_elements % 8 == 0 && aligned16(a) && aligned16(b) && aligned16(out);
    Ctx::RowPending& r = g.rows;
    const bool joins = fusable && r.active && (r.cur == a || r.cur == b) && !r.p.addend && !r.p.rms && !r.p.frag &&
                       (r.batch ? r.batch * r.len == total_elements && row_len_ok(r.len) : r.n_flat == total_elements);
    if (!joins && !settle()) return 0;
    if (fusable) {
        const void* other = a;
        if (joins) {
            other = r.cur == a ? b : a;
        } else {
            rows_begin(a, 0, 0);
            r.n_flat = total_elements;
            other = b;
        }
        r.p.addend = static_cast<const float*>(other);
        r.p.add_out = static_cast<float*>(out);
        r.cur = out;
        return finish(sync);
    }
    hipLaunchKernelGGL(add_kernel, dim3((unsigned)((total_elements + 255) / 256)), dim3(256), 0, g.stream,
                       static_cast<const float*>(a), static_cast<const float*>(b),
                       static_cast<float*>(out), (uint32_t)total_elements);
    return finish(sync);
}

int mlc_hip_silu_mul_batched(const void* gate, const void* up, void* out, size_t total_elements,
                             int sync) {
    if (!init_once()) return fail("GPU unavailable");
    if (!settle()) return 0;
    if (!sync && !g.pass_open) return fail("encode: no open forward pass");
    if (const char* why = flat3_problem(gate, up, out, total_elements, "silu mul")) return fail(why);  // :7048
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((total_elements + 255) / 256)), dim3(256), 0,
                       g.stream, static_cast<const float*>(gate), static_cast<const float*>(up),
                       static_cast<float*>(out), (uint32_t)total_elements);
    return finish(sync);
}

int mlc_hip_gate_up_split_silu_mul(const void* gate_up, void* gate, void* up, void* out, size_t batch,
                                   size_t ffn_inner, size_t ffn_gate_up_rows, int sync) {
    if (!init_once()) return fail("GPU unavailable");
    if (!sync && !g.pass_open) return fail("encode: no open forward pass");
    if (!gate_up) return fail("gate/up split: null buffer");
    if (batch == 0 || ffn_inner == 0) return fail("gate/up split: zero size");
    if (const char* why = flat3_problem(gate, up, out, batch * ffn_inner, "gate/up split")) return fail(why);
    if (2 * ffn_inner > ffn_gate_up_rows) return fail("gate/up split: 2 * ffn_inner > ffn_gate_up_rows");
    if (batch * ffn_gate_up_rows > 0x7FFFFFFFull) return fail("gate/up split: too many elements");
    const size_t kg = known_bytes(gate_up);
    if (kg && batch * ffn_gate_up_rows * 4 > kg) return fail("gate/up split: gate_up buffer too small");
    {
        Ctx::RowPending& r = g.rows;
        const bool joins = ffn_gate_up_rows == 2 * ffn_inner && row_len_ok(ffn_inner) && aligned16(gate) &&
                           aligned16(up) && aligned16(out) && !r.p.silu && !r.p.addend && !r.p.rms &&
                           rows_continue(gate_up, batch, ffn_gate_up_rows);
        if (joins) {
            r.p.silu = 1;
            r.p.gate_out = static_cast<float*>(gate);
            r.p.up_out = static_cast<float*>(up);
            r.p.silu_out = static_cast<float*>(out);
            r.len = ffn_inner;
            r.cur = out;
            return finish(sync);
        }
        if (!settle()) return 0;
        // nothing to join: the operator starts a chain of its own, so that the split of the
        // down-projection's input can join it
        if (g.opt_fuse_rows && ffn_gate_up_rows == 2 * ffn_inner && row_len_ok(ffn_inner) && aligned16(gate_up) &&
            aligned16(gate) && aligned16(up) && aligned16(out)) {
            rows_begin(gate_up, batch, ffn_gate_up_rows);
            r.p.silu = 1;
            r.p.gate_out = static_cast<float*>(gate);
            r.p.up_out = static_cast<float*>(up);
            r.p.silu_out = static_cast<float*>(out);
            r.len = ffn_inner;
            r.cur = out;
            return finish(sync);
        }
    }
    const size_t n = batch * ffn_inner;
    hipLaunchKernelGGL(gate_up_split_silu_mul_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       g.stream, static_cast<const float*>(gate_up), static_cast<float*>(gate),
                       static_cast<float*>(up), static_cast<float*>(out), (uint32_t)batch,
                       (uint32_t)ffn_inner, (uint32_t)ffn_gate_up_rows);
    return finish(sync);
}

// ---- batched Q4_0 matmul -------------------------------------------------------------------

namespace {

bool q4_fast_shape(size_t rows, size_t cols, size_t row_stride) {
    return rows % 64 == 0 && cols % 32 == 0 && row_stride >= cols / 32 * 18;
}

// Uploads the weight matrix on first use of its name (or when its size changed).
Ctx::Q4Weight* q4_weight(const char* name, const uint8_t* host, size_t bytes, size_t rows, size_t cols,
                         size_t stride) {
    Ctx::Q4Weight& w = g.q4_weights[name];
    if (w.raw && w.bytes == bytes && w.rows == rows && w.cols == cols && w.stride == stride) return &w;
    if (g_capturing) { fail("q4 matmul: the weights are not on the device yet (run the pass once uncaptured first)"); return nullptr; }
    (void)hipStreamSynchronize(g.stream);
    for (void** p : {&w.raw, &w.qs, &w.d})
        if (*p) { (void)hipFree(*p); *p = nullptr; ++g.buffer_generation; }
    w = Ctx::Q4Weight{};
    void* raw = nullptr;
    if (hipMalloc(&raw, bytes) != hipSuccess) { (void)hipGetLastError(); fail("q4 matmul: hipMalloc failed"); return nullptr; }
    if (hipMemcpy(raw, host, bytes, hipMemcpyHostToDevice) != hipSuccess) { (void)hipFree(raw); fail("q4 matmul: upload failed"); return nullptr; }
    w.raw = raw; w.bytes = bytes; w.rows = rows; w.cols = cols; w.stride = stride;
    if (q4_fast_shape(rows, cols, stride)) {
        const size_t nb = cols / 32, tiles = rows / 32;
        std::vector<uint8_t> qs(tiles * nb * 64 * 8);
        std::vector<uint16_t> d(tiles * nb * 32);
        for (size_t t = 0; t < tiles; ++t)
            for (size_t b = 0; b < nb; ++b)
                for (size_t m = 0; m < 32; ++m) {
                    const uint8_t* blk = host + (t * 32 + m) * stride + b * 18;
                    std::memcpy(&d[(t * nb + b) * 32 + m], blk, 2);
                    for (size_t h = 0; h < 2; ++h)
                        std::memcpy(&qs[((t * nb + b) * 64 + h * 32 + m) * 8], blk + 2 + h * 8, 8);
                }
        if (hipMalloc(&w.qs, qs.size()) != hipSuccess || hipMalloc(&w.d, d.size() * 2) != hipSuccess ||
            hipMemcpy(w.qs, qs.data(), qs.size(), hipMemcpyHostToDevice) != hipSuccess ||
            hipMemcpy(w.d, d.data(), d.size() * 2, hipMemcpyHostToDevice) != hipSuccess) {
            (void)hipGetLastError();
            fail("q4 matmul: repacked upload failed");
            return nullptr;
        }
    }
    return &w;
}

}  // namespace

int mlc_hip_matmul_q4_0_batched(const char* weight_name, const void* weights, size_t weight_bytes,
                                const void* in, size_t batch, size_t rows, size_t cols,
                                size_t row_stride, uint32_t quant_version, void* out, int sync) {
    (void)quant_version;  // one block format: quantization.cpp:228-246 ignores it as well
    if (!init_once()) return fail("GPU unavailable");
    if (!sync && !g.pass_open) return fail("encode: no open forward pass");
    if (!in || !out || batch == 0 || rows == 0 || cols == 0) return fail("q4 matmul: null buffer or zero size");  // :6940
    if (cols < 64 || (rows % 4u) != 0) return fail("q4 matmul: needs cols >= 64 and rows % 4 == 0");          // :6942
    if (!weight_name || !weights) return fail("q4 matmul: null weights");
    const size_t nb = (cols + 31) / 32;
    if (row_stride < nb * 18 || weight_bytes < (rows - 1) * row_stride + nb * 18)
        return fail("q4 matmul: weight bytes do not cover rows x row_stride");
    if (batch * rows > 0x7FFFFFFFull || batch * cols > 0x7FFFFFFFull) return fail("q4 matmul: too many elements");
    const size_t ki = known_bytes(in), ko = known_bytes(out);
    if ((ki && batch * cols * 4 > ki) || (ko && batch * rows * 4 > ko)) return fail("q4 matmul: buffer too small");
    // does the pending chain end in this matmul's input?  (decided before anything below can
    // replace a buffer the chain still refers to)
    const bool feeds = batch <= 64 && !g.opt_q4_force_generic && !(reinterpret_cast<uintptr_t>(out) & 15u) &&
                       q4_fast_shape(rows, cols, row_stride) && row_len_ok(cols) && rows_continue(in, batch, cols);
    if (!feeds && !settle()) return 0;
    Ctx::Q4Weight* w = q4_weight(weight_name, static_cast<const uint8_t*>(weights), weight_bytes, rows, cols, row_stride);
    if (!w) return 0;

    if (!w->qs || g.opt_q4_force_generic || (reinterpret_cast<uintptr_t>(out) & 15u)) {
        if (!settle()) return 0;
        const size_t waves = batch * rows;
        hipLaunchKernelGGL(q4_0_matmul_generic_kernel, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, g.stream,
                           static_cast<const uint8_t*>(w->raw), static_cast<const float*>(in),
                           static_cast<float*>(out), (uint32_t)batch, (uint32_t)rows, (uint32_t)cols,
                           (uint32_t)row_stride);
        return finish(sync);
    }

    // MFMA path, one pass over at most 64 requests at a time.  A workgroup takes one or two
    // 32-row tiles and, unless K is split, all of K; two tiles when one would give more
    // workgroups than CUs.  K is split only to fill CUs that would otherwise idle, and only as
    // far as a workgroup keeps about 64 blocks of work.
    const size_t nblocks = cols / 32, tiles = rows / 32;
    const int row_tiles = tiles > 256 ? 2 : 1;
    const size_t wgs = tiles / row_tiles;
    size_t ksplit = (size_t)g.opt_q4_ksplit;
    if (ksplit == 0)
        ksplit = std::max<size_t>(1, std::min<size_t>(256 / std::max<size_t>(wgs, 1), (nblocks * row_tiles + 63) / 64));
    ksplit = std::min(ksplit, std::max<size_t>(1, nblocks / 16));
    const size_t per_slice = (nblocks + ksplit - 1) / ksplit;
    ksplit = (nblocks + per_slice - 1) / per_slice;
    for (size_t bo = 0; bo < batch; bo += 64) {
        const size_t bn = std::min<size_t>(64, batch - bo);
        const size_t bpad = (bn + 31) / 32 * 32;
        _Float16* frag = static_cast<_Float16*>(cached_buffer("q4_x_fragments", bpad * cols * 4));
        float* inv = static_cast<float*>(cached_buffer("q4_x_inv_scale", 64 * 4));
        if (!frag || !inv) return fail("q4 matmul: scratch allocation failed");
        const float* xin = static_cast<const float*>(in) + bo * cols;
        float* o = static_cast<float*>(out) + bo * rows;
        if (feeds) {  // the chain that produces the input also splits it (batch <= 64: one round)
            g.rows.p.frag = frag;
            g.rows.p.inv_scale = inv;
            g.rows.grid_rows = bpad;
            if (!settle()) return 0;
        } else {
            hipLaunchKernelGGL(q4_split_activations_kernel, dim3((unsigned)bpad), dim3(256), 0, g.stream, xin, frag,
                               inv, (uint32_t)bn, (uint32_t)cols);
        }
        // (the chain has been launched: its K-slice source may be replaced now)
        float* slices = ksplit > 1 ? static_cast<float*>(cached_buffer("q4_k_slices", ksplit * bn * rows * 4)) : nullptr;
        if (ksplit > 1 && !slices) return fail("q4 matmul: scratch allocation failed");
        Q4Args a;
        a.qs = static_cast<const uint2*>(w->qs);
        a.d = static_cast<const _Float16*>(w->d);
        a.xfrag = frag;
        a.inv_scale = inv;
        a.out = ksplit > 1 ? slices : o;
        a.batch = (uint32_t)bn; a.rows = (uint32_t)rows; a.nblocks = (uint32_t)nblocks;
        a.blocks_per_slice = (uint32_t)per_slice; a.ksplit = (uint32_t)ksplit;
        a.rope_on = 0;
        a.rope = RopeArgs{};
        if (g.opt_fuse_rows && !sync && ksplit == 1 && batch <= 64) {
            // held back for one call: a split + RoPE + cast of this output becomes the epilogue
            Ctx::GemmPending& m = g.gemm;
            m.active = true;
            m.a = a;
            m.grid_x = (unsigned)wgs;
            m.nbt = bpad == 32 ? 1 : 2;
            m.rt = row_tiles;
            m.out = out;
            m.batch = batch;
            m.rows = rows;
            return finish(sync);
        }
        const dim3 grid((unsigned)wgs, (unsigned)ksplit);
        launch_q4_mfma(bpad == 32 ? 1 : 2, row_tiles, grid, a);
        if (ksplit > 1) {
            const uint32_t n = (uint32_t)(bn * rows);
            if (g.opt_fuse_rows && batch <= 64 && rows <= 2 * kRowMaxLen) {
                // the sum over the slices starts the next chain: whatever row-local operator
                // consumes this matmul's output joins it
                rows_begin(slices, bn, rows);
                g.rows.p.n_slices = (uint32_t)ksplit;
                g.rows.p.slice_stride = n;
                g.rows.p.src_store = o;
                g.rows.cur = o;
            } else {
                hipLaunchKernelGGL(q4_sum_slices_kernel, dim3((n + 255) / 256), dim3(256), 0, g.stream, slices, o, n,
                                   (uint32_t)ksplit);
            }
        }
    }
    return finish(sync);
}

// ---- batched Q6_K matmul -------------------------------------------------------------------

namespace {

bool q6k_fast_shape(size_t rows, size_t cols, size_t row_stride) {
    return rows % 32 == 0 && cols % 256 == 0 && row_stride >= cols / 256 * 210;
}

// Uploads the weight matrix on first use of its name (or when its size changed); shapes the
// matrix-core kernel takes are also repacked (layout: q6k_matmul_kernels.h).
Ctx::Q6KWeight* q6k_weight(const char* name, const uint8_t* host, size_t bytes, size_t rows, size_t cols,
                           size_t stride) {
    Ctx::Q6KWeight& w = g.q6k_weights[name];
    if (w.raw && w.bytes == bytes && w.rows == rows && w.cols == cols && w.stride == stride) return &w;
    if (g_capturing) { fail("q6_k matmul: the weights are not on the device yet (run the pass once uncaptured first)"); return nullptr; }
    (void)hipStreamSynchronize(g.stream);
    for (void** p : {&w.raw, &w.qa, &w.sc, &w.d})
        if (*p) { (void)hipFree(*p); *p = nullptr; ++g.buffer_generation; }
    w = Ctx::Q6KWeight{};
    void* raw = nullptr;
    if (hipMalloc(&raw, bytes) != hipSuccess) { (void)hipGetLastError(); fail("q6_k matmul: hipMalloc failed"); return nullptr; }
    if (hipMemcpy(raw, host, bytes, hipMemcpyHostToDevice) != hipSuccess) { (void)hipFree(raw); fail("q6_k matmul: upload failed"); return nullptr; }
    w.raw = raw; w.bytes = bytes; w.rows = rows; w.cols = cols; w.stride = stride;
    if (q6k_fast_shape(rows, cols, stride)) {
        const size_t nb = cols / 256, tiles = rows / 32, groups = nb * 4;
        std::vector<uint8_t> qa(tiles * groups * 3 * 64 * 8);
        std::vector<uint8_t> sc(tiles * groups * 32 * 4);
        std::vector<uint16_t> d(tiles * nb * 32);
        for (size_t t = 0; t < tiles; ++t)
            for (size_t m = 0; m < 32; ++m) {
                const uint8_t* row = host + (t * 32 + m) * stride;
                for (size_t b = 0; b < nb; ++b) {
                    const uint8_t* blk = row + b * 210;
                    std::memcpy(&d[(t * nb + b) * 32 + m], blk + 208, 2);
                    for (size_t hi = 0; hi < 2; ++hi)
                        for (size_t l0i = 0; l0i < 2; ++l0i) {
                            const size_t gi = b * 4 + hi * 2 + l0i, tg = t * groups + gi;
                            for (size_t h = 0; h < 2; ++h) {
                                const size_t lane = h * 32 + m, l = l0i * 16 + h * 8;
                                std::memcpy(&qa[((tg * 3 + 0) * 64 + lane) * 8], blk + hi * 64 + l, 8);
                                std::memcpy(&qa[((tg * 3 + 1) * 64 + lane) * 8], blk + hi * 64 + 32 + l, 8);
                                std::memcpy(&qa[((tg * 3 + 2) * 64 + lane) * 8], blk + 128 + hi * 32 + l, 8);
                            }
                            for (size_t q = 0; q < 4; ++q) sc[(tg * 32 + m) * 4 + q] = blk[192 + hi * 8 + q * 2 + l0i];
                        }
                }
            }
        if (hipMalloc(&w.qa, qa.size()) != hipSuccess || hipMalloc(&w.sc, sc.size()) != hipSuccess ||
            hipMalloc(&w.d, d.size() * 2) != hipSuccess ||
            hipMemcpy(w.qa, qa.data(), qa.size(), hipMemcpyHostToDevice) != hipSuccess ||
            hipMemcpy(w.sc, sc.data(), sc.size(), hipMemcpyHostToDevice) != hipSuccess ||
            hipMemcpy(w.d, d.data(), d.size() * 2, hipMemcpyHostToDevice) != hipSuccess) {
            (void)hipGetLastError();
            fail("q6_k matmul: repacked upload failed");
            return nullptr;
        }
    }
    return &w;
}

}  // namespace

int mlc_hip_matmul_q6_k_batched(const char* weight_name, const void* weights, size_t weight_bytes,
                                const void* in, size_t batch, size_t rows, size_t cols,
                                size_t row_stride, void* out, int sync) {
    if (!init_once()) return fail("GPU unavailable");
    if (!sync && !g.pass_open) return fail("encode: no open forward pass");
    if (!in || !out || batch == 0 || rows == 0 || cols == 0) return fail("q6_k matmul: null buffer or zero size");  // :6983
    if (cols < 64 || (rows % 4u) != 0) return fail("q6_k matmul: needs cols >= 64 and rows % 4 == 0");          // :6985
    if (!weight_name || !weights) return fail("q6_k matmul: null weights");
    const size_t nb = (cols + 255) / 256;
    if (row_stride < nb * 210 || weight_bytes < (rows - 1) * row_stride + nb * 210)
        return fail("q6_k matmul: weight bytes do not cover rows x row_stride");
    if (batch * rows > 0x7FFFFFFFull || batch * cols > 0x7FFFFFFFull) return fail("q6_k matmul: too many elements");
    const size_t ki = known_bytes(in), ko = known_bytes(out);
    if ((ki && batch * cols * 4 > ki) || (ko && batch * rows * 4 > ko)) return fail("q6_k matmul: buffer too small");
    const bool fast = q6k_fast_shape(rows, cols, row_stride) && !g.opt_q4_force_generic;
    const bool feeds = fast && batch <= 64 && row_len_ok(cols) && rows_continue(in, batch, cols);
    if (!feeds && !settle()) return 0;
    Ctx::Q6KWeight* w = q6k_weight(weight_name, static_cast<const uint8_t*>(weights), weight_bytes, rows, cols, row_stride);
    if (!w) return 0;

    if (!fast || !w->qa) {
        if (!settle()) return 0;
        const size_t waves = batch * rows;
        hipLaunchKernelGGL(q6_k_matmul_generic_kernel, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, g.stream,
                           static_cast<const uint8_t*>(w->raw), static_cast<const float*>(in),
                           static_cast<float*>(out), (uint32_t)batch, (uint32_t)rows, (uint32_t)cols,
                           (uint32_t)row_stride);
        return finish(sync);
    }

    // matrix cores, at most 64 requests per pass; two row tiles per workgroup when one would give
    // more workgroups than CUs (and the batch fits one batch tile)
    const size_t tiles = rows / 32;
    for (size_t bo = 0; bo < batch; bo += 64) {
        const size_t bn = std::min<size_t>(64, batch - bo);
        const size_t bpad = (bn + 31) / 32 * 32;
        _Float16* frag = static_cast<_Float16*>(cached_buffer("q4_x_fragments", bpad * cols * 4));
        float* inv = static_cast<float*>(cached_buffer("q4_x_inv_scale", 64 * 4));
        if (!frag || !inv) return fail("q6_k matmul: scratch allocation failed");
        const float* xin = static_cast<const float*>(in) + bo * cols;
        if (feeds) {
            g.rows.p.frag = frag;
            g.rows.p.inv_scale = inv;
            g.rows.grid_rows = bpad;
            if (!settle()) return 0;
        } else {
            hipLaunchKernelGGL(q4_split_activations_kernel, dim3((unsigned)bpad), dim3(256), 0, g.stream, xin, frag,
                               inv, (uint32_t)bn, (uint32_t)cols);
        }
        Q6KArgs a;
        a.qa = static_cast<const uint2*>(w->qa);
        a.sc = static_cast<const uint32_t*>(w->sc);
        a.d = static_cast<const _Float16*>(w->d);
        a.xfrag = frag;
        a.inv_scale = inv;
        a.out = static_cast<float*>(out) + bo * rows;
        a.batch = (uint32_t)bn; a.rows = (uint32_t)rows; a.nblocks = (uint32_t)(cols / 256);
        if (bpad == 32 && tiles > 256 && tiles % 2 == 0)
            hipLaunchKernelGGL((q6_k_matmul_mfma_kernel<1, 2>), dim3((unsigned)(tiles / 2)), dim3(512), 0, g.stream, a);
        else if (bpad == 32)
            hipLaunchKernelGGL((q6_k_matmul_mfma_kernel<1, 1>), dim3((unsigned)tiles), dim3(512), 0, g.stream, a);
        else
            hipLaunchKernelGGL((q6_k_matmul_mfma_kernel<2, 1>), dim3((unsigned)tiles), dim3(512), 0, g.stream, a);
    }
    return finish(sync);
}

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


void* mlc_hip_stream(void) {
    if (!init_once() || !settle()) return nullptr;  // the caller may enqueue behind what has been encoded
    return static_cast<void*>(g.stream);
}

int mlc_hip_timer_start(void) {
    if (!init_once()) return fail("GPU unavailable");
    NOT_WHILE_CAPTURING("timer");
    if (!settle()) return 0;
    HIP_OK(hipEventRecord(g.ev0, g.stream));
    return 1;
}

float mlc_hip_timer_stop(void) {
    if (!init_once()) return -1.f;
    if (g_capturing) { fail("timer: not possible while a pass is being captured"); return -1.f; }
    if (!settle()) return -1.f;
    if (hipEventRecord(g.ev1, g.stream) != hipSuccess) return -1.f;
    if (hipEventSynchronize(g.ev1) != hipSuccess) return -1.f;
    float ms = -1.f;
    if (hipEventElapsedTime(&ms, g.ev0, g.ev1) != hipSuccess) return -1.f;
    return ms;
}

int mlc_hip_last_decode_launches(void) { return g.last_launches; }
int mlc_hip_last_decode_work_items(void) { return g.last_items; }
const char* mlc_hip_last_decode_kernel(void) { return g.last_kernel; }
long mlc_hip_fused_kv_write_launches(void) { return g.kv_fused; }
long mlc_hip_fused_matmul_rope_launches(void) { return g.gemm_rope_fused; }
long mlc_hip_kv_writes_in_decode_launches(void) { return g.kv_in_decode; }
long mlc_hip_row_program_launches(void) { return g.row_launches; }
long mlc_hip_decode_table_uploads(void) { return g.table_uploads; }

#ifdef MLC_STREAM_PROBE
// timing probe build only: the per-workgroup time stamps of the last tile-balanced launch
int mlc_hip_debug_probe(uint64_t* dst, size_t n_wg) {
    if (!init_once()) return 0;
    HIP_OK(hipStreamSynchronize(g.stream));
    HIP_OK(hipMemcpy(dst, g.scratch_ptr + kStreamPartBytes, n_wg * 256, hipMemcpyDeviceToHost));
    return 1;
}
#endif

int mlc_hip_set_option(const char* name, long value) {
    if (!name) return 0;
    if (g.inited && g.available && !settle()) return 0;
    if (!std::strcmp(name, "fuse_row_ops")) { g.opt_fuse_rows = value ? 1 : 0; return 1; }
    if (!std::strcmp(name, "decode_force_generic")) { g.opt_force_generic = value; return 1; }
    if (!std::strcmp(name, "decode_stages")) {
        if (value != 0 && (value < 2 || value > 4)) return 0;
        g.opt_stream_stages = value;
        return 1;
    }
    if (!std::strcmp(name, "decode_grid_wgs")) {
        if (value < 0 || value > (long)kStreamMaxWgs) return 0;
        g.opt_grid_wgs = value;
        return 1;
    }
    if (!std::strcmp(name, "decode_wgs_per_cu")) {
        if (value < 0 || value > 8) return 0;
        g.opt_wgs_per_cu = value;
        return 1;
    }
    if (!std::strcmp(name, "decode_pv_fp16")) { g.opt_pv_fp16 = value ? 1 : 0; return 1; }
    if (!std::strcmp(name, "q4_force_generic")) { g.opt_q4_force_generic = value ? 1 : 0; return 1; }
    if (!std::strcmp(name, "q4_int_operand")) { g.opt_q4_int_operand = value ? 1 : 0; return 1; }
    if (!std::strcmp(name, "q4_ksplit")) {
        if (value < 0 || value > 64) return 0;
        g.opt_q4_ksplit = value;
        return 1;
    }
    if (!std::strcmp(name, "prefill_stages")) {
        if (value != 0 && value != 2 && value != 4 && value != 6 && value != 8) return 0;
        g.opt_prefill_stages = value;
        return 1;
    }
    if (!std::strcmp(name, "decode_pair_cost")) {
        if (value < -1 || value > 64) return 0;
        g.opt_pair_cost = value;
        return 1;
    }
    if (!std::strcmp(name, "decode_spin_limit")) {
        if (value < 1 || value > 0x7FFFFFFFl) return 0;
        g.opt_spin_limit = value;
        return 1;
    }
    if (!std::strcmp(name, "decode_test_flags")) {
        if (value < 0 || value > 1) return 0;
        g.opt_test_flags = value;
        return 1;
    }
    if (!std::strcmp(name, "decode_mfma")) {
        if (value != 0 && value != 1) return 0;
        g.opt_decode_mfma = value;
        return 1;
    }
    if (!std::strcmp(name, "prefill_rows64")) {
        if (value != 0 && value != 1) return 0;
        g.opt_prefill_rows64 = value;
        return 1;
    }
    if (!std::strcmp(name, "decode_heads_per_wave")) {
        if (value != 0 && value != 1 && value != 2 && value != 4 && value != 8) return 0;
        g.opt_hpw_max = value;
        return 1;
    }
    return 0;
}

}  // extern "C"
