// Entry points of the walker's small per-layer operators: RMSNorm, add, SiLU * up, gate/up split.
//
// A section of the one translation unit mlc_hip.hip, which includes it once, in order, after the
// sections before it; not a header for anybody else.

extern "C" {

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
    // A residual add on top of the held-back matmul's output (the out-projection): the matmul stays
    // held back while the chain add -> RMSNorm builds up behind it; if a Q4_0 matmul then reads the
    // norm, the two matmuls do the chain's work (mlc_hip_matmul_q4_0_batched), and if anything
    // else comes the matmul and the chain are launched one after the other, as always.
    const Ctx::GemmPending& m = g.gemm;
    const bool on_gemm = fusable && !sync && !joins && !r.active && !g.kv.active && !g.dec.active && m.active && !m.silu &&
                         m.rt == 1 && g.opt_q4_int_operand && (m.out == a || m.out == b) &&
                         m.batch * m.rows == total_elements && row_len_ok(m.rows);
    if (!joins && !on_gemm && !settle()) return 0;
    if (fusable) {
        const void* other = a;
        if (joins) {
            other = r.cur == a ? b : a;
        } else if (on_gemm) {
            rows_begin(m.out, 0, 0);
            r.n_flat = total_elements;
            other = m.out == a ? b : a;
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
        // The gate/up projection itself is still held back: the operator becomes its epilogue
        // (workgroup j takes row tile j of the gate half and row tile j of the up half).
        Ctx::GemmPending& m = g.gemm;
        if (g.opt_fuse_rows && g.opt_q4_int_operand && !sync && m.active && !m.silu && !g.rows.active && !g.kv.active &&
            m.rt == 2 && m.grid_z == 1 && !(m.block_scales && m.nbt != 1) && m.out == gate_up && m.batch == batch && m.rows == ffn_gate_up_rows &&
            ffn_gate_up_rows == 2 * ffn_inner && ffn_inner % 32 == 0 && aligned16(gate) && aligned16(up) && aligned16(out)) {
            m.silu = true;
            m.silu_out = out;
            m.ffn_inner = ffn_inner;
            m.a.tile_stride = (uint32_t)(ffn_inner / 32);
            m.a.ffn_inner = (uint32_t)ffn_inner;
            m.a.gate = static_cast<float*>(gate);
            m.a.up = static_cast<float*>(up);
            m.a.silu_out = static_cast<float*>(out);
            m.a.split_frag = nullptr;
            m.a.split_blk_exp = nullptr;
            return finish(sync);
        }
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

}  // extern "C"
