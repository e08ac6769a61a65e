// Entry points for the stream, the timer, what the last decode launched, the timing probe and the options.
//
// A section of the one translation unit mlc_hip.hip, which includes it once, in order, after the
// sections before it; not a header for anybody else.

extern "C" {

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
long mlc_hip_fused_matmul_silu_launches(void) { return g.gemm_silu_fused; }
long mlc_hip_fused_matmul_silu_split_launches(void) { return g.gemm_silu_split_fused; }
long mlc_hip_fused_decode_split_launches(void) { return g.decode_split_fused; }
long mlc_hip_fused_matmul_norm_launches(void) { return g.gemm_rms_fused; }
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
