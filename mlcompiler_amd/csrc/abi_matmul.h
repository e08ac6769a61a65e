// Entry points of the batched Q4_0 and Q6_K matmuls and their device-resident weights.
//
// A section of the one translation unit mlc_hip.hip, which includes it once, in order, after the
// sections before it; not a header for anybody else.

extern "C" {

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
    // ... and is that chain  held-back matmul -> + residual -> RMSNorm?  Then the held-back matmul's
    // epilogue adds, leaves the sums of squares and writes (sum * gamma) as this matmul's fragments,
    // block-wise scaled, and this matmul finishes the norm: no launch in between.
    // (block-wise scaled activations: not every shape of workgroup is built for them)
    const bool scales_fit = q4_block_scales_fit((batch + 31) / 32 * 32, rows / 32 > 256 ? 2 : 1);
    bool feeds_rms = false;
    if (feeds && scales_fit && g.gemm.active && g.opt_q4_int_operand) {
        const Ctx::GemmPending& m = g.gemm;
        const RowProgram& p = g.rows.p;
        const size_t tiles = rows / 32, row_tiles = tiles > 256 ? 2 : 1;
        feeds_rms = !m.silu && m.rt == 1 && m.a.rope_on == 0 && !g.kv.active && p.src == m.out && p.n_slices == 1 &&
                    !p.src_store && !p.silu && p.addend && p.rms && !p.frag && g.rows.batch == batch &&
                    g.rows.len == cols && m.batch == batch && m.rows == cols && cols / 32 <= (batch <= 32 ? 128u : 64u) &&
                    batch * cols <= (tiles / row_tiles) * 1024;   // (every workgroup of the reader writes 1024 elements of the norm)
    }
    // ... or is the input the SiLU * up product that the held-back gate/up projection's epilogue
    // will write?  Then that epilogue also splits it, per (request, block of 32 columns).
    const bool feeds_silu = !feeds && scales_fit && batch <= 64 && g.opt_fuse_rows && g.opt_q4_int_operand && !g.opt_q4_force_generic &&
                            !(reinterpret_cast<uintptr_t>(out) & 15u) && q4_fast_shape(rows, cols, row_stride) &&
                            g.gemm.active && g.gemm.silu && !g.rows.active && !g.kv.active && g.gemm.silu_out == in &&
                            g.gemm.batch == batch && g.gemm.ffn_inner == cols;
    // ... or the output of the held-back decode attention?  Then the attention kernel splits it.
    const bool feeds_attn = !feeds && !feeds_silu && scales_fit && batch <= 64 && g.opt_fuse_rows && g.opt_q4_int_operand &&
                            !g.opt_q4_force_generic && !(reinterpret_cast<uintptr_t>(out) & 15u) &&
                            q4_fast_shape(rows, cols, row_stride) && g.dec.active && g.dec.o == in &&
                            g.dec.batch == batch && g.dec.cols == cols;
    const bool block_scales = feeds_silu || feeds_attn || feeds_rms;
    if (!feeds && !block_scales && !settle()) return 0;
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
        // (the held-back projection still reads "q4_x_fragments": its products go to a buffer of their own)
        _Float16* frag = static_cast<_Float16*>(cached_buffer(
            feeds_silu ? "q4_x_fragments_silu" : feeds_attn ? "q4_x_fragments_attention" : feeds_rms ? "q4_x_fragments_norm" : "q4_x_fragments",
            bpad * cols * 4));
        float* inv = static_cast<float*>(cached_buffer("q4_x_inv_scale", 64 * 4));
        int8_t* blk_exp = !block_scales ? nullptr : static_cast<int8_t*>(cached_buffer(
            feeds_silu ? "q4_x_block_exponents_silu" : feeds_attn ? "q4_x_block_exponents_attention" : "q4_x_block_exponents_norm",
            bpad * nblocks));
        float* ssq = feeds_rms ? static_cast<float*>(cached_buffer("q4_norm_partial_sums", nblocks * 64 * 4)) : nullptr;
        if (feeds_rms && !ssq) return fail("q4 matmul: scratch allocation failed");
        Q4Args norm{};   // (what this matmul needs to finish the norm)
        if (!frag || !inv || (block_scales && !blk_exp)) return fail("q4 matmul: scratch allocation failed");
        const float* xin = static_cast<const float*>(in) + bo * cols;
        float* o = static_cast<float*>(out) + bo * rows;
        if (feeds_silu) {
            g.gemm.a.split_frag = frag;
            g.gemm.a.split_blk_exp = blk_exp;
            if (!settle()) return 0;
        } else if (feeds_attn) {
            g.dec.a.split_frag = frag;
            g.dec.a.split_exp = blk_exp;
            g.dec.a.split_rows = (uint32_t)bpad;
            if (!settle()) return 0;
        } else if (feeds_rms) {
            Ctx::GemmPending& m = g.gemm;
            const RowProgram& p = g.rows.p;
            m.a.add_resid = p.addend;
            m.a.add_out = p.add_out;
            m.a.gamma = p.rms_weight;
            m.a.n_gamma = p.n_weight;
            m.a.ssq_out = ssq;
            m.a.split_frag = frag;
            m.a.split_blk_exp = blk_exp;
            norm.ssq_in = ssq;
            norm.ssq_tiles = (uint32_t)nblocks;   // one partial per 32 columns of the norm's row
            norm.rms_len = (uint32_t)cols;
            norm.rms_eps = p.epsilon;
            norm.rms_src = p.add_out;
            norm.rms_out = p.rms_out;
            norm.gamma = p.rms_weight;
            norm.n_gamma = p.n_weight;
            g.rows.active = false;   // the two matmuls do the chain's work
            ++g.gemm_rms_fused;
            if (!settle()) return 0;
        } else if (feeds) {  // the chain that produces the input also splits it (batch <= 64: one round)
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
        Q4Args a{};
        a.qs = static_cast<const uint2*>(w->qs);
        a.blk_exp = blk_exp;
        a.ssq_in = norm.ssq_in; a.ssq_tiles = norm.ssq_tiles; a.rms_len = norm.rms_len; a.rms_eps = norm.rms_eps;
        a.rms_src = norm.rms_src; a.rms_out = norm.rms_out; a.gamma = norm.gamma; a.n_gamma = norm.n_gamma;
        a.d = static_cast<const _Float16*>(w->d);
        a.xfrag = frag;
        a.inv_scale = inv;
        a.out = ksplit > 1 ? slices : o;
        a.batch = (uint32_t)bn; a.rows = (uint32_t)rows; a.nblocks = (uint32_t)nblocks;
        a.blocks_per_slice = (uint32_t)per_slice; a.ksplit = (uint32_t)ksplit;
        a.rope_on = 0;
        a.rope = RopeArgs{};
        // one batch tile of more than 16 requests on a grid that fills at most half of the CUs: two
        // workgroups per (row tile, K slice), each with half of the tile's requests
        const unsigned bsplit = (bpad == 32 && bn > 16 && wgs * ksplit <= (size_t)g.n_cu / 2) ? 2u : 1u;
        a.bsplit = bsplit;
        if (g.opt_fuse_rows && !sync && ksplit == 1 && batch <= 64) {
            // held back for one call: a split + RoPE + cast of this output becomes the epilogue
            Ctx::GemmPending& m = g.gemm;
            m.active = true;
            m.silu = false;
            m.block_scales = block_scales;
            m.a = a;
            m.grid_x = (unsigned)wgs;
            m.grid_z = bsplit;
            m.nbt = bpad == 32 ? 1 : 2;
            m.rt = row_tiles;
            m.out = out;
            m.batch = batch;
            m.rows = rows;
            return finish(sync);
        }
        const dim3 grid((unsigned)wgs, (unsigned)ksplit, bsplit);
        if (block_scales)
            launch_q4_mfma_block_scales(bpad == 32 ? 1 : 2, row_tiles, grid, a);
        else
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

}  // extern "C"
