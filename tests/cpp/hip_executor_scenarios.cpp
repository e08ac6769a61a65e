// The scenarios of the reference's tests/test_paged_flash.cpp:214-275, driven through the C++
// HipExecutor (same method names and argument order as MetalExecutor), checked against the
// CPU oracle with the benchmark's bar (cosine >= 0.9999, max-abs <= 2e-3 per head).
// Also one decode step with KV write through encode* calls, and the feed-forward half of a
// layer plus final norm and lm_head.  Exit code 0 = all passed.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

#include "../../mlcompiler_amd/csrc/hip_executor.hpp"
#include "../../oracle/paged_oracle.h"

namespace {

struct Scenario {
    const char* name;
    uint32_t batch, heads, kv_heads, head_dim, page, capacity;
    std::vector<uint32_t> seq_lens;
    bool causal;
};

int run(const Scenario& sp) {
    auto& exec = mlc_amd::HipExecutor::Instance();
    const uint32_t D = sp.head_dim, H = sp.heads;
    std::mt19937 rng(0xBEEF);  // tests/test_paged_flash.cpp:127-128
    std::uniform_real_distribution<float> dist(-0.5f, 0.5f);
    std::vector<float> q(sp.batch * H * D);
    for (auto& v : q) v = dist(rng);
    const size_t n = (size_t)sp.capacity * sp.page * sp.kv_heads * D;
    std::vector<uint16_t> k(n), v(n);
    for (auto& x : k) x = oracle_float_to_fp16_ref(dist(rng));
    for (auto& x : v) x = oracle_float_to_fp16_ref(dist(rng));
    std::vector<uint32_t> flat, off(sp.batch + 1, 0), qpos(sp.batch);
    uint32_t next = 0;
    for (uint32_t r = 0; r < sp.batch; ++r) {
        off[r] = (uint32_t)flat.size();
        for (uint32_t p = 0; p < (sp.seq_lens[r] + sp.page - 1) / sp.page; ++p) flat.push_back(next++);
        qpos[r] = sp.seq_lens[r] ? sp.seq_lens[r] - 1 : 0;
    }
    off[sp.batch] = (uint32_t)flat.size();
    std::vector<float> want(q.size()), got(q.size(), NAN);
    if (!oracle_paged_attention_executor(q.data(), k.data(), v.data(), want.data(), flat.data(),
                                         flat.size(), off.data(), sp.seq_lens.data(), qpos.data(),
                                         sp.batch, H, sp.kv_heads, D, sp.page, sp.causal, 1))
        return 1;
    void* qb = exec.allocateScratchBuffer(q.size() * 4);
    void* kb = exec.allocateScratchBuffer(n * 2);
    void* vb = exec.allocateScratchBuffer(n * 2);
    void* ob = exec.allocateScratchBuffer(q.size() * 4);
    if (!qb || !kb || !vb || !ob) return 1;
    exec.uploadToBuffer(qb, q.data(), q.size() * 4);
    exec.uploadToBuffer(kb, k.data(), n * 2);
    exec.uploadToBuffer(vb, v.data(), n * 2);
    exec.uploadToBuffer(ob, got.data(), got.size() * 4);
    bool ok = exec.runPagedFlashAttention(qb, kb, vb, ob, flat, off, sp.seq_lens, qpos, sp.batch, H,
                                          sp.kv_heads, D, sp.page, sp.causal);
    exec.downloadFromBuffer(ob, got.data(), got.size() * 4);
    int bad = ok ? 0 : 1;
    for (uint32_t i = 0; i < sp.batch * H && !bad; ++i) {
        double mx, me, rms, cs;
        oracle_metrics(got.data() + (size_t)i * D, want.data() + (size_t)i * D, D, &mx, &me, &rms, &cs);
        if (!(cs >= 0.9999) || !(mx <= 2e-3)) bad = 1;
    }
    // wrong vector lengths are refused like metal_runtime.mm:7747-7748
    std::vector<uint32_t> short_off(off.begin(), off.end() - 1);
    if (exec.runPagedFlashAttention(qb, kb, vb, ob, flat, short_off, sp.seq_lens, qpos, sp.batch, H,
                                    sp.kv_heads, D, sp.page, sp.causal))
        bad = 1;
    exec.releaseScratchBuffer(qb);
    exec.releaseScratchBuffer(kb);
    exec.releaseScratchBuffer(vb);
    exec.releaseScratchBuffer(ob);
    std::printf("%-32s %s\n", sp.name, bad ? "FAIL" : "ok");
    return bad;
}

// scatter K, scatter V, attention on one open pass (batched_walker.cpp:304-331)
int decode_step() {
    auto& exec = mlc_amd::HipExecutor::Instance();
    const uint32_t B = 3, H = 32, Hkv = 4, D = 64, P = 64, cap = 8;
    std::mt19937 rng(7);
    std::normal_distribution<float> dist(0.f, 1.f);
    const size_t n = (size_t)cap * P * Hkv * D;
    std::vector<uint16_t> k(n), v(n), nk(B * Hkv * D), nv(B * Hkv * D);
    for (auto& x : k) x = oracle_float_to_fp16_rne(dist(rng));
    for (auto& x : v) x = oracle_float_to_fp16_rne(dist(rng));
    for (auto& x : nk) x = oracle_float_to_fp16_rne(dist(rng));
    for (auto& x : nv) x = oracle_float_to_fp16_rne(dist(rng));
    std::vector<float> q(B * H * D);
    for (auto& x : q) x = dist(rng);
    std::vector<uint32_t> seq{65, 130, 7}, flat{5, 2, 0, 7, 3, 1}, off{0, 2, 5, 6}, qpos{64, 129, 6};
    std::vector<uint32_t> ids{2, 3, 1}, slots{0, 1, 6};  // (seq-1) / P -th page, (seq-1) % P
    void* kb = exec.allocateScratchBuffer(n * 2);
    void* vb = exec.allocateScratchBuffer(n * 2);
    void* nkb = exec.allocateScratchBuffer(nk.size() * 2);
    void* nvb = exec.allocateScratchBuffer(nv.size() * 2);
    void* qb = exec.allocateScratchBuffer(q.size() * 4);
    void* ob = exec.allocateScratchBuffer(q.size() * 4);
    exec.uploadToBuffer(kb, k.data(), n * 2);
    exec.uploadToBuffer(vb, v.data(), n * 2);
    exec.uploadToBuffer(nkb, nk.data(), nk.size() * 2);
    exec.uploadToBuffer(nvb, nv.data(), nv.size() * 2);
    exec.uploadToBuffer(qb, q.data(), q.size() * 4);
    int bad = 0;
    if (exec.encodeScatterKVPagedBatched(kb, ids, slots, P, Hkv, D, B, nkb)) bad = 1;  // no open pass
    bad |= !exec.beginForwardPassCB();
    bad |= !exec.encodeScatterKVPagedBatched(kb, ids, slots, P, Hkv, D, B, nkb);
    bad |= !exec.encodeScatterKVPagedBatched(vb, ids, slots, P, Hkv, D, B, nvb);
    bad |= !exec.encodePagedFlashAttention(qb, kb, vb, ob, flat, off, seq, qpos, B, H, Hkv, D, P, true);
    bad |= !exec.flushForwardPassCB();
    oracle_scatter_kv_paged_batched_f16(k.data(), ids.data(), slots.data(), P, Hkv, D, B, nk.data());
    oracle_scatter_kv_paged_batched_f16(v.data(), ids.data(), slots.data(), P, Hkv, D, B, nv.data());
    std::vector<uint16_t> gk(n), gv(n);
    exec.downloadFromBuffer(kb, gk.data(), n * 2);
    exec.downloadFromBuffer(vb, gv.data(), n * 2);
    if (std::memcmp(gk.data(), k.data(), n * 2) || std::memcmp(gv.data(), v.data(), n * 2)) bad = 1;
    std::vector<float> want(q.size()), got(q.size());
    oracle_paged_attention_executor(q.data(), k.data(), v.data(), want.data(), flat.data(), flat.size(),
                                    off.data(), seq.data(), qpos.data(), B, H, Hkv, D, P, 1, 1);
    exec.downloadFromBuffer(ob, got.data(), got.size() * 4);
    for (uint32_t i = 0; i < B * H && !bad; ++i) {
        double mx, me, rms, cs;
        oracle_metrics(got.data() + (size_t)i * D, want.data() + (size_t)i * D, D, &mx, &me, &rms, &cs);
        if (!(cs >= 0.9999) || !(mx <= 2e-3)) bad = 1;
    }
    for (void* b : {kb, vb, nkb, nvb, qb, ob}) exec.releaseScratchBuffer(b);
    std::printf("%-32s %s\n", "DecodeStepWithKvWrite", bad ? "FAIL" : "ok");
    return bad;
}

// The feed-forward half of a layer and the end of the step through the C++ methods of the
// layer loop (batched_walker.cpp:346-431): RMSNorm -> Q4_0 gate/up -> gate/up split + SiLU ->
// Q4_0 down -> residual add -> final RMSNorm -> Q6_K lm_head, one open pass, against the oracles.
int ffn_and_head() {
    auto& exec = mlc_amd::HipExecutor::Instance();
    const size_t B = 5, HID = 256, FFN = 512, VOCAB = 128;
    std::mt19937 rng(11);
    std::normal_distribution<float> dist(0.f, 1.f);
    auto randv = [&](size_t n, float s) { std::vector<float> v(n); for (auto& x : v) x = dist(rng) * s; return v; };
    const std::vector<float> x = randv(B * HID, 1.f);
    std::vector<float> g1(HID), g2(HID);
    for (auto& w : g1) w = 0.5f + 0.01f * (float)(rng() % 100);
    for (auto& w : g2) w = 0.5f + 0.01f * (float)(rng() % 100);
    auto q4 = [&](size_t rows, size_t cols) {
        std::vector<uint8_t> w(rows * (cols / 32) * 18);
        const std::vector<float> f = randv(rows * cols, 0.05f);
        for (size_t r = 0; r < rows; ++r) oracle_quantize_row_q4_0(f.data() + r * cols, cols, w.data() + r * (cols / 32) * 18);
        return w;
    };
    const std::vector<uint8_t> w_gu = q4(2 * FFN, HID), w_down = q4(HID, FFN);
    std::vector<uint8_t> w_head(VOCAB * (HID / 256) * 210);
    {
        const std::vector<float> f = randv(VOCAB * HID, 0.05f);
        for (size_t r = 0; r < VOCAB; ++r) oracle_quantize_row_q6_k(f.data() + r * HID, HID, w_head.data() + r * (HID / 256) * 210);
    }
    // oracle chain
    std::vector<float> n1(B * HID), gu(B * 2 * FFN), gate(B * FFN), up(B * FFN), mix(B * FFN), down(B * HID),
        out(B * HID), n2(B * HID), logits(B * VOCAB);
    int ok = oracle_rms_norm_batched(x.data(), g1.data(), HID, 1e-5f, B, HID, n1.data());
    ok &= oracle_matmul_q4_0_batched(w_gu.data(), n1.data(), B, 2 * FFN, HID, HID / 32 * 18, gu.data(), 1);
    ok &= oracle_gate_up_split_silu_mul(gu.data(), gate.data(), up.data(), mix.data(), B, FFN, 2 * FFN);
    ok &= oracle_matmul_q4_0_batched(w_down.data(), mix.data(), B, HID, FFN, FFN / 32 * 18, down.data(), 1);
    ok &= oracle_add(x.data(), down.data(), out.data(), B * HID);
    ok &= oracle_rms_norm_batched(out.data(), g2.data(), HID, 1e-5f, B, HID, n2.data());
    ok &= oracle_matmul_q6_k_batched(w_head.data(), n2.data(), B, VOCAB, HID, HID / 256 * 210, logits.data(), 1);
    if (!ok) return 1;
    // device
    void* dx = exec.allocateScratchBuffer(B * HID * 4);
    void* dn = exec.allocateScratchBuffer(B * HID * 4);
    void* dgu = exec.allocateScratchBuffer(B * 2 * FFN * 4);
    void* dgate = exec.allocateScratchBuffer(B * FFN * 4);
    void* dup = exec.allocateScratchBuffer(B * FFN * 4);
    void* dmix = exec.allocateScratchBuffer(B * FFN * 4);
    void* ddown = exec.allocateScratchBuffer(B * HID * 4);
    void* dout = exec.allocateScratchBuffer(B * HID * 4);
    void* dlog = exec.allocateScratchBuffer(B * VOCAB * 4);
    exec.uploadToBuffer(dx, x.data(), B * HID * 4);
    int bad = 0;
    bad |= !exec.beginForwardPassCB();
    bad |= !exec.encodeRmsNormBatched(dx, g1, 1e-5f, B, HID, dn);
    bad |= !exec.encodeMatMulQ4_0Batched("cpp.ffn_gate_up", w_gu, dn, B, 2 * FFN, HID, HID / 32 * 18, 1, dgu);
    bad |= !exec.encodeGateUpSplitSiluMul(dgu, dgate, dup, dmix, B, FFN, 2 * FFN);
    bad |= !exec.encodeMatMulQ4_0Batched("cpp.ffn_down", w_down, dmix, B, HID, FFN, FFN / 32 * 18, 1, ddown);
    bad |= !exec.encodeAddBatched(dx, ddown, dout, B * HID);
    bad |= !exec.encodeRmsNormBatched(dout, g2, 1e-5f, B, HID, dn);
    bad |= !exec.encodeMatMulQ6KBatched("cpp.head", w_head, dn, B, VOCAB, HID, HID / 256 * 210, dlog);
    bad |= !exec.flushForwardPassCB();
    std::vector<float> got_out(B * HID), got_log(B * VOCAB);
    exec.downloadFromBuffer(dout, got_out.data(), got_out.size() * 4);
    exec.downloadFromBuffer(dlog, got_log.data(), got_log.size() * 4);
    auto close = [](const std::vector<float>& a, const std::vector<float>& b) {
        double worst = 0, scale = 0;
        for (size_t i = 0; i < a.size(); ++i) {
            worst = std::fmax(worst, std::fabs((double)a[i] - b[i]));
            scale = std::fmax(scale, std::fabs((double)b[i]));
        }
        return worst <= 1e-4 * scale;
    };
    if (!close(got_out, out) || !close(got_log, logits)) bad = 1;
    // the waiting form gives the same logits
    bad |= !exec.runMatMulQ6KBatched("cpp.head", w_head, dn, B, VOCAB, HID, HID / 256 * 210, dlog);
    std::vector<float> again(B * VOCAB);
    exec.downloadFromBuffer(dlog, again.data(), again.size() * 4);
    if (std::memcmp(again.data(), got_log.data(), again.size() * 4)) bad = 1;
    for (void* b : {dx, dn, dgu, dgate, dup, dmix, ddown, dout, dlog}) exec.releaseScratchBuffer(b);
    std::printf("%-32s %s\n", "FfnAndHead", bad ? "FAIL" : "ok");
    return bad;
}

}  // namespace

int main() {
    auto& exec = mlc_amd::HipExecutor::Instance();
    if (!exec.isAvailable()) {
        std::printf("no gfx950 device: %s\n", exec.lastError());
        return 2;
    }
    const Scenario all[] = {
        {"SingleRequestSmall", 1, 2, 2, 64, 4, 8, {8}, true},
        {"TwoRequestsDisjointPages", 2, 2, 2, 64, 4, 16, {10, 12}, true},
        {"FourRequestsGQA", 4, 8, 2, 64, 4, 32, {20, 14, 8, 18}, true},
        {"EightRequestsVariableLength", 8, 8, 2, 64, 8, 64, {4, 12, 20, 32, 7, 16, 28, 11}, true},
        {"MultiplePagesPerRequest", 4, 4, 2, 64, 16, 32, {64, 50, 40, 32}, true},
        {"TinyLlamaLikeShape", 4, 32, 4, 64, 64, 8, {32, 48, 64, 96}, true},
        {"NoCausal", 2, 4, 2, 64, 8, 16, {16, 24}, false},
    };
    int bad = 0;
    for (const auto& s : all) bad |= run(s);
    bad |= decode_step();
    bad |= ffn_and_head();
    return bad;
}
