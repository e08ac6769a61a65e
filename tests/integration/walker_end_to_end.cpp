// Drives the reference's unchanged BatchedWalker::step (compiler/runtime/batched_walker.cpp:81-479)
// over a GGUF model on top of libmlc_hip.so, the way the reference's own test does
// (tests/test_batched_walker_h1.cpp:62-180: a PagePool, a PagedKVStorage, one RequestSlot per
// request and step), and writes every step's logits to a file.  The same program computes the
// expected logits with the reference's single-stream CPU runner (DecodeRunner, the figure the
// reference's test compares against): that mode needs no GPU.
//
//   walker_end_to_end reference MODEL.gguf OUT.bin REQUESTS STEPS    (CPU, DecodeRunner)
//   walker_end_to_end walker    MODEL.gguf OUT.bin REQUESTS STEPS    (GPU, BatchedWalker)
//
// OUT.bin: uint32 requests, steps, vocab, then float32 logits [request][step][vocab].
// Request r's token at step i is (7 + 13 * r + 29 * i) % vocab, its position i.
// This file is test infrastructure of this repository; the reference's sources are compiled where
// they lie (tests/integration/Makefile) and nothing of them is part of it.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <string>
#include <vector>

#include "runtime/batched_executor.hpp"
#include "runtime/batched_walker.hpp"
#include "runtime/decode_runner.hpp"
#include "runtime/metal_runtime.hpp"
#include "runtime/paged_kv.hpp"
#include "runtime/session.hpp"

namespace rt = mlc::runtime;

static uint64_t token_of(size_t request, size_t step, size_t vocab) { return (7 + 13 * request + 29 * step) % vocab; }

static int fail(const char* what) {
    std::fprintf(stderr, "walker_end_to_end: %s\n", what);
    return 1;
}

int main(int argc, char** argv) {
    if (argc != 6) return fail("usage: walker_end_to_end reference|walker MODEL.gguf OUT.bin REQUESTS STEPS");
    const std::string mode = argv[1], model = argv[2], out_path = argv[3];
    const size_t n_req = (size_t)std::atoi(argv[4]), n_steps = (size_t)std::atoi(argv[5]);
    if (!n_req || !n_steps) return fail("REQUESTS and STEPS must be positive");
    std::vector<float> logits;   // [request][step][vocab]
    size_t vocab = 0;
    try {
        if (mode == "reference") {
            rt::DecodeRunner probe(model);
            {
                rt::Session session(model);
                rt::BatchedExecutor exec(session);
                vocab = exec.graph().modelConfig().vocab_size;
            }
            if (!vocab) return fail("the model has no vocabulary size");
            logits.assign(n_req * n_steps * vocab, 0.f);
            for (size_t r = 0; r < n_req; ++r) {
                rt::DecodeOptions opts;
                for (size_t i = 0; i < n_steps; ++i) opts.tokens.push_back(token_of(r, i, vocab));
                opts.max_steps = n_steps;
                rt::DecodeRunner runner(model);
                const rt::DecodeResult res = runner.run(opts);
                if (!res.success || res.steps.size() != n_steps) return fail("DecodeRunner failed");
                for (size_t i = 0; i < n_steps; ++i) {
                    if (res.steps[i].logits.size() != vocab) return fail("DecodeRunner: logits of another size");
                    std::copy(res.steps[i].logits.begin(), res.steps[i].logits.end(),
                              logits.begin() + (r * n_steps + i) * vocab);
                }
            }
        } else if (mode == "walker") {
            if (!rt::MetalExecutor::Instance().isAvailable()) return fail("no gfx950 device");
            rt::Session session(model);
            rt::BatchedExecutor exec(session);
            size_t kv_heads = 0, head_dim = 0, layers = 0;
            for (const auto& n : exec.graph().nodes()) {
                if (n.op != rt::ExecOpType::Attention) continue;
                kv_heads = (size_t)n.attributes.at("kv_heads");
                head_dim = (size_t)n.attributes.at("head_dim");
                ++layers;
            }
            vocab = exec.graph().modelConfig().vocab_size;
            if (!layers || !vocab) return fail("no attention layers or no vocabulary in the model graph");
            const uint32_t pages = 64, page_tokens = 64;
            rt::PagePool pool(pages);
            rt::PagedKVStorage storage(pages, layers, page_tokens, kv_heads, head_dim, 2);
            if (!storage.initialize()) return fail("PagedKVStorage::initialize failed");
            exec.attach_page_pool(&pool, page_tokens);
            exec.attach_paged_storage(&storage);
            rt::BatchedWalker walker(exec);
            logits.assign(n_req * n_steps * vocab, 0.f);
            for (size_t i = 0; i < n_steps; ++i) {
                std::vector<rt::RequestSlot> slots;
                for (size_t r = 0; r < n_req; ++r) slots.push_back({(uint32_t)(100 + r), token_of(r, i, vocab), i});
                const rt::BatchedDecodeOutput out = walker.step(slots);
                if (out.per_request.size() != n_req) return fail("BatchedWalker::step: wrong number of results");
                for (const auto& per : out.per_request) {
                    const size_t r = per.request_id - 100;
                    if (!per.success || per.logits.size() != vocab) return fail("BatchedWalker::step: a request failed");
                    std::copy(per.logits.begin(), per.logits.end(), logits.begin() + (r * n_steps + i) * vocab);
                }
            }
        } else {
            return fail("mode must be reference or walker");
        }
    } catch (const std::exception& e) {
        return fail(e.what());
    }
    FILE* f = std::fopen(out_path.c_str(), "wb");
    if (!f) return fail("cannot write the output file");
    const uint32_t head[3] = {(uint32_t)n_req, (uint32_t)n_steps, (uint32_t)vocab};
    std::fwrite(head, 4, 3, f);
    std::fwrite(logits.data(), 4, logits.size(), f);
    std::fclose(f);
    std::printf("walker_end_to_end: %s, %zu requests x %zu steps, vocab %zu -> %s\n", mode.c_str(), n_req, n_steps, vocab,
                out_path.c_str());
    return 0;
}
