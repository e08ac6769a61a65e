// Scripted driver around the REAL reference allocator, compiled from
// /root/reference/compiler/runtime/paged_kv.cpp (oracle/Makefile, target _ref).
// TEST INFRASTRUCTURE ONLY.  Reads one command per line on stdin and prints
// one result line per command, so a test can replay the same script through
// oracle_pool_* / oracle_req_* and compare the transcripts:
//   pool N | alloc | allocn K | release ID | req P | extend | reserve T |
//   locate POS | total | release_all | stats
// Only PagePool and RequestKVState (paged_kv.cpp:10-81) are referenced; the
// link drops the device-backed PagedKVStorage with --gc-sections.
#include <cstdio>
#include <cstring>
#include <memory>
#include <vector>

#include "runtime/paged_kv.hpp"

int main() {
    using namespace mlc::runtime;
    std::unique_ptr<PagePool> pool;
    RequestKVState req;
    char cmd[64];
    unsigned long long a = 0;
    char line[256];
    while (std::fgets(line, sizeof line, stdin)) {
        a = 0;
        cmd[0] = 0;
        if (std::sscanf(line, "%63s %llu", cmd, &a) < 1) continue;
        if (!std::strcmp(cmd, "pool")) {
            pool.reset(new PagePool(static_cast<uint32_t>(a)));
            std::printf("ok\n");
        } else if (!std::strcmp(cmd, "alloc")) {
            auto id = pool->allocate();
            if (id) std::printf("%u\n", *id); else std::printf("none\n");
        } else if (!std::strcmp(cmd, "allocn")) {
            std::vector<uint32_t> out;
            bool ok = pool->allocate_n(a, out);
            std::printf("%d", ok ? 1 : 0);
            for (uint32_t v : out) std::printf(" %u", v);
            std::printf("\n");
        } else if (!std::strcmp(cmd, "release")) {
            pool->release(static_cast<uint32_t>(a));
            std::printf("ok\n");
        } else if (!std::strcmp(cmd, "req")) {
            req = RequestKVState();
            req.page_size_tokens = static_cast<uint32_t>(a);
            std::printf("ok\n");
        } else if (!std::strcmp(cmd, "extend")) {
            auto r = req.extend_one_token(*pool);
            if (r) std::printf("%u %u\n", r->first, r->second); else std::printf("none\n");
        } else if (!std::strcmp(cmd, "reserve")) {
            bool ok = req.reserve(*pool, a);
            std::printf("%d %zu\n", ok ? 1 : 0, req.page_table.size());
        } else if (!std::strcmp(cmd, "locate")) {
            auto r = req.locate(a);
            if (r) std::printf("%u %u\n", r->first, r->second); else std::printf("none\n");
        } else if (!std::strcmp(cmd, "total")) {
            std::printf("%zu\n", req.total_tokens());
        } else if (!std::strcmp(cmd, "release_all")) {
            req.release_all(*pool);
            std::printf("ok\n");
        } else if (!std::strcmp(cmd, "stats")) {
            std::printf("%zu %zu\n", pool->pages_in_use(), pool->pages_free());
        }
    }
    return 0;
}
