// Host-only hardening check: mutated expert-index files (flipped bytes, truncations, random
// offsets, lengths, counts and payload sizes) through the container reader. Built by
// tests/test_artifact.py with the host-side address and undefined-behaviour sanitizers around the
// reader's own source file; a finding aborts the program. argv[1] = number of mutations.
#include "aeon_mi355.h"
#include <cstdio>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>
#include <unistd.h>

static void write_file(const std::string& p, const std::vector<uint8_t>& b) {
    FILE* f = fopen(p.c_str(), "wb"); fwrite(b.data(), 1, b.size(), f); fclose(f);
}
int main(int argc, char** argv) {
    const int mutations = argc > 1 ? atoi(argv[1]) : 20000;
    const uint32_t layers = 2, experts = 3, sector = 4096; const uint64_t payload = 8192;
    std::vector<uint8_t> idx(12 + 4 + 4 + 4 + 8 + layers * experts * 16);
    memcpy(idx.data(), "AEON_EXPERTS", 12);   // whatever the magic is, mutations cover the rest
    uint32_t v = 2; memcpy(&idx[12], &v, 4); memcpy(&idx[16], &layers, 4); memcpy(&idx[20], &experts, 4);
    memcpy(&idx[24], &payload, 8);
    for (uint32_t i = 0; i < layers * experts; ++i) {
        uint64_t off = uint64_t(i) * payload, len = payload;
        memcpy(&idx[32 + i * 16], &off, 8); memcpy(&idx[40 + i * 16], &len, 8);
    }
    std::vector<uint8_t> blob(layers * experts * payload, 7);
    const std::string dir = "/tmp/aeon_fuzz_" + std::to_string(getpid());
    std::string ip = dir + ".index", bp = dir + ".aeon";
    write_file(bp, blob);
    std::mt19937_64 rng(1);
    int opened = 0, rejected = 0;
    for (int iter = 0; iter < mutations; ++iter) {
        std::vector<uint8_t> m = idx;
        const int kind = iter % 5;
        if (kind == 0) { for (int k = 0; k < 1 + int(rng() % 4); ++k) m[rng() % m.size()] = uint8_t(rng()); }
        else if (kind == 1) { m.resize(rng() % (m.size() + 1)); }
        else if (kind == 2) { uint64_t x = rng(); memcpy(&m[32 + (rng() % (layers * experts)) * 16 + 8 * (rng() % 2)], &x, 8); }
        else if (kind == 3) { uint32_t x = uint32_t(rng()); memcpy(&m[12 + 4 * (rng() % 3)], &x, 4); }
        else { uint64_t x = rng() >> (rng() % 64); memcpy(&m[24], &x, 8); }
        write_file(ip, m);
        aeon_expert_catalog* c = nullptr;
        const int rc = aeon_expert_catalog_open(ip.c_str(), bp.c_str(), 2, sector, &c);
        if (rc == AEON_OK && c) {
            ++opened;
            uint32_t L, E, ver; uint64_t pb;
            aeon_expert_catalog_info(c, &L, &E, &pb, &ver);
            for (uint32_t l = 0; l < L && l < 4; ++l)
                for (uint32_t e = 0; e < E && e < 4; ++e) {
                    const void* p = nullptr; uint64_t n = 0;
                    if (aeon_expert_catalog_payload(c, l, e, &p, &n) == AEON_OK && n) {
                        volatile uint8_t a = static_cast<const uint8_t*>(p)[0], b = static_cast<const uint8_t*>(p)[n - 1];
                        (void)a; (void)b;
                    }
                }
            const void* p; uint64_t n;
            aeon_expert_catalog_payload(c, L, 0, &p, &n);
            aeon_expert_catalog_close(c);
        } else { ++rejected; }
    }
    unlink(ip.c_str()); unlink(bp.c_str());
    printf("opened %d rejected %d\n", opened, rejected);
    return 0;
}
