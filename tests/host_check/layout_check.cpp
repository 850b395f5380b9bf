// Host check of the packed block format's index arithmetic (turboquant_plus_amd/csrc/tq_layout.h, the header
// the kernels use), built with -fsanitize=address,undefined and run against exactly sized heap buffers, so an
// offset or shift that leaves its block or its dword is reported by the sanitizers.
//
// Input file (written by tests/test_host_sanitize.py from the oracle's layout_pack):
//   int32 bits, kind, tokens; uint8 idx[tokens][128]; uint16 norms[tokens]; uint8 packed[n_blocks * block_bytes]
// Checks: fetch_code of every (token, dim) of the oracle's bytes gives idx; put_code of every idx into a zeroed
// buffer plus the norms gives the oracle's bytes back (rows past `tokens` in the last block are the oracle's
// padding and are compared where the oracle left zeros).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "tq_layout.h"

// `layout_check fastdiv`: tqd::FastDiv against the division it replaces, for small divisors exhaustively over a
// range of numerators and for the extreme numerators and divisors.
static int check_fast_div() {
    const uint32_t edge[] = {0u, 1u, 2u, 3u, 127u, 128u, 255u, 65535u, 65536u, 0x7FFFFFFFu, 0x80000000u, 0xFFFFFFFEu, 0xFFFFFFFFu};
    auto one = [](uint32_t n, uint32_t d, const tqd::FastDiv &f) {
        if (f.div(n) != n / d) {
            printf("fastdiv: %u / %u gave %u\n", n, d, f.div(n));
            return 1;
        }
        return 0;
    };
    for (uint32_t d = 1; d <= 4100; ++d) {
        const tqd::FastDiv f = tqd::make_fast_div(d);
        for (uint32_t n = 0; n < 70000; ++n)
            if (one(n, d, f)) return 1;
        for (uint32_t e : edge) {
            if (one(e, d, f)) return 1;
            // numerators next to multiples of d near the top of the range
            const uint32_t q = 0xFFFFFFFFu / d;
            if (one(q * d, d, f) || one(q * d - 1u, d, f) || (q * d + (d - 1u) >= q * d && one(q * d + (d - 1u), d, f))) return 1;
        }
    }
    const uint32_t big[] = {4097u, 65535u, 65536u, 65537u, 1000003u, 0x40000000u, 0x7FFFFFFFu, 0x80000000u};
    for (uint32_t d : big) {
        const tqd::FastDiv f = tqd::make_fast_div(d);
        for (uint32_t e : edge)
            if (one(e, d, f)) return 1;
        for (uint32_t k = 0; k < 100000; ++k)
            if (one(k * 42949u + 7u, d, f)) return 1;
    }
    printf("fastdiv ok\n");
    return 0;
}

int main(int argc, char **argv) {
    if (argc == 2 && strcmp(argv[1], "fastdiv") == 0) return check_fast_div();
    if (argc != 2) return 2;
    FILE *f = fopen(argv[1], "rb");
    if (!f) return 2;
    int32_t hdr[3];
    if (fread(hdr, 4, 3, f) != 3) return 2;
    const int bits = hdr[0], kind = hdr[1], tokens = hdr[2];
    const int n_blocks = (tokens + TQ_ROWS_PER_BLOCK - 1) / TQ_ROWS_PER_BLOCK;
    const size_t bb = (size_t)tqd::block_bytes(bits);
    std::vector<uint8_t> idx((size_t)tokens * 128);
    std::vector<uint16_t> norms(tokens);
    std::vector<uint8_t> want(n_blocks * bb);
    if (fread(idx.data(), 1, idx.size(), f) != idx.size() || fread(norms.data(), 2, norms.size(), f) != norms.size() ||
        fread(want.data(), 1, want.size(), f) != want.size())
        return 2;
    fclose(f);

    // read side: exactly one block at a time on the heap, so that any offset past the block faults
    long bad = 0;
    for (int b = 0; b < n_blocks; ++b) {
        uint8_t *block = (uint8_t *)malloc(bb);
        memcpy(block, want.data() + b * bb, bb);
        for (int t = 0; t < TQ_ROWS_PER_BLOCK && b * TQ_ROWS_PER_BLOCK + t < tokens; ++t) {
            const int tok = b * TQ_ROWS_PER_BLOCK + t;
            for (int d = 0; d < 128; ++d) bad += tqd::fetch_code(block, bits, kind, t, d) != idx[(size_t)tok * 128 + d];
            uint16_t g;
            memcpy(&g, block + tqd::norm_offset(bits, t), 2);
            bad += g != norms[tok];
        }
        free(block);
    }
    if (bad) {
        printf("fetch_code: %ld mismatches\n", bad);
        return 1;
    }
    // write side
    for (int b = 0; b < n_blocks; ++b) {
        uint8_t *block = (uint8_t *)calloc(bb, 1);
        const int nt = tokens - b * TQ_ROWS_PER_BLOCK < TQ_ROWS_PER_BLOCK ? tokens - b * TQ_ROWS_PER_BLOCK : TQ_ROWS_PER_BLOCK;
        for (int t = 0; t < nt; ++t) {
            const int tok = b * TQ_ROWS_PER_BLOCK + t;
            for (int d = 0; d < 128; ++d) tqd::put_code(block, bits, kind, t, d, idx[(size_t)tok * 128 + d]);
            memcpy(block + tqd::norm_offset(bits, t), &norms[tok], 2);
        }
        if (nt == TQ_ROWS_PER_BLOCK) {
            if (memcmp(block, want.data() + b * bb, bb)) bad += 1;
        } else {
            // the oracle fills the rows past the end with the code of 0.0: compare the codes of the tokens that exist
            for (int t = 0; t < nt; ++t)
                for (int d = 0; d < 128; ++d)
                    bad += tqd::fetch_code(block, bits, kind, t, d) != tqd::fetch_code(want.data() + b * bb, bits, kind, t, d);
        }
        free(block);
    }
    if (bad) {
        printf("put_code: %ld mismatching blocks / codes\n", bad);
        return 1;
    }
    printf("layout ok: bits %d kind %d tokens %d\n", bits, kind, tokens);
    return 0;
}
