// Index arithmetic of the packed block format, usable from device code and from a plain host build (the host
// build runs it under AddressSanitizer / UBSan against exactly sized buffers: tests/host_check/).
//
// A row holds 64 pair codes (128 values) in 4*BITS dwords; pair = lo | hi << BITS.
// The row is four groups of 16 pairs; a group owns BITS dwords and dword j of group g
// is row dword 4j + g, so 16-byte chunk j of the row holds dword j of the four groups.
// Inside a group, pair k sits in
//   BITS 4: byte k%4 of dword k/4
//   BITS 2: nibble k%8 of dword k/8
//   BITS 3: bits 6*(k%4).. of dword k/4 for k < 12; pairs 12..15 form a 24-bit tail
//           (pair k at tail bit 6*(k-12)) whose byte j is the top byte of dword j
// Pairs 2q, 2q+1 ("quad" q, four values) are contiguous bits in every width, so a
// reader can index a table by a whole quad with one field extract.
// A block is 128 rows stored chunk-major [BITS][128][16 B] followed by 128 fp16
// norms.  K rows: row = token, pair p = dims (2p, 2p+1).  V rows are dim-major
// inside each 64-token tile: row (token & 64) | (dim & 63) holds dims r and 64+r
// of the tile's tokens; with tp = (token & 63) / 2 and hf = dim >> 6, tokens 2tp,
// 2tp+1 are pair 4*(tp/2) + 2*hf + tp%2, so a quad is four consecutive tokens of
// one dim.
#pragma once
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define TQ_HD __host__ __device__
#else
#define TQ_HD
#endif

#ifndef TQ_ROWS_PER_BLOCK
#define TQ_ROWS_PER_BLOCK 128
#endif
#ifndef TQ_KIND_K_VALUE
#define TQ_KIND_K_VALUE 0  // == TQ_KIND_K of tq.h
#endif

namespace tqd {

TQ_HD constexpr int row_dwords(int bits) { return 4 * bits; }
TQ_HD constexpr int block_bytes(int bits) { return TQ_ROWS_PER_BLOCK * (16 * bits + 2); }
TQ_HD constexpr int block_code_bytes(int bits) { return TQ_ROWS_PER_BLOCK * 16 * bits; }

// pairs per dword (BITS 3: of the 12 pairs outside the tail)
TQ_HD constexpr int pairs_per_dword(int bits) { return bits == 2 ? 8 : 4; }
// true for the four pairs of a 3-bit group that live in the split tail
TQ_HD constexpr bool pair_in_tail(int bits, int p) { return bits == 3 && (p & 15) >= 12; }
// row dword and bit position of pair p (not for tail pairs)
TQ_HD constexpr int pair_dword(int bits, int p) { return 4 * ((p & 15) / pairs_per_dword(bits)) + (p >> 4); }
TQ_HD constexpr int pair_shift(int bits, int p) { return 2 * bits * ((p & 15) % pairs_per_dword(bits)); }

// (row, pair, half) of the code of (token, dim) inside its 128-token block
TQ_HD inline void locate(int kind, int token, int dim, int &row, int &pair, int &half) {
    if (kind == TQ_KIND_K_VALUE) {
        row = token;
        pair = dim >> 1;
        half = dim & 1;
    } else {
        row = (token & 64) | (dim & 63);
        pair = ((token & 60) | ((dim >> 6) << 1)) | ((token >> 1) & 1);
        half = token & 1;
    }
}

// byte offset inside the block of dword q of a row (blocks are chunk-major)
TQ_HD constexpr int row_dword_offset(int row, int q) { return (q >> 2) * 2048 + row * 16 + (q & 3) * 4; }

TQ_HD inline uint32_t row_dword(const uint8_t *block, int row, int q) {
    uint32_t v;
    memcpy(&v, block + row_dword_offset(row, q), 4);
    return v;
}

// codebook index of (token, dim) of a packed block
TQ_HD inline uint32_t fetch_code(const uint8_t *block, int bits, int kind, int token, int dim) {
    int row = 0, p = 0, half = 0;
    locate(kind, token, dim, row, p, half);
    uint32_t pc;
    if (pair_in_tail(bits, p)) {
        const int g = p >> 4;
        const uint32_t tail = (row_dword(block, row, g) >> 24) | ((row_dword(block, row, 4 + g) >> 24) << 8) |
                              ((row_dword(block, row, 8 + g) >> 24) << 16);
        pc = (tail >> (6 * ((p & 15) - 12))) & 63u;
    } else {
        pc = (row_dword(block, row, pair_dword(bits, p)) >> pair_shift(bits, p)) & ((1u << (2 * bits)) - 1u);
    }
    return (pc >> (half * bits)) & ((1u << bits) - 1u);
}

// the inverse: or the codebook index of (token, dim) into a block whose bits at that position are zero
// (single-threaded use: host checks and one-off writers, not the store kernels)
TQ_HD inline void put_code(uint8_t *block, int bits, int kind, int token, int dim, uint32_t code) {
    int row = 0, p = 0, half = 0;
    locate(kind, token, dim, row, p, half);
    const uint32_t field = (code & ((1u << bits) - 1u)) << (half * bits);   // inside the 2*bits-wide pair code
    if (pair_in_tail(bits, p)) {
        const int g = p >> 4;
        const uint32_t tail = field << (6 * ((p & 15) - 12));               // 24-bit tail, byte j rides on dword 4j + g
        for (int j = 0; j < 3; ++j) {
            uint32_t v = row_dword(block, row, 4 * j + g);
            v |= ((tail >> (8 * j)) & 0xFFu) << 24;
            memcpy(block + row_dword_offset(row, 4 * j + g), &v, 4);
        }
    } else {
        uint32_t v = row_dword(block, row, pair_dword(bits, p));
        v |= field << pair_shift(bits, p);
        memcpy(block + row_dword_offset(row, pair_dword(bits, p)), &v, 4);
    }
}

// byte offset of token's fp16 norm inside the block
TQ_HD constexpr int norm_offset(int bits, int token) { return block_code_bytes(bits) + 2 * token; }

// Division of a 32-bit unit or block number by a divisor fixed at launch (blocks per sequence): a multiply-high,
// a subtraction, two shifts and an addition instead of the instruction sequence of a 32-bit division.  Exact for every
// n < 2^32 and 1 <= d <= 2^31 (round-up method: s = ceil(log2 d), m = floor(2^32 (2^s - d) / d) + 1,
// q = (t + ((n - t) >> min(s, 1))) >> (s - min(s, 1)) with t = high word of n m).
struct FastDiv {
    uint32_t d, m, s1, s2;
    TQ_HD uint32_t div(uint32_t n) const {
        const uint32_t t = (uint32_t)(((uint64_t)n * m) >> 32);
        return (t + ((n - t) >> s1)) >> s2;
    }
};
inline FastDiv make_fast_div(uint32_t d) {
    FastDiv f;
    d = d ? d : 1u;  // an empty launch divides nothing
    f.d = d;
    uint32_t s = 0;
    while ((1ull << s) < d) ++s;
    f.m = (uint32_t)((((1ull << s) - d) << 32) / d + 1);
    f.s1 = s < 1u ? s : 1u;
    f.s2 = s - f.s1;
    return f;
}

}  // namespace tqd
