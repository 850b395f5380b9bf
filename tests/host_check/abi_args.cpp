// Argument paths of the C ABI (include/tq.h) under AddressSanitizer / UBSan: every entry point is called with
// null pointers, negative sizes, bad enums and misaligned pointers and must return its error code without
// touching memory.  Built against a host-sanitised capi.o (tests/test_host_sanitize.py); runs with or without a
// GPU, since every case is rejected before any device work.
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "tq.h"

static int fails = 0;
#define EXPECT(cond)                                              \
    do {                                                          \
        if (!(cond)) {                                            \
            printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); \
            ++fails;                                              \
        }                                                         \
    } while (0)

int main() {
    alignas(16) static unsigned char buf[64];
    void *ok = buf, *odd = buf + 1;
    tq_handle *h = nullptr;

    EXPECT(tq_version() >= 100);
    if (tq_device_count() > 0) {
        // Every case below is meant to be refused before any device work; on a machine with a GPU a case that
        // slipped through would hand host pointers to a kernel, so the check only runs where no GPU is visible.
        printf("abi argument paths ok (skipped: a GPU is visible)\n");
        return 0;
    }
    EXPECT(tq_create(nullptr, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_create(&h, nullptr) == TQ_ERR_ARG && h == nullptr);
    double cent[2] = {-1.0, 1.0};
    tq_config cfg;
    memset(&cfg, 0, sizeof cfg);
    cfg.centroids = cent;
    cfg.d = 0; cfg.bits = 1;
    EXPECT(tq_create(&h, &cfg) == TQ_ERR_UNSUPPORTED);
    cfg.d = 8192;
    EXPECT(tq_create(&h, &cfg) == TQ_ERR_UNSUPPORTED);
    cfg.d = 128; cfg.bits = 9;
    EXPECT(tq_create(&h, &cfg) == TQ_ERR_ARG);
    cfg.bits = 1; cfg.rotation = TQ_ROT_WHT;      // sign tables missing
    EXPECT(tq_create(&h, &cfg) == TQ_ERR_ARG);
    cfg.rotation = 7;
    EXPECT(tq_create(&h, &cfg) == TQ_ERR_ARG);
    EXPECT(strlen(tq_last_error()) > 0);
    tq_destroy(nullptr);

    EXPECT(tq_fwht(nullptr, nullptr, 1, 8, TQ_F64, TQ_F64, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_fwht(ok, ok, 1, 12, TQ_F64, TQ_F64, nullptr) != TQ_OK);      // not a power of two
    EXPECT(tq_fwht(ok, ok, -1, 8, TQ_F64, TQ_F64, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_rotate(nullptr, ok, ok, 1, TQ_F32, TQ_F32, 0, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_nearest_centroid(nullptr, 1, cent, 2, nullptr, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_nearest_centroid((const double *)ok, 1, cent, 300, (int32_t *)ok, nullptr) == TQ_ERR_UNSUPPORTED);
    EXPECT(tq_quantize_indices(nullptr, ok, 1, TQ_F64, buf, (double *)ok, nullptr, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_dequantize_indices(nullptr, buf, (const double *)ok, 1, (double *)ok, nullptr, 0, nullptr, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_qjl_quantize(nullptr, ok, 1, TQ_F64, (int8_t *)ok, (double *)ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_qjl_dequantize(nullptr, (const int8_t *)ok, (const double *)ok, 1.0, 1, (double *)ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_pack_bits(nullptr, 1, 128, nullptr, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_pack_bits((const int8_t *)ok, -1, 128, buf, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_unpack_bits(nullptr, 1, 128, nullptr, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_pack_indices(buf, 4, 0, buf, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_pack_indices(buf, 4, 9, buf, nullptr) == TQ_ERR_ARG);

    EXPECT(tq_packed_bytes(3, 2, 129) == 2 * 2 * 128 * 50);
    EXPECT(tq_packed_bytes(5, 1, 1) < 0);
    EXPECT(tq_packed_bytes(3, -1, 1) < 0);
    EXPECT(tq_q8_0_bytes(1, 1) == 128 * 136);
    EXPECT(tq_q8_0_bytes(-1, 1) < 0);
    EXPECT(tq_fork_block_bytes(3) == 50 && tq_fork_block_bytes(4) == 68 && tq_fork_block_bytes(2) == 34 && tq_fork_block_bytes(5) < 0);

    EXPECT(tq_store(nullptr, ok, 1, 1, TQ_F16, TQ_KIND_K, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_store_kv(nullptr, nullptr, ok, ok, 1, 1, TQ_F16, ok, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_append(nullptr, ok, 1, 0, 1, 128, TQ_F16, TQ_KIND_K, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_append_kv(nullptr, nullptr, ok, ok, 1, 0, 1, 128, TQ_F16, ok, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_requantize(nullptr, nullptr, ok, 1, 1, TQ_KIND_K, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_export_fork_blocks(nullptr, ok, 1, 1, TQ_KIND_K, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_import_fork_blocks(nullptr, ok, 1, 1, TQ_KIND_K, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_load(nullptr, ok, 1, 1, TQ_KIND_K, ok, TQ_F32, TQ_DOMAIN_ORIGINAL, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_load_kv(nullptr, nullptr, ok, ok, 1, 1, ok, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_unpack_codes(nullptr, ok, 1, 1, TQ_KIND_K, buf, (float *)ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_store_qjl(nullptr, ok, 1, 1, TQ_F32, ok, buf, ok, nullptr) == TQ_ERR_ARG);

    EXPECT(tq_q8_0_store(nullptr, 1, 1, TQ_F16, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_q8_0_store(ok, 1, 1, 9, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_q8_0_store(odd, 1, 1, TQ_F16, ok, nullptr) == TQ_ERR_ALIGN);
    EXPECT(tq_q8_0_store_v(nullptr, 1, 1, TQ_F16, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_q8_0_unpack(nullptr, 1, 1, (int8_t *)ok, (float *)ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_q8_0_unpack_v(nullptr, 1, 1, (int8_t *)ok, (float *)ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_q8_0_append(nullptr, 1, 0, 1, 128, TQ_F16, TQ_KIND_K, ok, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_q8_0_append(ok, 1, 127, 2, 128, TQ_F16, TQ_KIND_K, ok, nullptr) == TQ_ERR_ARG);   // past the capacity
    // appends at a position in device memory: null position, misaligned position or overrun word, too many tokens
    EXPECT(tq_q8_0_append_at(ok, 1, nullptr, 1, 128, TQ_F16, TQ_KIND_K, ok, nullptr, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_q8_0_append_at(ok, 1, (const int64_t *)odd, 1, 128, TQ_F16, TQ_KIND_K, ok, nullptr, nullptr) == TQ_ERR_ALIGN);
    EXPECT(tq_q8_0_append_at(ok, 1, (const int64_t *)ok, 1, 128, TQ_F16, TQ_KIND_K, ok, (uint32_t *)odd, nullptr) == TQ_ERR_ALIGN);
    EXPECT(tq_q8_0_append_at(ok, 1, (const int64_t *)ok, 129, 128, TQ_F16, TQ_KIND_K, ok, nullptr, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_append_at(nullptr, ok, 1, (const int64_t *)ok, 1, 128, TQ_F16, TQ_KIND_K, ok, nullptr, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_append_kv_at(nullptr, nullptr, ok, ok, 1, (const int64_t *)ok, 1, 128, TQ_F16, ok, ok, nullptr, nullptr) == TQ_ERR_ARG);

    tq_attn_params p;
    memset(&p, 0, sizeof p);
    EXPECT(tq_attn_workspace_bytes(nullptr) < 0);
    EXPECT(tq_attn_workspace_bytes(&p) < 0);                 // sizes must be positive
    p.batch = 1; p.n_q_heads = 7; p.n_kv_heads = 2; p.tokens = 128; p.n_splits = 1; p.scale = 0.1f;
    EXPECT(tq_attn_workspace_bytes(&p) < 0);                 // ragged GQA group
    p.n_q_heads = 8;
    EXPECT(tq_attn_workspace_bytes(&p) > 0);
    p.k_format = 5;
    EXPECT(tq_decode_attention(nullptr, nullptr, &p, ok, TQ_F16, ok, nullptr, ok, nullptr, (float *)ok, nullptr, ok, 64, nullptr) == TQ_ERR_ARG);
    p.k_format = TQ_KFMT_Q8_0; p.v_format = TQ_KFMT_Q8_0;
    EXPECT(tq_decode_attention(nullptr, nullptr, &p, nullptr, TQ_F16, ok, nullptr, ok, nullptr, (float *)ok, nullptr, ok, 64, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_decode_attention(nullptr, nullptr, &p, ok, TQ_F16, odd, nullptr, ok, nullptr, (float *)ok, nullptr, ok, 64, nullptr) == TQ_ERR_ALIGN);
    EXPECT(tq_decode_attention(nullptr, nullptr, &p, ok, TQ_F16, ok, nullptr, ok, nullptr, (float *)ok, nullptr, ok, 64, nullptr) == TQ_ERR_ARG);  // workspace too small
    p.capacity = 64;                                         // capacity below tokens
    EXPECT(tq_decode_attention_static(nullptr, nullptr, &p, ok, TQ_F16, ok, ok, nullptr, (float *)ok, nullptr, nullptr) == TQ_ERR_ARG);
    p.capacity = 0; p.batch = 4096; p.n_q_heads = 8; p.n_kv_heads = 8; p.n_splits = 64;
    EXPECT(tq_decode_attention_static(nullptr, nullptr, &p, ok, TQ_F16, ok, ok, nullptr, (float *)ok, nullptr, nullptr) == TQ_ERR_UNSUPPORTED);
    p.k_format = TQ_KFMT_TURBO;                              // turbo K needs a handle
    EXPECT(tq_decode_attention_static(nullptr, nullptr, &p, ok, TQ_F16, ok, ok, nullptr, (float *)ok, nullptr, nullptr) == TQ_ERR_ARG);
    EXPECT(tq_score_tile(nullptr, ok, TQ_F16, 1, ok, buf, ok, 1, ok, TQ_F32, ok, 64, nullptr) == TQ_ERR_ARG);

    if (fails) {
        printf("%d checks failed\n", fails);
        return 1;
    }
    printf("abi argument paths ok\n");
    return 0;
}
