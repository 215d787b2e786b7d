/* A plain C client of include/zyx_hip.h: what a cgo / libloading / JNI binding sees. Built by the tests with
 * `gcc -std=c99` (the header must be valid C) and linked against libzyx_hip.so.
 *   client layout   prints sizeof / offsetof of every struct of the ABI (compared with the Python mirror)
 *   client softmax  runs config 2's fused kernel on a small tensor through the C ABI only and checks it
 *                   against a straightforward C restatement (needs a GPU) */
#include "zyx_hip.h"

#include <math.h>
#include <stddef.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define CHECK(call)                                                                              \
    do {                                                                                         \
        int32_t rc_ = (call);                                                                    \
        if (rc_ != ZHIP_OK) {                                                                    \
            fprintf(stderr, "%s -> status %d: %s\n", #call, (int)rc_, zhip_last_error(ctx));    \
            return 1;                                                                            \
        }                                                                                        \
    } while (0)

static int layout(void) {
    printf("zhip_kernel_desc %zu kind %zu dtype %zu out_dtype %zu flags %zu dims %zu fparams %zu iparams %zu\n",
           sizeof(zhip_kernel_desc), offsetof(zhip_kernel_desc, kind), offsetof(zhip_kernel_desc, dtype),
           offsetof(zhip_kernel_desc, out_dtype), offsetof(zhip_kernel_desc, flags), offsetof(zhip_kernel_desc, dims),
           offsetof(zhip_kernel_desc, fparams), offsetof(zhip_kernel_desc, iparams));
    printf("zhip_config %zu device_id %zu debug %zu cache_bytes %zu\n", sizeof(zhip_config), offsetof(zhip_config, device_id),
           offsetof(zhip_config, debug), offsetof(zhip_config, cache_bytes));
    printf("zhip_device_info %zu\n", sizeof(zhip_device_info));
    printf("kinds %d %d %d %d %d %d %d %d %d %d %d %d\n", ZHIP_K_SOFTMAX_ROWS, ZHIP_K_ELEMENTWISE, ZHIP_K_REDUCE, ZHIP_K_GEMM,
           ZHIP_K_NORM_ROWS, ZHIP_K_CROSS_ENTROPY, ZHIP_K_CONV2D, ZHIP_K_MAX_POOL2D, ZHIP_K_INDEX, ZHIP_K_ATTENTION,
           ZHIP_K_ATTENTION_BWD, ZHIP_K_NORM_ROWS_BWD);
    printf("zhip_ir_op %zu id %zu opcode %zu dtype %zu a %zu b %zu c %zu aux %zu imm %zu\n", sizeof(zhip_ir_op), offsetof(zhip_ir_op, id),
           offsetof(zhip_ir_op, opcode), offsetof(zhip_ir_op, dtype), offsetof(zhip_ir_op, a), offsetof(zhip_ir_op, b),
           offsetof(zhip_ir_op, c), offsetof(zhip_ir_op, aux), offsetof(zhip_ir_op, imm));
    printf("ir %zu %u %d %d %d %d %d %d\n", sizeof(zhip_ir_header), ZHIP_IR_MAGIC, ZHIP_IR_BARRIER, ZHIP_IR_REDUCE, ZHIP_IR_ABS, ZHIP_IR_EQ,
           ZHIP_IR_GLOBAL_MUT, ZHIP_IR_SCOPE_REGISTER);
    printf("zhip_ceilings %zu memcpy_d2d_GBps %zu read_kernel_GBps %zu mfma_bf16_const_TFLOPs %zu mfma_bf16_random_launch_us %zu\n",
           sizeof(zhip_ceilings), offsetof(zhip_ceilings, memcpy_d2d_GBps), offsetof(zhip_ceilings, read_kernel_GBps),
           offsetof(zhip_ceilings, mfma_bf16_const_TFLOPs), offsetof(zhip_ceilings, mfma_bf16_random_launch_us));
    printf("zhip_rng %zu kinds %d %d %d %d argmax %d ce_dense %d\n", sizeof(zhip_rng), ZHIP_RNG_RAND, ZHIP_RNG_UNIFORM, ZHIP_RNG_RANDN,
           ZHIP_RNG_RANDINT, ZHIP_K_ARGMAX, ZHIP_CE_DENSE);
    {   /* the generator needs no device: the reference's known answer starts from seed 42069 (zyx/tests/05_misc.rs:768-774) */
        zhip_rng r;
        uint64_t counts[3] = {0, 0, 0};
        zhip_rng_seed(&r, 42069);
        printf("rng %llu\n", (unsigned long long)zhip_rng_next_u64(&r));
        zhip_compile_cache_stats(counts);
        printf("cache %llu %llu %llu\n", (unsigned long long)counts[0], (unsigned long long)counts[1], (unsigned long long)counts[2]);
    }
    return 0;
}

static int softmax(void) {
    enum { ROWS = 64, COLS = 1024 };
    zhip_ctx *ctx = NULL;
    zhip_config cfg;
    memset(&cfg, 0, sizeof cfg);
    int32_t n = 0;
    CHECK(zhip_device_count(&n));
    if (n < 1) {
        fprintf(stderr, "no device\n");
        return 1;
    }
    CHECK(zhip_init(&cfg, &ctx));
    float *x = (float *)malloc(sizeof(float) * ROWS * COLS), *y = (float *)malloc(sizeof(float) * ROWS * COLS);
    float sum[ROWS];
    int32_t arg[ROWS];
    uint32_t s = 12345u;
    for (int i = 0; i < ROWS * COLS; i++) {
        s = s * 1664525u + 1013904223u;
        x[i] = ((float)(s >> 8) / 16777216.0f - 0.5f) * 12.0f;
    }
    zhip_buf bx, by, bs, ba;
    zhip_event e[4], up, done;
    CHECK(zhip_alloc(ctx, sizeof(float) * (ROWS * COLS + 1), &bx, &e[0]));
    CHECK(zhip_alloc(ctx, sizeof(float) * (ROWS * COLS + 1), &by, &e[1]));
    CHECK(zhip_alloc(ctx, sizeof(float) * (ROWS + 1), &bs, &e[2]));
    CHECK(zhip_alloc(ctx, sizeof(int32_t) * (ROWS + 1), &ba, &e[3]));
    CHECK(zhip_h2d(ctx, x, sizeof(float) * ROWS * COLS, bx, &e[0], 1, &up));
    zhip_kernel_desc d;
    memset(&d, 0, sizeof d);
    d.kind = ZHIP_K_SOFTMAX_ROWS;
    d.dtype = d.out_dtype = ZHIP_F32;
    d.flags = ZHIP_SOFTMAX_Y | ZHIP_SOFTMAX_ROWSUM | ZHIP_SOFTMAX_ARGMAX;
    d.dims[0] = ROWS;
    d.dims[1] = COLS;
    zhip_prog prog;
    CHECK(zhip_register_kernel(ctx, &d, &prog));
    zhip_buf args[4] = {bx, by, bs, ba};
    zhip_event waits[4] = {up, e[1], e[2], e[3]};
    CHECK(zhip_launch(ctx, prog, args, 4, waits, 4, &done));
    CHECK(zhip_d2h(ctx, by, y, sizeof(float) * ROWS * COLS, &done, 1));
    CHECK(zhip_d2h(ctx, bs, sum, sizeof(float) * ROWS, NULL, 0));
    CHECK(zhip_d2h(ctx, ba, arg, sizeof(int32_t) * ROWS, NULL, 0));
    int bad = 0;
    for (int r = 0; r < ROWS; r++) {
        double m = x[r * COLS], z = 0.0;
        int am = 0;
        for (int c = 1; c < COLS; c++)
            if (x[r * COLS + c] > m) m = x[r * COLS + c];
        for (int c = 0; c < COLS; c++) z += exp((double)x[r * COLS + c] - m);
        for (int c = 0; c < COLS; c++) {
            double want = exp((double)x[r * COLS + c] - m) / z;
            if (fabs(y[r * COLS + c] - want) > 1e-5 * want + 1e-12) bad++;
            if (x[r * COLS + c] >= x[r * COLS + am]) am = c; /* ties: the largest index */
        }
        if (fabs(sum[r] - 1.0) > 1e-5 || arg[r] != am) bad++;
    }
    /* a wrong argument count is reported, not executed */
    zhip_event ev2;
    int32_t rc = zhip_launch(ctx, prog, args, 3, NULL, 0, &ev2);
    if (rc != ZHIP_INCORRECT_KERNEL_ARG) bad++;
    CHECK(zhip_release_program(ctx, prog));
    CHECK(zhip_free(ctx, bx, NULL, 0));
    CHECK(zhip_free(ctx, by, NULL, 0));
    CHECK(zhip_free(ctx, bs, NULL, 0));
    CHECK(zhip_free(ctx, ba, NULL, 0));
    CHECK(zhip_deinit(ctx));
    free(x);
    free(y);
    printf("softmax through the C ABI: %s\n", bad ? "MISMATCH" : "ok");
    return bad != 0;
}

int main(int argc, char **argv) {
    if (argc > 1 && strcmp(argv[1], "layout") == 0) return layout();
    if (argc > 1 && strcmp(argv[1], "softmax") == 0) return softmax();
    fprintf(stderr, "usage: client layout | softmax\n");
    return 2;
}
