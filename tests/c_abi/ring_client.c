/* A client of the C ABI written in plain C: no C++, no Python, no PyTorch.  It registers the
 * per-rank graph files given on the command line (a ring allreduce over as many virtual ranks),
 * runs the operation in place and as a staged call on buffers it allocated with hipMalloc, and
 * checks the closed form of the reference's own correctness test (tests/test_correctness.py:142,
 * 170-171: every element of rank r is r + 1, so every element of the result is R (R + 1) / 2).
 *
 * usage: ring_client <elements per rank> <rank0.json> <rank1.json> ...      (bfloat16 graphs)
 * exit status 0 and a line "ok ..." on success. */
#include <hip/hip_runtime_api.h>
#include <pccl_hip.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define MAX_RANKS 64

static uint16_t bf16_of_small_int(int v) {   /* exact for |v| < 256 */
    float f = (float)v;
    uint32_t u;
    memcpy(&u, &f, 4);
    return (uint16_t)(u >> 16);
}

static int check_hip(hipError_t e, const char* what) {
    if (e != hipSuccess) { fprintf(stderr, "%s: %s\n", what, hipGetErrorString(e)); return 1; }
    return 0;
}

static int check_all(const uint16_t* host, size_t n, uint16_t want, const char* what, int rank) {
    for (size_t i = 0; i < n; ++i)
        if (host[i] != want) {
            fprintf(stderr, "%s: rank %d element %zu is 0x%04x, expected 0x%04x\n", what, rank, i, host[i], want);
            return 1;
        }
    return 0;
}

int main(int argc, char** argv) {
    if (argc < 4) { fprintf(stderr, "usage: %s <elements per rank> <rank0.json> <rank1.json> ...\n", argv[0]); return 2; }
    const size_t n = (size_t)strtoull(argv[1], NULL, 10);
    const int R = argc - 2;
    if (R > MAX_RANKS || n == 0) { fprintf(stderr, "bad arguments\n"); return 2; }
    const size_t bytes = n * sizeof(uint16_t);
    printf("%s\n", pccl_hip_version());

    pccl_hip_ctx* ctx = NULL;
    if (pccl_hip_create(&ctx, 0, R) < 0) { fprintf(stderr, "create: %s\n", pccl_hip_last_error()); return 1; }
    for (int r = 0; r < R; ++r)
        if (pccl_hip_register_file(ctx, "ar", r, argv[2 + r]) < 0) { fprintf(stderr, "register: %s\n", pccl_hip_last_error()); return 1; }

    /* errors come back as codes with a message, never as a crash */
    void* none[MAX_RANKS] = {0};
    if (pccl_hip_execute_inplace(ctx, "no such operation", none, bytes, NULL, 1) != PCCL_ERR_NOT_FOUND) {
        fprintf(stderr, "an unknown operation was not reported as PCCL_ERR_NOT_FOUND\n");
        return 1;
    }
    if (strlen(pccl_hip_last_error()) == 0) { fprintf(stderr, "no error message\n"); return 1; }

    void *in[MAX_RANKS], *out[MAX_RANKS];
    uint16_t* host = (uint16_t*)malloc(bytes);
    if (!host) return 1;
    for (int r = 0; r < R; ++r) {
        if (check_hip(hipMalloc(&in[r], bytes), "hipMalloc") || check_hip(hipMalloc(&out[r], bytes), "hipMalloc")) return 1;
        for (size_t i = 0; i < n; ++i) host[i] = bf16_of_small_int(r + 1);
        if (check_hip(hipMemcpy(in[r], host, bytes, hipMemcpyHostToDevice), "hipMemcpy")) return 1;
        if (check_hip(hipMemset(out[r], 0, bytes), "hipMemset")) return 1;
    }
    const uint16_t want = bf16_of_small_int(R * (R + 1) / 2);
    hipStream_t stream;
    if (check_hip(hipStreamCreate(&stream), "hipStreamCreate")) return 1;

    /* the reference's call shape: separate input and output tensors, inputs left untouched */
    if (pccl_hip_execute(ctx, "ar", (const void* const*)in, out, bytes, bytes, stream, 0) < 0) { fprintf(stderr, "execute: %s\n", pccl_hip_last_error()); return 1; }
    if (pccl_hip_sync(ctx, "ar") < 0) { fprintf(stderr, "sync: %s\n", pccl_hip_last_error()); return 1; }
    for (int r = 0; r < R; ++r) {
        if (check_hip(hipMemcpy(host, out[r], bytes, hipMemcpyDeviceToHost), "hipMemcpy")) return 1;
        if (check_all(host, n, want, "staged call", r)) return 1;
        if (check_hip(hipMemcpy(host, in[r], bytes, hipMemcpyDeviceToHost), "hipMemcpy")) return 1;
        if (check_all(host, n, bf16_of_small_int(r + 1), "staged call, input", r)) return 1;
    }

    /* zero copy: the caller's buffers are the rank buffers; once per runner */
    const char* modes[3] = {"auto", "stepwise", "persistent"};
    for (int m = 0; m < 3; ++m) {
        if (pccl_hip_set_option(ctx, "mode", modes[m]) < 0) { fprintf(stderr, "set_option: %s\n", pccl_hip_last_error()); return 1; }
        for (int r = 0; r < R; ++r) {
            for (size_t i = 0; i < n; ++i) host[i] = bf16_of_small_int(r + 1);
            if (check_hip(hipMemcpy(out[r], host, bytes, hipMemcpyHostToDevice), "hipMemcpy")) return 1;
        }
        if (pccl_hip_execute_inplace(ctx, "ar", out, bytes, stream, 1) < 0) { fprintf(stderr, "execute_inplace (%s): %s\n", modes[m], pccl_hip_last_error()); return 1; }
        for (int r = 0; r < R; ++r) {
            if (check_hip(hipMemcpy(host, out[r], bytes, hipMemcpyDeviceToHost), "hipMemcpy")) return 1;
            if (check_all(host, n, want, modes[m], r)) return 1;
        }
    }

    pccl_program_info info;
    if (pccl_hip_op_info(ctx, "ar", &info) < 0) { fprintf(stderr, "op_info: %s\n", pccl_hip_last_error()); return 1; }
    for (int r = 0; r < R; ++r) { (void)hipFree(in[r]); (void)hipFree(out[r]); }
    (void)hipStreamDestroy(stream);
    free(host);
    pccl_hip_destroy(ctx);
    printf("ok ranks=%d elements=%zu data_ops=%d levels=%d algorithmic_bytes=%lld\n", R, n, info.num_data_ops, info.num_levels,
           (long long)info.algorithmic_bytes);
    return 0;
}
