/*
 * C harness of the single-head fp16 backward: the counterpart of main() in cuda-src/mlstm_backward.cu:561-670.
 * srand(1678); fill dH, Q, K, V, F, I (:580-586); CPU reference; device buffers; ONE call of the C entry point where the
 * reference launches matmul_backward_db and matmul_backward (:620-628); the reference's check() printout for every
 * gradient (the reference stops at dB, dQ, dK: :641-646; dV, dF, dI are checked here as well).  M and B, which the
 * reference uploads from its CPU pass (:618-619), are passed as NULL: the entry point recomputes them.
 * The CPU side uses sign(b) for dB (mlstm_matmul.py:196), not the reference harness' signbit(b) (cpu_utils.cuh:195).
 * Usage: mlstm_backward_main [S]   (default 64 * 10)
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <hip/hip_runtime_api.h>
#include "mlstm_hip.h"

void oracle_srand(unsigned seed);
void oracle_fill_rand_half(uint16_t* A, int size);
int oracle_mlstm_backward_f16(const uint16_t* dH, const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* F,
                              const uint16_t* I, uint16_t* dQ, uint16_t* dK, uint16_t* dV, uint16_t* dF, uint16_t* dI, unsigned S,
                              unsigned D, int flags, int threads);
unsigned oracle_count_mismatch_f16(const uint16_t* a, const uint16_t* b, int size, float atol);

#define HIP_CHECK(call)                                                                        \
    do {                                                                                       \
        hipError_t e_ = (call);                                                                \
        if (e_ != hipSuccess) {                                                                \
            fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            return 2;                                                                          \
        }                                                                                      \
    } while (0)

static void check(const char* name, const uint16_t* a, const uint16_t* b, int size) {
    unsigned count = oracle_count_mismatch_f16(a, b, size, 0.01f);
    printf("Check %s \n", name);
    printf("Non_matching count: %u\n", count);
    printf("Non_matching percent: %g\n", 100.0 * (count / (float)size));
}

int main(int argc, char** argv) {
    const unsigned D = 128;
    const unsigned S = argc > 1 ? (unsigned)atoi(argv[1]) : 64 * 10;
    const size_t n = (size_t)S * D;
    uint16_t *in[6], *ref[5], *got[5];
    void *dev_in[6], *dev_out[5];
    const size_t in_n[6] = {n, n, n, n, S, S}, out_n[5] = {n, n, n, S, S};
    const char* names[5] = {"dQ", "dK", "dV", "dF", "dI"};
    oracle_srand(1678);
    for (int t = 0; t < 6; t++) {   /* dH, Q, K, V, F, I */
        in[t] = malloc(in_n[t] * 2);
        oracle_fill_rand_half(in[t], (int)in_n[t]);
    }
    for (int t = 0; t < 5; t++) { ref[t] = malloc(out_n[t] * 2); got[t] = malloc(out_n[t] * 2); }
    if (oracle_mlstm_backward_f16(in[0], in[1], in[2], in[3], in[4], in[5], ref[0], ref[1], ref[2], ref[3], ref[4], S, D, 0, 1)) return 3;

    for (int t = 0; t < 6; t++) {
        HIP_CHECK(hipMalloc(&dev_in[t], in_n[t] * 2));
        HIP_CHECK(hipMemcpy(dev_in[t], in[t], in_n[t] * 2, hipMemcpyHostToDevice));
    }
    for (int t = 0; t < 5; t++) HIP_CHECK(hipMalloc(&dev_out[t], out_n[t] * 2));

    const int rc = mlstm_backward(dev_in[0], dev_in[1], dev_in[2], dev_in[3], dev_in[4], dev_in[5], NULL, NULL, dev_out[0], dev_out[1],
                                  dev_out[2], dev_out[3], dev_out[4], S);
    if (rc != 0) { fprintf(stderr, "mlstm_backward returned %d\n", rc); return 4; }
    HIP_CHECK(hipDeviceSynchronize());
    HIP_CHECK(hipGetLastError());

    printf("%s, S = %u, D = %u\n", mlstm_version(), S, D);
    for (int t = 0; t < 5; t++) {
        HIP_CHECK(hipMemcpy(got[t], dev_out[t], out_n[t] * 2, hipMemcpyDeviceToHost));
        check(names[t], ref[t], got[t], (int)out_n[t]);
    }
    for (int t = 0; t < 6; t++) { free(in[t]); HIP_CHECK(hipFree(dev_in[t])); }
    for (int t = 0; t < 5; t++) { free(ref[t]); free(got[t]); HIP_CHECK(hipFree(dev_out[t])); }
    return 0;
}
