/*
 * C harness of the single-head fp16 forward: the counterpart of main() in cuda-src/mlstm_forward.cu:192-263.
 * Same order of events: srand(100); fill Q, K, V, F, I with uniform [-1, 1) halves (:210-215); CPU reference (:217);
 * device buffers and host-to-device copies (:219-233); ONE call of the C entry point where the reference launches its
 * kernel (:237-238); synchronise; copy back; the reference's check() printout (cpu_utils.cuh:30-40).
 * Plain C: it also shows that include/mlstm_hip.h compiles, and libmlstm_hip.so links, from C.
 * Usage: mlstm_forward_main [S]   (default S = 64 * 10, the README's shape; the reference's source constant is 64 * 20)
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <hip/hip_runtime_api.h>
#include "mlstm_hip.h"

/* CPU side: the test-suite's C restatement of the reference's CPU path (oracle/mlstm_cpu.c) */
void oracle_srand(unsigned seed);
void oracle_fill_rand_half(uint16_t* A, int size);
int oracle_mlstm_forward_f16(const uint16_t* Q, const uint16_t* K, const uint16_t* V, const uint16_t* F, const uint16_t* I,
                             uint16_t* H, float* M, float* B, unsigned S, unsigned D, int flags, int threads);
unsigned oracle_count_mismatch_f16(const uint16_t* a, const uint16_t* b, int size, float atol);
#define ORACLE_EPS_INSIDE_MAX 1

#define HIP_CHECK(call)                                                                        \
    do {                                                                                       \
        hipError_t e_ = (call);                                                                \
        if (e_ != hipSuccess) {                                                                \
            fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            return 2;                                                                          \
        }                                                                                      \
    } while (0)

static void check(const uint16_t* a, const uint16_t* b, int size) {
    unsigned count = oracle_count_mismatch_f16(a, b, size, 0.01f);
    printf("Non_matching count: %u\n", count);
    printf("Non_matching percent: %g\n", 100.0 * (count / (float)size));
}

int main(int argc, char** argv) {
    const unsigned D = 128;
    const unsigned S = argc > 1 ? (unsigned)atoi(argv[1]) : 64 * 10;
    const size_t n = (size_t)S * D;
    uint16_t *Q = malloc(n * 2), *K = malloc(n * 2), *V = malloc(n * 2), *F = malloc(S * 2), *I = malloc(S * 2), *H = malloc(n * 2);
    float *M = malloc(S * 4), *B = malloc(S * 4);
    oracle_srand(100);
    oracle_fill_rand_half(Q, (int)n);
    oracle_fill_rand_half(K, (int)n);
    oracle_fill_rand_half(V, (int)n);
    oracle_fill_rand_half(F, (int)S);
    oracle_fill_rand_half(I, (int)S);
    if (oracle_mlstm_forward_f16(Q, K, V, F, I, H, M, B, S, D, ORACLE_EPS_INSIDE_MAX, 1)) return 3;

    void *dev_Q, *dev_K, *dev_V, *dev_F, *dev_I, *dev_H;
    HIP_CHECK(hipMalloc(&dev_Q, n * 2));
    HIP_CHECK(hipMalloc(&dev_K, n * 2));
    HIP_CHECK(hipMalloc(&dev_V, n * 2));
    HIP_CHECK(hipMalloc(&dev_F, S * 2));
    HIP_CHECK(hipMalloc(&dev_I, S * 2));
    HIP_CHECK(hipMalloc(&dev_H, n * 2));
    HIP_CHECK(hipMemcpy(dev_Q, Q, n * 2, hipMemcpyHostToDevice));
    HIP_CHECK(hipMemcpy(dev_K, K, n * 2, hipMemcpyHostToDevice));
    HIP_CHECK(hipMemcpy(dev_V, V, n * 2, hipMemcpyHostToDevice));
    HIP_CHECK(hipMemcpy(dev_F, F, S * 2, hipMemcpyHostToDevice));
    HIP_CHECK(hipMemcpy(dev_I, I, S * 2, hipMemcpyHostToDevice));

    const int rc = mlstm_forward(dev_Q, dev_K, dev_V, dev_F, dev_I, dev_H, S);
    if (rc != 0) { fprintf(stderr, "mlstm_forward returned %d\n", rc); return 4; }
    HIP_CHECK(hipDeviceSynchronize());
    HIP_CHECK(hipGetLastError());

    uint16_t* hipH = malloc(n * 2);
    HIP_CHECK(hipMemcpy(hipH, dev_H, n * 2, hipMemcpyDeviceToHost));
    printf("%s, S = %u, D = %u\n", mlstm_version(), S, D);
    printf("Check H \n");
    check(H, hipH, (int)n);

    free(Q); free(K); free(V); free(F); free(I); free(H); free(M); free(B); free(hipH);
    HIP_CHECK(hipFree(dev_Q)); HIP_CHECK(hipFree(dev_K)); HIP_CHECK(hipFree(dev_V));
    HIP_CHECK(hipFree(dev_F)); HIP_CHECK(hipFree(dev_I)); HIP_CHECK(hipFree(dev_H));
    return 0;
}
