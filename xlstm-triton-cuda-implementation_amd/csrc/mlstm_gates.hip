// Gate pre-pass of the matmul form and of the scan form: everything that depends only on (f, i).
//
// Reference semantics: logsigmoid + cumulative sum of the forget gate and the row maximum of the log-decay
// matrix (mlstm_matmul.py:57-59,73-84; mlstm_scan.py:48-69 computes the same m by a max-plus scan).
//
// With lf = logsigmoid(f), Fc = cumsum(lf), a_j = i_j - Fc_j and A_i = max_{j<=i} a_j the stabilised decay is
//     D_ij - m_i = a_j - A_i,        m_i = Fc_i + A_i,
// so the row maximum is a prefix maximum and the tile kernels need no online rescaling.  Fc grows to 1e3..1e4
// in magnitude, so it is never stored in fp32: each 64-position granule g keeps an fp64 base G_g (Fc before the
// granule) and positions store granule-relative values
//     alpha_j = i_j - (Fc_j - G_g(j)),     beta_i = A_i + G_g(i),
// whence  a_j - A_i = alpha_j - beta_i + (G_g(i) - G_g(j))  with one fp64 subtraction per tile pair.
// alpha, beta and G are stored pre-multiplied by log2(e) (the kernels use exp2); m in natural units.
// alpha and beta have a row stride of ceil(S/64)*64 per head (padded to whole granules).
#include "mlstm_device.h"
#include "mlstm_kernels.h"

namespace mlstm {

constexpr int GATES_MAX_GRANULES = 2048;  // S <= 131072

// fp64 prefix over granules by the first wave, 64 granules at a time: exclusive sum G of the totals (sT), then the running
// maximum R of (P - G) over EARLIER granules (sP), by log-step lane shuffles (a serial loop of one lane costs a dependent
// LDS round trip per granule)
__device__ __forceinline__ void granule_prefix(double* sT, double* sP, int NG, int wave, int lane) {
    if (wave == 0) {
        double run = 0.0, rmax = -INFINITY;
        for (int g0 = 0; g0 < NG; g0 += 64) {
            const int g = g0 + lane;
            const double tot = g < NG ? sT[g] : 0.0, p = g < NG ? sP[g] : -INFINITY;
            double incl = tot;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const double up = __shfl_up(incl, d);
                if (lane >= d) incl += up;
            }
            const double excl = run + (incl - tot);       // G of this granule
            double mx = p - excl;                          // this granule's candidate for later granules
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const double up = __shfl_up(mx, d);
                if (lane >= d) mx = fmax(mx, up);
            }
            double before = __shfl_up(mx, 1);              // maximum over earlier granules of this chunk
            if (lane == 0) before = -INFINITY;
            if (g < NG) { sT[g] = excl; sP[g] = fmax(rmax, before); }
            run += __shfl(incl, 63);
            rmax = fmax(rmax, __shfl(mx, 63));
        }
    }
}

// per-position outputs of one granule from the in-granule cumulative sum c and alpha (natural units)
__device__ __forceinline__ void gates_outputs(float c, float al, bool ok, double Gg, double Rg, size_t pos, size_t mpos, size_t gidx, int lane,
                                              float* alpha2, float* beta2, double* G2, float* M, float* ek2, float* amax2) {
    const float loc = wave_scan_inclusive<OpMax>(al);
    const float carry = (float)(Rg + Gg);  // max over earlier granules of (alpha_j - G_g(j)) + G_g ; -inf for g == 0
    const float be = fmaxf(loc, carry);
    // alpha2 / beta2 rows are padded to whole granules: alpha = -inf there, so padded keys weigh nothing
    alpha2[pos] = ok ? al * LOG2E : -INFINITY;
    beta2[pos] = ok ? be * LOG2E : 0.0f;
    if (ok) M[mpos] = c + be;
    // Factorised weights for blocks of 32 keys that lie entirely below the diagonal: with c0 the block maximum of
    // alpha, exp2(alpha_j - beta_i + dG) = exp2(alpha_j - c0) * exp2(c0 - beta_i + dG); both factors are <= 1 there,
    // so the product under- or overflows only where the weight itself does.
    float lo, hi;
    wave_half_max(al * LOG2E, lo, hi);
    const float c0 = lane < 32 ? lo : hi;
    ek2[pos] = (ok && c0 > -INFINITY) ? fast_exp2(al * LOG2E - c0) : 0.0f;
    if ((lane & 31) == 0) amax2[gidx * 2 + (lane >> 5)] = c0;
    if (lane == 0) G2[gidx] = Gg * LOG2E_D;
}

// log-sigmoid of the forget gate at position t from what the caller's F holds (see launch_gates): the pre-activation,
// the log-sigmoid itself, or its cumulative sum over the head (then the difference of two neighbours)
template <typename TG>
__device__ __forceinline__ float forget_log(const TG* f, size_t ss, int t, int form) {
    const float x = (float)f[(size_t)t * ss];
    if (form == MLSTM_GATE_RAW) return log_sigmoid(x);
    if (form == MLSTM_GATE_LOGSIGMOID) return x;
    return t > 0 ? x - (float)f[(size_t)(t - 1) * ss] : x;
}

// Sequences of up to 16 * GPW granules (GPW = 4, 8, 16: S <= 16384): every wave keeps its granules' cumulative sums and alphas in registers
// between the two passes, and issues all its loads before the first scan (one memory round trip instead of one per granule
// and pass).
template <typename TG, int GPW>
__global__ __launch_bounds__(1024) void gates_kernel_reg(const TG* __restrict__ F, const TG* __restrict__ I, float* __restrict__ alpha2,
                                                        float* __restrict__ beta2, double* __restrict__ G2, float* __restrict__ M,
                                                        float* __restrict__ ek2, float* __restrict__ amax2, int S, int NG, Lay lg, int form,
                                                        SavedStamp stamp) {
    stamp_apply(stamp, blockIdx.x == 0, threadIdx.x);
    __shared__ double sT[16 * GPW];
    __shared__ double sP[16 * GPW];
    const int bh = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t gs = (size_t)lg.ss;
    const TG* f = F + lg.head(bh);
    const TG* ig = I + lg.head(bh);
    float fv[GPW], iv[GPW], c[GPW], al[GPW];
#pragma unroll
    for (int k = 0; k < GPW; k++) {
        const int t = (wave + 16 * k) * GRAN + lane;
        const bool ok = t < S;
        fv[k] = ok ? forget_log(f, gs, t, form) : 0.0f;
        iv[k] = ok ? (float)ig[(size_t)t * gs] : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < GPW; k++) {
        const int g = wave + 16 * k, t = g * GRAN + lane;
        const bool ok = t < S;
        const float lf = ok ? fv[k] : 0.0f;
        c[k] = wave_scan_inclusive<OpAdd>(lf);
        al[k] = ok ? iv[k] - c[k] : -INFINITY;
        const float p = wave_reduce<OpMax>(al[k]);
        const float tot = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, c[k]), 63));
        if (lane == 0 && g < NG) { sT[g] = (double)tot; sP[g] = (double)p; }
    }
    __syncthreads();
    granule_prefix(sT, sP, NG, wave, lane);
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GPW; k++) {
        const int g = wave + 16 * k, t = g * GRAN + lane;
        if (g < NG)
            gates_outputs(c[k], al[k], t < S, sT[g], sP[g], (size_t)bh * NG * GRAN + t, (size_t)bh * S + t, (size_t)bh * NG + g, lane, alpha2,
                          beta2, G2, M, ek2, amax2);
    }
}

template <typename TG>
__global__ __launch_bounds__(1024) void gates_kernel(const TG* __restrict__ F, const TG* __restrict__ I, float* __restrict__ alpha2,
                                                    float* __restrict__ beta2, double* __restrict__ G2, float* __restrict__ M,
                                                    float* __restrict__ ek2, float* __restrict__ amax2, int S, int NG, Lay lg, int form,
                                                    SavedStamp stamp) {
    stamp_apply(stamp, blockIdx.x == 0, threadIdx.x);
    __shared__ double sT[GATES_MAX_GRANULES];  // granule totals of lf, then exclusive prefix G
    __shared__ double sP[GATES_MAX_GRANULES];  // granule maxima of alpha, then running max R of (P - G) over earlier granules
    const int bh = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const size_t gs = (size_t)lg.ss;
    const TG* f = F + lg.head(bh);
    const TG* ig = I + lg.head(bh);

    // pass 1: per-granule total of lf and maximum of alpha
    for (int g = wave; g < NG; g += 16) {
        int t = g * GRAN + lane;
        bool ok = t < S;
        float lf = ok ? forget_log(f, gs, t, form) : 0.0f;
        float c = wave_scan_inclusive<OpAdd>(lf);
        float al = ok ? (float)ig[(size_t)t * gs] - c : -INFINITY;
        float p = wave_reduce<OpMax>(al);
        float tot = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, c), 63));
        if (lane == 0) { sT[g] = (double)tot; sP[g] = (double)p; }
    }
    __syncthreads();
    granule_prefix(sT, sP, NG, wave, lane);
    __syncthreads();
    // pass 2: per-position outputs
    for (int g = wave; g < NG; g += 16) {
        int t = g * GRAN + lane;
        bool ok = t < S;
        float lf = ok ? forget_log(f, gs, t, form) : 0.0f;
        float c = wave_scan_inclusive<OpAdd>(lf);
        float al = ok ? (float)ig[(size_t)t * gs] - c : -INFINITY;
        gates_outputs(c, al, ok, sT[g], sP[g], (size_t)bh * NG * GRAN + t, (size_t)bh * S + t, (size_t)bh * NG + g, lane, alpha2, beta2, G2, M,
                      ek2, amax2);
    }
}

template <typename TG>
static hipError_t launch_gates_t(const void* F, const void* I, float* alpha2, float* beta2, double* G2, float* M, float* ek2,
                                 float* amax2, int BH, int S, hipStream_t st, const Lay& lg, int form, const SavedStamp& stamp) {
    int NG = (S + GRAN - 1) / GRAN;
    if (NG <= 16 * 4)
        hipLaunchKernelGGL((gates_kernel_reg<TG, 4>), dim3(BH), dim3(1024), 0, st, (const TG*)F, (const TG*)I, alpha2, beta2, G2, M, ek2, amax2, S, NG, lg, form, stamp);
    else if (NG <= 16 * 8)
        hipLaunchKernelGGL((gates_kernel_reg<TG, 8>), dim3(BH), dim3(1024), 0, st, (const TG*)F, (const TG*)I, alpha2, beta2, G2, M, ek2, amax2, S, NG, lg, form, stamp);
    else if (NG <= 16 * 16)
        hipLaunchKernelGGL((gates_kernel_reg<TG, 16>), dim3(BH), dim3(1024), 0, st, (const TG*)F, (const TG*)I, alpha2, beta2, G2, M, ek2, amax2, S, NG, lg, form, stamp);
    else
        hipLaunchKernelGGL(gates_kernel<TG>, dim3(BH), dim3(1024), 0, st, (const TG*)F, (const TG*)I, alpha2, beta2, G2, M, ek2, amax2, S, NG, lg, form, stamp);
    return hipGetLastError();
}

hipError_t launch_gates(int gate_dtype, const void* F, const void* I, float* alpha2, float* beta2, double* G2, float* M, float* ek2,
                        float* amax2, int BH, int S, hipStream_t st, const Lay& lg, int form, const SavedStamp* stamp_in) {
    const SavedStamp stamp = stamp_in ? *stamp_in : SavedStamp{};
    if ((S + GRAN - 1) / GRAN > GATES_MAX_GRANULES) return hipErrorInvalidValue;
    if (form == MLSTM_GATE_CUMSUM && gate_dtype != MLSTM_F32) return hipErrorInvalidValue;   // (16-bit types cannot hold the sum)
    switch (gate_dtype) {
        case MLSTM_F32: return launch_gates_t<float>(F, I, alpha2, beta2, G2, M, ek2, amax2, BH, S, st, lg, form, stamp);
        case MLSTM_F16: return launch_gates_t<_Float16>(F, I, alpha2, beta2, G2, M, ek2, amax2, BH, S, st, lg, form, stamp);
        case MLSTM_BF16: return launch_gates_t<__bf16>(F, I, alpha2, beta2, G2, M, ek2, amax2, BH, S, st, lg, form, stamp);
    }
    return hipErrorInvalidValue;
}

}  // namespace mlstm
