// Small O(S) passes after the tile kernels of the backward (the per-row n, dn, db live in the dQ kernel).
//
//   rowreduce_kernel: x_t = col_t - sum_J rowpart[J][t]  and dI = col  (mlstm_matmul.py:309,316).
//   dfscan_kernel   : dF_t = sigmoid(-f_t) * sum_{s<t} x_s, dF_0 = 0  (mlstm_matmul_kernel_df,
//                     mlstm_matmul.py:320-333): wave64 DPP scans, LDS carry across waves, fp64 carry across blocks.
#include "mlstm_device.h"
#include "mlstm_kernels.h"

namespace mlstm {

// x_t overwrites slice 0 of rowpart.  One workgroup per 64 positions: wave w adds the key tiles J = w, w+4, ... (the
// slices at or below the position's own tile), the four partial sums meet in LDS.
template <typename TG>
__global__ __launch_bounds__(256) void rowreduce_kernel(const float* __restrict__ colsum, float* rowpart, TG* __restrict__ dI,
                                                        int S, int NG, int RS, int chunk_tiles, const float* __restrict__ rowinter, Lay lg,
                                                        SavedStamp stamp) {
    stamp_apply(stamp, blockIdx.x == 0 && blockIdx.y == 0, threadIdx.x);
    __shared__ float part[4][GRAN];
    const int bh = blockIdx.y, g = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = GRAN * g + lane, tc = t < S ? t : S - 1;
    // in chunks the slices hold the key tiles of the position's own chunk only: slice = key tile - first tile of the chunk
    const int j0 = chunk_tiles > 0 ? g / chunk_tiles * chunk_tiles : 0;
    const int joff = RS == NG ? 0 : j0;
    const float* rp = rowpart + (size_t)bh * RS * S + tc;
    float r0 = 0.f, r1 = 0.f, r2 = 0.f, r3 = 0.f;
    int j = j0 + wave;
    for (; j + 12 <= g; j += 16) {  // four independent loads in flight per lane
        r0 += rp[(size_t)(j - joff) * S];
        r1 += rp[(size_t)(j + 4 - joff) * S];
        r2 += rp[(size_t)(j + 8 - joff) * S];
        r3 += rp[(size_t)(j + 12 - joff) * S];
    }
    for (; j <= g; j += 4) r0 += rp[(size_t)(j - joff) * S];
    part[wave][lane] = (r0 + r1) + (r2 + r3);
    __syncthreads();
    if (wave == 0 && t < S) {
        const float col = colsum[(size_t)bh * S + t];
        const float row = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]) + (rowinter ? rowinter[(size_t)bh * S + t] : 0.f);
        rowpart[(size_t)bh * RS * S + t] = col - row;
        dI[lg.head(bh) + (size_t)t * lg.ss] = (TG)col;
    }
}

// The gradient of what the caller's F holds (DfArgs::gate_form) from the running sum excl_t = sum_{s<t} x_s and x_t itself:
// the pre-activation sees it through the log-sigmoid's derivative sigmoid(-f); the log-sigmoid lf_t takes it as it is;
// the cumulative sum Fc (lf_t = Fc_t - Fc_{t-1}) gets excl_t - excl_{t+1} = -x_t, at every position.
__device__ __forceinline__ float forget_grad(int form, float f, float excl, float x, int t) {
    if (form == MLSTM_GATE_CUMSUM) return -x;
    if (t == 0) return 0.f;
    return form == MLSTM_GATE_RAW ? excl / (1.0f + __expf(f)) : excl;
}

// In chunks the running sum is re-anchored at every chunk start: sum_{s<t} (col_s - row_s) is the sum of dD over the pairs
// (i >= t, j < t), and for t = a chunk's first position that is <C~, E> + n~ . g of the two states at the boundary
// (anchor_kernel), free of the rounding the per-position sums of the state parts carry (the states are 16-bit: each
// position's sum is off by some 2^-9 of its size, independently, and a plain running sum would add those up).
template <typename TG>
__global__ __launch_bounds__(1024) void dfscan_kernel(const TG* __restrict__ F, const float* __restrict__ rowpart, TG* __restrict__ dF,
                                                      int S, int RS, int chunk_len, const float* __restrict__ anchor, int n_states, Lay lg,
                                                      int form) {
    __shared__ float wt[2][16];
    const int bh = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float* x = rowpart + (size_t)bh * RS * S;
    double carry = 0.0;
    int par = 0;
    const int step = chunk_len > 0 && chunk_len < 1024 ? chunk_len : 1024;   // (a chunk is a multiple of 128 positions)
    for (int base = 0; base < S; base += step, par ^= 1) {
        if (chunk_len > 0 && base > 0 && base % chunk_len == 0) carry = (double)anchor[(size_t)bh * n_states + base / chunk_len - 1];
        const int t = base + tid;
        const float v = t < S && tid < step ? x[t] : 0.f;
        const float f = t < S ? (float)F[lg.head(bh) + (size_t)t * lg.ss] : 0.f;
        const float incl = wave_scan_inclusive<OpAdd>(v);
        if (lane == 63) wt[par][wave] = incl;
        __syncthreads();  // (the totals alternate between two buffers: one barrier per block of 1024 positions)
        float pre = 0.f, tot = 0.f;
#pragma unroll
        for (int w = 0; w < 16; w++) {
            float s = wt[par][w];
            if (w < wave) pre += s;
            tot += s;
        }
        // A chunk that is scanned in one go and has an anchor behind it: the sum at its end is known, and what the
        // chunk's own (rounded) per-position sums miss of it is spread evenly over its positions
        float bridge = 0.f;
        if (chunk_len > 0 && step == chunk_len && base / chunk_len < n_states)
            bridge = (float)((double)anchor[(size_t)bh * n_states + base / chunk_len] - (carry + (double)tot)) / (float)step;
        if (t < S && tid < step) {
            const float excl = (float)(carry + (double)(pre + (incl - v))) + bridge * (float)tid;
            dF[lg.head(bh) + (size_t)t * lg.ss] = (TG)forget_grad(form, f, excl, v, t);
        }
        carry += (double)tot;
    }
}

// Row reduction and dF scan of a sequence that ran in chunks, in one kernel and one workgroup per (chunk, head): with
// the running sum known at every chunk's first position (the anchors) the chunks are independent of each other, and a
// position has at most chunk_len / 64 row partials.  chunk_len <= 1024.
template <typename TG>
__global__ __launch_bounds__(1024) void dfchunk_kernel(const TG* __restrict__ F, const float* __restrict__ colsum, const float* __restrict__ rowpart,
                                                       const float* __restrict__ rowinter, const float* __restrict__ anchor,
                                                       TG* __restrict__ dF, TG* __restrict__ dI, int S, int RS, int chunk_len, int n_states,
                                                       Lay lg, int form, const float* __restrict__ anchor_part, int anchor_parts,
                                                       const float* __restrict__ va, const float* __restrict__ vb, int D, SavedStamp stamp) {
    __shared__ float wt[16];
    __shared__ float at[2][16];
    const int c = blockIdx.x, bh = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    stamp_apply(stamp, c == 0 && bh == 0, tid);
    // the two anchors of this chunk (its first position, and the next chunk's) from their parts: the partial sums of the
    // matrix states' contraction and the product of the vector states; both states carry the factor 1 / sqrt(D) of the
    // scores, dD has it once
    float a_start = 0.f, a_next = 0.f;
    if (anchor_part) {
#pragma unroll
        for (int w = 0; w < 2; w++) {
            const int cs = c - 1 + w;
            float x = 0.f;
            if (cs >= 0 && cs < n_states) {
                const size_t o = (size_t)bh * n_states + cs;
                if (tid < D) x = va[o * D + tid] * vb[o * D + tid];
                if (tid < anchor_parts) x += anchor_part[o * anchor_parts + tid];
            }
            x = wave_scan_inclusive<OpAdd>(x);
            if (lane == 63) at[w][wave] = x;
        }
    }
    const int t = c * chunk_len + tid;
    const bool live = tid < chunk_len && t < S;
    float v = 0.f, col = 0.f, f = 0.f;
    if (live) {
        const int g = t / GRAN, g0 = c * (chunk_len / GRAN);
        const float* rp = rowpart + (size_t)bh * RS * S + t;     // slice = key tile - first tile of the chunk
        float row = rowinter[(size_t)bh * S + t];
        float part[16];   // (a fixed count, so that the loads leave together: chunk_len <= 1024 is at most 16 slices)
#pragma unroll
        for (int j = 0; j < 16; j++) part[j] = j <= g - g0 ? rp[(size_t)j * S] : 0.f;
#pragma unroll
        for (int j = 0; j < 16; j++) row += part[j];
        col = colsum[(size_t)bh * S + t];
        f = (float)F[lg.head(bh) + (size_t)t * lg.ss];
        v = col - row;
    }
    const float incl = wave_scan_inclusive<OpAdd>(v);
    if (lane == 63) wt[wave] = incl;
    __syncthreads();
    float pre = 0.f, tot = 0.f;
#pragma unroll
    for (int w = 0; w < 16; w++) {
        const float s = wt[w];
        if (w < wave) pre += s;
        tot += s;
    }
    if (anchor_part) {
        const float rs = sqrtf((float)D);
#pragma unroll
        for (int w = 0; w < 16; w++) { a_start += at[0][w]; a_next += at[1][w]; }
        a_start *= rs; a_next *= rs;
    } else {
        a_start = c > 0 ? anchor[(size_t)bh * n_states + c - 1] : 0.f;
        a_next = c < n_states ? anchor[(size_t)bh * n_states + c] : 0.f;
    }
    const float start = c > 0 ? a_start : 0.f;
    // what the chunk's own (rounded) sums miss of the next anchor is spread evenly over its positions
    const float bridge = c < n_states ? (a_next - (start + tot)) / (float)chunk_len : 0.f;
    if (live) {
        const float excl = start + (pre + (incl - v)) + bridge * (float)tid;
        dF[lg.head(bh) + (size_t)t * lg.ss] = (TG)forget_grad(form, f, excl, v, t);
        dI[lg.head(bh) + (size_t)t * lg.ss] = (TG)col;
    }
}

template <typename TG>
static int launch_df_t(const DfArgs& a, hipStream_t st) {
    if (a.chunk_len > 0 && a.chunk_len <= 1024) {
        hipLaunchKernelGGL(dfchunk_kernel<TG>, dim3((a.S + a.chunk_len - 1) / a.chunk_len, a.BH), dim3(1024), 0, st, reinterpret_cast<const TG*>(a.F),
                           a.colsum, a.rowpart, a.rowinter, a.anchor, reinterpret_cast<TG*>(a.dF), reinterpret_cast<TG*>(a.dI), a.S, a.RS,
                           a.chunk_len, a.n_states, a.lg, a.gate_form, a.anchor_part, a.anchor_parts, a.anchor_va, a.anchor_vb, a.D, a.stamp);
        return (int)hipGetLastError();
    }
    if (a.anchor_part) return MLSTM_EINVAL;   // (only the one-kernel form adds the parts up)
    hipLaunchKernelGGL(rowreduce_kernel<TG>, dim3((a.S + GRAN - 1) / GRAN, a.BH), dim3(256), 0, st, a.colsum, const_cast<float*>(a.rowpart),
                       reinterpret_cast<TG*>(a.dI), a.S, a.NG, a.RS, a.chunk_len / GRAN, a.chunk_len > 0 ? a.rowinter : nullptr, a.lg, a.stamp);
    hipLaunchKernelGGL(dfscan_kernel<TG>, dim3(a.BH), dim3(1024), 0, st, reinterpret_cast<const TG*>(a.F), a.rowpart,
                       reinterpret_cast<TG*>(a.dF), a.S, a.RS, a.chunk_len, a.anchor, a.n_states, a.lg, a.gate_form);
    return (int)hipGetLastError();
}

int launch_dfscan_plain(int gate_dtype, const void* F, const float* x, void* dF, int BH, int S, hipStream_t st) {
    if (gate_dtype != MLSTM_F32) return MLSTM_ESHAPE;
    hipLaunchKernelGGL(dfscan_kernel<float>, dim3(BH), dim3(1024), 0, st, reinterpret_cast<const float*>(F), x, reinterpret_cast<float*>(dF), S,
                       1, 0, nullptr, 0, dense_layout(BH, S, 1), MLSTM_GATE_RAW);
    return (int)hipGetLastError();
}

int launch_df(int gate_dtype, const DfArgs& a, hipStream_t st) {
    switch (gate_dtype) {
        case MLSTM_F32: return launch_df_t<float>(a, st);
        case MLSTM_F16: return launch_df_t<_Float16>(a, st);
        case MLSTM_BF16: return launch_df_t<__bf16>(a, st);
    }
    return MLSTM_EINVAL;
}

// Backward of the output gate h_out = silu(o) * h (the gate of mlstm_scan.py:277 applied to the matmul form): with
// s = sigmoid(o),  dh = dh_out * o s  and  d_o = dh_out * h * s (1 + o (1 - s)).  Streams 16 bytes per tensor and lane.
template <typename T>
__global__ __launch_bounds__(256) void gate_backward_kernel(const T* __restrict__ dh_out, const T* __restrict__ o, const T* __restrict__ h,
                                                            T* __restrict__ dh, T* __restrict__ d_o, size_t nvec) {
    constexpr int EPV = 16 / (int)sizeof(T);
    typedef T Vec __attribute__((ext_vector_type(EPV)));
    typedef float FVec __attribute__((ext_vector_type(EPV)));
    for (size_t v = (size_t)blockIdx.x * 256 + threadIdx.x; v < nvec; v += (size_t)gridDim.x * 256) {
        const FVec g = __builtin_convertvector(reinterpret_cast<const Vec*>(dh_out)[v], FVec);
        const FVec ov = __builtin_convertvector(reinterpret_cast<const Vec*>(o)[v], FVec);
        const FVec hv = __builtin_convertvector(reinterpret_cast<const Vec*>(h)[v], FVec);
        FVec a, b;
#pragma unroll
        for (int e = 0; e < EPV; e++) {
            const float s = 1.0f / (1.0f + __expf(-ov[e]));
            a[e] = g[e] * ov[e] * s;
            b[e] = g[e] * hv[e] * s * (1.0f + ov[e] * (1.0f - s));
        }
        reinterpret_cast<Vec*>(dh)[v] = __builtin_convertvector(a, Vec);
        reinterpret_cast<Vec*>(d_o)[v] = __builtin_convertvector(b, Vec);
    }
}

// The same over [BH, S, D] tensors that lie where the caller keeps them: dh_out, o and d_o in layout lx, h in layout lh, dh
// (the library's own) in layout ld; rows of D contiguous elements, 16 bytes per lane.
template <typename T>
__global__ __launch_bounds__(256) void gate_backward_rows_kernel(const T* __restrict__ dh_out, const T* __restrict__ o, const T* __restrict__ h,
                                                                 T* __restrict__ dh, T* __restrict__ d_o, int S, int D, size_t nvec, Lay lx,
                                                                 Lay lh, Lay ld) {
    constexpr int EPV = 16 / (int)sizeof(T);
    typedef T Vec __attribute__((ext_vector_type(EPV)));
    typedef float FVec __attribute__((ext_vector_type(EPV)));
    const int vpr = D / EPV;   // vectors per row
    for (size_t v = (size_t)blockIdx.x * 256 + threadIdx.x; v < nvec; v += (size_t)gridDim.x * 256) {
        const size_t row = v / vpr;
        const int c = (int)(v % vpr) * EPV, bh = (int)(row / S), s = (int)(row % S);
        const size_t ox = lx.head(bh) + (size_t)s * lx.ss + c, oh = lh.head(bh) + (size_t)s * lh.ss + c, od = ld.head(bh) + (size_t)s * ld.ss + c;
        const FVec g = __builtin_convertvector(*reinterpret_cast<const Vec*>(dh_out + ox), FVec);
        const FVec ov = __builtin_convertvector(*reinterpret_cast<const Vec*>(o + ox), FVec);
        const FVec hv = __builtin_convertvector(*reinterpret_cast<const Vec*>(h + oh), FVec);
        FVec a, b;
#pragma unroll
        for (int e = 0; e < EPV; e++) {
            const float sg = 1.0f / (1.0f + __expf(-ov[e]));
            a[e] = g[e] * ov[e] * sg;
            b[e] = g[e] * hv[e] * sg * (1.0f + ov[e] * (1.0f - sg));
        }
        *reinterpret_cast<Vec*>(dh + od) = __builtin_convertvector(a, Vec);
        *reinterpret_cast<Vec*>(d_o + ox) = __builtin_convertvector(b, Vec);
    }
}

template <typename T>
static int launch_gate_backward_rows_t(const void* dh_out, const void* o, const void* h, void* dh, void* d_o, int BH, int S, int D,
                                       const Lay& lx, const Lay& lh, const Lay& ld, hipStream_t st) {
    const size_t nvec = (size_t)BH * S * D / (16 / sizeof(T));
    const size_t want = (nvec + 255) / 256;
    const unsigned blocks = (unsigned)(want < 256 * 16 ? (want ? want : 1) : 256 * 16);
    hipLaunchKernelGGL(gate_backward_rows_kernel<T>, dim3(blocks), dim3(256), 0, st, reinterpret_cast<const T*>(dh_out),
                       reinterpret_cast<const T*>(o), reinterpret_cast<const T*>(h), reinterpret_cast<T*>(dh), reinterpret_cast<T*>(d_o), S, D,
                       nvec, lx, lh, ld);
    return (int)hipGetLastError();
}

int launch_gate_backward_rows(int dtype, const void* dh_out, const void* o, const void* h, void* dh, void* d_o, int BH, int S, int D,
                              const Lay& lx, const Lay& lh, const Lay& ld, hipStream_t st) {
    if (D % 8) return MLSTM_EINVAL;
    switch (dtype) {
        case MLSTM_F32: return launch_gate_backward_rows_t<float>(dh_out, o, h, dh, d_o, BH, S, D, lx, lh, ld, st);
        case MLSTM_F16: return launch_gate_backward_rows_t<_Float16>(dh_out, o, h, dh, d_o, BH, S, D, lx, lh, ld, st);
        case MLSTM_BF16: return launch_gate_backward_rows_t<__bf16>(dh_out, o, h, dh, d_o, BH, S, D, lx, lh, ld, st);
    }
    return MLSTM_EINVAL;
}

template <typename T>
static int launch_gate_backward_t(const void* dh_out, const void* o, const void* h, void* dh, void* d_o, size_t n, hipStream_t st) {
    const size_t nvec = n / (16 / sizeof(T));
    const size_t want = (nvec + 255) / 256;
    const unsigned blocks = (unsigned)(want < 256 * 16 ? (want ? want : 1) : 256 * 16);
    hipLaunchKernelGGL(gate_backward_kernel<T>, dim3(blocks), dim3(256), 0, st, reinterpret_cast<const T*>(dh_out),
                       reinterpret_cast<const T*>(o), reinterpret_cast<const T*>(h), reinterpret_cast<T*>(dh), reinterpret_cast<T*>(d_o), nvec);
    return (int)hipGetLastError();
}

int launch_gate_backward(int dtype, const void* dh_out, const void* o, const void* h, void* dh, void* d_o, size_t n, hipStream_t st) {
    if (n % 8) return MLSTM_EINVAL;
    switch (dtype) {
        case MLSTM_F32: return launch_gate_backward_t<float>(dh_out, o, h, dh, d_o, n, st);
        case MLSTM_F16: return launch_gate_backward_t<_Float16>(dh_out, o, h, dh, d_o, n, st);
        case MLSTM_BF16: return launch_gate_backward_t<__bf16>(dh_out, o, h, dh, d_o, n, st);
    }
    return MLSTM_EINVAL;
}

}  // namespace mlstm
