// sLSTM cell, forward and backward, fp32.  The reference lists the cell as an open item (README.md:9) and holds no code for
// it; this implements the published cell (Beck et al., "xLSTM: Extended Long Short-Term Memory", arXiv:2405.04517,
// section 2.2, with the stabilised exponential gating of appendix A.2), per head (block-diagonal recurrent matrices):
//     i~, f~, z~, o~ = Wx_t[g] + R_g h_{t-1} + b_g
//     m_t  = max(log f_t + m_{t-1}, i~)                 log f_t = f~ (exponential gate) or logsigmoid(f~)
//     i'_t = exp(i~ - m_t),  f'_t = exp(log f_t + m_{t-1} - m_t)
//     c_t  = f'_t c_{t-1} + i'_t tanh(z~),  n_t = f'_t n_{t-1} + i'_t,  h_t = sigmoid(o~) c_t / n_t
// The recurrence through h makes the cell sequential in t, so the kernels are latency machines, not throughput ones: one
// workgroup per (batch, head) walks the sequence with the head's four recurrent matrices in registers.
//   slstm_forward_kernel   four lanes per unit j, each with a quarter of row j of all four R_g: partial pre-activations from
//                          h_{t-1} (LDS), summed over the four lanes; every lane then updates the cell of its unit.
//                          Gate values and (c, n, m) are kept for the backward.
//   slstm_backward_kernel  back through time: rows of 16 lanes form R^T delta_{t+1} for their four units (a sixteenth of the
//                          gradient vector per lane, summed over the row), which is what step t+1 sent back to h_t; every
//                          lane of a unit's quad turns (dh_t + that, dc, dn) into the four pre-activation gradients (= dWx_t).  The stabiliser m is a common scale of c and n that h
//                          does not depend on, so it is held constant.
//   slstm_dr_kernel        dR_g = sum_{b,t} dWx_t[g] h_{t-1}^T and db_g = sum_{b,t} dWx_t[g]: off the sequential path, in
//                          slices of (b, t) whose partial sums a second kernel adds in a fixed order.
// Layouts: wx, dwx [B,S,4,NH,DH] (gates i, f, z, o); r, dr [NH,4,DH,DH] (r[h][g][j][k]: unit j from unit k); b, db [NH,4,DH];
// h, dh [B,S,NH,DH]; saved [B,S,7,NH,DH] (i~, log f, tanh(z~), sigmoid(o~), c, n, m).
#include <hip/hip_runtime.h>
#include <stddef.h>
#include "../../include/mlstm_hip.h"
#include "mlstm_device.h"
#include "mlstm_kernels.h"

namespace slstm {

typedef float f32x4 __attribute__((ext_vector_type(4)));

// The nonlinearities from the hardware's exp2 / reciprocal (a few instructions each, relative error around 1e-6): they sit
// on the critical path of every step of a sequential kernel.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896340736f); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }
__device__ __forceinline__ float sigmoid_fast(float x) { return fast_rcp(1.0f + fast_exp(-x)); }
__device__ __forceinline__ float tanh_fast(float x) {
    const float e = fast_exp(-2.0f * fabsf(x));   // in (0, 1]: no overflow
    const float t = (1.0f - e) * fast_rcp(1.0f + e);
    return x < 0.f ? -t : t;
}
__device__ __forceinline__ float log_sigmoid_fast(float x) {
    // min(x, 0) - log(1 + exp(-|x|)); the log through the hardware log2
    return fminf(x, 0.0f) - __builtin_amdgcn_logf(1.0f + fast_exp(-fabsf(x))) * 0.69314718055994530942f;
}

// Inputs of a step come from memory PF steps ahead of it, as direct-to-LDS loads into a ring (a trip to memory is several
// steps long, and a step must not wait for one).  The loads are issued and waited for by hand: every wave issues the same
// number of memory operations per step, in the same order (OPS: its stores, then its ring loads, none under a branch), so
// "the loads of step t have landed" is a counted wait -- memory operations of a wave complete in the order issued.  The
// kernels' own code has only stores besides, for which the compiler places no waits.  (Left to the compiler, ordinary
// loads into a ring of registers ended in a wait for everything at every step.)  A lane only ever reads ring values that
// its own wave loaded, so the wait needs no barrier behind it.
constexpr int PF = 8;
__device__ __forceinline__ void ring_load(const float* g, unsigned lds_off) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(g), "s"(lds_off) : "memory", "m0");
}
// (n is a constant once the step loops are unrolled; anything out of range waits for everything)
__device__ __forceinline__ void ring_wait(int n) {
    switch (n) {
        case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
        case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
        case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
        case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
        case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
        case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
        case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
        case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
        case 9: asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); break;
        case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
        case 11: asm volatile("s_waitcnt vmcnt(11)" ::: "memory"); break;
        case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
        case 13: asm volatile("s_waitcnt vmcnt(13)" ::: "memory"); break;
        case 14: asm volatile("s_waitcnt vmcnt(14)" ::: "memory"); break;
        case 15: asm volatile("s_waitcnt vmcnt(15)" ::: "memory"); break;
        case 16: asm volatile("s_waitcnt vmcnt(16)" ::: "memory"); break;
        case 17: asm volatile("s_waitcnt vmcnt(17)" ::: "memory"); break;
        case 18: asm volatile("s_waitcnt vmcnt(18)" ::: "memory"); break;
        case 19: asm volatile("s_waitcnt vmcnt(19)" ::: "memory"); break;
        case 20: asm volatile("s_waitcnt vmcnt(20)" ::: "memory"); break;
        case 21: asm volatile("s_waitcnt vmcnt(21)" ::: "memory"); break;
        case 22: asm volatile("s_waitcnt vmcnt(22)" ::: "memory"); break;
        case 23: asm volatile("s_waitcnt vmcnt(23)" ::: "memory"); break;
        case 24: asm volatile("s_waitcnt vmcnt(24)" ::: "memory"); break;
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
}

// Sum over the four lanes of a quad (lanes 4a .. 4a+3), the same bits in all four: two exchanges inside the quad.
template <int CTRL>
__device__ __forceinline__ float quad_perm(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float quad_sum(float x) {
    x += quad_perm<0xB1>(x);   // lanes 1, 0, 3, 2
    x += quad_perm<0x4E>(x);   // lanes 2, 3, 0, 1
    return x;
}
// Sum over the 16 lanes of a row (lanes 16a .. 16a+15), the same bits in all of them: rotations by 8 and 4, then the quad.
__device__ __forceinline__ float row_sum(float x) {
    x += quad_perm<0x128>(x);   // row_ror:8
    x += quad_perm<0x124>(x);   // row_ror:4
    return quad_sum(x);
}
// the value of lane q of a quad (three selects; is0..is2: q == 0, 1, 2)
__device__ __forceinline__ float pick(bool is0, bool is1, bool is2, float a, float b, float c, float d) {
    float x = is2 ? c : d;
    x = is1 ? b : x;
    return is0 ? a : x;
}

// A quad of lanes owns a unit j: lane q of it keeps, for all four gates, the quarter q of row j of R_g, forms its quarter of
// the four pre-activations from its quarter of h_{t-1}, and after the sum over the quad every lane has all four and
// updates the cell, all four alike (c, n, m are kept four times, the same bits).  So a step has no hand-over between
// threads but h itself: one LDS write, one barrier (h in two buffers, taken in turns).  Lane q loads gate q's input of its
// unit into the ring, and stores saved value q and value 4 + q (c, n, m; for q = 3, h itself).
template <int DH, bool SAVE, bool FS>
__global__ __launch_bounds__(4 * DH) void slstm_forward_kernel(const float* __restrict__ wx, const float* __restrict__ r,
                                                               const float* __restrict__ bias, float* __restrict__ h,
                                                               float* __restrict__ saved, int NH, int S) {
    constexpr int KQ = DH / 4;
    __shared__ __attribute__((aligned(16))) float hs[2][DH];
    __shared__ __attribute__((aligned(16))) float ring[PF][4 * DH];   // wx of the next PF steps: [slot][unit * 4 + gate]
    const int tid = threadIdx.x, j = tid >> 2, q = tid & 3, wave = tid >> 6;
    const bool is0 = q == 0, is1 = q == 1, is2 = q == 2;
    const int b = blockIdx.x / NH, hd = blockIdx.x % NH;
    float rr[4][KQ], bq[4];
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const float* src = r + (((size_t)hd * 4 + g) * DH + j) * DH + q * KQ;
#pragma unroll
        for (int k = 0; k < KQ; k += 4) {
            const f32x4 v = *reinterpret_cast<const f32x4*>(src + k);
            rr[g][k] = v[0]; rr[g][k + 1] = v[1]; rr[g][k + 2] = v[2]; rr[g][k + 3] = v[3];
        }
        bq[g] = bias[((size_t)hd * 4 + g) * DH + j];
    }
    const size_t step_wx = (size_t)4 * NH * DH, step_h = (size_t)NH * DH, step_s = (size_t)7 * NH * DH;
    // (pointers that walk with the steps: a lone wave per SIMD pays for every instruction of address arithmetic)
    const float* wnext = wx + (size_t)b * S * step_wx + ((size_t)q * NH + hd) * DH + j;   // the row the ring takes next
    float* own = SAVE ? saved + (size_t)b * S * step_s + ((size_t)q * NH + hd) * DH + j : nullptr;
    float* out2 = q == 3 ? h + (size_t)b * S * step_h + (size_t)hd * DH + j
                         : (SAVE ? saved + (size_t)b * S * step_s + ((size_t)(4 + q) * NH + hd) * DH + j : nullptr);
    const size_t step2 = q == 3 ? step_h : step_s;
    if (tid < DH) hs[0][tid] = 0.f;
    // (the stabiliser starts at -inf rather than the paper's 0: with c_0 = n_0 = 0 it only sets the scale of the first
    // step, and this way the first input gate is exp(0) whatever the first forget gate says)
    float c = 0.f, n = 0.f, m = -INFINITY;
    // Memory operations per wave and step, the same in every wave: two stores (without the saved state one: every wave has
    // lanes with q = 3), then the ring load.
    constexpr int OPS = SAVE ? 3 : 2;
    const unsigned ring_base = __builtin_amdgcn_readfirstlane(mlstm::lds_offset_of(&ring[0][0]) + wave * 256);
#pragma unroll
    for (int u = 0; u < PF; u++) {   // (past the end of the sequence the last row is loaded again)
        ring_load(wnext, ring_base + u * (4 * DH * 4));
        if (u + 1 < S) wnext += step_wx;
    }
    ring_wait(PF - 1);
    f32x4 wv = *reinterpret_cast<const f32x4*>(&ring[0][4 * j]);   // the quad's four inputs: its own wave's loads
    __syncthreads();
    // One step, u = t mod PF.  wait_n: how many of the wave's memory operations may still be under way when the NEXT
    // step's inputs are taken from the ring, before the barrier rather than after it.
    auto step = [&](int u, int t, int wait_n) __attribute__((always_inline)) {
        const float* hcur = hs[u & 1] + q * KQ;   // (PF is even: the buffers alternate across rounds too)
        f32x4 hv[KQ / 4];
#pragma unroll
        for (int k = 0; k < KQ / 4; k++) hv[k] = *reinterpret_cast<const f32x4*>(hcur + 4 * k);
        float a[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int k = 0; k < KQ / 4; k++)
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int g = 0; g < 4; g++) a[g] += rr[g][4 * k + e] * hv[k][e];
        const float it = quad_sum(a[0]) + (wv[0] + bq[0]);
        const float ft = quad_sum(a[1]) + (wv[1] + bq[1]);
        const float zt = quad_sum(a[2]) + (wv[2] + bq[2]);
        const float ot = quad_sum(a[3]) + (wv[3] + bq[3]);
        const float logf = FS ? log_sigmoid_fast(ft) : ft;
        const float z = tanh_fast(zt), o = sigmoid_fast(ot);
        const float mn = fmaxf(logf + m, it);
        const float ip = fast_exp(it - mn), fp = fast_exp(logf + m - mn);
        c = fp * c + ip * z;
        n = fp * n + ip;
        m = mn;
        const float hnew = o * c * fast_rcp(n);
        hs[(u & 1) ^ 1][j] = hnew;   // (the quad's four lanes write the same bits)
        if (SAVE) { *own = pick(is0, is1, is2, it, logf, z, o); own += step_s; }
        if (SAVE || q == 3) { *out2 = pick(is0, is1, is2, c, n, m, hnew); out2 += step2; }
        // (the ring's values of this step went into the stores above: its slot takes the row PF steps on)
        ring_load(wnext, ring_base + u * (4 * DH * 4));
        if (t + PF + 1 < S) wnext += step_wx;
        ring_wait(wait_n);
        wv = *reinterpret_cast<const f32x4*>(&ring[(u + 1) % PF][4 * j]);
        __syncthreads();
    };
    // The ring load of step t + 1 was issued at the end of step t + 1 - PF: when step t asks for it, the OPS operations of
    // each of the PF - 1 steps since are younger (the wait allows one step's fewer).  In the first round the loads come
    // from the prologue, and only the later slots' loads are counted as younger.
#pragma unroll
    for (int u = 0; u < PF; u++)
        if (u < S) step(u, u, u + 1 < PF ? PF - 2 - u : OPS * (PF - 2));
    for (int t0 = PF; t0 < S; t0 += PF) {
#pragma unroll
        for (int u = 0; u < PF; u++)
            if (t0 + u < S) step(u, t0 + u, OPS * (PF - 2));
    }
}

// Back through time with the same quads, but what step t + 1 sends back to h_t -- R^T delta_{t+1}, a vector of 4 DH gradients
// against DH outputs -- is formed by rows of 16 lanes: the four quads of a row own four units k, and lane p of the row takes
// a sixteenth of the gradient vector for all four of them (DH / 4 gradients x 4 columns of R: DH registers, DH multiply-adds,
// but only DH / 4 floats of LDS reads where a lane that served one unit alone read DH: the LDS pipeline was what the step
// waited for).  The four sums meet over the row in four DPP exchanges; every lane keeps its own unit's, and all four lanes
// of a quad then form the unit's four pre-activation gradients alike; lane q hands on and stores gradient q (delta in two
// buffers, taken in turns: one barrier per step).  Lane q loads saved value q, and value 4 + q or, for q = 3, dh.
template <int DH, bool FS>
__global__ __launch_bounds__(4 * DH) void slstm_backward_kernel(const float* __restrict__ dh, const float* __restrict__ r,
                                                                const float* __restrict__ saved, float* __restrict__ dwx, int NH,
                                                                int S) {
    constexpr int PE = DH / 4;       // gradients per lane: a sixteenth of the 4 DH (in the order unit * 4 + gate)
    constexpr int PS = PE + 4;       // ... and four floats, so that the 16 parts of a row's read start in different banks
    __shared__ __attribute__((aligned(16))) float delta[2][16 * PS];       // [buffer][part][unit * 4 + gate within the part]
    __shared__ __attribute__((aligned(16))) float ring[PF][2][4 * DH];     // [slot][0: saved 0..3 | 1: saved 4..6, dh][unit * 4 + q]
    const int tid = threadIdx.x, k = tid >> 2, q = tid & 3, wave = tid >> 6;
    const bool is0 = q == 0, is1 = q == 1, is2 = q == 2;
    const int b = blockIdx.x / NH, hd = blockIdx.x % NH;
    const int part = tid & 15, k4 = (tid >> 4) * 4;   // the lane's part of the gradient vector; the first of its row's four units
    float rc[PE][4];   // [gradient of the part][unit of the row]: R_g[j][k4 + u] for the part's (j, g)
#pragma unroll
    for (int e = 0; e < PE; e++) {
        const int f = part * PE + e, j = f >> 2, g = f & 3;
        const f32x4 v = *reinterpret_cast<const f32x4*>(r + (((size_t)hd * 4 + g) * DH + j) * DH + k4);
        rc[e][0] = v[0]; rc[e][1] = v[1]; rc[e][2] = v[2]; rc[e][3] = v[3];
    }
    const int urow = k & 3;   // which of the row's units is this lane's own
    const size_t step_wx = (size_t)4 * NH * DH, step_h = (size_t)NH * DH, step_s = (size_t)7 * NH * DH;
    // (pointers that walk with the steps, from the last row down; f0, f1: the rows the ring takes next)
    const float* f0 = saved + ((size_t)b * S + S - 1) * step_s + ((size_t)q * NH + hd) * DH + k;
    const float* f1 = q < 3 ? saved + ((size_t)b * S + S - 1) * step_s + ((size_t)(4 + q) * NH + hd) * DH + k
                            : dh + ((size_t)b * S + S - 1) * step_h + (size_t)hd * DH + k;
    const size_t step1 = q < 3 ? step_s : step_h;
    float* dwp = dwx + ((size_t)b * S + S - 1) * step_wx + ((size_t)q * NH + hd) * DH + k;
    const int mine_at = ((4 * k + q) / PE) * PS + (4 * k + q) % PE;   // where this lane's gradient goes in a delta buffer
    const unsigned ring_base = __builtin_amdgcn_readfirstlane(mlstm::lds_offset_of(&ring[0][0][0]) + wave * 256);
    auto fetch = [&](int u, bool more) __attribute__((always_inline)) {   // (before the start of the sequence: row 0 again)
        ring_load(f0, ring_base + (2 * u) * (4 * DH * 4));
        ring_load(f1, ring_base + (2 * u + 1) * (4 * DH * 4));
        if (more) { f0 -= step_s; f1 -= step1; }
    };
    constexpr int OPS = 3;   // per wave and step: the store of dwx, then two ring loads
#pragma unroll
    for (int u = 0; u < PF; u++) fetch(u, S - 2 - u >= 0);
    for (int e = tid; e < 16 * PS; e += 4 * DH) delta[0][e] = 0.f;   // (nothing comes back to the last step)
    float dc_next = 0.f, dn_next = 0.f;
    __syncthreads();
    // One step, the u-th of its round.  wait_n: how many of the wave's memory operations may still be under way when
    // the step takes its values from the ring.
    auto step = [&](int u, int t, int wait_n) __attribute__((always_inline)) {
        const float* dcur = delta[u & 1] + part * PS;
        f32x4 dl[PE / 4];
#pragma unroll
        for (int e = 0; e < PE / 4; e++) dl[e] = *reinterpret_cast<const f32x4*>(dcur + 4 * e);
        float a[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < PE; e++)
#pragma unroll
            for (int x = 0; x < 4; x++) a[x] += rc[e][x] * dl[e >> 2][e & 3];
        const float r0 = row_sum(a[0]), r1 = row_sum(a[1]), r2 = row_sum(a[2]), r3 = row_sum(a[3]);
        const float dhrec = urow == 0 ? r0 : urow == 1 ? r1 : urow == 2 ? r2 : r3;
        ring_wait(wait_n);
        const int un = (u + 1) % PF;
        const f32x4 s0 = *reinterpret_cast<const f32x4*>(&ring[u][0][4 * k]);    // i~, log f, z, o
        const f32x4 s1 = *reinterpret_cast<const f32x4*>(&ring[u][1][4 * k]);    // c, n, m, dh
        f32x4 sp = *reinterpret_cast<const f32x4*>(&ring[un][1][4 * k]);         // c, n, m of step t - 1
        if (t == 0) { sp[0] = 0.f; sp[1] = 0.f; sp[2] = -INFINITY; }
        const float it = s0[0], logf = s0[1], z = s0[2], o = s0[3], ct = s1[0], nt = s1[1], mt = s1[2];
        const float ip = fast_exp(it - mt), fp = fast_exp(logf + sp[2] - mt);
        const float d_h = s1[3] + dhrec;
        const float inv_n = fast_rcp(nt), psi = ct * inv_n;
        const float d_o = d_h * psi * o * (1.0f - o);
        const float dpsi = d_h * o;
        const float dc = dpsi * inv_n + dc_next;
        const float dn = -dpsi * psi * inv_n + dn_next;
        const float d_z = dc * ip * (1.0f - z * z);
        const float d_i = (dc * z + dn) * ip;
        float d_f = (dc * sp[0] + dn * sp[1]) * fp;
        if (FS) d_f *= 1.0f - fast_exp(logf);   // d logsigmoid(f~) / d f~ = sigmoid(-f~) = 1 - exp(log f)
        dc_next = dc * fp;
        dn_next = dn * fp;
        const float mine = pick(is0, is1, is2, d_i, d_f, d_z, d_o);
        delta[(u & 1) ^ 1][mine_at] = mine;
        *dwp = mine;
        dwp -= step_wx;
        fetch(u, t - PF >= 1);   // (the slot's values of this step are in registers: the store took them)
        __syncthreads();
    };
    // Step t needs its own values (loaded PF steps ago) and c, n, m of step t - 1 (the next slot, loaded PF - 1 steps ago,
    // as the last operations of that step): behind them lie the OPS operations of each of PF - 2 steps (the wait allows one
    // step's fewer).  In the first round both come from the prologue, where only the later slots' loads are counted as
    // younger; its last step's next slot is the first step's refill.  All of them are the quad's own wave's loads.
#pragma unroll
    for (int u = 0; u < PF; u++)
        if (S - 1 - u >= 0) step(u, S - 1 - u, u + 1 < PF ? 2 * (PF - 2 - u) : OPS * (PF - 3));
    for (int t0 = S - 1 - PF; t0 >= 0; t0 -= PF) {
#pragma unroll
        for (int u = 0; u < PF; u++)
            if (t0 - u >= 0) step(u, t0 - u, OPS * (PF - 3));
    }
}

constexpr int dr_parts(int DH) { return DH <= 64 ? 4 : 1; }   // partial sums per slice (slstm_dr_kernel's PARTS)
// dR[h][g][j][k] and db[h][g][j] over one slice of the (b, t) pairs, on the matrix units: per head and gate this is the
// product of dWx[g] ([pairs] x DH, taken transposed) with h_{t-1} ([pairs] x DH), the pairs being the inner dimension.
// v_mfma_f32_32x32x2_f32 takes per lane one element of each operand -- row or column l % 32 at inner index l / 32 -- so both
// come straight from global memory, one dword per lane, rows of 128 bytes; nothing passes through LDS.  One workgroup per
// (head, gate, slice), four waves: up to DH = 64 every wave forms the whole DH x DH block over a quarter of the slice's
// pairs (chunks of 16, taken in turns) and leaves it as a partial sum of its own; at DH = 128 every wave forms one 64 x 64
// quadrant over all the pairs.
template <int DH>
__global__ __launch_bounds__(256, 2) void slstm_dr_kernel(const float* __restrict__ dwx, const float* __restrict__ h, float* __restrict__ part_r,
                                                       float* __restrict__ part_b, int B, int NH, int S, int nslice) {
    using mlstm::f32x16;
    constexpr int W = DH < 64 ? DH : 64;   // a wave's block is W x W
    constexpr int T = W / 32;               // in T x T tiles
    constexpr int PARTS = dr_parts(DH);     // waves that share a block, each with its part of the pairs
    constexpr int U = 8, CH = 2 * U;        // matrix instructions along the pairs per round, and the pairs they take
    const int hg = blockIdx.x, hd = hg / 4, g = hg % 4, slice = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, l32 = lane & 31, hh = lane >> 5;
    const int part = PARTS > 1 ? wave : 0, quad = PARTS > 1 ? 0 : wave;
    const int j0 = (quad >> 1) * 64, k0 = (quad & 1) * 64;   // the block's corner
    const long long total = (long long)B * S, per = (total + nslice - 1) / nslice;
    const long long lo = slice * per, hi = lo + per < total ? lo + per : total;
    const size_t step_wx = (size_t)4 * NH * DH, step_h = (size_t)NH * DH;
    // (a lane's place inside a pair of rows, as one 32-bit offset: the rows' own addresses are the same for the whole wave)
    const unsigned la = (unsigned)(hh * step_wx + ((size_t)g * NH + hd) * DH + j0 + l32);
    const unsigned lb = (unsigned)(hh * step_h + (size_t)hd * DH + k0 + l32);
    f32x16 acc[T][T];
    float bsum[T];
#pragma unroll
    for (int x = 0; x < T; x++) {
        bsum[x] = 0.f;
#pragma unroll
        for (int y = 0; y < T; y++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[x][y][e] = 0.f;
    }
    float a[2][T][U], bv[2][T][U];
    // the operands of the round that starts at pair p0 (this lane's first pair: p0 + hh, t0 steps into its sequence)
    auto load = [&](int set, long long p0, int t0) __attribute__((always_inline)) {
#pragma unroll
        for (int e = 0; e < U; e++) {
            const long long pp = p0 + 2 * e + hh;
            int t = t0 + 2 * e;
            if (t >= S) t %= S;
            const bool in = pp < hi, prev = in && t != 0;   // (h_{-1} = 0: the first step of a sequence adds nothing to dR)
            const float* ra = dwx + (p0 + 2 * e) * (long long)step_wx;
            const float* rb = h + (p0 + 2 * e - 1) * (long long)step_h;
#pragma unroll
            for (int x = 0; x < T; x++) {
                a[set][x][e] = in ? ra[la + 32 * x] : 0.f;
                bv[set][x][e] = prev ? rb[lb + 32 * x] : 0.f;
            }
        }
    };
    long long p0 = lo + (long long)part * CH;
    int t0 = (int)((p0 + hh) % S);
    if (p0 < hi) load(0, p0, t0);
    // one round on operand set `set` (a constant at each call); the next round's operands are under way while it multiplies
    auto round = [&](int set) __attribute__((always_inline)) {
        const long long pn = p0 + (long long)PARTS * CH;
        int tn = t0 + PARTS * CH;
        if (tn >= S) tn %= S;
        if (pn < hi) load(set ^ 1, pn, tn);
#pragma unroll
        for (int e = 0; e < U; e++) {
#pragma unroll
            for (int x = 0; x < T; x++) {
                bsum[x] += a[set][x][e];
#pragma unroll
                for (int y = 0; y < T; y++) acc[x][y] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[set][x][e], bv[set][y][e], acc[x][y], 0, 0, 0);
            }
        }
        p0 = pn;
        t0 = tn;
    };
    while (p0 < hi) {
        round(0);
        if (p0 >= hi) break;
        round(1);
    }
    // db: a lane's sum covers its half of the pairs (inner index l / 32) for row l % 32
#pragma unroll
    for (int x = 0; x < T; x++) bsum[x] += __shfl_xor(bsum[x], 32);
    // accumulator register e of a lane: column l % 32, row 8 (e / 4) + 4 (l / 32) + e % 4 of its tile
    // (every wave's partial sum is a slice of its own for the kernel that adds the slices)
    const size_t sl = (size_t)slice * PARTS + part;
    float* out = part_r + ((sl * NH * 4 + hg) * DH) * DH;
#pragma unroll
    for (int x = 0; x < T; x++)
#pragma unroll
        for (int y = 0; y < T; y++)
#pragma unroll
            for (int e = 0; e < 16; e++)
                out[(size_t)(j0 + 32 * x + 8 * (e / 4) + 4 * hh + e % 4) * DH + k0 + 32 * y + l32] = acc[x][y][e];
    if (k0 == 0 && hh == 0) {
#pragma unroll
        for (int x = 0; x < T; x++) part_b[(sl * NH * 4 + hg) * DH + j0 + 32 * x + l32] = bsum[x];
    }
}

// out[e] = sum over the partial sums, in a fixed order: 64 elements per workgroup, four threads per element with every
// fourth partial sum each, their four sums added in order.
__global__ __launch_bounds__(256) void slstm_reduce_kernel(const float* __restrict__ part, float* __restrict__ out, size_t n, int nslice) {
    __shared__ float red[4][64];
    const int x = threadIdx.x & 63, y = threadIdx.x >> 6;
    const size_t e = (size_t)blockIdx.x * 64 + x;
    float s0 = 0.f, s1 = 0.f;
    if (e < n) {
        int i = y;
        for (; i + 4 < nslice; i += 8) { s0 += part[(size_t)i * n + e]; s1 += part[(size_t)(i + 4) * n + e]; }
        if (i < nslice) s0 += part[(size_t)i * n + e];
    }
    red[y][x] = s0 + s1;
    __syncthreads();
    if (y == 0 && e < n) out[e] = (red[0][x] + red[1][x]) + (red[2][x] + red[3][x]);
}

int slices_for(int B, int NH, int S) {
    const size_t total = (size_t)B * S;
    size_t n = 512 / ((size_t)NH * 4);   // about two workgroups for each of the 256 compute units
    if (n < 1) n = 1;
    if (n > (total + 255) / 256) n = (total + 255) / 256;   // at least 256 (b, t) pairs per slice
    return (int)(n < 1 ? 1 : n);
}

// (the step kernels count their waits for the input ring by hand: see no_scratch_once)
template <int DH, bool SAVE, bool FS>
int forward_launch(const float* wx, const float* r, const float* b, float* h, float* saved, int B, int NH, int S, hipStream_t st) {
    if (int rc = mlstm::no_scratch_once<slstm_forward_kernel<DH, SAVE, FS>>()) return rc;
    hipLaunchKernelGGL((slstm_forward_kernel<DH, SAVE, FS>), dim3(B * NH), dim3(4 * DH), 0, st, wx, r, b, h, saved, NH, S);
    return (int)hipGetLastError();
}

template <int DH>
int forward_t(const float* wx, const float* r, const float* b, float* h, float* saved, int B, int NH, int S, int fs, hipStream_t st) {
    if (saved && fs) return forward_launch<DH, true, true>(wx, r, b, h, saved, B, NH, S, st);
    if (saved) return forward_launch<DH, true, false>(wx, r, b, h, saved, B, NH, S, st);
    if (fs) return forward_launch<DH, false, true>(wx, r, b, h, saved, B, NH, S, st);
    return forward_launch<DH, false, false>(wx, r, b, h, saved, B, NH, S, st);
}

template <int DH>
int backward_t(const float* dh, const float* h, const float* r, const float* saved, float* dwx, float* dr, float* db, int B, int NH, int S,
               int fs, char* ws, hipStream_t st) {
    if (fs) {
        if (int rc = mlstm::no_scratch_once<slstm_backward_kernel<DH, true>>()) return rc;
        hipLaunchKernelGGL((slstm_backward_kernel<DH, true>), dim3(B * NH), dim3(4 * DH), 0, st, dh, r, saved, dwx, NH, S);
    } else {
        if (int rc = mlstm::no_scratch_once<slstm_backward_kernel<DH, false>>()) return rc;
        hipLaunchKernelGGL((slstm_backward_kernel<DH, false>), dim3(B * NH), dim3(4 * DH), 0, st, dh, r, saved, dwx, NH, S);
    }
    const int ns = slices_for(B, NH, S);
    const size_t nr = (size_t)NH * 4 * DH * DH, nb = (size_t)NH * 4 * DH;
    float* part_r = reinterpret_cast<float*>(ws);
    const int np = ns * dr_parts(DH);   // partial sums to add
    float* part_b = part_r + (size_t)np * nr;
    hipLaunchKernelGGL(slstm_dr_kernel<DH>, dim3(NH * 4, ns), dim3(256), 0, st, dwx, h, part_r, part_b, B, NH, S, ns);
    hipLaunchKernelGGL(slstm_reduce_kernel, dim3((unsigned)((nr + 63) / 64)), dim3(256), 0, st, part_r, dr, nr, np);
    hipLaunchKernelGGL(slstm_reduce_kernel, dim3((unsigned)((nb + 63) / 64)), dim3(256), 0, st, part_b, db, nb, np);
    return (int)hipGetLastError();
}

bool good_dh(int DH) { return DH == 32 || DH == 64 || DH == 128; }

}  // namespace slstm

extern "C" {

size_t slstm_saved_bytes(int B, int NH, int S, int DH) {
    if (B <= 0 || NH <= 0 || S <= 0 || !slstm::good_dh(DH)) return 0;
    return (size_t)B * S * 7 * NH * DH * sizeof(float);
}

size_t slstm_workspace_bytes(int B, int NH, int S, int DH) {
    if (B <= 0 || NH <= 0 || S <= 0 || !slstm::good_dh(DH)) return 0;
    return (size_t)slstm::slices_for(B, NH, S) * slstm::dr_parts(DH) * NH * 4 * ((size_t)DH * DH + DH) * sizeof(float);
}

int slstm_forward_ex(const float* wx, const float* r, const float* b, float* h, float* saved, int B, int NH, int S, int DH,
                     int forget_sigmoid, void* stream) {
    if (!wx || !r || !b || !h || B <= 0 || NH <= 0 || S <= 0) return MLSTM_EINVAL;
    if (!slstm::good_dh(DH)) return MLSTM_ESHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const int fs = forget_sigmoid ? 1 : 0;
    switch (DH) {
        case 32: return slstm::forward_t<32>(wx, r, b, h, saved, B, NH, S, fs, st);
        case 64: return slstm::forward_t<64>(wx, r, b, h, saved, B, NH, S, fs, st);
        default: return slstm::forward_t<128>(wx, r, b, h, saved, B, NH, S, fs, st);
    }
}

int slstm_backward_ex(const float* dh, const float* h, const float* r, const float* saved, float* dwx, float* dr, float* db, int B,
                      int NH, int S, int DH, int forget_sigmoid, void* workspace, size_t workspace_bytes, void* stream) {
    if (!dh || !h || !r || !saved || !dwx || !dr || !db || B <= 0 || NH <= 0 || S <= 0) return MLSTM_EINVAL;
    if (!slstm::good_dh(DH)) return MLSTM_ESHAPE;
    if (!workspace || workspace_bytes < slstm_workspace_bytes(B, NH, S, DH)) return MLSTM_EWORKSPACE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const int fs = forget_sigmoid ? 1 : 0;
    char* ws = reinterpret_cast<char*>(workspace);
    switch (DH) {
        case 32: return slstm::backward_t<32>(dh, h, r, saved, dwx, dr, db, B, NH, S, fs, ws, st);
        case 64: return slstm::backward_t<64>(dh, h, r, saved, dwx, dr, db, B, NH, S, fs, ws, st);
        default: return slstm::backward_t<128>(dh, h, r, saved, dwx, dr, db, B, NH, S, fs, ws, st);
    }
}

}  // extern "C"
