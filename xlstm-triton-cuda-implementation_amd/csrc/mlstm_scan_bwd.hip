// Backward of the scan form (fp32, every head dimension the scan form takes), built from the scan form's own pipeline.
// The reference has a forward only for this form (mlstm_scan.py:281-327); the gradients are those of the matmul form
// (mlstm_matmul.py:150-333, same function) with the silu(o) gate of mlstm_scan.py:277 in front.
//
// With a_j = i_j - Fc_j, A_t = max_{j<=t} a_j, w(t, j) = exp(a_j - A_t) / sqrt(D), the scan pipeline evaluates
//     N(x, y, z)_t = sum_{j<=t} w(t, j) (x_t . y_j) z_j                                        (finish mode 2)
// for any three [S, D] operands; the forward output is N(q, k, v)_t / n_t with n_t = max(|b_t|, exp(-m_t)) + 1e-6.
// With dh the gradient of the ungated output, u_t = dh_t / n_t, db_t the gradient of the normaliser sum
// (row_stats in mlstm_device.h) and n~_t = sum_{j<=t} w(t, j) k_j:
//     dQ_t = N(u, v, k)_t + db_t n~_t
//     dV_j = exp(a_j - A_j) R(k, q, u)_j
//     dK_j = exp(a_j - A_j) (R(v, u, q)_j + g_j)
// where R(x, y, z)_j = sum_{t>=j} exp(A_j - A_t) / sqrt(D) (x_j . y_t) z_t and g_j = sum_{t>=j} exp(A_j - A_t) / sqrt(D) db_t q_t.
// R is N on the time-reversed sequence with the gate arrays of reverse_gates_kernel (a' = A' = -A reversed: that
// sequence is non-decreasing, so it is its own running maximum and every weight stays <= 1).  The vector sums n~ and g
// run chunk-wise (vecscan_local_kernel, the carry of the scan form, and a term of the combine kernels).
//     dI_j = k_j . dK_j,   dF_t = sigmoid(-f_t) sum_{s<t} (k_s . dK_s - q_s . dQ_s)            (mlstm_matmul.py:309-333)
#include "mlstm_device.h"
#include "mlstm_kernels.h"

namespace mlstm {

namespace {

constexpr int ROWS_PER_WG = 4;  // one wave per row in the row-wise kernels

__device__ __forceinline__ float row_sum(float x) { return wave_reduce<OpAdd>(x); }

// inv_n, db per row; u = dh / n; db also in reversed order (the reversed vector scan scales its rows by it)
__global__ __launch_bounds__(256) void scanbwd_rowstats_kernel(const float* __restrict__ dh, const float* __restrict__ h,
                                                               const float* __restrict__ b, const float* __restrict__ m,
                                                               float* __restrict__ u, float* __restrict__ db, float* __restrict__ db_rev,
                                                               int BH, int S, int D) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t rows = (size_t)BH * S;
    for (size_t row = (size_t)blockIdx.x * ROWS_PER_WG + wave; row < rows; row += (size_t)gridDim.x * ROWS_PER_WG) {
        float acc = 0.f;
        for (int k = 4 * lane; k < D; k += 256) {
            const f32x4 x = *reinterpret_cast<const f32x4*>(dh + row * D + k);
            const f32x4 y = *reinterpret_cast<const f32x4*>(h + row * D + k);
            acc += x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3];
        }
        const float delta = row_sum(acc);
        const float bv = b[row], em = __expf(-m[row]);
        const float inv_n = 1.0f / (fmaxf(fabsf(bv), em) + 1e-6f);
        const float dn = -delta * inv_n;
        const float sg = (bv > 0.f) ? 1.f : ((bv < 0.f) ? -1.f : 0.f);
        const float dbv = (fabsf(bv) > em) ? sg * dn : 0.f;
        for (int k = 4 * lane; k < D; k += 256) {
            f32x4 x = *reinterpret_cast<const f32x4*>(dh + row * D + k);
            x *= inv_n;
            *reinterpret_cast<f32x4*>(u + row * D + k) = x;
        }
        if (lane == 0) {
            const size_t bh = row / S, t = row % S;
            db[row] = dbv;
            db_rev[bh * S + (S - 1 - t)] = dbv;
        }
    }
}

// out[bh][s][:] = in[bh][S-1-s][:]
__global__ __launch_bounds__(256) void scanbwd_flip_kernel(const float* __restrict__ in, float* __restrict__ out, int BH, int S, int D) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t rows = (size_t)BH * S;
    for (size_t row = (size_t)blockIdx.x * ROWS_PER_WG + wave; row < rows; row += (size_t)gridDim.x * ROWS_PER_WG) {
        const size_t bh = row / S, s = row % S, src = bh * S + (S - 1 - s);
        for (int k = 4 * lane; k < D; k += 256)
            *reinterpret_cast<f32x4*>(out + row * D + k) = *reinterpret_cast<const f32x4*>(in + src * D + k);
    }
}

// Gate arrays of the reversed sequence, in the layout of the gate pre-pass (granule-relative fp32 values over fp64 bases, in
// log2 units, rows padded to whole granules with alpha = -inf, beta = 0).  Reversed position s is position t = S-1-s;
// a'_s = A'_s = -A_t with A_t = beta2_t - G2_g(t); the base of a reversed granule is -(its first a'), so alpha' = beta' =
// A_t0 - A_t >= 0 with t0 the granule's first (latest in time) position.
__global__ __launch_bounds__(256) void scanbwd_reverse_gates_kernel(const float* __restrict__ beta2, const double* __restrict__ G2,
                                                                    float* __restrict__ alpha2r, float* __restrict__ beta2r,
                                                                    double* __restrict__ G2r, int BH, int S, int NG) {
    const size_t n = (size_t)BH * NG * GRAN;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= n) return;
    const size_t bh = idx / ((size_t)NG * GRAN);
    const int s = (int)(idx % ((size_t)NG * GRAN)), s0 = s & ~(GRAN - 1);
    const size_t poff = bh * NG * GRAN;
    auto A_of = [&](int rs) {  // A (log2 units) of the position that reversed position rs < S stands for
        const int t = S - 1 - rs;
        return (double)beta2[poff + t] - G2[bh * NG + t / GRAN];
    };
    const double A0 = A_of(s0);  // (s0 < S: the rows are padded to ceil(S/64) granules, so every granule starts inside)
    if (s == s0) G2r[bh * NG + s / GRAN] = A0;
    if (s < S) {
        const float rel = (float)(A0 - A_of(s));
        alpha2r[idx] = rel;
        beta2r[idx] = rel;
    } else {
        alpha2r[idx] = -INFINITY;
        beta2r[idx] = 0.0f;
    }
}

// Causal vector sums inside each 64-position chunk, from zero at the chunk start:
//   y_t = sum_{j in chunk, j<=t} exp(a_j - A_t) / sqrt(D) s_j x_j        (s: optional per-position scale)
// and the chunk's own sum at its last position into Z (what scan_ncarry_kernel carries from chunk to chunk).
// One thread per column walks the positions: y_t = exp(A_{t-1} - A_t) y_{t-1} + exp(a_t - A_t)/sqrt(D) s_t x_t.
__global__ __launch_bounds__(256) void scanbwd_vecscan_local_kernel(const float* __restrict__ x, const float* __restrict__ scale,
                                                                    const float* __restrict__ alpha2, const float* __restrict__ beta2,
                                                                    float* __restrict__ y, float* __restrict__ Z, int S, int D, int NC) {
    __shared__ float sw[GRAN], sg[GRAN];
    const int c = blockIdx.x, bh = blockIdx.z, tid = threadIdx.x, col = blockIdx.y * 256 + tid;
    const size_t hoff = (size_t)bh * S, poff = (size_t)bh * NC * GRAN + (size_t)GRAN * c;
    const float log2scale = -0.5f * __log2f((float)D);
    if (tid < GRAN) {
        const int t = GRAN * c + tid;
        const bool ok = t < S;
        const float be = beta2[poff + tid];
        float w = ok ? fast_exp2(alpha2[poff + tid] - be + log2scale) : 0.f;
        if (ok && scale) w *= scale[hoff + t];
        sw[tid] = w;
        sg[tid] = (ok && tid > 0) ? fast_exp2(beta2[poff + tid - 1] - be) : (ok ? 0.f : 1.f);
    }
    __syncthreads();
    if (col >= D) return;
    float run = 0.f;
#pragma unroll 8
    for (int j = 0; j < GRAN; j++) {
        const int t = GRAN * c + j;
        const int tc = t < S ? t : S - 1;
        const float xv = x[(hoff + tc) * D + col];
        run = sg[j] * run + sw[j] * xv;
        if (t < S) y[(hoff + t) * D + col] = run;
    }
    Z[((size_t)bh * NC + c) * D + col] = run;
}

// decay of the previous chunk's end state at position t of chunk c > 0: exp(A_{64c-1} - A_t)
__device__ __forceinline__ float carry_decay(const float* beta2, const double* G2, size_t poff, size_t goff, int c, int t) {
    return fast_exp2(beta2[poff + GRAN * c - 1] - beta2[poff + t] + (float)(G2[goff + c] - G2[goff + c - 1]));
}

// dQ_t = N(u, v, k)_t (in dq already) + db_t (y_t + decay_t carry_{c-1});  rowdot_t = q_t . dQ_t
__global__ __launch_bounds__(256) void scanbwd_dq_combine_kernel(float* __restrict__ dq, const float* __restrict__ q,
                                                                 const float* __restrict__ yloc, const float* __restrict__ carry,
                                                                 const float* __restrict__ db, const float* __restrict__ beta2,
                                                                 const double* __restrict__ G2, float* __restrict__ rowdot, int BH, int S,
                                                                 int D, int NC) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t rows = (size_t)BH * S;
    for (size_t row = (size_t)blockIdx.x * ROWS_PER_WG + wave; row < rows; row += (size_t)gridDim.x * ROWS_PER_WG) {
        const size_t bh = row / S;
        const int t = (int)(row % S), c = t / GRAN;
        const float dbv = db[row];
        const float dec = c > 0 ? carry_decay(beta2, G2, bh * NC * GRAN, bh * NC, c, t) : 0.f;
        const float* cr = carry + (bh * NC + (c > 0 ? c - 1 : 0)) * D;
        float acc = 0.f;
        for (int k = 4 * lane; k < D; k += 256) {
            f32x4 g = *reinterpret_cast<const f32x4*>(dq + row * D + k);
            const f32x4 yv = *reinterpret_cast<const f32x4*>(yloc + row * D + k);
            const f32x4 cv = *reinterpret_cast<const f32x4*>(cr + k);
            const f32x4 qv = *reinterpret_cast<const f32x4*>(q + row * D + k);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                g[e] += dbv * (yv[e] + dec * cv[e]);
                acc += qv[e] * g[e];
            }
            *reinterpret_cast<f32x4*>(dq + row * D + k) = g;
        }
        acc = row_sum(acc);
        if (lane == 0) rowdot[row] = acc;
    }
}

// dV_j = wd_j RV_s,  dK_j = wd_j (RK_s + y_s + decay_s carry_{c-1}) with s = S-1-j the reversed position and
// wd_j = exp(a_j - A_j);  dI_j = k_j . dK_j;  x_j = dI_j - rowdot_j (the summand of dF)
__global__ __launch_bounds__(256) void scanbwd_dkdv_combine_kernel(const float* __restrict__ RV, const float* __restrict__ RK,
                                                                   const float* __restrict__ yloc, const float* __restrict__ carry,
                                                                   const float* __restrict__ k, const float* __restrict__ alpha2,
                                                                   const float* __restrict__ beta2, const float* __restrict__ beta2r,
                                                                   const double* __restrict__ G2r, const float* __restrict__ rowdot,
                                                                   float* __restrict__ dk, float* __restrict__ dv, float* __restrict__ di,
                                                                   float* __restrict__ x, int BH, int S, int D, int NC) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t rows = (size_t)BH * S;
    for (size_t row = (size_t)blockIdx.x * ROWS_PER_WG + wave; row < rows; row += (size_t)gridDim.x * ROWS_PER_WG) {
        const size_t bh = row / S;
        const int j = (int)(row % S), s = S - 1 - j, c = s / GRAN;
        const size_t poff = bh * NC * GRAN, rrow = bh * S + s;
        const float wd = fast_exp2(alpha2[poff + j] - beta2[poff + j]);
        const float dec = c > 0 ? carry_decay(beta2r, G2r, poff, bh * NC, c, s) : 0.f;
        const float* cr = carry + (bh * NC + (c > 0 ? c - 1 : 0)) * D;
        float acc = 0.f;
        for (int e0 = 4 * lane; e0 < D; e0 += 256) {
            const f32x4 rv = *reinterpret_cast<const f32x4*>(RV + rrow * D + e0);
            const f32x4 rk = *reinterpret_cast<const f32x4*>(RK + rrow * D + e0);
            const f32x4 yv = *reinterpret_cast<const f32x4*>(yloc + rrow * D + e0);
            const f32x4 cv = *reinterpret_cast<const f32x4*>(cr + e0);
            const f32x4 kv = *reinterpret_cast<const f32x4*>(k + row * D + e0);
            f32x4 gk, gv;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                gv[e] = wd * rv[e];
                gk[e] = wd * (rk[e] + yv[e] + dec * cv[e]);
                acc += kv[e] * gk[e];
            }
            *reinterpret_cast<f32x4*>(dk + row * D + e0) = gk;
            *reinterpret_cast<f32x4*>(dv + row * D + e0) = gv;
        }
        acc = row_sum(acc);
        if (lane == 0) {
            di[row] = acc;
            x[row] = acc - rowdot[row];
        }
    }
}

struct Carve {
    char* base; size_t off;
    template <typename T> T* take(size_t n) {
        T* p = base ? reinterpret_cast<T*>(base + off) : nullptr;
        off += (n * sizeof(T) + 255) / 256 * 256;
        return p;
    }
};

struct Plan {
    double *G2, *G2r;
    float *alpha2, *beta2, *ek2, *amax2, *m, *alpha2r, *beta2r;
    float *b, *db, *db_rev, *rowdot, *x;
    float *P, *Nst, *Z, *hpart, *seg_state;
    float *T[8];
    size_t bytes;
};

Plan plan_of(char* ws, int BH_, int S_, int D_) {
    const size_t BH = BH_, S = S_, D = D_, NG = (S + GRAN - 1) / GRAN, N = BH * S * D;
    Carve c{ws, 0};
    Plan p;
    p.G2 = c.take<double>(BH * NG);
    p.G2r = c.take<double>(BH * NG);
    p.alpha2 = c.take<float>(BH * NG * GRAN);
    p.beta2 = c.take<float>(BH * NG * GRAN);
    p.ek2 = c.take<float>(BH * NG * GRAN);
    p.amax2 = c.take<float>(BH * NG * 2 + 64);
    p.m = c.take<float>(BH * S);
    p.alpha2r = c.take<float>(BH * NG * GRAN);
    p.beta2r = c.take<float>(BH * NG * GRAN);
    p.b = c.take<float>(BH * S);
    p.db = c.take<float>(BH * S);
    p.db_rev = c.take<float>(BH * S);
    p.rowdot = c.take<float>(BH * S);
    p.x = c.take<float>(BH * S);
    p.P = c.take<float>(BH * NG * GRAN * GRAN);
    p.Nst = c.take<float>(BH * NG * D);
    p.Z = c.take<float>(BH * NG * D);
    const int KS = scan_key_splits(BH_, D_);
    p.hpart = nullptr;
    for (int s = 1; s < KS; s++) { float* t = c.take<float>(N); if (s == 1) p.hpart = t; }
    p.seg_state = c.take<float>(scan_segment_state_bytes(BH_, S_, D_) / 4);
    for (int t = 0; t < 8; t++) p.T[t] = c.take<float>(N);
    p.bytes = c.off;
    return p;
}

int row_blocks(size_t rows) {
    const size_t want = (rows + ROWS_PER_WG - 1) / ROWS_PER_WG;
    return (int)(want < 16384 ? want : 16384);
}

}  // namespace

size_t scan_backward_workspace_bytes(int BH, int S, int D) { return plan_of(nullptr, BH, S, D).bytes; }

int launch_scan_backward(const ScanBwdArgs& a, char* ws, hipStream_t st, void (*mark)(int, hipStream_t, bool)) {
    const int BH = a.BH, S = a.S, D = a.D, NG = (S + GRAN - 1) / GRAN;
    if (D % 64 || D < 64 || BH <= 0 || S <= 0) return MLSTM_ESHAPE;
    const Plan p = plan_of(ws, BH, S, D);
    const size_t rows = (size_t)BH * S, N = rows * D;
    const int KS = scan_key_splits(BH, D), rb = row_blocks(rows);
    float *u = p.T[2], *yloc = p.T[3], *qr = p.T[4], *kr = p.T[5], *vr = p.T[6], *ur = p.T[7];
    const float* h = a.h_kept ? a.h_kept : p.T[0];
    const float* bsum = a.h_kept ? a.b_kept : p.b;
    float *RV = p.T[0], *RK = p.T[1];  // (h and dh are done with by then)

    mark(MLSTM_K_GATES, st, true);
    const hipError_t ge = launch_gates(MLSTM_F32, a.f, a.i, p.alpha2, p.beta2, p.G2, p.m, p.ek2, p.amax2, BH, S, st);
    mark(MLSTM_K_GATES, st, false);
    if (ge != hipSuccess) return (int)ge;

    ScanArgs base{};
    base.hpart = p.hpart; base.P = p.P; base.Nst = p.Nst; base.M = p.m; base.o = a.o; base.seg_state = p.seg_state;
    base.BH = BH; base.S = S; base.D = D; base.NC = NG;
    auto fwd_gates = [&](ScanArgs& s) { s.alpha2 = p.alpha2; s.beta2 = p.beta2; s.G2 = p.G2; };
    auto rev_gates = [&](ScanArgs& s) { s.alpha2 = p.alpha2r; s.beta2 = p.beta2r; s.G2 = p.G2r; };

    // the ungated forward output and its normaliser sums, unless the caller kept them
    if (!a.h_kept) {
        ScanArgs s = base; fwd_gates(s);
        s.q = a.q; s.k = a.k; s.v = a.v; s.h = p.T[0]; s.finish_mode = 1; s.Bout = p.b;
        if (int rc = launch_scan(s, KS, st, mark)) return rc;
    }
    // the gradient of the ungated output: through the gate's backward, or, without a gate (o == null: the matmul
    // form's backward at head dimensions only these kernels serve), the caller's own
    const float* dh = a.dhg;
    if (a.o) {
        mark(MLSTM_K_GATE_BWD, st, true);
        const int gb = launch_gate_backward(MLSTM_F32, a.dhg, a.o, h, p.T[1], a.d_o, N, st);
        mark(MLSTM_K_GATE_BWD, st, false);
        if (gb) return gb;
        dh = p.T[1];
    }

    mark(MLSTM_K_SCAN_GLUE, st, true);
    hipLaunchKernelGGL(scanbwd_rowstats_kernel, dim3(rb), dim3(256), 0, st, dh, h, bsum, p.m, u, p.db, p.db_rev, BH, S, D);
    hipLaunchKernelGGL(scanbwd_reverse_gates_kernel, dim3((unsigned)(((size_t)BH * NG * GRAN + 255) / 256)), dim3(256), 0, st, p.beta2, p.G2,
                       p.alpha2r, p.beta2r, p.G2r, BH, S, NG);
    hipLaunchKernelGGL(scanbwd_flip_kernel, dim3(rb), dim3(256), 0, st, a.q, qr, BH, S, D);
    hipLaunchKernelGGL(scanbwd_flip_kernel, dim3(rb), dim3(256), 0, st, a.k, kr, BH, S, D);
    hipLaunchKernelGGL(scanbwd_flip_kernel, dim3(rb), dim3(256), 0, st, a.v, vr, BH, S, D);
    hipLaunchKernelGGL(scanbwd_flip_kernel, dim3(rb), dim3(256), 0, st, u, ur, BH, S, D);
    // n~ within the chunks, and at the chunk ends
    hipLaunchKernelGGL(scanbwd_vecscan_local_kernel, dim3(NG, (D + 255) / 256, BH), dim3(256), 0, st, a.k, (const float*)nullptr, p.alpha2,
                       p.beta2, yloc, p.Z, S, D, NG);
    {
        ScanArgs s = base; fwd_gates(s); s.Nst = p.Z;
        launch_scan_ncarry(s, st);
    }
    mark(MLSTM_K_SCAN_GLUE, st, false);

    // dQ
    {
        ScanArgs s = base; fwd_gates(s);
        s.q = u; s.k = a.v; s.v = a.k; s.h = a.dq; s.finish_mode = 2;
        if (int rc = launch_scan(s, KS, st, mark)) return rc;
    }
    mark(MLSTM_K_SCAN_GLUE, st, true);
    hipLaunchKernelGGL(scanbwd_dq_combine_kernel, dim3(rb), dim3(256), 0, st, a.dq, a.q, yloc, p.Z, p.db, p.beta2, p.G2, p.rowdot, BH, S, D, NG);
    // g within the reversed chunks, and at their ends (yloc and Z are free again)
    hipLaunchKernelGGL(scanbwd_vecscan_local_kernel, dim3(NG, (D + 255) / 256, BH), dim3(256), 0, st, qr, p.db_rev, p.alpha2r, p.beta2r, yloc,
                       p.Z, S, D, NG);
    {
        ScanArgs s = base; rev_gates(s); s.Nst = p.Z;
        launch_scan_ncarry(s, st);
    }
    mark(MLSTM_K_SCAN_GLUE, st, false);

    // dV and dK on the reversed sequence
    {
        ScanArgs s = base; rev_gates(s);
        s.q = kr; s.k = qr; s.v = ur; s.h = RV; s.finish_mode = 2;
        if (int rc = launch_scan(s, KS, st, mark)) return rc;
    }
    {
        ScanArgs s = base; rev_gates(s);
        s.q = vr; s.k = ur; s.v = qr; s.h = RK; s.finish_mode = 2;
        if (int rc = launch_scan(s, KS, st, mark)) return rc;
    }
    mark(MLSTM_K_SCAN_GLUE, st, true);
    hipLaunchKernelGGL(scanbwd_dkdv_combine_kernel, dim3(rb), dim3(256), 0, st, RV, RK, yloc, p.Z, a.k, p.alpha2, p.beta2, p.beta2r, p.G2r,
                       p.rowdot, a.dk, a.dv, a.di, p.x, BH, S, D, NG);
    mark(MLSTM_K_SCAN_GLUE, st, false);
    mark(MLSTM_K_DF, st, true);
    const int dfrc = launch_dfscan_plain(MLSTM_F32, a.f, p.x, a.df, BH, S, st);
    mark(MLSTM_K_DF, st, false);
    return dfrc;
}

}  // namespace mlstm
