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
// sequence is non-decreasing, so it is its own running maximum and every weight stays <= 1); the pipeline reads q, k, v
// and u from their last row backwards (ScanArgs::rev), nothing is copied into reversed order.  The vector sums n~ and g
// ride along with the matrix sums: db_t n~_t and g_j are N and R with (x . y) + db in the place of (x . y), so the pairs
// inside a chunk take db into their weights and the chunks before it come through the scan form's vector carry
// (ScanArgs::Epilogue::vec).  The pipeline's last kernel applies exp(a_j - A_j), writes dQ, dK, dV where they belong and
// takes the row dot products.
//     dI_j = k_j . dK_j,   dF_t = sigmoid(-f_t) sum_{s<t} (k_s . dK_s - q_s . dQ_s)            (mlstm_matmul.py:309-333)
#include "mlstm_device.h"
#include "mlstm_kernels.h"

namespace mlstm {

namespace {

constexpr int ROWS_PER_WG = 4;  // one wave per row in the row-wise kernels

__device__ __forceinline__ float row_sum(float x) { return wave_reduce<OpAdd>(x); }

// Per row: 1/n, db and u = dh / n.  With an output gate (o != null) g is the gradient of the gated output: dh = g o s with
// s = sigmoid(o) is formed here and d_o = g h s (1 + o (1 - s)) written (the gate of mlstm_scan.py:277); without one g is dh.
// A lane keeps its values of dh between the two passes over the row (D <= 1024: sixteen).
__global__ __launch_bounds__(256) void scanbwd_rowstats_kernel(const float* __restrict__ g, const float* __restrict__ o,
                                                               const float* __restrict__ h, const float* __restrict__ b,
                                                               const float* __restrict__ m, float* __restrict__ u, float* __restrict__ d_o,
                                                               float* __restrict__ db, int BH, int S, int D) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t rows = (size_t)BH * S;
    for (size_t row = (size_t)blockIdx.x * ROWS_PER_WG + wave; row < rows; row += (size_t)gridDim.x * ROWS_PER_WG) {
        f32x4 dh[4];
        float acc = 0.f;
#pragma unroll
        for (int n = 0; n < 4; n++) {
            const int k = 4 * lane + 256 * n;
            if (k < D) {
                f32x4 x = *reinterpret_cast<const f32x4*>(g + row * D + k);
                const f32x4 y = *reinterpret_cast<const f32x4*>(h + row * D + k);
                if (o) {
                    const f32x4 ov = *reinterpret_cast<const f32x4*>(o + row * D + k);
                    f32x4 dov;
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const float sg = 1.0f / (1.0f + __expf(-ov[e]));
                        dov[e] = x[e] * y[e] * sg * (1.0f + ov[e] * (1.0f - sg));
                        x[e] = x[e] * ov[e] * sg;
                    }
                    *reinterpret_cast<f32x4*>(d_o + row * D + k) = dov;
                }
                dh[n] = x;
                acc += x[0] * y[0] + x[1] * y[1] + x[2] * y[2] + x[3] * y[3];
            }
        }
        const float delta = row_sum(acc);
        const float bv = b[row], em = __expf(-m[row]);
        const float inv_n = 1.0f / (fmaxf(fabsf(bv), em) + 1e-6f);
        const float dn = -delta * inv_n;
        const float sg = (bv > 0.f) ? 1.f : ((bv < 0.f) ? -1.f : 0.f);
        const float dbv = (fabsf(bv) > em) ? sg * dn : 0.f;
#pragma unroll
        for (int n = 0; n < 4; n++) {
            const int k = 4 * lane + 256 * n;
            if (k < D) *reinterpret_cast<f32x4*>(u + row * D + k) = dh[n] * inv_n;
        }
        if (lane == 0) db[row] = dbv;
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
    float *b, *db, *rowdot, *x;
    float *P, *Nst, *hpart, *seg_state;
    float *T[2];
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
    p.rowdot = c.take<float>(BH * S);
    p.x = c.take<float>(BH * S);
    p.P = c.take<float>(BH * NG * GRAN * GRAN);
    p.Nst = c.take<float>(BH * NG * D);
    const int KS = scan_key_splits(BH_, D_);
    p.hpart = nullptr;
    for (int s = 1; s < KS; s++) { float* t = c.take<float>(N); if (s == 1) p.hpart = t; }
    p.seg_state = c.take<float>(scan_segment_state_bytes(BH_, S_, D_) / 4);
    for (int t = 0; t < 2; t++) p.T[t] = c.take<float>(N);
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
    if (D % 64 || D < 64 || D > 1024 || BH <= 0 || S <= 0) return MLSTM_ESHAPE;
    const Plan p = plan_of(ws, BH, S, D);
    const size_t rows = (size_t)BH * S;
    const int KS = scan_key_splits(BH, D), rb = row_blocks(rows);
    // T[0]: the recomputed forward output, then the numerators of the reversed passes; T[1]: u
    float *u = p.T[1], *num = p.T[0];
    const float* h = a.h_kept ? a.h_kept : p.T[0];
    const float* bsum = a.h_kept ? a.b_kept : p.b;

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
    // u, db and (with a gate: o != null, else the matmul form's backward at head dimensions only these kernels serve) d_o
    mark(MLSTM_K_SCAN_GLUE, st, true);
    hipLaunchKernelGGL(scanbwd_rowstats_kernel, dim3(rb), dim3(256), 0, st, a.dhg, a.o, h, bsum, p.m, u, a.d_o, p.db, BH, S, D);
    hipLaunchKernelGGL(scanbwd_reverse_gates_kernel, dim3((unsigned)(((size_t)BH * NG * GRAN + 255) / 256)), dim3(256), 0, st, p.beta2, p.G2,
                       p.alpha2r, p.beta2r, p.G2r, BH, S, NG);
    mark(MLSTM_K_SCAN_GLUE, st, false);

    // dQ_t = N(u, v, k)_t + db_t n~_t, and rowdot_t = q_t . dQ_t
    {
        ScanArgs s = base; fwd_gates(s);
        s.q = u; s.k = a.v; s.v = a.k; s.h = a.dq; s.finish_mode = 2;
        s.ep.vec = 1; s.ep.row_scale = p.db; s.ep.dot_with = a.q; s.ep.dot_out = p.rowdot;
        if (int rc = launch_scan(s, KS, st, mark)) return rc;
    }
    // dV_j = wd_j R(k, q, u)_j and dK_j = wd_j (R(v, u, q)_j + g_j) from the end of the sequence backwards (wd_j =
    // exp(a_j - A_j)); dI_j = k_j . dK_j; x_j = dI_j - rowdot_j, the summand of dF
    {
        ScanArgs s = base; rev_gates(s); s.rev = 1;
        s.q = a.k; s.k = a.q; s.v = u; s.h = num; s.finish_mode = 2;
        s.ep.out = a.dv; s.ep.out_rev = 1; s.ep.wd_alpha2 = p.alpha2; s.ep.wd_beta2 = p.beta2;
        if (int rc = launch_scan(s, KS, st, mark)) return rc;
    }
    {
        ScanArgs s = base; rev_gates(s); s.rev = 1;
        s.q = a.v; s.k = u; s.v = a.q; s.h = num; s.finish_mode = 2;
        s.ep.out = a.dk; s.ep.out_rev = 1; s.ep.wd_alpha2 = p.alpha2; s.ep.wd_beta2 = p.beta2;
        s.ep.vec = 1; s.col_scale = p.db; s.ep.dot_with = a.k; s.ep.dot_out = a.di; s.ep.dot_minus = p.rowdot; s.ep.x_out = p.x;
        if (int rc = launch_scan(s, KS, st, mark)) return rc;
    }
    mark(MLSTM_K_DF, st, true);
    const int dfrc = launch_dfscan_plain(MLSTM_F32, a.f, p.x, a.df, BH, S, st);
    mark(MLSTM_K_DF, st, false);
    return dfrc;
}

}  // namespace mlstm
