// Internal launch interface between the C ABI (mlstm_api.hip) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include "../../include/mlstm_hip.h"

namespace mlstm {

inline size_t dtype_size(int dt) { return dt == MLSTM_F32 ? 4 : 2; }

// Raises a kernel's dynamic LDS limit, once per process and kernel; the initialisation of a function-local static is
// thread-safe, so concurrent first calls do not race.  Returns the status of that one call.
template <auto KERN>
inline hipError_t lds_limit_once(int bytes) {
    static const hipError_t rc = hipFuncSetAttribute(reinterpret_cast<const void*>(KERN), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    return rc;
}
// For kernels whose waits for memory are counted by hand (s_waitcnt vmcnt(n) with n derived from the operations the SOURCE
// issues): a register spill adds memory operations of the compiler's that the count does not know, and the wait would then
// let a load pass as landed that has not.  Asked once per process and kernel: the launch is refused (MLSTM_EBUILD) if the
// compiled kernel uses any scratch memory at all.
template <auto KERN>
inline int no_scratch_once() {
    static const int rc = [] {
        hipFuncAttributes attr;
        const hipError_t e = hipFuncGetAttributes(&attr, reinterpret_cast<const void*>(KERN));
        if (e != hipSuccess) return (int)e;
        return attr.localSizeBytes == 0 ? 0 : MLSTM_EBUILD;
    }();
    return rc;
}
constexpr int GATE_GRANULE = 64;  // positions per gate granule (== mlstm::GRAN in the device code)

// Where a [B,NH,S,D] (or [B,NH,S]) tensor of the caller's keeps position s of head bh = b * NH + h: at element
// b * sb + h * sh + s * ss (+ the column: the last dimension is contiguous).  Everything the library owns (workspace,
// statistics m and b, chunk states) is dense.
struct Lay {
    long long sb, sh, ss;
    int NH;
    __host__ __device__ size_t head(int bh) const { return (size_t)((long long)(bh / NH) * sb + (long long)(bh % NH) * sh); }
};
inline Lay dense_layout(int NH, long long S, long long D) { return Lay{(long long)NH * S * D, S * D, D, NH}; }
// dense [B,NH,S,D]?  (The tile kernels keep a variant with the strides as compile-time constants for that case: run-time
// strides cost them address arithmetic in loops that are bound by instruction issue.)
inline bool is_dense(const Lay& l, long long S, long long D) { return l.ss == D && l.sh == S * D && l.sb == (long long)l.NH * S * D; }

// Eight words that one kernel of the forward leaves at the head of a caller-kept buffer (dst) and one kernel of the backward
// compares with what it finds there (src; a difference sets bit 1 of *err): rides along in kernels that run anyway.
struct SavedStamp {
    int* dst = nullptr;
    const int* src = nullptr;
    int* err = nullptr;
    int v[8] = {};
};
#if defined(__HIPCC__)
__device__ __forceinline__ void stamp_apply(const SavedStamp& s, bool first_block, int tid) {
    if (!first_block || tid >= 8) return;
    if (s.dst) s.dst[tid] = s.v[tid];
    if (s.src && s.src[tid] != s.v[tid]) atomicOr(s.err, 2);
}
#endif

// Gate pre-pass: alpha2, beta2 [BH, NG*64] fp32 (NG = ceil(S/64), rows padded), G2 [BH, NG] fp64, M [BH,S] fp32.
// ek2 [BH, NG*64] = exp2(alpha2 - block max), amax2 [BH, NG*2] = the maxima of alpha2 over blocks of 32 positions.
// lg: layout of F and I.  gate_form: what F holds (MLSTM_GATE_RAW: the forget gate's pre-activation, _LOGSIGMOID: its
// log-sigmoid, _CUMSUM: the cumulative sum of that over the positions of a head).
hipError_t launch_gates(int gate_dtype, const void* F, const void* I, float* alpha2, float* beta2, double* G2, float* M, float* ek2,
                        float* amax2, int BH, int S, hipStream_t st, const Lay& lg, int gate_form, const SavedStamp* stamp = nullptr);
inline hipError_t launch_gates(int gate_dtype, const void* F, const void* I, float* alpha2, float* beta2, double* G2, float* M, float* ek2,
                               float* amax2, int BH, int S, hipStream_t st) {
    return launch_gates(gate_dtype, F, I, alpha2, beta2, G2, M, ek2, amax2, BH, S, st, dense_layout(BH, S, 1), MLSTM_GATE_RAW);
}

extern bool g_force_generic;  // see mlstm_force_generic_kernels

struct RowArgs {
    const void* X;    // row operand held in registers: Q (forward) or dH (dQ pass)      [BH,S,D]
    const void* Y1;   // contracted over D with X:       K (forward) or V (dQ pass)
    const void* Y2;   // contracted over keys:           V (forward) or K (dQ pass)
    void* out;        // H (forward) or dQ
    // forward with an output gate: when O is set the kernel also writes silu(O) * H to out_gated (H itself, which the
    // backward needs, still goes to out)
    const void* O;
    void* out_gated;
    // long sequences in chunks (eight-wave kernel only): with chunk_len = L > 0 a row takes the keys of its own chunk of
    // L positions from Y1 / Y2 and everything before the chunk from the state at the end of the previous chunk
    // (launch_chunk_states).  L is a multiple of 128.
    int chunk_len;
    int n_states;         // states per head (chunks but the last)
    const void* Qrow;     // dQ pass in chunks: Q [BH,S,D] and
    float* rowinter;      //   [BH,S] out: q_i . dQ_i of the state part = the row sums of dD over the keys before the chunk
    const void* Cst;      // [BH][n_states][D][D] matrix states in the element type of X, rows in contraction order:
                          // key-major for the forward, value-major (ChunkArgs::CstT) for the dQ pass
    const void* Cst_lo;   // split mode: the states' low-order terms, same layout (the state enters its product as Cst + Cst_lo)
    const float* Nst;     // [BH][n_states][D] vector states
    const float* alpha2;
    const float* beta2;
    const double* G2;
    const float* ek2;     // factorised key weights and their block maxima (see launch_gates)
    const float* amax2;
    const float* M;       // forward: stabiliser, for the normaliser
    float* Bsum;          // forward: row sums b
    // dQ pass: the kernel derives 1/n and db per row from (dh, h, m, b) and also writes them, [BH, NG*64], for the
    // column kernel that runs after it
    const void* Hin;      // forward output h [BH,S,D]
    const float* Bin;     // forward row sums b [BH,S]
    float* inv_n;
    float* db;
    int BH, S, NG;
    // Split mode (16-bit types, generic kernel only): the weights of the second product enter it as two terms, hi + lo,
    // each in the element type (two MFMAs per fragment), so that their rounding no longer limits the result.  The
    // forward then also leaves h - (h rounded) in out_lo; the dQ pass reads it back through Hin_lo for dh . h.
    int precise;
    void* out_lo;
    const void* Hin_lo;
    // eight-wave kernel: the producers' wait for their P buffer is bounded; a wait that expires sets *err (sticky,
    // see mlstm_kernel_error) and the kernel runs on to its end.  spin_limit < 0 (test aid) lets every wait expire.
    int* err;
    int spin_limit;
    // layouts of the caller's tensors: la for q, k, v (forward: X, Y1, Y2; dQ pass: Y1, Y2, Qrow and out),
    // lb for h, dh, o (forward: out, O, out_gated; dQ pass: X), lh for Hin (the caller's h, or a dense recomputed one)
    Lay la, lb, lh;
};
// mode 0 = forward (H, b), mode 1 = dQ
int launch_row_kernel(int mode, int dtype, int D, const RowArgs& a, hipStream_t st);
// eight waves (producer / consumer pairs per SIMD); 16-bit types and D in {128, 256} only
int launch_row8_kernel(int mode, int dtype, int D, const RowArgs& a, hipStream_t st);
// (the four-wave kernel serves every other case: fp32, D = 64, split mode -- in chunks too -- and the test switch)
inline int launch_row_best(int mode, int dtype, int D, const RowArgs& a, hipStream_t st) {
    if (dtype != MLSTM_F32 && (D == 128 || D == 256) && !g_force_generic && !a.precise) {
        int rc = launch_row8_kernel(mode, dtype, D, a, st);
        if (rc != MLSTM_ESHAPE) return rc;  // extremely long sequences do not fit its LDS budget
    }
    return launch_row_kernel(mode, dtype, D, a, st);
}

struct ColArgs {
    const void* Q; const void* K; const void* V; const void* dH;
    void* dK; void* dV;
    float* colsum;    // [BH,S] fp32 column sums of dD (= dI before the cast)
    float* rowpart;   // [BH,RS,S] fp32 partial row sums of dD, one slice per key tile (RS = NG), or, in chunks, per key
                      // tile of the position's own chunk (RS = chunk_len / 64: slice = key tile modulo RS)
    int RS;
    const float* alpha2; const float* beta2; const double* G2;
    const float* inv_n; const float* db;
    int BH, S, NG;
    // long sequences in chunks (col16_kernel only): with chunk_len > 0 the keys walk the queries of their own chunk and
    // take the contribution of the queries behind it from the chunk's reverse states (ChunkArgs::reverse); rowpart is then
    // written for the key tiles of the query's own chunk only
    int chunk_len;
    int n_states;
    const void* Ev;          // [BH][n_states][D][D] reverse states, value-major (ChunkArgs::CstT of the reverse pass)
    const void* Ev_lo;       // split mode: their low-order terms
    const float* gvec;       // [BH][n_states][D]
    int precise;             // split mode (see RowArgs): G and W enter phase B as hi + lo
    Lay la, lb;              // layouts of Q, K, V, dK, dV (la) and of dH (lb)
};
int launch_col_kernel(int dtype, int D, const ColArgs& a, hipStream_t st);
// phase A as 16x16x32 products on two query halves, the element-wise part of the first between the MFMAs of the second;
// 16-bit types at D = 128 and 256 only
int launch_col16_kernel(int dtype, int D, const ColArgs& a, hipStream_t st);
// weights kept in registers between the two phases (no G / W tiles in LDS); 16-bit types at D = 128 and 256, split mode included
int launch_cold_kernel(int dtype, int D, const ColArgs& a, hipStream_t st);
extern int g_col_variant;   // see mlstm_set_column_kernel: 0 = the library's choice, 1 = col16_kernel, 2 = cold_kernel, 3 = col_kernel
inline int launch_col_best(int dtype, int D, const ColArgs& a, hipStream_t st) {
    const bool half_big = dtype != MLSTM_F32 && (D == 128 || D == 256);
    int variant = g_force_generic ? 3 : g_col_variant;
    if (!half_big || variant < 0 || variant > 3) variant = 3;
    if (variant == 0) variant = 2;   // (measured faster than col16_kernel at D = 128 and 256, chunked and not)
    if (variant == 1 && a.precise) variant = 2;   // (col16_kernel has no split mode)
    if (variant == 1 || variant == 2) {
        int rc = variant == 1 ? launch_col16_kernel(dtype, D, a, st) : launch_cold_kernel(dtype, D, a, st);
        if (rc != MLSTM_ESHAPE) return rc;  // extremely long sequences do not fit their LDS budget
    }
    return launch_col_kernel(dtype, D, a, st);
}

struct DfArgs {
    const void* F; const float* colsum; const float* rowpart;
    void* dF; void* dI;
    int BH, S, NG;
    int RS;                  // row-partial slices per head (see ColArgs)
    // in chunks: rowpart holds the slices of the key tiles of the position's own chunk only, rowinter the rest
    int chunk_len;
    const float* rowinter;
    const float* anchor;     // [BH][n_states]: the running sum of (col - row) at the first position of chunks 1, 2, ...
    int n_states;
    Lay lg;                  // layout of F, dF and dI
    int gate_form;           // what F holds (see launch_gates); dF is the gradient of that same quantity
    // chunk_len <= 1024: the anchors come as partial sums instead (ChunkArgs::dot_part of the reverse states) and the
    // vector states of both directions, and the kernel adds them up itself
    const float* anchor_part = nullptr;   // [BH][n_states][anchor_parts]
    int anchor_parts = 0;
    const float* anchor_va = nullptr;     // [BH][n_states][D] each
    const float* anchor_vb = nullptr;
    int D = 0;
    SavedStamp stamp;        // compared by the first workgroup (src), if set
};
int launch_df(int gate_dtype, const DfArgs& a, hipStream_t st);

// States at the ends of the first NCS chunks of L positions of every head (16-bit types, D = 128 or 256), for the
// chunked forward of RowArgs: dC is scratch, Nst and Cst receive the states.
struct ChunkArgs {
    const void* K;
    const void* V;        // [BH,S,D]
    const float* alpha2;
    const float* beta2;
    const double* G2;
    float* dC;            // [BH][NCS][D][D] fp32 scratch: the chunks' own sums
    float* Nst;           // [BH][NCS][D]
    void* Cst;            // [BH][NCS][D][D], key-major: the forward contracts it over the key index; may be null
    void* CstT;           // the same states value-major, for the dQ pass; may be null
    int BH, S, NG, L, NCS;
    // reverse states for the keys of a chunk, summed over the queries behind it: K = Q, V = dH,
    //   E_c = sum_{i > e_c} exp(A_{e_c} - A_i) q_i (dh_i / n_i)^T / sqrt(D)  (Cst / CstT),  g_c likewise with db_i (Nst);
    // inv_n and db are the per-row scalars the dQ pass leaves
    int reverse;
    const float* inv_n;
    const float* db;
    Lay lk, lv;           // layouts of K and V
    // Split mode: the weighted V rows enter the chunk sums as two terms (hi + lo, two MFMAs per fragment) and every state
    // is written as two terms as well: Cst_lo / CstT_lo receive state - (state rounded to the element type), rounded.
    int precise;
    void* Cst_lo;
    void* CstT_lo;
    // The value-major carry can contract the states it forms (before rounding) with another set in the same layout
    // (dot_with, dot_with_lo: its low-order terms or null): dot_part[bh][c][workgroup of the head] receives the partial
    // sums of <state_c, dot_with_c>, (D / 64)^2 per state.
    const void* dot_with = nullptr;
    const void* dot_with_lo = nullptr;
    float* dot_part = nullptr;
};
int launch_chunk_states(int dtype, int D, const ChunkArgs& a, hipStream_t st);
// whether the carry of these shapes takes ChunkArgs::dot_part (otherwise launch_anchor forms the contraction)
bool chunk_states_fused_dot(int dtype, int D);
// partial sums per state that the launch with these arguments leaves in ChunkArgs::dot_part
int chunk_states_dot_parts(int dtype, int D, const ChunkArgs& a);
// test and measurement aid: 0 = the library's choice by the size of the launch, 1 = chunk sums and carry (two kernels),
// 2 = the one-pass kernel wherever it can serve
int set_state_kernel(int variant);

// anchor[bh][c] = <A_c, B_c> + va_c . vb_c over two sets of states in the same layout; A_lo, B_lo (both or neither):
// their low-order terms (split mode)
int launch_anchor(int dtype, int D, const void* A, const void* B, const void* A_lo, const void* B_lo, const float* va, const float* vb,
                  float* anchor, int BH, int NCS, hipStream_t st);

// Backward of the output gate h_out = silu(o) * h, element-wise over n elements (n a multiple of 8):
//   dh = dh_out * silu(o)   (the upstream gradient of the ungated form),   d_o = dh_out * h * silu'(o).
int launch_gate_backward(int dtype, const void* dh_out, const void* o, const void* h, void* dh, void* d_o, size_t n, hipStream_t st);
// the same over [BH, S, D] tensors in layouts: dh_out, o, d_o in lx, h in lh, dh in ld
int launch_gate_backward_rows(int dtype, const void* dh_out, const void* o, const void* h, void* dh, void* d_o, int BH, int S, int D,
                              const Lay& lx, const Lay& lh, const Lay& ld, hipStream_t st);

struct ScanArgs {
    const float* q; const float* k; const float* v; const float* o;
    float* h;             // unnormalised numerator (first key range), then the output
    float* hpart;         // [KS-1, BH, S, D] numerators of the other key ranges
    const float* alpha2; const float* beta2; const double* G2; const float* M;
    float* P;             // [BH, NC, 64, 64] in-chunk pair weights
    float* Nst;           // [BH, NC, D] vector state n~ at every chunk end
    int BH, S, D, NC;
    // What the last kernel writes to h: 0 = silu(o) * numerator / n (the scan form's output), 1 = numerator / n (ungated),
    // 2 = the numerator itself, sum_j exp(a_j - A_t) (q_t . k_j) / sqrt(D) v_j: the causal weighted sum the backward pass
    // reuses with other operands in the places of q, k and v, finished as `ep` says.  Bout (may be null): the normaliser
    // sums b_t, modes 0 and 1.
    int finish_mode;
    float* Bout;
    float* Hun;           // mode 0 only, may be null: numerator / n next to the gated output (what a backward wants kept)
    // rev (mode 2 only): q, k and v hold the sequence in its own order and the pipeline walks it from the end: position t
    // of the walk is row S-1-t of q, k and v.  Gate arrays, P, Nst, h and hpart are in walk order.
    int rev;
    // Mode 2 can carry a vector sum along with the matrix one (ep.vec):
    //   numerator_t = sum_{j<=t} exp(a_j - A_t) / sqrt(D) ((q_t . k_j) + rs_t cs_j) v_j
    // rs = ep.row_scale ([BH,S], walk order; null: 1), cs = col_scale ([BH,S], in the order of the rows of q, k, v; null: 1).
    // The pairs inside a chunk take the term into their weights P; the chunks before it come through Nst, which then holds
    // sum_j exp(a_j - A_end) / sqrt(D) cs_j v_j at the chunk ends.  What the last kernel then does with row t:
    //   x = numerator_t (+ rs_t decay_t Nst_{c-1}),  x *= exp2(wd_alpha2_j - wd_beta2_j)  (gate arrays of the output row j; may be null)
    //   out_j = x  with j = t, or S-1-t when out_rev             (out null: h, in place; out_rev needs out != h)
    //   dot_out_j = dot_with_j . x,  x_out_j = dot_out_j - dot_minus_j                              (each may be null)
    const float* col_scale;
    struct Epilogue {
        float* out; int out_rev;
        int vec; const float* row_scale;
        const float* wd_alpha2; const float* wd_beta2;
        const float* dot_with; float* dot_out; const float* dot_minus; float* x_out;
    } ep;
    // segments of the sequence that the state kernel runs side by side (filled in by launch_scan from scan_segments);
    // seg_state: scan_segment_state_bytes() bytes of scratch for the states at the segment ends, needed when nseg > 1
    float* seg_state;
    int nseg, seg_chunks;
};
int scan_key_splits(int BH, int D);
void scan_segments(int BH, int S, int D, int* nseg, int* seg_chunks);
size_t scan_segment_state_bytes(int BH, int S, int D);
// mark(kernel id, stream, begin?) brackets groups of launches for the optional event timing
int launch_scan(const ScanArgs& a, int KS, hipStream_t st, void (*mark)(int, hipStream_t, bool));
// n~ at every chunk end from the chunks' own sums, in place (ScanArgs::Nst, beta2, G2, BH, NC, D are read)
void launch_scan_ncarry(const ScanArgs& a, hipStream_t st);

// Backward of the scan form (mlstm_scan_bwd.hip): every pointer fp32, [B,NH,S,D] or [B,NH,S]; ws holds
// scan_backward_workspace_bytes(BH, S, D) bytes.  o == null: no output gate (dhg is the gradient of the ungated
// output, d_o is not written)
struct ScanBwdArgs {
    const float* dhg; const float* q; const float* k; const float* v; const float* f; const float* i; const float* o;
    float* dq; float* dk; float* dv; float* df; float* di; float* d_o;
    int BH, S, D;
    // the forward's ungated output and normaliser sums, if the caller kept them (both or neither): the forward is then not
    // run again
    const float* h_kept; const float* b_kept;
};
size_t scan_backward_workspace_bytes(int BH, int S, int D);
int launch_scan_backward(const ScanBwdArgs& a, char* ws, hipStream_t st, void (*mark)(int, hipStream_t, bool));
// dF_t = sigmoid(-f_t) * sum_{s<t} x_s over each head (x: [BH,S] fp32; dF_0 = 0): the scan of launch_df on its own
int launch_dfscan_plain(int gate_dtype, const void* F, const float* x, void* dF, int BH, int S, hipStream_t st);

}  // namespace mlstm
