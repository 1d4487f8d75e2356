/*
 * libmlstm_hip.so -- C ABI of the MI355X (gfx950) mLSTM kernels.
 *
 * Every pointer is caller-owned DEVICE memory, row-major contiguous; the library never frees or keeps it.
 * Calls are asynchronous on the given HIP stream (NULL = the default stream) and return 0 on success, a positive
 * hipError_t on a runtime failure, or a negative MLSTM_E* code for a rejected argument.  They never abort and never
 * throw.  The compute entry points may be called from several threads at once (on different streams and buffers);
 * the process-wide settings further down (timing, chunk length, generic kernels, spin limit) are test and
 * measurement aids: they are not synchronised with calls in flight and must not change between a forward and the
 * backward that reads its `saved` buffer.  Shapes: q, k, v, h, dh, o and their gradients are [B, NH, S, D];
 * f, i, m, b and their gradients are [B, NH, S].
 *
 * Each entry point names the interface of the reference it replaces (paths relative to the reference
 * checkout, LukasBluebaum/xLSTM-Triton-CUDA-Implementation).
 */
#ifndef MLSTM_HIP_H
#define MLSTM_HIP_H
#include <stddef.h>
#ifdef __cplusplus
extern "C" {
#endif

/* element types */
#define MLSTM_F32 0
#define MLSTM_F16 1
#define MLSTM_BF16 2

/*
 * Split mode, or-ed into the `dtype` argument of the *_ex entry points (16-bit types; no effect on MLSTM_F32).
 * The 16-bit kernels round the weights C~ (and their backward counterparts) to the element type before the second
 * product of a tile, as every tensor-core implementation does; an output element is a sum of terms that can be far
 * larger than the element itself, so that rounding shows as an absolute error of about 2^-9 (bf16) of the terms'
 * size.  With MLSTM_PRECISE every such operand enters its product as two terms, hi + lo, each in the element type
 * (two MFMAs per fragment), and the forward hands the low-order part of h to the backward (the `saved` buffer of
 * mlstm_forward_save_ex, or a recomputation), which makes the results agree with an fp32 evaluation of the
 * reference's formulas (mlstm_matmul.py:104-118, :336-365) to rtol 2e-2 / atol 2e-3 element by element.  Long
 * sequences run in chunks in this mode too, with every chunk state kept as two terms.  Price: the four-wave kernels
 * instead of the eight-wave ones, and half as many MFMAs again.
 */
#define MLSTM_PRECISE 0x100

/*
 * Layout of the caller's tensors, for the entry points that take one (names ending in _lx).  Element (b, h, s, d) of
 * a [B,NH,S,D] tensor lies at  b * stride_b + h * stride_h + s * stride_s + d  elements from its base pointer: the
 * head dimension is contiguous, everything else is free, so the [B,S,NH,D] activations of a projection (stride_b =
 * S*NH*D, stride_h = D, stride_s = NH*D), or the q / k / v slices of one fused [B,S,3,NH,D] projection, are taken as
 * they are, without the transposing copy the reference needs in front of its kernels (the step the reference's
 * cutlass-src-hopper/mlstm_forward.cu:201 suggests fusing away).  One layout for q, k, v and their gradients, one for
 * h and its gradient, one (without d) for the gates f, i and their gradients.  Rows must start on 16-byte boundaries:
 * base pointers 16-byte aligned, qkv / out strides multiples of 8 elements (16-bit types) or 4 (fp32).
 * A layout in which the library WRITES (out for the forward's h; qkv and gates for the backward's gradients) must not
 * overlap itself: an expanded view (a stride of 0 over more than one index) or interleaved rows would have several
 * workgroups write one address, so such a layout is refused with MLSTM_EINVAL (pass a dense copy instead).  Tensors that
 * are only read may overlap.
 * gate_form says what `f` holds: the forget gate's pre-activation (the reference's input, mlstm_matmul.py:57), its
 * log-sigmoid, or the cumulative sum of the log-sigmoid over the positions of each head (what mlstm_matmul.py:57-58
 * compute first; fp32 gates only: the sum reaches 1e3..1e4 and 16-bit types cannot hold it).  The backward returns
 * in `df` the gradient of whatever `f` held.  m and b (statistics) are always dense [B,NH,S] fp32.
 */
#define MLSTM_GATE_RAW 0
#define MLSTM_GATE_LOGSIGMOID 1
#define MLSTM_GATE_CUMSUM 2
typedef struct mlstm_layout {
    long long qkv_stride_b, qkv_stride_h, qkv_stride_s;
    long long out_stride_b, out_stride_h, out_stride_s;
    long long gate_stride_b, gate_stride_h, gate_stride_s;
    int gate_form;
} mlstm_layout;

/* argument errors */
#define MLSTM_EINVAL (-1)      /* null pointer, non-positive size, unknown dtype */
#define MLSTM_ESHAPE (-2)      /* head dimension / sequence length not supported by this build */
#define MLSTM_EWORKSPACE (-3)  /* caller workspace smaller than mlstm_workspace_bytes() */
#define MLSTM_EKERNEL (-4)     /* a kernel's bounded wait expired (mlstm_kernel_error) */
#define MLSTM_EBUILD (-6)      /* a kernel with hand-counted memory waits was compiled with register spills: refused */
#define MLSTM_ESAVED (-5)      /* a backward was given a `saved` buffer written for another shape or setting (mlstm_kernel_error) */

/* operations, for mlstm_workspace_bytes */
#define MLSTM_OP_FORWARD 0
#define MLSTM_OP_BACKWARD 1
#define MLSTM_OP_SCAN_FORWARD 2
#define MLSTM_OP_FORWARD_GATED 3
#define MLSTM_OP_BACKWARD_GATED 4
#define MLSTM_OP_SCAN_BACKWARD 5

/*
 * Single-head fp16 forward, D = 128, default stream: the launch of the CUDA harness,
 *   mlstm_forward<64,16,128,16,8,8><<<S/64,128,smem>>>(Q,K,V,F,I,H,S)
 * (cuda-src/mlstm_forward.cu:12-15, launched at :237-238).  Q, K, V, H are [S,128] halves, F, I are [S].
 */
int mlstm_forward(const void* Q, const void* K, const void* V, const void* F, const void* I, void* H, unsigned S);

/*
 * Single-head fp16 backward, D = 128, default stream: the two launches of the CUDA backward harness,
 *   matmul_backward_db(dH,Q,K,V,F,I,M,B,dB,S)  and  matmul_backward(dH,dB,Q,K,V,dQ,dK,dV,F,I,dI,M,B,S)
 * (cuda-src/mlstm_backward.cu:11-12,177-178, launched at :620-628), completed with dV, dF and dI, which the
 * reference kernels leave unwritten.  M and B (the harness takes them from its CPU pass, in half precision)
 * are accepted for signature compatibility and may be NULL: the stabiliser and normaliser are recomputed in
 * fp32.  dB follows sign(b) (mlstm_matmul.py:196), not the harness' signbit(b).
 */
int mlstm_backward(const void* dH, const void* Q, const void* K, const void* V, const void* F, const void* I,
                   const void* M, const void* B, void* dQ, void* dK, void* dV, void* dF, void* dI, unsigned S);

/*
 * General forward: what Triton_mLSTM.forward / mlstm_matmul launch,
 *   mlstm_matmul_kernel[grid](q,k,v,f,i,m,b,h,NH,S,D,SB)        (mlstm_matmul.py:38-101, :121-129, :371-381).
 * dtype is the element type of q, k, v and h; gate_dtype that of f and i; m and b are always fp32.
 * D in {64,128,256} for fp16 / bf16, {64,...,1024} (powers of two) for fp32; any S >= 1.  fp32 at D >= 256 runs on
 * the scan form's kernels (same function, see mlstm_scan_forward_ex): the tile kernels hold a row block's D columns
 * in accumulator registers and two D-wide tiles per stage in LDS, which ends at D = 128 in fp32 and at D = 256 in
 * 16 bits; a D = 512 16-bit variant would need the head dimension tiled as well (a second kernel family), and is not
 * built.  (The Python wrappers serve what lies outside these sets on the same entry points: D = 16 and 32 zero-padded to
 * four times D with q scaled by 2, which is exact; 16-bit tensors at D = 512 / 1024 widened to fp32.)  At those fp32 sizes the tensors must be dense, the gates fp32 pre-activations, and the backward recomputes
 * the forward (h, m, b are ignored); the gated entry points and layouts of the caller's return MLSTM_ESHAPE there.
 * workspace may be NULL (the library then allocates and frees stream-ordered); otherwise it must hold
 * mlstm_workspace_bytes(MLSTM_OP_FORWARD, ...) bytes.
 */
int mlstm_forward_ex(const void* q, const void* k, const void* v, const void* f, const void* i, void* h, float* m,
                     float* b, int B, int NH, int S, int D, int dtype, int gate_dtype, void* workspace,
                     size_t workspace_bytes, void* stream);

/*
 * mlstm_forward_ex for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  Same arguments and results as
 * mlstm_forward_ex without the workspace: the scratch is a static device array of MLSTM_NOALLOC_MAX_WORKSPACE bytes
 * inside the library (each GPU the library runs on holds one until the process ends), and the call performs no
 * hipMalloc / hipFree, stream-ordered or otherwise.  Shapes whose mlstm_workspace_bytes(MLSTM_OP_FORWARD, ...) exceeds
 * that size are rejected with MLSTM_EWORKSPACE.  All calls on one GPU share the one array: two calls that overlap in
 * time on the same GPU (different streams or threads) race; calls on one stream are ordered and safe.
 * (With mlstm_timing_enable on, events are created around the launches; leave it off in such callers.)
 * The first call on a device looks up the array's address (a mutex and a runtime query) and the first launch of each
 * kernel variant raises that kernel's LDS limit (hipFuncSetAttribute): neither belongs inside a stream capture.  Make
 * one ordinary call per device and shape class before capturing (mlstm_init() does the address lookup alone).
 */
#define MLSTM_NOALLOC_MAX_WORKSPACE (8u << 20)
int mlstm_forward_noalloc_ex(const void* q, const void* k, const void* v, const void* f, const void* i, void* h, float* m,
                             float* b, int B, int NH, int S, int D, int dtype, int gate_dtype, void* stream);

/*
 * General backward: what Triton_mLSTM.backward launches,
 *   mlstm_matmul_kernel_backward_db / _backward / _df           (mlstm_matmul.py:133-333, :384-405).
 * h, m, b are the forward's outputs (h in `dtype`, m and b fp32); any of them may be NULL, in which case all
 * three are recomputed.  dq, dk, dv are written in `dtype`, df and di in `gate_dtype`; df[..., 0] = 0.
 */
int mlstm_backward_ex(const void* dh, const void* q, const void* k, const void* v, const void* f, const void* i,
                      const void* h, const float* m, const float* b, void* dq, void* dk, void* dv, void* df, void* di,
                      int B, int NH, int S, int D, int dtype, int gate_dtype, void* workspace, size_t workspace_bytes,
                      void* stream);

/*
 * Forward and backward of a training step that hand the chunk states over: what Triton_mLSTM.forward keeps for its
 * backward with ctx.save_for_backward (mlstm_matmul.py:379: q, k, v, f, i, m, b), plus, for sequences that run in
 * chunks, the states at the chunk ends and the gate pre-pass, so that the backward does not form them again.  `saved` is caller-owned device
 * memory of mlstm_saved_state_bytes(...) bytes (0 for shapes that do not run in chunks: saved may then be NULL), written
 * by mlstm_forward_save_ex and read by mlstm_backward_saved_ex for the same inputs and the same dtype argument; the
 * process-wide settings (mlstm_set_chunk_length, mlstm_force_generic_kernels) must not change in between.  saved_bytes
 * must equal mlstm_saved_state_bytes at the time of either call (checked on the host), and the buffer starts with a
 * header -- shape, dtype argument, chunk length, kernel switch -- that the forward writes and the backward compares ON
 * THE DEVICE, without a host round trip: a mismatch sets the per-GPU error word, the backward's results are then
 * garbage (all reads stay inside the buffers), and mlstm_kernel_error() reports MLSTM_ESAVED.  Otherwise as mlstm_forward_ex / mlstm_backward_ex, with h, m
 * and b required in the backward.  MLSTM_EWORKSPACE also reports a `saved` buffer that is missing or too small.
 */
size_t mlstm_saved_state_bytes(int B, int NH, int S, int D, int dtype);
int mlstm_forward_save_ex(const void* q, const void* k, const void* v, const void* f, const void* i, void* h, float* m,
                          float* b, void* saved, size_t saved_bytes, int B, int NH, int S, int D, int dtype,
                          int gate_dtype, void* workspace, size_t workspace_bytes, void* stream);
int mlstm_backward_saved_ex(const void* dh, const void* q, const void* k, const void* v, const void* f, const void* i,
                            const void* h, const float* m, const float* b, const void* saved, size_t saved_bytes,
                            void* dq, void* dk, void* dv, void* df, void* di, int B, int NH, int S, int D, int dtype,
                            int gate_dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * The four entry points above for tensors in a layout of the caller's (see mlstm_layout; null = dense, which makes
 * each identical to its _ex namesake): the activations of a [B,S,NH,D] projection, or the slices of a fused q/k/v
 * projection, go in without a transposing copy, the forget gate may come as its log-sigmoid or as the cumulative sum
 * of that, and h, dq, dk, dv, df, di are written in the same layouts.  The kernels address rows through the layout's
 * strides; nothing else changes, and results are bit-identical to a run on dense copies.  No counterpart in the
 * reference, whose kernels take contiguous [B,NH,S,D] only (mlstm_matmul.py:121-129, :368-405); the hint to take the
 * step before the kernel into it is at cutlass-src-hopper/mlstm_forward.cu:201.
 */
int mlstm_forward_lx(const void* q, const void* k, const void* v, const void* f, const void* i, void* h, float* m, float* b,
                     int B, int NH, int S, int D, int dtype, int gate_dtype, const mlstm_layout* layout, void* workspace,
                     size_t workspace_bytes, void* stream);
int mlstm_backward_lx(const void* dh, const void* q, const void* k, const void* v, const void* f, const void* i, const void* h,
                      const float* m, const float* b, void* dq, void* dk, void* dv, void* df, void* di, int B, int NH, int S,
                      int D, int dtype, int gate_dtype, const mlstm_layout* layout, void* workspace, size_t workspace_bytes,
                      void* stream);
int mlstm_forward_save_lx(const void* q, const void* k, const void* v, const void* f, const void* i, void* h, float* m, float* b,
                          void* saved, size_t saved_bytes, int B, int NH, int S, int D, int dtype, int gate_dtype,
                          const mlstm_layout* layout, void* workspace, size_t workspace_bytes, void* stream);
int mlstm_backward_saved_lx(const void* dh, const void* q, const void* k, const void* v, const void* f, const void* i, const void* h,
                            const float* m, const float* b, const void* saved, size_t saved_bytes, void* dq, void* dk, void* dv,
                            void* df, void* di, int B, int NH, int S, int D, int dtype, int gate_dtype, const mlstm_layout* layout,
                            void* workspace, size_t workspace_bytes, void* stream);

/*
 * Matmul form with the output gate of the scan form, h_gated = silu(o) * h (mlstm_scan.py:277): the item the
 * reference leaves open for its matmul kernels ("Integrate o", mlstm_matmul.py:36; "could add multiplication by o
 * here", cuda-src/cpu_utils.cuh:161).  With it the matmul form returns what mlstm_scan() returns, and has a
 * backward.  The forward kernel writes both the ungated h (an input of the backward) and h_gated from the same
 * accumulators; o and h_gated are [B, NH, S, D] in `dtype`.  Other arguments as in mlstm_forward_ex.
 */
int mlstm_forward_gated_ex(const void* q, const void* k, const void* v, const void* f, const void* i, const void* o,
                           void* h, void* h_gated, float* m, float* b, int B, int NH, int S, int D, int dtype,
                           int gate_dtype, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward of mlstm_forward_gated_ex.  dh_gated is the gradient of h_gated; d_o receives the gradient of o, in
 * `dtype`.  h, m, b are the forward's ungated outputs (all three, or NULL to have them recomputed).  One
 * element-wise pass forms dh = dh_gated * silu(o) and d_o = dh_gated * h * silu'(o); the rest is mlstm_backward_ex
 * on dh.  Workspace: mlstm_workspace_bytes(MLSTM_OP_BACKWARD_GATED, ...).
 */
int mlstm_backward_gated_ex(const void* dh_gated, const void* q, const void* k, const void* v, const void* f,
                            const void* i, const void* o, const void* h, const float* m, const float* b, void* dq,
                            void* dk, void* dv, void* df, void* di, void* d_o, int B, int NH, int S, int D, int dtype,
                            int gate_dtype, void* workspace, size_t workspace_bytes, void* stream);
/*
 * The two gated entry points on tensors that lie where the caller keeps them (struct mlstm_layout, as for
 * mlstm_forward_lx / mlstm_backward_lx): q, k, v and dq, dk, dv in the qkv layout; h, h_gated, o, dh_gated and d_o in the
 * out layout; the gates and their gradients in the gate layout.  layout == NULL: dense tensors.  The backward's written
 * tensors must not overlap (MLSTM_EINVAL).  Not for fp32 at D >= 256 (MLSTM_ESHAPE).  No counterpart in the reference
 * (its gate is part of mlstm_scan only).
 */
int mlstm_forward_gated_lx(const void* q, const void* k, const void* v, const void* f, const void* i, const void* o,
                           void* h, void* h_gated, float* m, float* b, int B, int NH, int S, int D, int dtype,
                           int gate_dtype, const mlstm_layout* layout, void* workspace, size_t workspace_bytes,
                           void* stream);
int mlstm_backward_gated_lx(const void* dh_gated, const void* q, const void* k, const void* v, const void* f,
                            const void* i, const void* o, const void* h, const float* m, const float* b, void* dq,
                            void* dk, void* dv, void* df, void* di, void* d_o, int B, int NH, int S, int D, int dtype,
                            int gate_dtype, const mlstm_layout* layout, void* workspace, size_t workspace_bytes,
                            void* stream);

/*
 * Scan-form forward with the silu(o) output gate: what mlstm_scan() launches,
 *   stabilize_fi / precompute_mlstm_triton_scan / reduce_mlstm_triton / mlstm_triton_scan
 * (mlstm_scan.py:48-278, host :281-327).  fp32 only, like the reference; D in {64,...,1024} multiple of 64.
 */
int mlstm_scan_forward_ex(const void* q, const void* k, const void* v, const void* f, const void* i, const void* o,
                          void* h, int B, int NH, int S, int D, int dtype, void* workspace, size_t workspace_bytes,
                          void* stream);

/*
 * Backward of mlstm_scan(): gradients of q, k, v, f, i, o from the gradient of the gated output.  The reference has
 * no kernel for it (mlstm_scan.py holds a forward only; its differentiable counterpart is the PyTorch
 * mlstm_scan_pytorch, mlstm_scan.py:343-380); the gradients are those of mlstm_matmul.py:150-333 behind the gate of
 * mlstm_scan.py:277, evaluated with the scan form's own kernels (causal weighted sums with a matrix state carried
 * over chunks of 64 positions), so every head dimension of the forward is served.  Recomputes the forward: only the
 * inputs are needed.  fp32 only; dF[..., 0] = 0.  Workspace: mlstm_workspace_bytes(MLSTM_OP_SCAN_BACKWARD, ...).
 */
int mlstm_scan_backward_ex(const void* dh_gated, const void* q, const void* k, const void* v, const void* f, const void* i,
                           const void* o, void* dq, void* dk, void* dv, void* df, void* di, void* d_o, int B, int NH, int S,
                           int D, int dtype, void* workspace, size_t workspace_bytes, void* stream);
/* The same pair for a training step that keeps what its backward would otherwise form again: the forward also leaves the
 * ungated output h_ungated ([B,NH,S,D] fp32: numerator / n, before silu(o)) and the normaliser sums b ([B,NH,S]); the backward
 * that is handed both skips its forward pass (one of its four walks over the sequence) and returns the same bits.  Null
 * h_ungated and b make mlstm_scan_backward_saved_ex identical to mlstm_scan_backward_ex. */
int mlstm_scan_forward_save_ex(const void* q, const void* k, const void* v, const void* f, const void* i, const void* o, void* h,
                               void* h_ungated, float* b, int B, int NH, int S, int D, int dtype, void* workspace,
                               size_t workspace_bytes, void* stream);
int mlstm_scan_backward_saved_ex(const void* dh_gated, const void* q, const void* k, const void* v, const void* f, const void* i,
                                 const void* o, const void* h_ungated, const float* b, void* dq, void* dk, void* dv, void* df,
                                 void* di, void* d_o, int B, int NH, int S, int D, int dtype, void* workspace,
                                 size_t workspace_bytes, void* stream);

/*
 * sLSTM cell, forward and backward (fp32).  The reference lists the cell as an open item (README.md:9) and has no code
 * for it; these implement the published cell (Beck et al., arXiv:2405.04517, section 2.2 and appendix A.2) per head:
 *   pre_g = wx[b,t,g,h,:] + r[h,g] h_{t-1} + b[h,g]   (g = i, f, z, o),  m_t = max(log f_t + m_{t-1}, i~),
 *   c_t = exp(log f_t + m_{t-1} - m_t) c_{t-1} + exp(i~ - m_t) tanh(z~),  n_t likewise with 1,  h_t = sigmoid(o~) c_t / n_t,
 * log f_t = f~ or, with forget_sigmoid != 0, logsigmoid(f~); zero initial state.
 * wx, dwx: [B,S,4,NH,DH] (the input projections of the four gates, computed by the caller's GEMM); r, dr: [NH,4,DH,DH]
 * (r[h][g][j][k]: unit j from unit k); b, db: [NH,4,DH]; h, dh: [B,S,NH,DH]; DH in {32, 64, 128}.
 * slstm_forward_ex writes what the backward needs into `saved` (slstm_saved_bytes; may be NULL for inference; opaque:
 * written and read by the same build of the library).  All tensors dense.
 * slstm_backward_ex needs a workspace of slstm_workspace_bytes.  One workgroup per (batch, head) walks the sequence:
 * the cell is sequential in t by construction.
 */
size_t slstm_saved_bytes(int B, int NH, int S, int DH);
size_t slstm_workspace_bytes(int B, int NH, int S, int DH);
int slstm_forward_ex(const float* wx, const float* r, const float* b, float* h, float* saved, int B, int NH, int S, int DH,
                     int forget_sigmoid, void* stream);
int slstm_backward_ex(const float* dh, const float* h, const float* r, const float* saved, float* dwx, float* dr, float* db,
                      int B, int NH, int S, int DH, int forget_sigmoid, void* workspace, size_t workspace_bytes,
                      void* stream);

/* Bytes of scratch the operation needs for this shape (the torch.zeros workspaces of mlstm_scan.py:299-307 and
 * the db buffer of mlstm_matmul.py:394 are the reference's counterparts). */
size_t mlstm_workspace_bytes(int op, int B, int NH, int S, int D, int dtype);

/*
 * Measurement aid with no counterpart in the reference (which has no timing code at all): when enabled, every
 * kernel launch of the entry points above is bracketed by HIP events recorded on the launch stream.
 * mlstm_timing_read waits for the recorded launches of one kernel, returns their summed duration and count, and
 * forgets them.  Off by default; enabling it is process-wide.
 */
#define MLSTM_K_GATES 0     /* gate pre-pass */
#define MLSTM_K_ROW_FWD 1   /* forward tile kernel (H, b) */
#define MLSTM_K_COL 3       /* backward tile kernel (dK, dV, dI, row partials) */
#define MLSTM_K_ROW_DQ 4    /* backward tile kernel (dQ) */
#define MLSTM_K_DF 5        /* row reduce + dF scan */
#define MLSTM_K_SCAN_STATE 6
#define MLSTM_K_SCAN_CARRY 7
#define MLSTM_K_SCAN_OUT 8
#define MLSTM_K_GATE_BWD 9  /* element-wise backward of the output gate (gated matmul form only) */
#define MLSTM_K_CHUNK_STATES 10  /* chunk sums + carry (forward and reverse states) of sequences that run in chunks */
#define MLSTM_K_SCAN_GLUE 11     /* row-wise and vector-sum kernels between the scans of the scan form's backward */
int mlstm_timing_enable(int on);
/* An event pair costs the stream about 10 us of idle time around the launch it brackets.  mlstm_timing_select narrows
 * the timing to the kernels whose bit (1u << MLSTM_K_...) is set in `mask` and, of their launches, to every
 * `every`-th one (>= 1), so that a timed run is disturbed as little as the measurement needs.  Default: all
 * kernels, every launch.  Process-wide; resets the launch counters. */
int mlstm_timing_select(unsigned mask, int every);
int mlstm_timing_read(int kernel, double* total_ms, int* launches);

/*
 * Test aid with no counterpart in the reference: the 16-bit types at D >= 128 are normally served by an eight-wave
 * row kernel and fall back to the generic four-wave kernel only when a sequence is too long for its LDS budget.  With
 * `on` != 0 every shape goes through the generic kernels, so that the fallback can be tested at sizes the CPU oracle
 * can check.  Process-wide; returns the previous setting.
 */
int mlstm_force_generic_kernels(int on);

/*
 * Test and measurement aid with no counterpart in the reference.  The tile kernels (every type; D = 64, 128, and 256 in
 * 16 bits) cut sequences of 1024 positions and more into chunks -- 512 positions for the 16-bit types at D = 128 / 256,
 * 256 at D = 64, 128 for fp32 -- : a row walks the keys of its own chunk and takes everything
 * before it from the matrix state at the end of the previous chunk (the state of mlstm_scan.py:16-26; both forms are
 * the same function); the backward's keys likewise take the queries behind their chunk from a reverse state.  length > 0 (a multiple of 128) forces that chunk length, length < 0 switches chunking off,
 * 0 restores the default.  Process-wide; returns 0, or MLSTM_EINVAL for a length that is not a multiple of 128.
 * Workspace sizes depend on it: query mlstm_workspace_bytes after changing it.
 */
int mlstm_set_chunk_length(int length);
/*
 * Measurement and test aid: which column kernel (dK, dV, dI) serves the 16-bit types at D = 128 and 256.
 * 0 = the library's choice, 1 = col16_kernel (G / W through LDS, 16x16 MFMA chains), 2 = cold_kernel (G / W stay in
 * registers; the only one of the two with a split mode), 3 = the generic four-wave col_kernel.  Process-wide; returns 0,
 * or MLSTM_EINVAL.  No counterpart in the reference.
 */
int mlstm_set_column_kernel(int variant);
/*
 * Measurement and test aid: which kernels form the chunk states of the 16-bit types at D = 128 and 256.
 * 0 = the library's choice (chunk sums and carry today), 1 = chunk sums and carry (two kernels, any size, split mode),
 * 2 = the one-pass kernel ((D / 64) * 2 workgroups per head walk the chunks in order, no fp32 sums through memory)
 * wherever it can serve (not in split mode, at most 256 states per head).  The two weight different operands (V, K), so
 * their states differ by the rounding of a weighted 16-bit operand, like two runs of different tilings.
 * Process-wide; returns 0, or MLSTM_EINVAL.  No counterpart in the reference.
 */
int mlstm_set_state_kernel(int variant);
/* The chunk length the entry points use for this shape under the current setting, 0 = the sequence is not cut
 * (measurement aid: the work a chunked kernel executes depends on it). */
int mlstm_chunk_length_for(int S, int D, int dtype);

/*
 * Fail-safe of the eight-wave row kernel, no counterpart in the reference.  Inside a workgroup its producer waves wait
 * for an LDS counter before they reuse a buffer; the wait is bounded, and if it ever expires (a bug: it cannot in a
 * correct build) the kernel sets a per-GPU error word and runs on to its end instead of hanging the GPU.
 * mlstm_kernel_error waits for ALL work of the current device (hipDeviceSynchronize: every stream, the non-blocking
 * ones included), returns MLSTM_EKERNEL if an expired wait set the word (MLSTM_ESAVED if only a mismatched `saved`
 * buffer did, see mlstm_forward_save_ex) (results since the last call are then not to be trusted) and
 * clears it, 0 otherwise.  Work launched by other threads between its read and its clear can lose an error.  mlstm_set_spin_limit is the test aid for it:
 * limit > 0 replaces the bound (loop iterations), limit < 0 makes every such wait count as expired without waiting
 * (the results of that run are undefined), 0 restores the default.  Process-wide.
 */
int mlstm_kernel_error(void);
int mlstm_set_spin_limit(int limit);

/* Per-device set-up that the first call on a device would otherwise do (the addresses of the library's static device
 * arrays): call with that device current; returns 0 or a HIP error.  Optional, and idempotent. */
int mlstm_init(void);

/* Library version string, e.g. "mlstm_hip 0.1 gfx950". */
const char* mlstm_version(void);

#ifdef __cplusplus
}
#endif
#endif
