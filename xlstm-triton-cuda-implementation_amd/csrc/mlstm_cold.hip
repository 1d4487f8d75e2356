// Column-parallel backward kernel for the 16-bit types at D = 128 and 256 whose weights never leave the registers.
// Phase A is computed NOT transposed, S = Q K^T and dC = dH V^T with the queries along the accumulator rows and the keys
// along the lanes, so that the element-wise results G and W, still in accumulator layout, ARE the second operands of
// phase B (dK^T += Q^T G, dV^T += dH^T W: contraction over the queries, which are the accumulator's registers) -- the
// same trick the row kernels use between their two products.  There is no G / W tile in LDS, no transposing read of one,
// no barrier between the phases, and split mode (ColArgs::precise: G and W as hi + lo) costs registers only.
//
//   workgroup: 128 keys, four waves with 32 keys each (kb = wave), query tiles of 32 rows.
//   phase A:   S, dC for the wave's 32 keys x the tile's 32 queries (K fragments stationary in registers, V fragments
//              from an LDS tile that stays for the whole kernel), then per element
//              E = exp2(alpha_j - beta_i + dG) / sqrt(D),  C~ = S E,  dC~ = dC / n_i + db_i,  G = dC~ E,  W = C~ / n_i,  dD = C~ dC~.
//   phase B:   dK^T[:, its keys] += Q^T G,  dV^T[:, its keys] += dH^T W over all D columns: a wave owns its keys' rows of dK
//              and dV outright (256 accumulator registers at D = 256), nothing is exchanged between waves.
// A lane holds one key and 16 queries of a block, so the key's scalars are one register each and the column sums of dD one
// accumulating register; the queries' scalars (beta, 1/n, db) come from LDS four at a time, and the row sums of dD are
// reduced across the lanes (v_permlane16_swap folds register pairs, DPP row shifts add up 16 lanes) between the MFMAs of
// phase B.  A query tile is 32 rows so that two stages of Q and dH (64 KB at D = 256) and the V tile (64 KB) fit the LDS.
// In chunks (ColArgs::chunk_len) a state phase precedes the query loop:  dK_j = w_j (E v_j + g),  dV_j = w_j E^T k_j  with the
// chunk's reverse state E, which streams through the (then idle) query stages.
// Replaces the dK/dV/dI loop of mlstm_matmul_kernel_backward (mlstm_matmul.py:269-316) and matmul_backward
// (cuda-src/mlstm_backward.cu:402-518).
#include <type_traits>
#include "mlstm_device.h"
#include "mlstm_kernels.h"

namespace mlstm {

constexpr int CD_KEYS = 128, CD_QT = 32;

template <typename T, int D>
struct ColdCfg {
    static constexpr size_t V_BYTES = (size_t)CD_KEYS * D * sizeof(T);                 // the keys' V rows, resident
    static constexpr size_t QT_BYTES = (size_t)CD_QT * D * sizeof(T);                  // a 32-row tile of Q or dH
    static constexpr size_t STAGES_BYTES = 4 * QT_BYTES;                               // two stages of (Q, dH); the state tiles before them
    static constexpr size_t ROW_BYTES = 2 * 3 * GRAN * sizeof(float);                  // per stage: beta, 1/n, db (64 floats copied, 32 used)
    static constexpr size_t MISC_BYTES = (2 * 4 * CD_QT + 64 + D) * sizeof(float);     // row sums [2 parities][4 key blocks][32], 64 sink words, the vector state
    static constexpr size_t LDS_BYTES = V_BYTES + STAGES_BYTES + ROW_BYTES + MISC_BYTES;   // plus one float per 64-position granule
};

// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its second: one swap and one
// add fold a pair of registers (a, b) into one that holds a(l) + a(l ^ 16) in the even rows and b(l) + b(l ^ 16) in the odd ones.
__device__ __forceinline__ float fold_pair(float a, float b) {
    auto r = __builtin_amdgcn_permlane16_swap(__builtin_bit_cast(int, a), __builtin_bit_cast(int, b), false, false);
    return __builtin_bit_cast(float, (int)r[0]) + __builtin_bit_cast(float, (int)r[1]);
}
__device__ __forceinline__ float row_total(float v) {   // lane 15 of each 16-lane row: the row's sum
    v += dpp_f<0x111>(0.f, v);
    v += dpp_f<0x112>(0.f, v);
    v += dpp_f<0x114>(0.f, v);
    v += dpp_f<0x118>(0.f, v);
    return v;
}

// 32x32x16 MFMA whose accumulator is held in ordinary vector registers, for D = 256.  With a budget of 512 registers per
// lane the compiler gives every MFMA it emits an accumulator in the second half of the register file (AGPRs), which this
// kernel's output accumulators fill to the last register at D = 256; the 32 registers of phase A's two products would push
// two output blocks out to scratch memory at every step.  Issued from inline assembly they stay where the element-wise part
// wants them anyway.  The compiler does not know what the instruction is, so the wait states it would insert are written
// out: two in front of every MFMA (an operand written by a vector instruction just before it) and four behind it (an
// operand overwritten just after it), both in the shadow of the MFMA that is executing; settle() before the first ordinary
// instruction that reads the result (an MFMA of 8 passes needs 11 wait states; 2 x 16 are given).  Two chains issued in
// turns need none between their MFMAs.  At D = 128 the accumulators leave room and the compiler's own MFMAs are used: there
// it parks the stationary K fragments in AGPRs and moves them in and out right next to the MFMAs, which only it can pad.
template <typename T> struct MmaV;
template <> struct MmaV<__bf16> {
    static __device__ __forceinline__ void first(f32x16& c, bf16x8 a, bf16x8 b) {
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, 0\n\ts_nop 3" : "=&v"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void next(f32x16& c, bf16x8 a, bf16x8 b) {
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_bf16 %0, %1, %2, %0\n\ts_nop 3" : "+v"(c) : "v"(a), "v"(b));
    }
};
template <> struct MmaV<_Float16> {
    static __device__ __forceinline__ void first(f32x16& c, f16x8 a, f16x8 b) {
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, 0\n\ts_nop 3" : "=&v"(c) : "v"(a), "v"(b));
    }
    static __device__ __forceinline__ void next(f32x16& c, f16x8 a, f16x8 b) {
        asm volatile("s_nop 1\n\tv_mfma_f32_32x32x16_f16 %0, %1, %2, %0\n\ts_nop 3" : "+v"(c) : "v"(a), "v"(b));
    }
};
__device__ __forceinline__ void settle(f32x16& c0, f32x16& c1) { asm volatile("s_nop 15\n\ts_nop 15" : "+v"(c0), "+v"(c1)); }

// Profiling builds (-DMLSTM_COLD_PROF): waves 0 and 3 add up the shader-clock cycles they spend in each part of the
// kernel and leave the sums, as floats, in the first two rows of the workgroup's dK tile (the results are then wrong, the
// timing is what the build is for).  s_memtime is only trustworthy with one wave per SIMD, which this kernel has.
#ifdef MLSTM_COLD_PROF
#define CP_DECL float prof_[12] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}; long long last_ = (long long)__builtin_amdgcn_s_memtime()
#define CP_STAMP(k) do { const long long now_ = (long long)__builtin_amdgcn_s_memtime(); prof_[k] += (float)(now_ - last_); last_ = now_; } while (0)
#define CP_COUNT(k) do { prof_[k] += 1.f; } while (0)
#else
#define CP_DECL do {} while (0)
#define CP_STAMP(k) do {} while (0)
#define CP_COUNT(k) do {} while (0)
#endif

template <typename T, int D, bool STRICT, bool DENSE>
__global__ __launch_bounds__(256, 1) void cold_kernel(ColArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses device-only builtins; the host pass only needs the stub
    CP_DECL;
    using R = Tr<T>;
    using Cfg = ColdCfg<T, D>;
    using Z = Swz<T, D>;
    typedef typename R::frag frag;
    static_assert(R::HALF && (D == 128 || D == 256), "16-bit types, D = 128 or 256");
    constexpr int KW = R::KW, NS = D / KW, NXD = D / 32;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    // The stages come first: their tiles are read with instruction offsets (16 bits), which reach the first 64 KB only
    char* const stg = smem;
    T* const Vt = reinterpret_cast<T*>(smem + Cfg::STAGES_BYTES);
    char* const tail = smem + Cfg::STAGES_BYTES + Cfg::V_BYTES;
#define ST_Q(st) (reinterpret_cast<T*>(stg + (size_t)(2 * (st)) * Cfg::QT_BYTES))
#define ST_DH(st) (reinterpret_cast<T*>(stg + (size_t)(2 * (st) + 1) * Cfg::QT_BYTES))
#define ST_ROW(st) (reinterpret_cast<float*>(tail) + (st) * 3 * GRAN)
    float* const rowtmp = reinterpret_cast<float*>(tail + Cfg::ROW_BYTES);   // [2][4][32]
    float* const gvl = rowtmp + 2 * 4 * CD_QT + 64;   // (behind the sink words) the chunk's vector state g
    float* const sG = gvl + D;                         // granule bases minus that of the tile's first granule

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, h = lane >> 5, c32 = lane & 31;
    const int kb = wave;
    const int S = a.S, NG = a.NG;
    const int NK = (S + CD_KEYS - 1) / CD_KEYS;            // key tiles per head
    const int NQ = (S + CD_QT - 1) / CD_QT;                // query tiles per head
    int bh, jt;
    {
        const int bid = blockIdx.x;  // key tile 0 has the longest loop: ascending order is heaviest first
        const int tpc = a.chunk_len / CD_KEYS;   // key tiles per chunk
        if ((a.BH & 7) == 0 && a.chunk_len > 0 && NK % tpc == 0) {
            // Groups = (head, chunk) pairs of this XCD (bid & 7), chunk-major; the key tiles of GB groups run together, one
            // per CU of the XCD, heaviest first: what they share (query tiles, reverse states) stays in the XCD's L2.
            const int GB = tpc >= 32 ? 1 : 32 / tpc;
            const int rest = bid >> 3, ngrp = a.BH >> 3, nch = NK / tpc;
            const int G = ngrp * nch, head_n = (G / GB) * GB;
            int g, cls;
            if (rest < head_n * tpc) {
                const int batch = rest / (GB * tpc), r2 = rest % (GB * tpc);
                cls = r2 / GB; g = batch * GB + r2 % GB;
            } else {   // the groups left over form a last, smaller set
                const int r2 = rest - head_n * tpc, n2 = G - head_n;
                cls = r2 / n2; g = head_n + r2 % n2;
            }
            bh = (g % ngrp) * 8 + (bid & 7);
            jt = (g / ngrp) * tpc + cls;
        } else if ((a.BH & 7) == 0) {
            int rest = bid >> 3;
            bh = (rest / NK) * 8 + (bid & 7);
            jt = rest % NK;
        } else {
            bh = bid % a.BH;
            jt = bid / a.BH;
        }
    }
    const size_t hoff = (size_t)bh * S, poff = (size_t)bh * NG * GRAN, goff = (size_t)bh * NG;
    const size_t rsA = DENSE ? (size_t)D : (size_t)a.la.ss, rsB = DENSE ? (size_t)D : (size_t)a.lb.ss;
    const size_t offA = DENSE ? hoff * D : a.la.head(bh), offB = DENSE ? hoff * D : a.lb.head(bh);
    const T* Q = reinterpret_cast<const T*>(a.Q) + offA;
    const T* dH = reinterpret_cast<const T*>(a.dH) + offB;
    const T* K = reinterpret_cast<const T*>(a.K) + offA;
    const T* V = reinterpret_cast<const T*>(a.V) + offA;
    const int key0 = CD_KEYS * jt + 32 * kb;       // the wave's first key
    const int key = key0 + c32;                    // the lane's key
    const int keyc = key < S ? key : S - 1;

    TileDma<T, D, CD_QT, 256> qdma;
    qdma.init(tid);
    const auto ra = qdma.rows(tid, (unsigned)(rsA * sizeof(T))), rb = qdma.rows(tid, (unsigned)(rsB * sizeof(T)));
    RowVec3Dma rvdma;   // beta, 1/n, db of a query tile (padded arrays: always readable)
    rvdma.init(tid, a.beta2 + poff, a.inv_n + poff, a.db + poff, CD_QT, CD_QT, CD_QT);
    const int full_q = S / CD_QT;   // query tiles whose 32 rows all exist
    const int tpc = a.chunk_len > 0 ? a.chunk_len / CD_KEYS : 0;
    const int chunk = a.chunk_len > 0 ? jt / tpc : 0;
    // one past the last query tile the keys meet: the end of their chunk, or of the sequence
    const int NQe = a.chunk_len > 0 ? ((chunk + 1) * (a.chunk_len / CD_QT) < NQ ? (chunk + 1) * (a.chunk_len / CD_QT) : NQ) : NQ;
    const bool has_state = a.chunk_len > 0 && chunk < a.n_states;   // (uniform over the workgroup)
    const int it0 = jt * (CD_KEYS / CD_QT);        // the first query tile: the keys' own
#define COLD_DMA(it, st)                                                          \
    do {                                                                          \
        if ((it) < full_q) {                                                      \
            qdma.issue(ST_Q(st), Q + (size_t)CD_QT * (it) * rsA, ra);              \
            qdma.issue(ST_DH(st), dH + (size_t)CD_QT * (it) * rsB, rb);            \
        } else {                                                                  \
            tile_dma<T, D, CD_QT, 256>(ST_Q(st), Q, CD_QT * (it), S, tid, rsA);    \
            tile_dma<T, D, CD_QT, 256>(ST_DH(st), dH, CD_QT * (it), S, tid, rsB);  \
        }                                                                         \
        rvdma.issue(ST_ROW(st), (it));                                             \
    } while (0)

    // ---- prologue: the V tile (stays), the first state tiles or the first query tile, the wave's K rows into registers
    tile_dma<T, D, CD_KEYS, 256>(Vt, V, CD_KEYS * jt, S, tid, rsA);   // (rows past the end are clamped)
    const size_t sbase = has_state ? ((size_t)bh * a.n_states + chunk) * D * D : 0;
    const T* const Evc = reinterpret_cast<const T*>(a.Ev) + sbase;
    const T* const Evl = STRICT ? reinterpret_cast<const T*>(a.Ev_lo) + sbase : nullptr;
    // The reverse state streams through the query stages in pieces of 32 rows, two pieces in flight (slots 0 / 1 of the four
    // 32-row slots; in split mode the pieces' low-order terms in slots 2 / 3).
    constexpr int SROWS = 32, NPIECE = D / SROWS;
    TileDma<T, D, SROWS, 256> sdma;
    sdma.init(tid);
    auto piece_hi = [&](int p) { return reinterpret_cast<T*>(stg + (size_t)(p & 1) * Cfg::QT_BYTES); };
    auto piece_lo = [&](int p) { return reinterpret_cast<T*>(stg + (size_t)(2 + (p & 1)) * Cfg::QT_BYTES); };
    auto state_issue = [&](int p) {
        sdma.issue(piece_hi(p), Evc + (size_t)SROWS * p * D);
        if constexpr (STRICT) sdma.issue(piece_lo(p), Evl + (size_t)SROWS * p * D);
    };
    if (has_state) state_issue(0);
    else COLD_DMA(it0, 0);
    frag kf[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) kf[s] = frag_rowmajor<T>(K + (size_t)keyc * rsA, s, h);
    const int pe = has_state ? (chunk + 1) * a.chunk_len - 1 : 0;   // the chunk's last position
    const int g0 = 2 * jt;                                          // the tile's first granule
    const double gbase = a.G2[goff + g0];
    const double gkey = a.G2[goff + (key0 / GRAN < NG ? key0 / GRAN : NG - 1)];
    const double g_first = tid < NG ? a.G2[goff + tid] : 0.0;
    const float bend = a.beta2[poff + pe];
    const double Gend = a.G2[goff + pe / GRAN];
    const float al = key < S ? a.alpha2[poff + key] : -INFINITY;   // (a key past the end weighs nothing)

    f32x16 dkacc[NXD], dvacc[NXD];
#pragma unroll
    for (int x = 0; x < NXD; x++)
#pragma unroll
        for (int r = 0; r < 16; r++) { dkacc[x][r] = 0.f; dvacc[x][r] = 0.f; }
    SwzTransReader<T, D> trd;
    trd.init(lane, 0);
    SwzRowReaderX<T, D> rrd;
    rrd.init(lane);

    if (has_state && tid < D) gvl[tid] = a.gvec[((size_t)bh * a.n_states + chunk) * D + tid];
    if (tid < NG) sG[tid] = (float)(g_first - gbase);
    for (int g = tid + 256; g < NG; g += 256) sG[g] = (float)(a.G2[goff + g] - gbase);
    const float gcorr = (float)(gbase - gkey);   // granule base of the tile's first granule minus that of the wave's keys
#pragma unroll
    for (int s = 0; s < NS; s++) pin(kf[s]);
    dma_wait();
    __syncthreads();   // V of the keys and the first state piece (or the first query tile) have landed; sG is visible
    CP_STAMP(0);

    // ---- state phase (sequences in chunks): E is stored value-major (row = value index, rows in the contraction order of
    // the transposing reads).  Per piece of SROWS rows: dK contracts over the piece's rows (values) with V out of LDS; dV
    // is owed by the piece's own rows (SROWS / 32 blocks of output columns), contracted over the whole key index with the
    // K fragments in registers.
    float colacc = 0.f;   // the lane's share of the column sum of dD of its key
    // Scaling by the keys' weights w_j.  bf16 (END_SCALE): instead of multiplying all 2 D accumulators of a lane by w_j
    // behind the state phase (some two thousand instructions: every accumulator through the vector registers and back), the
    // query loop divides ITS contributions by s_j = w_j (the weights' exponent subtracts log2 s_j, exact in fp32, and bf16 has
    // fp32's range), and the epilogue multiplies the sums by s_j once, where it touches every element anyway, and adds
    // w_j g there.  A key whose weight is below 2^-40 drops the state part instead (its operands are zeroed) and uses
    // s_j = 1: what it loses is below 2^-40 of the state product.  fp16 cannot hold G / s_j and scales the accumulators.
    constexpr bool END_SCALE = std::is_same<T, __bf16>::value;
    float scale_s = 1.f, log2_s = 0.f, wkg = 0.f;   // s_j, its log2, and w_j for the epilogue's w_j g (0 without a state)
    if (has_state) {
        const float wk = fast_exp2(al - bend + (float)(Gend - gkey));
        const bool use = !END_SCALE || wk > 0x1p-40f;
        if constexpr (END_SCALE) {
            if (use) { scale_s = wk; log2_s = al - bend + (float)(Gend - gkey); }
            wkg = wk;
        }
        // the stored place of the lane's own row c32 inside a 32-row block (rows are kept in the contraction order of the
        // transposing reads: the two middle groups of four of every 16 swap places), as a byte offset with the column half
        const int own_row = (c32 & ~15) | ((c32 & 3) | ((c32 & 4) << 1) | ((c32 & 8) >> 1));
        const int own_off = Z::off(own_row, R::EPL * h);
        typedef int i32x4 __attribute__((ext_vector_type(4)));
        auto masked = [&](frag f) {   // (END_SCALE: a key that drops the state part multiplies with zeros)
            if constexpr (END_SCALE) {
                i32x4 bits = __builtin_bit_cast(i32x4, f);
#pragma unroll
                for (int e = 0; e < 4; e++) bits[e] = use ? bits[e] : 0;
                return __builtin_bit_cast(frag, bits);
            } else {
                return f;
            }
        };
#pragma unroll
        for (int p = 0; p < NPIECE; p++) {
            if (p + 1 < NPIECE) state_issue(p + 1);   // (into the slots piece p - 1 left behind the last barrier)
            const T* th = piece_hi(p);
            const T* tl = piece_lo(p);
#pragma unroll
            for (int t16 = 0; t16 < SROWS / KW; t16++) {
                const frag vB = masked(rrd.read(Vt, kb, (SROWS / KW) * p + t16));
#pragma unroll
                for (int x = 0; x < NXD; x++) {
                    R::mma(dkacc[x], trd.read(th, KW * t16, x), vB);
                    if constexpr (STRICT) R::mma(dkacc[x], trd.read(tl, KW * t16, x), vB);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int xx = 0; xx < SROWS / 32; xx++) {
                // (own_off: the lane's own row of a 32-row block, first chunk; step t is 32 t bytes on, modulo the swizzle)
                const char* eh = reinterpret_cast<const char*>(th) + 32 * xx * Z::ROW_BYTES;
                const char* el = reinterpret_cast<const char*>(tl) + 32 * xx * Z::ROW_BYTES;
#pragma unroll
                for (int t = 0; t < NS; t++) {
                    const int o = (own_off ^ ((t % 8) << 5)) + (t / 8) * 256;
                    const frag kB = masked(kf[t]);
                    R::mma(dvacc[(SROWS / 32) * p + xx], *reinterpret_cast<const frag*>(eh + o), kB);
                    if constexpr (STRICT) R::mma(dvacc[(SROWS / 32) * p + xx], *reinterpret_cast<const frag*>(el + o), kB);
                    if (t % 4 == 3) __builtin_amdgcn_sched_barrier(0);
                }
            }
            dma_wait();
            __syncthreads();   // every wave is done with piece p, and piece p + 1 has landed
        }
        CP_STAMP(1);
        COLD_DMA(it0, 0);   // the first query tile follows the state into stage 0
        // k_j . (E v_j + g) w_j, the column sums of dD over the queries behind the chunk (and, for fp16, the scaling itself).
        // The K values a lane needs (its accumulators' rows 8 a4 + 4 h + c of every block) are in the K fragments of the two
        // lanes of its key (which hold columns 16 s + 8 h + 0..7): one v_permlane32_swap per register pair sorts them out.
        float cp = 0.f;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const int x = s >> 1, a4a = 2 * (s & 1);
            const i32x4 w = __builtin_bit_cast(i32x4, kf[s]);
            const auto r0 = __builtin_amdgcn_permlane32_swap(w[0], w[2], false, false);
            const auto r1 = __builtin_amdgcn_permlane32_swap(w[1], w[3], false, false);
            typedef int i32x2 __attribute__((ext_vector_type(2)));
            // first results: columns 16 s + 4 h + c (own low half for h = 0, the partner's high half for h = 1); second
            // results: columns 16 s + 8 + 4 h + c
            const f32x4 ka = __builtin_convertvector(__builtin_bit_cast(typename R::vec4, i32x2{(int)r0[0], (int)r1[0]}), f32x4);
            const f32x4 kc = __builtin_convertvector(__builtin_bit_cast(typename R::vec4, i32x2{(int)r0[1], (int)r1[1]}), f32x4);
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int a4 = a4a + u;
                const f32x4 g4v = *reinterpret_cast<const f32x4*>(gvl + 32 * x + 8 * a4 + 4 * h);
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const float kval = u ? kc[c] : ka[c];
                    if constexpr (END_SCALE) {
                        cp += (dkacc[x][4 * a4 + c] + g4v[c]) * kval;
                    } else {
                        const float dkv = (dkacc[x][4 * a4 + c] + g4v[c]) * wk;
                        dkacc[x][4 * a4 + c] = dkv;
                        dvacc[x][4 * a4 + c] *= wk;
                        cp += dkv * kval;
                    }
                }
            }
            if (s % 2 == 1) __builtin_amdgcn_sched_barrier(0);   // (one block of the accumulators at a time through the vector registers)
        }
        colacc = END_SCALE ? cp * wk : cp;   // (starts the lane's column accumulator: the two halves of the wave meet in the epilogue)
        CP_STAMP(2);
    }
    const float log2scale = -0.5f * __log2f((float)D);

    // row sums go to the slice of the 64-key tile of the workgroup's first keys (the dF pass adds up one slice per 64 keys),
    // zeros to the slice of its second half wherever that pass reads it
    const int j64 = 2 * jt;
    float* const rowpart_slice = a.rowpart + ((size_t)bh * a.RS + (a.RS == NG ? j64 : j64 % a.RS)) * S;
    // One step = one 32-query tile.  A lane computes E = exp2(alpha_key + crow_query) per element (a lane holds one key and
    // 16 queries: the factorised form of the other kernels would need one exponential per query and lane as well) and
    // masks it where the key lies behind the query, so diagonal tiles need no code of their own.
    constexpr int PW = TileDma<T, D, CD_QT, 256>::PER_WAVE;
    auto step = [&](auto spread_tag, int it) {
        constexpr bool SPREAD = decltype(spread_tag)::value;  // copy of tile it+1 interleaved with this step's MFMAs
        const int qi0 = CD_QT * it;
        const int stage = (it - it0) & 1, stn = stage ^ 1;
        dma_wait();
        __syncthreads();   // tile `it` has landed and every wave is past phase B of the previous step
        CP_STAMP(3);
        CP_COUNT(8);
        if constexpr (SPREAD) {
            rvdma.issue(ST_ROW(stn), it + 1);
        } else {
            if (it + 1 < NQe) { if (stage) COLD_DMA(it + 1, 0); else COLD_DMA(it + 1, 1); }
        }
        // row sums of the previous step: the four key blocks' shares are in LDS
        if (it > it0 && tid < CD_QT && qi0 - CD_QT + tid < S) {
            const float* rt = rowtmp + ((it - 1) & 1) * 4 * CD_QT;
            float* rp = rowpart_slice + qi0 - CD_QT + tid;
            rp[0] = (rt[tid] + rt[CD_QT + tid]) + (rt[2 * CD_QT + tid] + rt[3 * CD_QT + tid]);
            if (j64 + 1 < NG && (qi0 - CD_QT) / GRAN >= j64 + 1) rp[S] = 0.f;
        }
        const T* gq = Q + (size_t)CD_QT * (it + 1) * rsA;
        const T* gdh = dH + (size_t)CD_QT * (it + 1) * rsB;
        T* const lq = ST_Q(stn);
        T* const ldh = ST_DH(stn);
        const T* Qs = ST_Q(stage);
        const T* dHs = ST_DH(stage);
        const float* srow = ST_ROW(stage);
        float* const rt = rowtmp + (it & 1) * 4 * CD_QT + kb * CD_QT;

        const bool active = key0 <= qi0 + CD_QT - 1;   // some key of the wave lies at or before some query of the tile
        f32x16 gacc, wacc;   // dC, then G = dC~ E;  S, then W = C~ / n   (rows = queries 8 (r / 4) + 4 h + r % 4, column = key c32)
        if (active) {
            // ---- phase A
            constexpr int AHEAD = 4;
            frag qf[NS], hf[NS], vf[NS];
#pragma unroll
            for (int s = 0; s < AHEAD; s++) { qf[s] = rrd.read(Qs, 0, s); hf[s] = rrd.read(dHs, 0, s); vf[s] = rrd.read(Vt, kb, s); }
#pragma unroll
            for (int s = 0; s < NS; s++) {
                if constexpr (SPREAD) {
                    if (s % AHEAD == 0) qdma.issue_range(lq, gq, (s / AHEAD) * PW / (NS / AHEAD), (s / AHEAD + 1) * PW / (NS / AHEAD), ra);
                }
                if (s + AHEAD < NS) {
                    qf[s + AHEAD] = rrd.read(Qs, 0, s + AHEAD);
                    hf[s + AHEAD] = rrd.read(dHs, 0, s + AHEAD);
                    vf[s + AHEAD] = rrd.read(Vt, kb, s + AHEAD);
                }
                if constexpr (D == 256) {   // (accumulators in vector registers: see MmaV)
                    if (s == 0) { MmaV<T>::first(wacc, qf[s], kf[s]); MmaV<T>::first(gacc, hf[s], vf[s]); }
                    else { MmaV<T>::next(wacc, qf[s], kf[s]); MmaV<T>::next(gacc, hf[s], vf[s]); }
                } else {
                    if (s == 0) {
                        const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                        wacc = z; gacc = z;
                    }
                    R::mma(wacc, qf[s], kf[s]);
                    R::mma(gacc, hf[s], vf[s]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (D == 256) settle(wacc, gacc);
            CP_STAMP(4);
            CP_COUNT(9);
            // ---- element-wise part and phase B, by halves of the tile's queries: registers 8t .. 8t+7 of a block are the 16
            // queries of contraction step t of phase B, so the second half's element-wise work, and all the lane reductions
            // of the row sums, are placed between the MFMAs of phase B.  Everything is branch-free: a masked element (key
            // behind the query, or a query past the end) gets the exponent -inf.
            const float argbase = al + (sG[it >> 1] + gcorr + log2scale) - log2_s;   // (weights over s_j: see END_SCALE)
            const unsigned span = (unsigned)(S - key);    // query q takes part iff 0 <= q - key < S - key (unsigned compare)
            const int dq0 = qi0 + 4 * h - key;            // q - key of register r: dq0 + 8 (r / 4) + r % 4
            float dd[16];
            f32x4 beta4[2], inv4[2], db4[2];   // the scalars of the half's eight queries (two groups of four registers)
            auto ew_scalars = [&](int t) {
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const int ql = 8 * (2 * t + u) + 4 * h;
                    beta4[u] = *reinterpret_cast<const f32x4*>(srow + ql);
                    inv4[u] = *reinterpret_cast<const f32x4*>(srow + GRAN + ql);
                    db4[u] = *reinterpret_cast<const f32x4*>(srow + 2 * GRAN + ql);
                }
            };
            auto ew_one = [&](int r) {
                const int u = (r >> 2) & 1, c = r & 3;
                const bool live = (unsigned)(dq0 + 8 * (r >> 2) + c) < span;
                const float e = fast_exp2(live ? argbase - beta4[u][c] : -INFINITY);
                const float ct = wacc[r] * e;
                const float dct = gacc[r] * inv4[u][c] + db4[u][c];
                dd[r] = END_SCALE ? (ct * scale_s) * dct : ct * dct;
                gacc[r] = dct * e;
                wacc[r] = ct * inv4[u][c];
                colacc += dd[r];
            };
            // lane 15 of a 16-lane row holds the row's total: rows 0 / 2 (h = 0 / 1) carry register 2p, rows 1 / 3 register
            // 2p + 1 of the folded pair; the other lanes write to a word of their own that nobody reads
            float* const sink = rowtmp + 2 * 4 * CD_QT + lane;
            auto row_sum_out = [&](int p, float folded) {
                const float tot = row_total(folded);
                const int r = 2 * p + ((lane >> 4) & 1);
                float* dst = (lane & 15) == 15 ? rt + (8 * (r >> 2) + 4 * h + (r & 3)) : sink;
                *dst = tot;
            };
            ew_scalars(0);
#pragma unroll
            for (int r = 0; r < 8; r++) ew_one(r);
            ew_scalars(1);   // (for the second half, whose work rides on phase B below)
            float rs[8];
#pragma unroll
            for (int p = 0; p < 4; p++) rs[p] = fold_pair(dd[2 * p], dd[2 * p + 1]);
            CP_STAMP(5);
#pragma unroll
            for (int t = 0; t < 2; t++) {
                frag ghi, glo, whi, wlo;
                if constexpr (STRICT) { R::from_acc_split(gacc, t, ghi, glo); R::from_acc_split(wacc, t, whi, wlo); }
                else { ghi = R::from_acc(gacc, t); whi = R::from_acc(wacc, t); }
                frag qa[2], ha[2];
                qa[0] = trd.read(Qs, KW * t, 0);
                ha[0] = trd.read(dHs, KW * t, 0);
#pragma unroll
                for (int x = 0; x < NXD; x++) {
                    if constexpr (SPREAD) {
                        constexpr int HOOKS = 2 * NXD / 2;   // one hook per two column blocks, over both halves
                        if (x % 2 == 0) {
                            const int k = t * (NXD / 2) + x / 2;
                            qdma.issue_range(ldh, gdh, k * PW / HOOKS, (k + 1) * PW / HOOKS, rb);
                        }
                    }
                    if (x + 1 < NXD) { qa[(x + 1) & 1] = trd.read(Qs, KW * t, x + 1); ha[(x + 1) & 1] = trd.read(dHs, KW * t, x + 1); }
                    R::mma(dkacc[x], qa[x & 1], ghi);
                    R::mma(dvacc[x], ha[x & 1], whi);
                    if constexpr (STRICT) {
                        R::mma(dkacc[x], qa[x & 1], glo);
                        R::mma(dvacc[x], ha[x & 1], wlo);
                    }
                    // behind the MFMAs: 8 / NXD registers of the second half's element-wise work (t = 0 only) and 4 / NXD
                    // folded row sums of this half
                    if (t == 0) {
#pragma unroll
                        for (int u = 0; u < 8 / NXD; u++) ew_one(8 + x * (8 / NXD) + u);
                    }
                    if constexpr (NXD == 8) { if (x % 2 == 1) row_sum_out(4 * t + x / 2, rs[4 * t + x / 2]); }
                    else row_sum_out(4 * t + x, rs[4 * t + x]);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if (t == 0) {
#pragma unroll
                    for (int p = 4; p < 8; p++) rs[p] = fold_pair(dd[2 * p], dd[2 * p + 1]);
                }
            }
            CP_STAMP(6);
        } else {
            if constexpr (SPREAD) { qdma.issue(lq, gq, ra); qdma.issue(ldh, gdh, rb); }
            if (lane < CD_QT) rt[lane] = 0.f;
        }
    };
    const int lim = (NQe < full_q ? NQe : full_q) - 1;   // last step index that may spread is lim - 1
    int it = it0;
    for (; it < lim; it++) step(std::true_type{}, it);
    for (; it < NQe; it++) step(std::false_type{}, it);
#undef COLD_DMA

    // ---- epilogue: column sums, the last step's row sums, then dK and dV through LDS (the V tile and the stages are free
    // once every wave is past its last phase B): rows of D elements, 16-byte chunk c of row r at chunk c ^ (r & 31), so that
    // the lanes' 8-byte pieces of 32 different rows spread over the banks; the rows leave 16 bytes at a time.
    colacc = sum_halves(colacc);
    if (h == 0 && key < S) a.colsum[hoff + key] = colacc;
    __syncthreads();
    {
        const int last = NQe - 1;
        if (tid < CD_QT && CD_QT * last + tid < S) {
            const float* rt = rowtmp + (last & 1) * 4 * CD_QT;
            float* rp = rowpart_slice + CD_QT * last + tid;
            rp[0] = (rt[tid] + rt[CD_QT + tid]) + (rt[2 * CD_QT + tid] + rt[3 * CD_QT + tid]);
            if (j64 + 1 < NG && (CD_QT * last) / GRAN >= j64 + 1) rp[S] = 0.f;
        }
    }
    {
        constexpr int ROWB = D * (int)sizeof(T), CPR = ROWB / 16, NPC = CD_KEYS * CPR / 256;
        static_assert(2 * (size_t)CD_KEYS * ROWB <= Cfg::V_BYTES + Cfg::STAGES_BYTES, "both staged outputs fit the V tile and the stages");
#pragma unroll
        for (int which = 0; which < 2; which++) {
            char* const out = smem + (size_t)which * CD_KEYS * ROWB;
            const int row = 32 * kb + c32;
#pragma unroll
            for (int x = 0; x < NXD; x++)
#pragma unroll
                for (int a4 = 0; a4 < 4; a4++) {
                    const int d = 32 * x + 8 * a4 + 4 * h;               // first of the four columns
                    f32x4 v;
#pragma unroll
                    for (int c = 0; c < 4; c++) v[c] = which ? dvacc[x][4 * a4 + c] : dkacc[x][4 * a4 + c];
                    if constexpr (END_SCALE) {   // the keys' weights: see the state phase
                        v *= scale_s;
                        if (!which && has_state) v += *reinterpret_cast<const f32x4*>(gvl + d) * wkg;
                    }
                    const int chunk16 = (d * (int)sizeof(T)) >> 4, within = (d * (int)sizeof(T)) & 15;
                    *reinterpret_cast<typename R::vec4*>(out + row * ROWB + (((chunk16 ^ (row & 31)) & (CPR - 1)) << 4) + within) = R::cvt4(v);
                }
        }
        __syncthreads();
#pragma unroll
        for (int which = 0; which < 2; which++) {
            const char* const out = smem + (size_t)which * CD_KEYS * ROWB;
            char* const gout = reinterpret_cast<char*>(which ? a.dV : a.dK) + (offA + (size_t)CD_KEYS * jt * rsA) * sizeof(T);
#pragma unroll
            for (int i = 0; i < NPC; i++) {
                const int c = tid + 256 * i, row = c / CPR, cc = c % CPR;
                if (CD_KEYS * jt + row < S)
                    *reinterpret_cast<uint4*>(gout + (size_t)row * rsA * sizeof(T) + 16 * cc) =
                        *reinterpret_cast<const uint4*>(out + row * ROWB + (((cc ^ (row & 31)) & (CPR - 1)) << 4));
            }
        }
    }
#ifdef MLSTM_COLD_PROF
    CP_STAMP(7);
    if ((wave == 0 || wave == 3) && lane < 12 && CD_KEYS * jt + 1 < S) {
        float v = 0.f;
#pragma unroll
        for (int k = 0; k < 12; k++) v = lane == k ? prof_[k] : v;
        reinterpret_cast<float*>(reinterpret_cast<char*>(a.dK) + (offA + ((size_t)CD_KEYS * jt + (wave == 3)) * rsA) * sizeof(T))[lane] = v;
    }
#endif
#undef ST_Q
#undef ST_DH
#undef ST_ROW
#endif
}

template <typename T, int D, bool STRICT, bool DENSE>
static int launch_cold_t(const ColArgs& a, hipStream_t st) {
    using Cfg = ColdCfg<T, D>;
    auto kern = cold_kernel<T, D, STRICT, DENSE>;
    if (hipError_t e = lds_limit_once<cold_kernel<T, D, STRICT, DENSE>>((int)(Cfg::LDS_BYTES + 2048 * sizeof(float))); e != hipSuccess) return (int)e;
    if (a.NG > 2048) return MLSTM_ESHAPE;
    if (a.chunk_len > 0 && (a.chunk_len % CD_KEYS != 0 || (a.n_states > 0 && (!a.Ev || !a.gvec || (STRICT && !a.Ev_lo))))) return MLSTM_EINVAL;
    const int NK = (a.S + CD_KEYS - 1) / CD_KEYS;
    hipLaunchKernelGGL(kern, dim3(a.BH * NK), dim3(256), Cfg::LDS_BYTES + (size_t)a.NG * sizeof(float), st, a);
    return (int)hipGetLastError();
}

template <typename T, int D>
static int launch_cold_d(const ColArgs& a, hipStream_t st) {
    const bool dense = is_dense(a.la, a.S, D) && is_dense(a.lb, a.S, D);
    if (a.precise) return dense ? launch_cold_t<T, D, true, true>(a, st) : launch_cold_t<T, D, true, false>(a, st);
    return dense ? launch_cold_t<T, D, false, true>(a, st) : launch_cold_t<T, D, false, false>(a, st);
}

int launch_cold_kernel(int dtype, int D, const ColArgs& a, hipStream_t st) {
    if (dtype == MLSTM_F16 && D == 128) return launch_cold_d<_Float16, 128>(a, st);
    if (dtype == MLSTM_F16 && D == 256) return launch_cold_d<_Float16, 256>(a, st);
    if (dtype == MLSTM_BF16 && D == 128) return launch_cold_d<__bf16, 128>(a, st);
    if (dtype == MLSTM_BF16 && D == 256) return launch_cold_d<__bf16, 256>(a, st);
    return MLSTM_ESHAPE;
}

}  // namespace mlstm
