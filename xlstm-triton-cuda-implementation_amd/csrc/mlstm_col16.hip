// Column-parallel backward kernel for the 16-bit types at D = 128 and 256: mlstm_col.hip with phase A done as
// v_mfma_f32_16x16x32 products on two halves of 16 queries, so that the element-wise part of the first half runs
// between the MFMAs of the second (a wave issues in order and an MFMA executes asynchronously: vector work placed
// between MFMAs is free, whereas after them the matrix unit idles).  With 32x32 blocks all 16 accumulator registers of
// a lane complete together at the end of the contraction and nothing can start early.
// Same tile layouts, phase B, epilogue and outputs as col_kernel; replaces the dK/dV/dI loop of
// mlstm_matmul_kernel_backward (mlstm_matmul.py:269-316) and matmul_backward (cuda-src/mlstm_backward.cu:402-518).
//
// Phase A of wave (kbA, qbA): keys 32*kbA.., queries 32*qbA.. of the 64 x 64 tile pair, as [2 key sub-blocks of 16] x
// [2 query halves of 16].  16x16x32 operand layout: A row (key) = lane % 16, contraction elements 8*(lane/16)..+7;
// B column (query) = lane % 16, same contraction elements; C column (query) = lane % 16, rows (keys) 4*(lane/16) + r.
#include <type_traits>
#include "mlstm_device.h"
#include "mlstm_kernels.h"

namespace mlstm {

// v(l) + v(l^16) + v(l^32) + v(l^48): the four lanes that share a query in the 16x16 accumulator layout
__device__ __forceinline__ float sum_quarters(float v) {
    int x = __builtin_bit_cast(int, sum_halves(v));
    auto r = __builtin_amdgcn_permlane16_swap(x, x, false, false);
    return __builtin_bit_cast(float, (int)r[0]) + __builtin_bit_cast(float, (int)r[1]);
}

template <typename T> struct Mma16;
template <> struct Mma16<__bf16> {
    static __device__ __forceinline__ f32x4 mma(f32x4 c, bf16x8 a, bf16x8 b) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Mma16<_Float16> {
    static __device__ __forceinline__ f32x4 mma(f32x4 c, f16x8 a, f16x8 b) { return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0); }
};

template <typename T, int D>
struct Col16Cfg {
    // G / W tiles [query][key], written by lanes in phase A and read transposed in phase B.  16-bit: 128-byte rows,
    // 16-byte chunk c of row q stored at chunk c ^ gkey16(q); fp32: rows padded by 8 floats.
    static constexpr int LDG = Tr<T>::HALF ? GRAN : GRAN + 8;
    static constexpr size_t TILE_ELEMS = (size_t)GRAN * D;
    static constexpr size_t STAGE_BYTES = 2 * TILE_ELEMS * sizeof(T) + 3 * GRAN * sizeof(float);  // Q, dH, (beta, 1/n, db)
    static constexpr size_t G_BYTES = (size_t)GRAN * LDG * sizeof(T);
    static constexpr size_t FIXED_BYTES = 2 * G_BYTES + 2 * GRAN * sizeof(float);                  // G, W, row-sum scratch
    static constexpr int STAGES = (2 * STAGE_BYTES + FIXED_BYTES + 2048 * sizeof(float) <= 160 * 1024) ? 2 : 1;
    static constexpr size_t LDS_BYTES = STAGES * STAGE_BYTES + FIXED_BYTES;  // plus one float per key tile, appended at launch
};

// Swizzle key of the 16-bit G / W tiles: bits (q>>1)&1 and (q>>2)&3 of the query row.  Phase A writes one chunk of
// 32 consecutive rows per instruction (all 16 residues of q spread over both 128-byte bank windows x 8 chunks);
// phase B gathers 4 consecutive rows x 64 bytes (rows q and q+2 land in different halves of the row).
__device__ __forceinline__ int gkey16(int q) { return (((q >> 1) & 1) << 2) | ((q >> 2) & 3); }

template <typename T, int D, bool DENSE>
__global__ __launch_bounds__(256, 1) void col16_kernel(ColArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses device-only builtins; the host pass only needs the stub
    using R = Tr<T>;
    using Cfg = Col16Cfg<T, D>;
    typedef typename R::frag frag;
    static_assert(R::HALF && D >= 128 && D % 64 == 0, "16-bit types, D >= 128");
    constexpr int KW = R::KW, NX = D / 64, NQS = GRAN / KW;
    constexpr int NS32 = D / 32;   // contraction steps of the 16x16x32 products
    // Phase B ownership.  D >= 128: wave w accumulates output column blocks {w*NXW .. } for BOTH key blocks, so each
    // transposed Q / dH fragment (the expensive ds_read_b64_tr_b16 traffic) is read by exactly one wave and feeds two
    // MFMAs.  D = 64 has only two column blocks: there a wave owns one key block and one column block.
    constexpr bool BOTH_KB = D >= 128;
    constexpr int NXW = BOTH_KB ? D / 128 : NX;   // column blocks per wave
    constexpr int NKB = BOTH_KB ? 2 : 1;          // key blocks per wave in phase B
    constexpr int LDG = Cfg::LDG, STAGES = Cfg::STAGES;
    static_assert(STAGES == 2 && NQS == 4 && BOTH_KB, "two tile stages, 64-query tiles");
    extern __shared__ __attribute__((aligned(16))) char smem[];
#define ST_Q(st) (reinterpret_cast<T*>(smem + (st) * Cfg::STAGE_BYTES))
#define ST_DH(st) (ST_Q(st) + Cfg::TILE_ELEMS)
#define ST_ROW(st) (reinterpret_cast<float*>(ST_DH(st) + Cfg::TILE_ELEMS))
    T* const Gs = reinterpret_cast<T*>(smem + STAGES * Cfg::STAGE_BYTES);
    T* const Ws = Gs + GRAN * LDG;
    float* const rowtmp = reinterpret_cast<float*>(Ws + GRAN * LDG);  // [2][64]
    float* const sG = reinterpret_cast<float*>(smem + Cfg::LDS_BYTES);  // granule bases minus this key tile's (see row kernel)

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, h = lane >> 5, c32 = lane & 31;
    const int S = a.S, NG = a.NG;
    int bh, jt;
    {
        const int bid = blockIdx.x;  // key tile 0 has the longest loop: ascending order is heaviest first
        const int tpc = a.chunk_len / GRAN;   // key tiles per chunk
        if ((a.BH & 7) == 0 && a.chunk_len > 0 && NG % tpc == 0) {
            // In chunks a key tile's loop length is set by its place in the chunk, and the key tiles of a chunk share
            // the chunk's reverse states and query tiles.  Groups = (head, chunk) pairs of this XCD (bid & 7), chunk-major,
            // so that the last chunks of the heads (no state phase) come last; the key tiles of COL_GB groups run
            // together -- one per CU of the XCD, and what they share stays in its L2 -- heaviest first.
            const int COL_GB = tpc >= 32 ? 1 : 32 / tpc;   // (an XCD has 32 CUs, a CU holds one workgroup)
            const int rest = bid >> 3, ngrp = a.BH >> 3, nch = NG / tpc;
            const int G = ngrp * nch, head_n = (G / COL_GB) * COL_GB;
            int g, cls;
            if (rest < head_n * tpc) {
                const int batch = rest / (COL_GB * tpc), r2 = rest % (COL_GB * tpc);
                cls = r2 / COL_GB; g = batch * COL_GB + r2 % COL_GB;
            } else {   // the groups left over form a last, smaller set
                const int r2 = rest - head_n * tpc, n2 = G - head_n;
                cls = r2 / n2; g = head_n + r2 % n2;
            }
            bh = (g % ngrp) * 8 + (bid & 7);
            jt = (g / ngrp) * tpc + cls;
        } else if ((a.BH & 7) == 0) {
            int rest = bid >> 3;
            bh = (rest / NG) * 8 + (bid & 7);
            jt = rest % NG;
        } else {
            bh = bid % a.BH;
            jt = bid / a.BH;
        }
    }
    const int kbA = wave >> 1, qbA = wave & 1;   // phase A block
    const int kbB = wave & 1, dsel = wave >> 1;  // phase B: keys 32*kbB.., column blocks dsel, dsel+2, ...
    const size_t hoff = (size_t)bh * S, poff = (size_t)bh * NG * GRAN;
    // the caller's tensors: q, k, v, dk, dv in layout la, dh in lb (element offset of the head, elements per position)
    // (DENSE: contiguous [BH,S,D] tensors, strides as compile-time constants)
    const size_t rsA = DENSE ? (size_t)D : (size_t)a.la.ss, rsB = DENSE ? (size_t)D : (size_t)a.lb.ss;
    const size_t offA = DENSE ? hoff * D : a.la.head(bh), offB = DENSE ? hoff * D : a.lb.head(bh);
    const T* Q = reinterpret_cast<const T*>(a.Q) + offA;
    const T* dH = reinterpret_cast<const T*>(a.dH) + offB;
    const T* K = reinterpret_cast<const T*>(a.K) + offA;
    const T* V = reinterpret_cast<const T*>(a.V) + offA;
    const float* const beta_head = a.beta2 + poff;
    const float* const inv_head = a.inv_n + poff;
    const float* const db_head = a.db + poff;

    TileDma<T, D, GRAN, 256> tdma;
    tdma.init(tid);
    const auto ra = tdma.rows(tid, (unsigned)(rsA * sizeof(T))), rb = tdma.rows(tid, (unsigned)(rsB * sizeof(T)));
    RowVec3Dma rvdma;   // beta, 1/n, db of a query tile (padded arrays: always readable)
    rvdma.init(tid, beta_head, inv_head, db_head);
    const int full_tiles = S / GRAN;  // query tiles whose 64 rows all exist
    // In chunks the keys walk the query tiles of their own chunk only (NGe: one past the last of them); what the queries
    // behind the chunk contribute comes through the chunk's reverse states (state phase below).
    const int NGe = a.chunk_len > 0 ? ((GRAN * jt) / a.chunk_len + 1) * (a.chunk_len / GRAN) < NG ? ((GRAN * jt) / a.chunk_len + 1) * (a.chunk_len / GRAN) : NG
                                    : NG;
#define COL_DMA(it, st)                                                          \
    do {                                                                         \
        if ((it) < full_tiles) {                                                 \
            tdma.issue(ST_Q(st), Q + (size_t)GRAN * (it) * rsA, ra);              \
            tdma.issue(ST_DH(st), dH + (size_t)GRAN * (it) * rsB, rb);            \
        } else {                                                                 \
            tile_dma<T, D, GRAN, 256>(ST_Q(st), Q, GRAN * (it), S, tid, rsA);     \
            tile_dma<T, D, GRAN, 256>(ST_DH(st), dH, GRAN * (it), S, tid, rsB);   \
        }                                                                        \
        rvdma.issue(ST_ROW(st), (it));                                            \
    } while (0)
    const int chunk = a.chunk_len > 0 ? (GRAN * jt) / a.chunk_len : 0;
    const bool has_state = a.chunk_len > 0 && chunk < a.n_states;   // (uniform over the workgroup)
    // The keys' own K and V rows go through LDS once (stage 1, which the query loop only needs from its second tile on):
    // every wave wants all of them, as the second operand of the state phase below and as the stationary fragments of
    // the query loop.  With a state phase ahead, stage 0 first carries the reverse state (two 64-row tiles at a time) and
    // the first query tile follows when the state is done with; otherwise the first query tile travels right away.
    // The copies are issued before anything else: the time to pull these bytes into the CU is what the prologue costs.
    T* const Kt = ST_Q(1);
    T* const Vt = ST_DH(1);
    constexpr int NTL = D / GRAN;   // 64-row tiles of a state
    const T* const Evc = has_state ? reinterpret_cast<const T*>(a.Ev) + ((size_t)bh * a.n_states + chunk) * D * D : nullptr;
    if (GRAN * (jt + 1) <= S) {
        tdma.issue(Kt, K + (size_t)GRAN * jt * rsA, ra);
        tdma.issue(Vt, V + (size_t)GRAN * jt * rsA, ra);
    } else {   // rows past the end are clamped
        tile_dma<T, D, GRAN, 256>(Kt, K, GRAN * jt, S, tid, rsA);
        tile_dma<T, D, GRAN, 256>(Vt, V, GRAN * jt, S, tid, rsA);
    }
    if (has_state) {
        tdma.issue(ST_Q(0), Evc);
        tdma.issue(ST_DH(0), Evc + (size_t)GRAN * D);
    } else {
        COL_DMA(jt, 0);
    }
    // every scalar the prologue needs, requested in one batch (each dependent trip to memory costs a few thousand cycles here)
    const int pe = has_state ? (chunk + 1) * a.chunk_len - 1 : 0;   // the chunk's last position
    const double gj = a.G2[(size_t)bh * a.NG + jt];
    const double g_first = tid < a.NG ? a.G2[(size_t)bh * a.NG + tid] : 0.0;
    const float bend = a.beta2[poff + pe];
    const double Gend = a.G2[(size_t)bh * a.NG + pe / GRAN];
    float akey[2];
    {
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            int key = GRAN * jt + 32 * kb + c32;
            key = key < S ? key : S - 1;
            akey[kb] = a.alpha2[poff + key];
        }
    }
    f32x16 dkacc[NKB][NXW], dvacc[NKB][NXW];
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
        for (int x = 0; x < NXW; x++)
#pragma unroll
            for (int r = 0; r < 16; r++) { dkacc[kb][x][r] = 0.f; dvacc[kb][x][r] = 0.f; }
    constexpr bool FAST_TR = R::HALF && Swz<T, D>::CPR >= 16;
    SwzTransReader<typename std::conditional<FAST_TR, T, __bf16>::type, FAST_TR ? D : 256> trd;
    // Phase B column blocks of a wave: wave, wave + 4, ... (XS apart), so that its blocks are spread over the 64-row tiles of
    // the state: with two tiles at a time in LDS every wave finds one of its own blocks in either round of the state phase
    constexpr int XS = 4;
    if constexpr (FAST_TR) trd.init(lane, BOTH_KB ? wave : 0);

    // ---- state phase (sequences in chunks): what the queries behind the keys' chunk contribute comes through the reverse
    // state of the chunk, E[k][v] = sum_i rho_i / n_i q_i[k] dh_i[v] / sqrt(D):  dK_j = w_j (E v_j + g),  dV_j = w_j E^T k_j
    // with w_j = exp(a_j - A_e), e the chunk's last position.  The state is stored once, value-major (row = value index,
    // 16-row groups in the contraction order of the transposing reads), and streams through stage 0 as D/64 tiles of 64
    // rows, two at a time.  A wave owns output columns: for dV those are rows of the state -- its own 32-row blocks, read
    // row-major and contracted over the key index with K; for dK they are columns of the state, read with transposing
    // loads from every tile and contracted over the tile's rows (values) with V.  The other operand of both products is
    // the keys' K / V rows out of LDS.
    // colfar: k_j . dK_j of that part = the column sums of dD over those queries.
    float colfar = 0.f;   // thread tid < 64: key tid of the tile
    constexpr int NT16 = D / KW;   // contraction steps of a whole row
    float wk[NKB];
    const float* gv = nullptr;
    if (has_state) gv = a.gvec + ((size_t)bh * a.n_states + chunk) * D;
    // granule bases minus this key tile's
    if (tid < a.NG) sG[tid] = (float)(g_first - gj);
    for (int g = tid + 256; g < a.NG; g += 256) sG[g] = (float)(a.G2[(size_t)bh * a.NG + g] - gj);
    if (has_state) {
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) wk[kb] = fast_exp2(akey[kb] - bend + (float)(Gend - gj));   // (the keys' granule is jt)
    }
    dma_wait();
    __syncthreads();   // K, V of the keys and the first state tiles (or the first query tile) have landed
    if (has_state) {
        // the wave's own rows: column block cb holds stored rows 32 cb + c32 -> tile (32 cb) / 64, local row (32 cb) % 64 + c32
        int own_row[NXW];
#pragma unroll
        for (int x = 0; x < NXW; x++) {
            const int rl = (32 * (wave + XS * x)) % GRAN + c32;
            own_row[x] = (rl & ~15) | ((rl & 3) | ((rl & 4) << 1) | ((rl & 8) >> 1));
        }
#pragma unroll
        for (int round = 0; round < (NTL + 1) / 2; round++) {
            if (round > 0) {
                tdma.issue(ST_Q(0), Evc + (size_t)GRAN * (2 * round) * D);
                if (2 * round + 1 < NTL) tdma.issue(ST_DH(0), Evc + (size_t)GRAN * (2 * round + 1) * D);
                dma_wait();
                __syncthreads();
            }
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const int tau = 2 * round + half;
                if (tau >= NTL) break;
                const T* tile = half ? ST_DH(0) : ST_Q(0);
                // dK: contraction over this tile's 64 rows (values 64 tau ..), the wave's columns of the state.  Operand reads
                // run one step ahead of the MFMAs that consume them.
                {
                    constexpr int NTT = GRAN / KW;
                    frag vB[2][NKB], ea[2][NXW];
                    auto rd = [&](int tt) {
#pragma unroll
                        for (int kb = 0; kb < NKB; kb++) vB[tt & 1][kb] = swz_frag_rowmajor<T, D>(Vt, 32 * kb + c32, NTT * tau + tt, h);
#pragma unroll
                        for (int x = 0; x < NXW; x++) ea[tt & 1][x] = trd.read(tile, KW * tt, XS * x);
                    };
                    rd(0);
#pragma unroll
                    for (int tt = 0; tt < NTT; tt++) {
                        if (tt + 1 < NTT) rd(tt + 1);
#pragma unroll
                        for (int x = 0; x < NXW; x++)
#pragma unroll
                            for (int kb = 0; kb < NKB; kb++) R::mma(dkacc[kb][x], ea[tt & 1][x], vB[tt & 1][kb]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                // dV: the wave's own rows, if this tile holds them, contracted over the whole key index
#pragma unroll
                for (int x = 0; x < NXW; x++) {
                    if ((32 * (wave + XS * x)) / GRAN != tau) continue;
                    frag kB[2][NKB], eb[2];
                    auto rd = [&](int t) {
#pragma unroll
                        for (int kb = 0; kb < NKB; kb++) kB[t & 1][kb] = swz_frag_rowmajor<T, D>(Kt, 32 * kb + c32, t, h);
                        eb[t & 1] = swz_frag_rowmajor<T, D>(tile, own_row[x], t, h);
                    };
                    rd(0);
#pragma unroll
                    for (int t = 0; t < NT16; t++) {
                        if (t + 1 < NT16) rd(t + 1);
#pragma unroll
                        for (int kb = 0; kb < NKB; kb++) R::mma(dvacc[kb][x], eb[t & 1], kB[t & 1][kb]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
            __syncthreads();   // every wave is done with the two tiles
        }
        // The first query tile follows the state into stage 0.  Its copy is issued a block at a time between the pieces of
        // the arithmetic below (a wave that issues it in one go sits in the memory pipeline's queue for its whole length)
        const bool first_full = jt < full_tiles;
        if (first_full) rvdma.issue(ST_ROW(0), jt);
        else COL_DMA(jt, 0);
        constexpr int PW0 = TileDma<T, D, GRAN, 256>::PER_WAVE;
        constexpr int PIECES = NKB * NXW * 4;     // bodies of the loop below; both tiles' blocks are dealt out over them
        float* const cpart = reinterpret_cast<float*>(Gs);   // [4 waves][64 keys]; G / W are not in use yet
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) {
            float cp = 0.f;
#pragma unroll
            for (int x = 0; x < NXW; x++)
#pragma unroll
                for (int a4 = 0; a4 < 4; a4++) {
                    if (first_full) {
                        const int piece = (kb * NXW + x) * 4 + a4;
                        const int b0 = piece * 2 * PW0 / PIECES, b1 = (piece + 1) * 2 * PW0 / PIECES;   // of 2 PW0 blocks: Q then dH
                        if (b0 < PW0) tdma.issue_range(ST_Q(0), Q + (size_t)GRAN * jt * rsA, b0, b1 < PW0 ? b1 : PW0, ra);
                        if (b1 > PW0) tdma.issue_range(ST_DH(0), dH + (size_t)GRAN * jt * rsB, b0 > PW0 ? b0 - PW0 : 0, b1 - PW0, rb);
                    }
                    const int d = 32 * (wave + XS * x) + 8 * a4 + 4 * h;
                    const f32x4 g4v = *reinterpret_cast<const f32x4*>(gv + d);
                    const char* kp = reinterpret_cast<const char*>(Kt) + Swz<T, D>::off(32 * kb + c32, d & ~7) + (d & 7) * (int)sizeof(T);
                    const f32x4 kv = __builtin_convertvector(*reinterpret_cast<const typename R::vec4*>(kp), f32x4);
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        const float dkv = (dkacc[kb][x][4 * a4 + c] + g4v[c]) * wk[kb];
                        dkacc[kb][x][4 * a4 + c] = dkv;
                        dvacc[kb][x][4 * a4 + c] *= wk[kb];
                        cp += dkv * kv[c];
                    }
                }
            cp = sum_halves(cp);
            if (h == 0) cpart[wave * GRAN + 32 * kb + c32] = cp;
        }
        __syncthreads();   // the waves' shares of k . dK lie in LDS
        if (tid < GRAN) colfar = (cpart[tid] + cpart[GRAN + tid]) + (cpart[2 * GRAN + tid] + cpart[3 * GRAN + tid]);
        // (G / W get written behind the barrier that opens the first step)
    }

    const int kstartA = GRAN * jt + 32 * kbA;
    const int l16 = lane & 15, g4 = lane >> 4;
    frag kf[2][NS32], vf[2][NS32];   // [key sub-block][contraction step]
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
        const int krow = 32 * kbA + 16 * kt + l16;   // (rows past the end of the sequence hold the last row)
#pragma unroll
        for (int s = 0; s < NS32; s++) {
            kf[kt][s] = *reinterpret_cast<const frag*>(reinterpret_cast<const char*>(Kt) + Swz<T, D>::off(krow, 32 * s + 8 * g4));
            vf[kt][s] = *reinterpret_cast<const frag*>(reinterpret_cast<const char*>(Vt) + Swz<T, D>::off(krow, 32 * s + 8 * g4));
        }
    }
    // element r of a lane: key 16*(r>>2) + 4*g4 + (r&3) of the block
    float al[8];
#pragma unroll
    for (int r = 0; r < 8; r++) al[r] = a.alpha2[poff + kstartA + 16 * (r >> 2) + 4 * g4 + (r & 3)];
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int s = 0; s < NS32; s++) { pin(kf[kt][s]); pin(vf[kt][s]); }
    // factorised weights for the steps below the diagonal: ekr[r] = exp2(alpha_key(r) - c0), c0 the block maximum
    float ekr[8], amaxA;
    {
        float mx = al[0];
#pragma unroll
        for (int r = 1; r < 8; r++) mx = fmaxf(mx, al[r]);
        mx = fmaxf(mx, __shfl_xor(mx, 16));
        amaxA = fmaxf(mx, __shfl_xor(mx, 32));
#pragma unroll
        for (int r = 0; r < 8; r++) ekr[r] = amaxA > -INFINITY ? fast_exp2(al[r] - amaxA) : 0.f;
    }
#pragma unroll
    for (int r = 0; r < 8; r++) { pin(al[r]); pin(ekr[r]); }
    pin(amaxA);
    int qoff[4];  // byte offsets of the lane's Q / dH fragment, contraction steps 0..3 (step s + 4 is 256 bytes on)
#pragma unroll
    for (int s = 0; s < 4; s++) qoff[s] = Swz<T, D>::off(l16, 32 * s + 8 * g4);
    // (sG and the first tile are visible since the barrier above; the stationary fragments have left LDS -- pin -- before
    // the barrier that opens the first step, behind which stage 1 is overwritten)
    const float log2scale = -0.5f * __log2f((float)D);

    float colacc[8];
#pragma unroll
    for (int r = 0; r < 8; r++) colacc[r] = 0.f;

    // transposing read of the swizzled 16-bit G / W tiles: contraction rows 16t + 8x + 4h + (j>>2), keys 32*kbB + ..
    int gwoff[NKB][2];
    {
        const int j = lane & 15, sub = (lane >> 4) & 1;
#pragma unroll
        for (int kb = 0; kb < NKB; kb++)
#pragma unroll
            for (int x = 0; x < 2; x++) {
                const int q = 8 * x + 4 * h + (j >> 2);
                const int c = 4 * (BOTH_KB ? kb : kbB) + 2 * sub + ((j & 3) >> 1);
                gwoff[kb][x] = q * GRAN + ((c ^ gkey16(q)) << 3) + 4 * (j & 1);
            }
    }
    auto gw_read = [&](const T* tile, int t, int kb) {
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(tile + gwoff[kb][0] + 16 * t * GRAN));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(tile + gwoff[kb][1] + 16 * t * GRAN));
        s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(frag, both);
    };

    // One step = one 64-query tile.  FIRST (the diagonal tile, it == jt) carries the causal masks and the skipped
    // block; every later tile takes the mask-free path.  Two instantiations instead of a run-time branch keep each
    // loop body a single code path.
    constexpr int PW = TileDma<T, D, GRAN, 256>::PER_WAVE;
    auto step = [&](auto first_tag, auto spread_tag, int it) {
        constexpr bool FIRST = decltype(first_tag)::value;
        constexpr bool SPREAD = decltype(spread_tag)::value;  // copy of tile it+1 interleaved with this step's MFMAs
        const int qi0 = GRAN * it;
        const int stage = (it - jt) & (STAGES - 1);
        // tile `it` has landed and every wave is past phase B of the previous step
        dma_wait();
        __syncthreads();
        const int stn = stage ^ 1;
        if constexpr (STAGES == 2) {
            if constexpr (SPREAD) {
                rvdma.issue(ST_ROW(stn), it + 1);
            } else {
                if (it + 1 < NGe) { if (stage) COL_DMA(it + 1, 0); else COL_DMA(it + 1, 1); }
            }
        }
        const T* gq = Q + (size_t)GRAN * (it + 1) * rsA;
        const T* gdh = dH + (size_t)GRAN * (it + 1) * rsB;
        T* const lq = ST_Q(stn);
        T* const ldh = ST_DH(stn);
        const T* Qs = ST_Q(stage);
        const T* dHs = ST_DH(stage);
        const float* srow = ST_ROW(stage);

        // ---- phase A
        const int qstart = qi0 + 32 * qbA;
        const bool skip = FIRST && kstartA > qstart;   // the block above the diagonal
        const bool diag = FIRST && kstartA == qstart;
        f32x4 sacc[2][2], dacc[2][2];   // [query half][key sub-block]
#pragma unroll
        for (int qh = 0; qh < 2; qh++)
#pragma unroll
            for (int kt = 0; kt < 2; kt++) { sacc[qh][kt] = f32x4{0.f, 0.f, 0.f, 0.f}; dacc[qh][kt] = f32x4{0.f, 0.f, 0.f, 0.f}; }
        float g[2][8], w[2][8];
        // per-query scalars of the lane's query in each half: read now, first used after the first half's MFMAs
        float crow[2], inv[2], dbv[2], er[2], beta_q[2];
        bool qvalid[2];
        const float sg_it = sG[it];
#pragma unroll
        for (int qh = 0; qh < 2; qh++) {
            const int ql = 32 * qbA + 16 * qh + l16;
            beta_q[qh] = srow[ql];
            inv[qh] = srow[GRAN + ql];
            dbv[qh] = srow[2 * GRAN + ql];
            qvalid[qh] = qi0 + ql < S;
        }
        auto query_scalars = [&]() {
#pragma unroll
            for (int qh = 0; qh < 2; qh++) {
                crow[qh] = log2scale - beta_q[qh] + sg_it;
                const float e = fast_exp2(crow[qh] + amaxA);
                er[qh] = qvalid[qh] ? e : 0.f;
            }
        };
        // element r of query half qh; mask-free steps: E = ekr[key] * er[query], the query factor goes into the per-lane
        // scalars, which leaves seven operations per element (G = dC~ E, W = C~ / n, dD = C~ dC~)
        float rsum[2] = {0.f, 0.f};
        auto elem = [&](int qh, int r) {
            float dd;
            const float sv = sacc[qh][r >> 2][r & 3], dv = dacc[qh][r >> 2][r & 3];
            if constexpr (FIRST) {
                float e = fast_exp2(al[r] + crow[qh]);
                const int kl = 32 * kbA + 16 * (r >> 2) + 4 * g4 + (r & 3), ql = 32 * qbA + 16 * qh + l16;
                if (!qvalid[qh] || skip || (diag && kl > ql)) e = 0.f;
                const float ct = sv * e;
                const float dct = dv * inv[qh] + dbv[qh];
                dd = ct * dct;
                g[qh][r] = dct * e;
                w[qh][r] = ct * inv[qh];
            } else {
                const float inv_er = inv[qh] * er[qh], dbv_er = dbv[qh] * er[qh];
                const float dct_er = dv * inv_er + dbv_er;
                const float sk = sv * ekr[r];
                g[qh][r] = dct_er * ekr[r];
                w[qh][r] = sk * inv_er;
                dd = sk * dct_er;
            }
            rsum[qh] += dd;
            colacc[r] += dd;
        };
        // Each of the four accumulators of a query half is the target of NS32 MFMAs in a row: measured, a 16x16x32 MFMA
        // issues every 17 cycles when it accumulates into the register the previous one wrote, but only every 23 (31)
        // when 4 (8) accumulators take turns.  Order per half: S (keys 0..15), S (keys 16..31), dC, dC.  The Q fragments
        // of the second half are read (into the same registers) once the first half's S chains are issued, its dH
        // fragments after the first half's dC chains; `between(chain, s)` is vector work placed behind an MFMA.
        frag qf[NS32], hf[NS32];
        auto rd = [&](const T* tile, int qh, int s) {
            return *reinterpret_cast<const frag*>(reinterpret_cast<const char*>(tile) + (32 * qbA + 16 * qh) * Swz<T, D>::ROW_BYTES +
                                                  qoff[s & 3] + (s >> 2) * 256);
        };
        auto chain = [&](int idx, f32x4& acc, const frag (&kk)[NS32], const frag (&xx)[NS32], auto&& between) {
#pragma unroll
            for (int s = 0; s < NS32; s++) {
                acc = Mma16<T>::mma(acc, kk[s], xx[s]);
                between(idx, s);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // copy of the next Q tile: one hook every four MFMAs of the first half
        constexpr int NH = NS32 >= 4 ? NS32 / 4 : 1;
        auto copy_hook = [&](int idx, int s) {
            if constexpr (SPREAD && STAGES == 2) {
                if (s % 4 == 0 && s / 4 < NH) {
                    const int k = idx * NH + s / 4;
                    tdma.issue_range(lq, gq, k * PW / (4 * NH), (k + 1) * PW / (4 * NH), ra);
                }
            }
        };
        // element-wise part of the first half, one element every four MFMAs of the second half
        auto ew_hook = [&](int idx, int s) {
            if constexpr (!FIRST) {
                constexpr int EPC = 2;   // elements per chain
#pragma unroll
                for (int e = 0; e < EPC; e++)
                    if (s == e * (NS32 / EPC)) elem(0, idx * EPC + e);
            }
        };
        // LDS operand reads, one per MFMA, each a few MFMAs ahead of its use (16 reads issued together would fill the
        // LDS queue and hold the wave for the time the four waves' 64 KB take):
        //   half 0: S chains read the rest of Q(0) and dH(0); the first dC chain reads Q(1) into the Q registers;
        //   half 1: the first S chain reads dH(1) into the dH registers.
        constexpr int LEAD = NS32 < 4 ? NS32 : 4;
        auto reads_h0 = [&](int idx, int s) {
            if (idx == 0) {
                if (s + LEAD < NS32) qf[s + LEAD] = rd(Qs, 0, s + LEAD);
                else hf[s + LEAD - NS32] = rd(dHs, 0, s + LEAD - NS32);
            } else if (idx == 1) {
                if (s + LEAD < NS32) hf[s + LEAD] = rd(dHs, 0, s + LEAD);
            } else if (idx == 2) {
                qf[s] = rd(Qs, 1, s);
            }
            copy_hook(idx, s);
        };
        auto reads_h1 = [&](int idx, int s) {
            if (idx == 0) hf[s] = rd(dHs, 1, s);
            ew_hook(idx, s);
            // first half of the copy of the next dH tile (the second half goes with phase B: issued any later it is not
            // there at the next barrier, measured 6 % slower with both tiles' copies in phase B)
            if constexpr (SPREAD) {
                if (idx < 2 && s % 4 == 2 && s / 4 < NH) {
                    const int k = idx * NH + s / 4;
                    tdma.issue_range(ldh, gdh, k * PW / (4 * NH), (k + 1) * PW / (4 * NH), rb);
                }
            }
        };
        // operand fragments of contraction step t: the next step's are read while this step's MFMAs run
        frag gB[2][NKB], wB[2][NKB], qa[2][NXW], ha[2][NXW];
        auto read_gw = [&](int t, int kb) {
            gB[t & 1][kb] = gw_read(Gs, t, kb);
            wB[t & 1][kb] = gw_read(Ws, t, kb);
        };
        auto read_qh = [&](int t, int x) {
            qa[t & 1][x] = trd.read(Qs, KW * t, XS * x);   // reader based at column block `wave`
            ha[t & 1][x] = trd.read(dHs, KW * t, XS * x);
        };
        if (!skip) {
#pragma unroll
            for (int s = 0; s < LEAD; s++) qf[s] = rd(Qs, 0, s);
            __builtin_amdgcn_sched_barrier(0);
            chain(0, sacc[0][0], kf[0], qf, reads_h0);
            chain(1, sacc[0][1], kf[1], qf, reads_h0);
            chain(2, dacc[0][0], vf[0], hf, reads_h0);
            chain(3, dacc[0][1], vf[1], hf, reads_h0);
            query_scalars();
            chain(0, sacc[1][0], kf[0], qf, reads_h1);
            chain(1, sacc[1][1], kf[1], qf, reads_h1);
            chain(2, dacc[1][0], vf[0], hf, reads_h1);
            chain(3, dacc[1][1], vf[1], hf, reads_h1);
            if constexpr (FIRST) {
#pragma unroll
                for (int r = 0; r < 8; r++) elem(0, r);
            }
            // phase B's first Q / dH fragments do not depend on G / W: their latency passes under the vector work below
#pragma unroll
            for (int x = 0; x < NXW; x++) read_qh(0, x);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int r = 0; r < 8; r++) elem(1, r);
        } else {
            if constexpr (SPREAD) {   // (no MFMA chains to carry this wave's share of the next tile's copy)
                tdma.issue(lq, gq, ra);
                tdma.issue_range(ldh, gdh, 0, PW / 2, rb);
            }
#pragma unroll
            for (int x = 0; x < NXW; x++) read_qh(0, x);
#pragma unroll
            for (int qh = 0; qh < 2; qh++)
#pragma unroll
                for (int r = 0; r < 8; r++) { g[qh][r] = 0.f; w[qh][r] = 0.f; }
        }
#pragma unroll
        for (int qh = 0; qh < 2; qh++) {
            const int ql = 32 * qbA + 16 * qh + l16;
#pragma unroll
            for (int kt = 0; kt < 2; kt++) {
                f32x4 gv, wv;
#pragma unroll
                for (int c = 0; c < 4; c++) { gv[c] = g[qh][4 * kt + c]; wv[c] = w[qh][4 * kt + c]; }
                const int chunk = 4 * kbA + 2 * kt + (g4 >> 1);  // keys 32*kbA + 16*kt + 4*g4 .. +3 of row ql
                const int off = ql * GRAN + ((chunk ^ gkey16(ql)) << 3) + 4 * (g4 & 1);
                *reinterpret_cast<typename R::vec4*>(Gs + off) = R::cvt4(gv);
                *reinterpret_cast<typename R::vec4*>(Ws + off) = R::cvt4(wv);
            }
            const float rs = sum_quarters(rsum[qh]);
            if (g4 == 0) rowtmp[kbA * GRAN + ql] = rs;
        }
        __syncthreads();

        // ---- phase B
        // row sums of this step: read now, stored after the MFMAs are issued (the wait for the two values would
        // otherwise hold the first wave, and with it the next barrier, for an LDS round trip)
        float rp0 = 0.f, rp1 = 0.f;
        if (tid < GRAN) { rp0 = rowtmp[tid]; rp1 = rowtmp[GRAN + tid]; }
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) read_gw(0, kb);
#pragma unroll
        for (int t = 0; t < NQS; t++) {
            if constexpr (SPREAD) { if (t < 2) tdma.issue_range(ldh, gdh, PW / 2 + t * PW / 4, PW / 2 + (t + 1) * PW / 4, rb); }
#pragma unroll
            for (int x = 0; x < NXW; x++) {
#pragma unroll
                for (int kb = 0; kb < NKB; kb++) {
                    if (t + 1 < NQS) {  // one quarter (or so) of the next step's reads per MFMA pair
                        if (x == 0) read_gw(t + 1, kb);
                        if (kb == 0) read_qh(t + 1, x);
                    }
                    R::mma(dkacc[kb][x], qa[t & 1][x], gB[t & 1][kb]);
                    R::mma(dvacc[kb][x], ha[t & 1][x], wB[t & 1][kb]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        if (tid < GRAN && qi0 + tid < S) a.rowpart[((size_t)bh * a.RS + (a.RS == NG ? jt : jt % a.RS)) * S + qi0 + tid] = rp0 + rp1;
    };
    // steps whose successor tile exists and is complete spread its copy over their MFMAs; the others copy in one go
    const int lim = (NGe < full_tiles ? NGe : full_tiles) - 1;   // last step index that may spread is lim - 1
    if (jt < lim) step(std::true_type{}, std::true_type{}, jt);
    else step(std::true_type{}, std::false_type{}, jt);
    int it = jt + 1;
    for (; it < lim; it++) step(std::false_type{}, std::true_type{}, it);
    for (; it < NGe; it++) step(std::false_type{}, std::false_type{}, it);
#undef COL_DMA
#undef ST_Q
#undef ST_DH
#undef ST_ROW

    // ---- epilogue: dK, dV.  A lane holds 4 consecutive columns of its key's row: stored directly that would be 8-byte
    // pieces scattered over 32 rows per instruction.  Each tensor goes through an LDS tile of its own (rows padded by 16
    // bytes; dK in the first query stage, dV in the second: both are free once every wave is past its last phase B) and
    // leaves in 16-byte pieces, a row at a time.
    {
        constexpr int RB = D * (int)sizeof(T) + 16, CPR = D * (int)sizeof(T) / 16, NPC = GRAN * CPR / 256;
        static_assert((size_t)GRAN * RB <= Cfg::STAGE_BYTES, "a staged output tile fits a query stage");
        __syncthreads();
#pragma unroll
        for (int which = 0; which < 2; which++) {
            char* const stage = smem + which * Cfg::STAGE_BYTES;
#pragma unroll
            for (int kb = 0; kb < NKB; kb++)
#pragma unroll
                for (int x = 0; x < NXW; x++)
#pragma unroll
                    for (int a4 = 0; a4 < 4; a4++) {
                        f32x4 v;
#pragma unroll
                        for (int c = 0; c < 4; c++) v[c] = which ? dvacc[kb][x][4 * a4 + c] : dkacc[kb][x][4 * a4 + c];
                        const int d = 32 * (BOTH_KB ? wave + XS * x : dsel + 2 * x) + 8 * a4 + 4 * h;
                        *reinterpret_cast<typename R::vec4*>(stage + (32 * (BOTH_KB ? kb : kbB) + c32) * RB + d * (int)sizeof(T)) = R::cvt4(v);
                    }
        }
        __syncthreads();
#pragma unroll
        for (int which = 0; which < 2; which++) {
            const char* const stage = smem + which * Cfg::STAGE_BYTES;
            char* const gout = reinterpret_cast<char*>(which ? a.dV : a.dK) + (offA + (size_t)GRAN * jt * rsA) * sizeof(T);
#pragma unroll
            for (int i = 0; i < NPC; i++) {
                const int c = tid + 256 * i, row = c / CPR, cc = c % CPR;
                if (GRAN * jt + row < S) {
                    *reinterpret_cast<uint4*>(gout + (size_t)row * rsA * sizeof(T) + 16 * cc) = *reinterpret_cast<const uint4*>(stage + row * RB + 16 * cc);
                }
            }
        }
    }
    // ---- column sums: reduce over the 16 query lanes and the two query halves are already in one register; then
    // over the two query blocks through LDS
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 8; r++) {
        // sum over the 16 query lanes of a DPP row: after the four shifted adds lane 15 of the row holds the total
        float v = colacc[r];
        v += dpp_f<0x111>(0.f, v);
        v += dpp_f<0x112>(0.f, v);
        v += dpp_f<0x114>(0.f, v);
        v += dpp_f<0x118>(0.f, v);
        if (l16 == 15) rowtmp[qbA * GRAN + 32 * kbA + 16 * (r >> 2) + 4 * g4 + (r & 3)] = v;
    }
    __syncthreads();
    if (tid < GRAN && GRAN * jt + tid < S)
        a.colsum[hoff + GRAN * jt + tid] = rowtmp[tid] + rowtmp[GRAN + tid] + colfar;
#endif
}

template <typename T, int D, bool DENSE>
static int launch_col16_t(const ColArgs& a, hipStream_t st) {
    using Cfg = Col16Cfg<T, D>;
    auto kern = col16_kernel<T, D, DENSE>;
    if (hipError_t e = lds_limit_once<col16_kernel<T, D, DENSE>>((int)(Cfg::LDS_BYTES + 2048 * sizeof(float))); e != hipSuccess) return (int)e;
    if (a.NG > 2048) return MLSTM_ESHAPE;
    hipLaunchKernelGGL(kern, dim3(a.BH * a.NG), dim3(256), Cfg::LDS_BYTES + (size_t)a.NG * sizeof(float), st, a);
    return (int)hipGetLastError();
}

int launch_col16_kernel(int dtype, int D, const ColArgs& a, hipStream_t st) {
    const bool dense = is_dense(a.la, a.S, D) && is_dense(a.lb, a.S, D);
    if (D == 128) {
        if (dtype == MLSTM_F16) return dense ? launch_col16_t<_Float16, 128, true>(a, st) : launch_col16_t<_Float16, 128, false>(a, st);
        if (dtype == MLSTM_BF16) return dense ? launch_col16_t<__bf16, 128, true>(a, st) : launch_col16_t<__bf16, 128, false>(a, st);
    }
    if (D == 256) {
        if (dtype == MLSTM_F16) return dense ? launch_col16_t<_Float16, 256, true>(a, st) : launch_col16_t<_Float16, 256, false>(a, st);
        if (dtype == MLSTM_BF16) return dense ? launch_col16_t<__bf16, 256, true>(a, st) : launch_col16_t<__bf16, 256, false>(a, st);
    }
    return MLSTM_ESHAPE;
}

}  // namespace mlstm
