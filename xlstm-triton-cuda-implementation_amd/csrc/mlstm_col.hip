// Column-parallel backward kernel of the matmul form: one workgroup owns a 64-key tile, keeps dK and dV for it in
// registers and walks the query tiles at or below the diagonal.  Replaces the dK/dV/dI loop of
// mlstm_matmul_kernel_backward (mlstm_matmul.py:269-316) and the fp16 CUDA kernel matmul_backward
// (cuda-src/mlstm_backward.cu:402-518, which stops at dK).
//
// Per 64x64 tile pair:
//   phase A (wave = one 32-key x 32-query block):  S^T = K Q^T, dC^T = V dH^T, then in registers
//       E = exp2(alpha_j - beta_i + dG) / sqrt(D),  C~ = S E,  dC~ = dC / n_i + db_i,
//       G = dC~ E (operand of dK),  W = C~ / n_i (operand of dV),  dD = C~ dC~ (row and column sums);
//       G and W go to LDS as [query][key].
//   phase B (wave = 32 keys x D/2 columns):  dK^T += Q^T G,  dV^T += dH^T W, both operands read from LDS with
//       transposing loads.
// Column sums of dD (= dI) stay in registers for the whole kernel; row sums leave the kernel as one partial per
// (key tile, query) and are added up by the dF pass, so rows and columns are sums of the very same fp32 products
// and the cancellation in dF = sigmoid(-f) * cumsum(col - row) stays exact to fp32 round-off.
//
// Long sequences in chunks (ColArgs::chunk_len): the keys walk the query tiles of their own chunk only; what the queries
// behind the chunk contribute comes through the chunk's reverse state E (value-major, mlstm_chunk.hip) in a state phase
// ahead of the query loop:  dK_j = w_j (E v_j + g),  dV_j = w_j E^T k_j,  w_j = exp(a_j - A_e), e the chunk's last
// position, and k_j . dK_j of that part goes into the column sums.  In split mode E comes as two terms, hi + lo.
#include <mutex>
#include <type_traits>
#include "mlstm_device.h"
#include "mlstm_kernels.h"

namespace mlstm {

template <typename T, int D, bool STRICT = false>
struct ColCfg {
    // G / W tiles [query][key], written by lanes in phase A and read transposed in phase B.  16-bit: 128-byte rows,
    // 16-byte chunk c of row q stored at chunk c ^ gkey(q); fp32: rows padded by 8 floats.
    static constexpr int LDG = Tr<T>::HALF ? GRAN : GRAN + 8;
    static constexpr size_t TILE_ELEMS = (size_t)GRAN * D;
    static constexpr size_t STAGE_BYTES = 2 * TILE_ELEMS * sizeof(T) + 3 * GRAN * sizeof(float);  // Q, dH, (beta, 1/n, db)
    static constexpr size_t G_BYTES = (size_t)GRAN * LDG * sizeof(T);
    // G, W (split mode: and their low-order terms), row-sum scratch.  With the two extra tiles the 16-bit D = 256 case
    // no longer fits two query stages and runs single-staged.
    static constexpr size_t GW_BYTES = (STRICT ? 4 : 2) * G_BYTES;
    static constexpr size_t FIXED_BYTES = GW_BYTES + 6 * GRAN * sizeof(float);   // + row sums [2][64], far column sums [4][64]
    static constexpr int STAGES = (2 * STAGE_BYTES + FIXED_BYTES + 2048 * sizeof(float) <= 160 * 1024) ? 2 : 1;
    static constexpr size_t LDS_BYTES = STAGES * STAGE_BYTES + FIXED_BYTES;  // plus one float per key tile, appended at launch
    // In chunks the keys' own K and V tiles lie in LDS during the state phase: in the second stage where there is one;
    // otherwise K in the (not yet used) G / W area and V in an extra tile between the fixed part and the granule bases
    static constexpr size_t TILE_BYTES = TILE_ELEMS * sizeof(T);
    static constexpr size_t EXTRA_CHUNK_BYTES = STAGES == 2 ? 0 : TILE_BYTES;
    static_assert(STAGES == 2 || GW_BYTES >= TILE_BYTES, "the keys' K tile fits the G / W area");
};

// Swizzle key of the 16-bit G / W tiles: bits (q>>1)&1 and (q>>2)&3 of the query row.  Phase A writes one chunk of
// 32 consecutive rows per instruction (all 16 residues of q spread over both 128-byte bank windows x 8 chunks);
// phase B gathers 4 consecutive rows x 64 bytes (rows q and q+2 land in different halves of the row).
__device__ __forceinline__ int gkey(int q) { return (((q >> 1) & 1) << 2) | ((q >> 2) & 3); }

// STRICT (16-bit types): split mode, see ColArgs::precise.
template <typename T, int D, bool STRICT>
__global__ __launch_bounds__(256, 1) void col_kernel(ColArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses device-only builtins; the host pass only needs the stub
    using R = Tr<T>;
    using Cfg = ColCfg<T, D, STRICT>;
    typedef typename R::frag frag;
    constexpr int KW = R::KW, NS = D / KW, NX = D / 64, NQS = GRAN / KW;
    // Phase B ownership.  D >= 128: wave w accumulates output column blocks {w*NXW .. } for BOTH key blocks, so each
    // transposed Q / dH fragment (the expensive ds_read_b64_tr_b16 traffic) is read by exactly one wave and feeds two
    // MFMAs.  D = 64 has only two column blocks: there a wave owns one key block and one column block.
    constexpr bool BOTH_KB = D >= 128;
    constexpr int NXW = BOTH_KB ? D / 128 : NX;   // column blocks per wave
    constexpr int NKB = BOTH_KB ? 2 : 1;          // key blocks per wave in phase B
    constexpr int LDG = Cfg::LDG, STAGES = Cfg::STAGES;
    extern __shared__ __attribute__((aligned(16))) char smem[];
#define ST_Q(st) (reinterpret_cast<T*>(smem + (st) * Cfg::STAGE_BYTES))
#define ST_DH(st) (ST_Q(st) + Cfg::TILE_ELEMS)
#define ST_ROW(st) (reinterpret_cast<float*>(ST_DH(st) + Cfg::TILE_ELEMS))
    T* const Gs = reinterpret_cast<T*>(smem + STAGES * Cfg::STAGE_BYTES);
    T* const Ws = Gs + GRAN * LDG;
    T* const Gl = Ws + GRAN * LDG;                                    // split mode: low-order terms of G and W
    T* const Wl = Gl + GRAN * LDG;
    float* const rowtmp = reinterpret_cast<float*>(Gs + (STRICT ? 4 : 2) * GRAN * LDG);  // [2][64]
    float* const cpart = rowtmp + 2 * GRAN;                                               // [4][64]
    // granule bases minus this key tile's (see row kernel)
    float* const sG = reinterpret_cast<float*>(smem + Cfg::LDS_BYTES + (a.chunk_len > 0 ? Cfg::EXTRA_CHUNK_BYTES : 0));

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, h = lane >> 5, c32 = lane & 31;
    const int S = a.S, NG = a.NG;
    int bh, jt;
    {
        const int bid = blockIdx.x;  // key tile 0 has the longest loop: ascending order is heaviest first
        if ((a.BH & 7) == 0) {
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
    const size_t rsA = (size_t)a.la.ss, rsB = (size_t)a.lb.ss, offA = a.la.head(bh), offB = a.lb.head(bh);
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
    // In chunks the keys walk the query tiles of their own chunk only (NGe: one past the last of them)
    const int tpc = a.chunk_len > 0 ? a.chunk_len / GRAN : 0;
    const int chunk = a.chunk_len > 0 ? jt / tpc : 0;
    const int NGe = a.chunk_len > 0 ? ((chunk + 1) * tpc < NG ? (chunk + 1) * tpc : NG) : NG;
    const bool has_state = a.chunk_len > 0 && chunk < a.n_states;   // (uniform over the workgroup)
    constexpr int NTL = D / GRAN;   // 64-row tiles of a state
    T* const Kt = STAGES == 2 ? ST_Q(1) : Gs;
    T* const Vt = STAGES == 2 ? ST_DH(1) : reinterpret_cast<T*>(smem + Cfg::LDS_BYTES);
    const size_t sbase = has_state ? ((size_t)bh * a.n_states + chunk) * D * D : 0;
    const T* const Evc = reinterpret_cast<const T*>(a.Ev) + sbase;
    const T* const Evl = STRICT ? reinterpret_cast<const T*>(a.Ev_lo) + sbase : nullptr;
    // state tile tau: split mode hi -> Q slot, lo -> dH slot of stage 0, one tile per round; otherwise tile tau -> slot
    // tau & 1, the next tile travelling while this one is worked on
    auto state_issue = [&](int tau) {
        if constexpr (STRICT) {
            tdma.issue(ST_Q(0), Evc + (size_t)GRAN * tau * D);
            tdma.issue(ST_DH(0), Evl + (size_t)GRAN * tau * D);
        } else {
            tdma.issue((tau & 1) ? ST_DH(0) : ST_Q(0), Evc + (size_t)GRAN * tau * D);
        }
    };
    if (has_state) {   // (a chunk with a successor is complete: its key tiles have all their rows)
        tdma.issue(Kt, K + (size_t)GRAN * jt * rsA, ra);
        tdma.issue(Vt, V + (size_t)GRAN * jt * rsA, ra);
        state_issue(0);
    } else {
        COL_DMA(jt, 0);  // first of all: its latency then overlaps that of the plain loads below
    }
    {
        const double gj = a.G2[(size_t)bh * a.NG + jt];
        for (int g = threadIdx.x; g < a.NG; g += 256) sG[g] = (float)(a.G2[(size_t)bh * a.NG + g] - gj);
    }

    const int kstartA = GRAN * jt + 32 * kbA;
    const int keyA = kstartA + c32, keyAc = keyA < S ? keyA : S - 1;
    frag kf[NS], vf[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) {
        kf[s] = frag_rowmajor<T>(K + (size_t)keyAc * rsA, s, h);
        vf[s] = frag_rowmajor<T>(V + (size_t)keyAc * rsA, s, h);
    }
    float al[16];
#pragma unroll
    for (int r = 0; r < 16; r++) al[r] = a.alpha2[poff + kstartA + 8 * (r >> 2) + 4 * h + (r & 3)];
#pragma unroll
    for (int s = 0; s < NS; s++) { pin(kf[s]); pin(vf[s]); }
    // factorised weights for the steps below the diagonal: ekr[r] = exp2(alpha_key(r) - c0), c0 the block maximum
    float ekr[16], amaxA;
    {
        float mx = al[0];
#pragma unroll
        for (int r = 1; r < 16; r++) mx = fmaxf(mx, al[r]);
        amaxA = fmaxf(mx, __shfl_xor(mx, 32));
#pragma unroll
        for (int r = 0; r < 16; r++) ekr[r] = amaxA > -INFINITY ? fast_exp2(al[r] - amaxA) : 0.f;
    }
#pragma unroll
    for (int r = 0; r < 16; r++) { pin(al[r]); pin(ekr[r]); }
    pin(amaxA);
    // (sG becomes visible, and the first tile is waited for, at the barrier that opens the first step; every plain
    // global load above has been waited for by pin)
    const float log2scale = -0.5f * __log2f((float)D);

    float colacc[16];
#pragma unroll
    for (int r = 0; r < 16; r++) colacc[r] = 0.f;
    f32x16 dkacc[NKB][NXW], dvacc[NKB][NXW];
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
        for (int x = 0; x < NXW; x++)
#pragma unroll
            for (int r = 0; r < 16; r++) { dkacc[kb][x][r] = 0.f; dvacc[kb][x][r] = 0.f; }

    constexpr bool FAST_TR = R::HALF && Swz<T, D>::CPR >= 16;
    SwzRowReader<T, D> qrd;
    qrd.init(lane);
    SwzTransReader<typename std::conditional<FAST_TR, T, __bf16>::type, FAST_TR ? D : 256> trd;
    if constexpr (FAST_TR) trd.init(lane, BOTH_KB ? wave * NXW : 0);

    // ---- state phase (sequences in chunks)
    // (k_j . dK_j of the state part, the far column sums, stay in cpart[0..63] until the end of the kernel)
    if (has_state) {
        constexpr int NGRP = GRAN / KW;
        const int pe = (chunk + 1) * a.chunk_len - 1;   // the chunk's last position
        const float bend = a.beta2[poff + pe];
        const double dG = a.G2[(size_t)bh * a.NG + pe / GRAN] - a.G2[(size_t)bh * a.NG + jt];   // (the keys' granule is jt)
        float wk[NKB];
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) wk[kb] = fast_exp2(a.alpha2[poff + GRAN * jt + 32 * (BOTH_KB ? kb : kbB) + c32] - bend + (float)dG);
        auto col_block = [&](int x) { return BOTH_KB ? wave * NXW + x : dsel + 2 * x; };
        auto rd_tr = [&](const T* tile, int tt, int x) {
            if constexpr (FAST_TR) return trd.read(tile, KW * tt, BOTH_KB ? x : col_block(x));
            else return swz_frag_transposed<T, D>(tile, KW * tt, 32 * col_block(x), lane);
        };
#pragma unroll
        for (int tau = 0; tau < NTL; tau++) {
            dma_wait();
            __syncthreads();   // tile tau (and, the first time, the keys' K and V) have landed
            const T* th = STRICT ? ST_Q(0) : ((tau & 1) ? ST_DH(0) : ST_Q(0));
            const T* tl = ST_DH(0);
            if constexpr (!STRICT) { if (tau + 1 < NTL) state_issue(tau + 1); }
            // dK: contraction over this tile's 64 rows (values 64 tau ..), the wave's columns of the state
#pragma unroll
            for (int tt = 0; tt < NGRP; tt++) {
                frag vB[NKB], ea[NXW], el[STRICT ? NXW : 1];
#pragma unroll
                for (int kb = 0; kb < NKB; kb++) vB[kb] = swz_frag_rowmajor<T, D>(Vt, 32 * (BOTH_KB ? kb : kbB) + c32, NGRP * tau + tt, h);
#pragma unroll
                for (int x = 0; x < NXW; x++) {
                    ea[x] = rd_tr(th, tt, x);
                    if constexpr (STRICT) el[x] = rd_tr(tl, tt, x);
                }
#pragma unroll
                for (int x = 0; x < NXW; x++)
#pragma unroll
                    for (int kb = 0; kb < NKB; kb++) {
                        R::mma(dkacc[kb][x], ea[x], vB[kb]);
                        if constexpr (STRICT) R::mma(dkacc[kb][x], el[x], vB[kb]);
                    }
            }
            // dV: the wave's own rows of the state, if this tile holds them, contracted over the whole key index
#pragma unroll
            for (int x = 0; x < NXW; x++) {
                const int r0v = 32 * col_block(x);
                if (r0v / GRAN != tau) continue;
                const int rl = r0v % GRAN + c32;
                // (16-bit states keep their rows in the contraction order of the transposing reads, see mlstm_chunk.hip)
                const int own = R::HALF ? ((rl & ~15) | ((rl & 3) | ((rl & 4) << 1) | ((rl & 8) >> 1))) : rl;
#pragma unroll
                for (int t = 0; t < NS; t++) {
                    frag kB[NKB];
#pragma unroll
                    for (int kb = 0; kb < NKB; kb++) kB[kb] = swz_frag_rowmajor<T, D>(Kt, 32 * (BOTH_KB ? kb : kbB) + c32, t, h);
                    const frag eb = swz_frag_rowmajor<T, D>(th, own, t, h);
#pragma unroll
                    for (int kb = 0; kb < NKB; kb++) R::mma(dvacc[kb][x], eb, kB[kb]);
                    if constexpr (STRICT) {
                        const frag ebl = swz_frag_rowmajor<T, D>(tl, own, t, h);
#pragma unroll
                        for (int kb = 0; kb < NKB; kb++) R::mma(dvacc[kb][x], ebl, kB[kb]);
                    }
                }
            }
            if constexpr (STRICT) {
                __syncthreads();   // every wave is done with the tile: the next one may overwrite it
                if (tau + 1 < NTL) state_issue(tau + 1);
            }
        }
        if constexpr (!STRICT) __syncthreads();   // every wave is done with stage 0
        COL_DMA(jt, 0);   // the first query tile follows the state into stage 0
        // the keys' weights, the vector state, and k_j . dK_j for the column sums
        const float* gv = a.gvec + ((size_t)bh * a.n_states + chunk) * D;
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) {
            float cp = 0.f;
            const int krow = 32 * (BOTH_KB ? kb : kbB) + c32;
#pragma unroll
            for (int x = 0; x < NXW; x++)
#pragma unroll
                for (int a4 = 0; a4 < 4; a4++) {
                    const int d = 32 * col_block(x) + 8 * a4 + 4 * h;
                    const f32x4 g4v = *reinterpret_cast<const f32x4*>(gv + d);
                    const char* kp = reinterpret_cast<const char*>(Kt) + Swz<T, D>::off(krow, d & ~(Swz<T, D>::EPC - 1)) + (d & (Swz<T, D>::EPC - 1)) * (int)sizeof(T);
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
            if (h == 0) {
                cpart[wave * GRAN + krow] = cp;
                if constexpr (!BOTH_KB) cpart[wave * GRAN + (krow ^ 32)] = 0.f;
            }
        }
        __syncthreads();   // the waves' shares of k . dK lie in LDS (and Kt, in the G / W area, is done with)
        if (tid < GRAN) cpart[tid] = (cpart[tid] + cpart[GRAN + tid]) + (cpart[2 * GRAN + tid] + cpart[3 * GRAN + tid]);
    }

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
                gwoff[kb][x] = q * GRAN + ((c ^ gkey(q)) << 3) + 4 * (j & 1);
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
        const int qrow = qstart + c32;
        f32x16 g, w;
        float rsum = 0.f;
        if (!FIRST || kstartA <= qstart) {
            const bool diag = FIRST && kstartA == qstart;
            f32x16 sacc, dacc;
            // The operand reads run AHEAD fragments in front of the MFMAs that consume them (a wave issues in order:
            // without the explicit interleave the reads of a batch and its MFMAs would take turns).
            constexpr int AHEAD = NS < 4 ? NS : 4;
            frag qf[NS], hf[NS];
#pragma unroll
            for (int s = 0; s < AHEAD; s++) { qf[s] = qrd.read(Qs, qbA, s); hf[s] = qrd.read(dHs, qbA, s); }
#pragma unroll
            for (int s = 0; s < NS; s++) {
                if constexpr (SPREAD && STAGES == 2) {
                    if (s % AHEAD == 0) tdma.issue_range(lq, gq, (s / AHEAD) * PW / (NS / AHEAD), (s / AHEAD + 1) * PW / (NS / AHEAD), ra);
                }
                if (s + AHEAD < NS) { qf[s + AHEAD] = qrd.read(Qs, qbA, s + AHEAD); hf[s + AHEAD] = qrd.read(dHs, qbA, s + AHEAD); }
                if (s == 0) {
                    const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                    sacc = z; dacc = z;
                }
                R::mma(sacc, kf[s], qf[s]);
                R::mma(dacc, vf[s], hf[s]);
                __builtin_amdgcn_sched_barrier(0);
            }
            const float crow = log2scale - srow[32 * qbA + c32] + sG[it];
            const float inv = srow[GRAN + 32 * qbA + c32], dbv = srow[2 * GRAN + 32 * qbA + c32];
            const bool qvalid = qrow < S;
            const float er = qvalid ? fast_exp2(crow + amaxA) : 0.f;
            // below the diagonal E = ekr[key] * er[query]: the query factor goes into the per-lane scalars, which leaves
            // seven operations per element (G = dC~ E, W = C~ / n, dD = C~ dC~ with C~ = S E, dC~ = dC / n + db)
            const float inv_er = inv * er, dbv_er = dbv * er;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float dd;
                if constexpr (FIRST) {
                    float e = fast_exp2(al[r] + crow);
                    if (!qvalid || (diag && (8 * (r >> 2) + 4 * h + (r & 3) > c32))) e = 0.f;
                    const float ct = sacc[r] * e;
                    const float dct = dacc[r] * inv + dbv;
                    dd = ct * dct;
                    g[r] = dct * e;
                    w[r] = ct * inv;
                } else {
                    const float dct_er = dacc[r] * inv_er + dbv_er;
                    const float sk = sacc[r] * ekr[r];
                    g[r] = dct_er * ekr[r];
                    w[r] = sk * inv_er;
                    dd = sk * dct_er;
                }
                rsum += dd;
                colacc[r] += dd;
            }
        } else {
#pragma unroll
            for (int r = 0; r < 16; r++) { g[r] = 0.f; w[r] = 0.f; }
        }
        {
#pragma unroll
            for (int a4 = 0; a4 < 4; a4++) {
                f32x4 gv, wv;
#pragma unroll
                for (int c = 0; c < 4; c++) { gv[c] = g[4 * a4 + c]; wv[c] = w[4 * a4 + c]; }
                int off;  // element offset of keys 32*kbA + 8*a4 + 4*h .. +3 of row 32*qbA + c32
                if constexpr (R::HALF) off = (32 * qbA + c32) * GRAN + (((4 * kbA + a4) ^ gkey(c32)) << 3) + 4 * h;
                else off = (32 * qbA + c32) * LDG + 32 * kbA + 8 * a4 + 4 * h;
                if constexpr (STRICT) {
                    typename R::vec4 ghi, glo, whi, wlo;
                    R::cvt4_split(gv, ghi, glo);
                    R::cvt4_split(wv, whi, wlo);
                    *reinterpret_cast<typename R::vec4*>(Gs + off) = ghi;
                    *reinterpret_cast<typename R::vec4*>(Ws + off) = whi;
                    *reinterpret_cast<typename R::vec4*>(Gl + off) = glo;
                    *reinterpret_cast<typename R::vec4*>(Wl + off) = wlo;
                } else {
                    *reinterpret_cast<typename R::vec4*>(Gs + off) = R::cvt4(gv);
                    *reinterpret_cast<typename R::vec4*>(Ws + off) = R::cvt4(wv);
                }
            }
            const float rs = sum_halves(rsum);
            if (h == 0) rowtmp[kbA * GRAN + 32 * qbA + c32] = rs;
        }
        __syncthreads();

        // ---- phase B
        // row sums of this step: read now, stored after the MFMAs are issued (the wait for the two values would
        // otherwise hold the first wave, and with it the next barrier, for an LDS round trip)
        float rp0 = 0.f, rp1 = 0.f;
        if (tid < GRAN) { rp0 = rowtmp[tid]; rp1 = rowtmp[GRAN + tid]; }
        // operand fragments of contraction step t: the next step's are read while this step's MFMAs run
        frag gB[2][NKB], wB[2][NKB], qa[2][NXW], ha[2][NXW];
        // (split mode: the low-order fragments are single-buffered, read at the start of their own step behind the
        // MFMAs on the high-order ones: a second set of them does not fit the registers at D = 256)
        frag gL[STRICT ? NKB : 1], wL[STRICT ? NKB : 1];
        auto read_gw = [&](int t, int kb) {
            if constexpr (R::HALF) {
                gB[t & 1][kb] = gw_read(Gs, t, kb);
                wB[t & 1][kb] = gw_read(Ws, t, kb);
            } else {
                gB[t & 1][kb] = frag_transposed<T>(Gs, LDG, KW * t, 32 * (BOTH_KB ? kb : kbB), lane);
                wB[t & 1][kb] = frag_transposed<T>(Ws, LDG, KW * t, 32 * (BOTH_KB ? kb : kbB), lane);
            }
        };
        auto read_qh = [&](int t, int x) {
            const int dblk = BOTH_KB ? wave * NXW + x : dsel + 2 * x;
            if constexpr (FAST_TR) {
                if constexpr (BOTH_KB) { qa[t & 1][x] = trd.read(Qs, KW * t, x); ha[t & 1][x] = trd.read(dHs, KW * t, x); }   // reader based at wave*NXW
                else { qa[t & 1][x] = trd.read(Qs, KW * t, dblk); ha[t & 1][x] = trd.read(dHs, KW * t, dblk); }
            } else {
                qa[t & 1][x] = swz_frag_transposed<T, D>(Qs, KW * t, 32 * dblk, lane);
                ha[t & 1][x] = swz_frag_transposed<T, D>(dHs, KW * t, 32 * dblk, lane);
            }
        };
#pragma unroll
        for (int kb = 0; kb < NKB; kb++) read_gw(0, kb);
#pragma unroll
        for (int x = 0; x < NXW; x++) read_qh(0, x);
#pragma unroll
        for (int t = 0; t < NQS; t++) {
            if constexpr (SPREAD && STAGES == 2) tdma.issue_range(ldh, gdh, t * PW / NQS, (t + 1) * PW / NQS, rb);
#pragma unroll
            for (int x = 0; x < NXW; x++) {
#pragma unroll
                for (int kb = 0; kb < NKB; kb++) {
                    if (t + 1 < NQS) {  // one quarter (or so) of the next step's reads per MFMA pair
                        if (x == 0) read_gw(t + 1, kb);
                        if (kb == 0) read_qh(t + 1, x);
                    }
                    if constexpr (STRICT) {
                        if (x == 0) { gL[kb] = gw_read(Gl, t, kb); wL[kb] = gw_read(Wl, t, kb); }
                    }
                    R::mma(dkacc[kb][x], qa[t & 1][x], gB[t & 1][kb]);
                    R::mma(dvacc[kb][x], ha[t & 1][x], wB[t & 1][kb]);
                    if constexpr (STRICT) {
                        R::mma(dkacc[kb][x], qa[t & 1][x], gL[kb]);
                        R::mma(dvacc[kb][x], ha[t & 1][x], wL[kb]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
        if (tid < GRAN && qi0 + tid < S) a.rowpart[((size_t)bh * a.RS + (a.RS == NG ? jt : jt % a.RS)) * S + qi0 + tid] = rp0 + rp1;
        if constexpr (STAGES == 1) {
            __syncthreads();  // single stage: everyone is done reading before the overwrite, which the next top barrier awaits
            if (it + 1 < NGe) COL_DMA(it + 1, 0);
        }
    };
    // steps whose successor tile exists and is complete spread its copy over their MFMAs; the others copy in one go
    const int lim = (NGe < full_tiles ? NGe : full_tiles) - 1;   // last step index that may spread is lim - 1
    step(std::true_type{}, std::false_type{}, jt);  // the diagonal step skips a block in some waves: it copies in one go
    int it = jt + 1;
    for (; it < lim; it++) step(std::false_type{}, std::true_type{}, it);
    for (; it < NGe; it++) step(std::false_type{}, std::false_type{}, it);
#undef COL_DMA
#undef ST_Q
#undef ST_DH
#undef ST_ROW

    // ---- epilogue: dK, dV.  A lane holds 4 consecutive columns of its key's row: stored directly that would be 8-byte
    // pieces scattered over 32 rows per instruction.  Each tensor goes through an LDS tile (rows padded by 16 bytes)
    // and leaves in 16-byte pieces, a row at a time.
    {
        constexpr int RB = D * (int)sizeof(T) + 16, CPR = D * (int)sizeof(T) / 16;
        char* const stage = smem;  // the Q / dH stages are free once every wave is past its last phase B
#pragma unroll
        for (int which = 0; which < 2; which++) {
            __syncthreads();
#pragma unroll
            for (int kb = 0; kb < NKB; kb++)
#pragma unroll
                for (int x = 0; x < NXW; x++)
#pragma unroll
                    for (int a4 = 0; a4 < 4; a4++) {
                        f32x4 v;
#pragma unroll
                        for (int c = 0; c < 4; c++) v[c] = which ? dvacc[kb][x][4 * a4 + c] : dkacc[kb][x][4 * a4 + c];
                        const int d = 32 * (BOTH_KB ? wave * NXW + x : dsel + 2 * x) + 8 * a4 + 4 * h;
                        *reinterpret_cast<typename R::vec4*>(stage + (32 * (BOTH_KB ? kb : kbB) + c32) * RB + d * (int)sizeof(T)) = R::cvt4(v);
                    }
            __syncthreads();
            char* const gout = reinterpret_cast<char*>(which ? a.dV : a.dK) + (offA + (size_t)GRAN * jt * rsA) * sizeof(T);
#pragma unroll
            for (int i = 0; i < GRAN * CPR / 256; i++) {
                const int c = tid + 256 * i, row = c / CPR, cc = c % CPR;
                if (GRAN * jt + row < S)
                    *reinterpret_cast<uint4*>(gout + (size_t)row * rsA * sizeof(T) + 16 * cc) = *reinterpret_cast<const uint4*>(stage + row * RB + 16 * cc);
            }
        }
    }
    // ---- column sums: reduce over the 32 query lanes, then over the two query blocks through LDS
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 16; r++) {
        float v = colacc[r];
        v += __shfl_xor(v, 1);
        v += __shfl_xor(v, 2);
        v += __shfl_xor(v, 4);
        v += __shfl_xor(v, 8);
        v += __shfl_xor(v, 16);
        if (c32 == 0) rowtmp[qbA * GRAN + 32 * kbA + 8 * (r >> 2) + 4 * h + (r & 3)] = v;
    }
    __syncthreads();
    if (tid < GRAN && GRAN * jt + tid < S) a.colsum[hoff + GRAN * jt + tid] = rowtmp[tid] + rowtmp[GRAN + tid] + (has_state ? cpart[tid] : 0.f);
#endif
}

template <typename T, int D, bool STRICT>
static int launch_col_ts(const ColArgs& a, hipStream_t st) {
    using Cfg = ColCfg<T, D, STRICT>;
    auto kern = col_kernel<T, D, STRICT>;
    static std::once_flag once;
    static hipError_t attr_rc = hipSuccess;
    std::call_once(once, [&] {
        attr_rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      (int)(Cfg::LDS_BYTES + Cfg::EXTRA_CHUNK_BYTES + 2048 * sizeof(float)));
    });
    if (attr_rc != hipSuccess) return (int)attr_rc;
    if (a.NG > 2048) return MLSTM_ESHAPE;
    if (a.chunk_len > 0 && (a.chunk_len % GRAN != 0 || (a.n_states > 0 && (!a.Ev || !a.gvec || (STRICT && !a.Ev_lo))))) return MLSTM_EINVAL;
    const size_t lds = Cfg::LDS_BYTES + (a.chunk_len > 0 ? Cfg::EXTRA_CHUNK_BYTES : 0) + (size_t)a.NG * sizeof(float);
    if (lds > 160 * 1024) return MLSTM_ESHAPE;
    hipLaunchKernelGGL(kern, dim3(a.BH * a.NG), dim3(256), lds, st, a);
    return (int)hipGetLastError();
}

template <typename T, int D>
static int launch_col_t(const ColArgs& a, hipStream_t st) {
    if constexpr (Tr<T>::HALF) {
        if (a.precise) return launch_col_ts<T, D, true>(a, st);
    }
    return launch_col_ts<T, D, false>(a, st);
}

template <typename T>
static int launch_col_d(int D, const ColArgs& a, hipStream_t st) {
    switch (D) {
        case 64: return launch_col_t<T, 64>(a, st);
        case 128: return launch_col_t<T, 128>(a, st);
        case 256:
            if constexpr (Tr<T>::HALF) return launch_col_t<T, 256>(a, st);
            else return MLSTM_ESHAPE;
    }
    return MLSTM_ESHAPE;
}

int launch_col_kernel(int dtype, int D, const ColArgs& a, hipStream_t st) {
    switch (dtype) {
        case MLSTM_F32: return launch_col_d<float>(D, a, st);
        case MLSTM_F16: return launch_col_d<_Float16>(D, a, st);
        case MLSTM_BF16: return launch_col_d<__bf16>(D, a, st);
    }
    return MLSTM_EINVAL;
}

}  // namespace mlstm
