// Row-parallel tile kernel of the matmul form: one workgroup owns 128 query rows (4 waves x 32 rows) and walks
// the causal key tiles.  Two instantiations share the body:
//
//   MODE_FWD  X=Q, Y1=K, Y2=V:  S^T = K Q^T, P = S * exp2(alpha_j - beta_i + dG) / sqrt(D), b += rowsum P,
//             H^T += V^T P^T, epilogue h = H / (max(|b|, exp(-m)) + 1e-6).
//             Replaces mlstm_matmul_kernel (mlstm_matmul.py:38-101) and the CUDA kernel mlstm_forward
//             (cuda-src/mlstm_forward.cu:14-189).
//   MODE_DQ   X=dH, Y1=V, Y2=K: dC^T = V dH^T, G = (dC / n_i + db_i) * exp2(...) / sqrt(D), dQ^T += K^T G^T.
//             Replaces the dQ loop of mlstm_matmul_kernel_backward (mlstm_matmul.py:239-267).
//
// The products are computed transposed (keys along accumulator rows, queries along lanes) so that the
// accumulator of the first product is already laid out as the B operand of the second one: no lane exchange
// and every per-query scalar (beta, 1/n, db, the running row sum) lives in one register of one lane.
// There is no online max: the row maximum comes from the gate pre-pass as a prefix maximum.
//
// Memory pipeline: the two 64-key tiles of step j+1 are copied global->LDS by direct loads (no registers) into
// the other of two LDS stages while step j is consumed; one barrier per step.  Tiles are XOR-swizzled.
//
// Long sequences in chunks (RowArgs::chunk_len): a row tile walks the key tiles of its own chunk only; what lies before
// the chunk enters through the state at the end of the previous chunk (mlstm_chunk.hip), D/64 tiles of 64 state rows
// that pass through the same LDS stages ahead of the key tiles and are contracted with the rows' own X fragments:
//   forward  H^T += C~^T-tiles x Q^T, then the rows' decay exp(A_e - A_i), and b += decay (q_i . n~);
//   dQ pass  dQ^T += C~-tiles (value-major) x dH^T, then decay / n_i, the rank-one term decay db_i n~, and the row sums
//            q_i . dQ_i of dD over the keys before the chunk.
// In split mode the state comes as two terms, hi + lo (one tile each per stage), and takes two MFMAs per fragment.
#include <mutex>
#include <type_traits>
#include "mlstm_device.h"
#include "mlstm_kernels.h"

namespace mlstm {

constexpr int MODE_FWD = 0, MODE_DQ = 1;
constexpr int ROW_BQ = 128;

template <typename T, int D>
struct RowCfg {
    static constexpr size_t TILE_ELEMS = (size_t)GRAN * D;
    static constexpr size_t STAGE_BYTES = 2 * TILE_ELEMS * sizeof(T) + 3 * GRAN * sizeof(float);  // Y1, Y2, alpha, ek, amax
    static constexpr size_t STAGES_BYTES = 2 * STAGE_BYTES;
    // plus one double per key tile of the head (the granule bases), appended at launch
};

// STRICT (16-bit types): split mode, see RowArgs::precise.
template <typename T, int D, int MODE, bool STRICT>
__global__ __launch_bounds__(256, 1) void row_kernel(RowArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses device-only builtins; the host pass only needs the stub
    using R = Tr<T>;
    using Cfg = RowCfg<T, D>;
    typedef typename R::frag frag;
    constexpr int KW = R::KW, NS = D / KW, NDB = D / 32, NSTEP32 = 32 / KW;
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, h = lane >> 5, c32 = lane & 31;
    int S = a.S, NG = a.NG;
    const int nQT = (S + ROW_BQ - 1) / ROW_BQ;
    int bh, qt;
    {
        // heaviest query tiles first over ALL heads (a per-head-group order leaves heavy tiles of the last group for the end); all tiles of a head run on one XCD
        // (workgroups are dealt round-robin to the 8 XCDs) so that its K/V stay in that XCD's L2
        const int bid = blockIdx.x;
        if ((a.BH & 7) == 0) {
            int rest = bid >> 3;
            const int ngrp = a.BH >> 3;
            bh = (rest % ngrp) * 8 + (bid & 7);
            qt = nQT - 1 - rest / ngrp;
        } else {
            bh = bid % a.BH;
            qt = nQT - 1 - bid / a.BH;
        }
    }
    size_t hoff = (size_t)bh * S, poff = (size_t)bh * NG * GRAN, goff = (size_t)bh * NG;
    // the caller's tensors: q, k, v, dq in layout la, h, dh, o in lb (element offset of the head, elements per position)
    const size_t rsA = (size_t)a.la.ss, rsB = (size_t)a.lb.ss, rsH = (size_t)a.lh.ss;
    size_t offA = a.la.head(bh), offB = a.lb.head(bh), offH = a.lh.head(bh);
    // In chunks the workgroup's rows lie in chunk `chunk`, and everything below addresses positions relative to the chunk's
    // first one: the sequence "starts" there (offsets move forward; S, NG and the row tile index shrink).
    int chunk = 0;
    if (a.chunk_len > 0) {
        chunk = (qt * ROW_BQ) / a.chunk_len;
        const int p0 = chunk * a.chunk_len;
        hoff += p0; poff += p0; goff += p0 / GRAN;
        offA += (size_t)p0 * rsA; offB += (size_t)p0 * rsB; offH += (size_t)p0 * rsH;
        S -= p0; NG -= p0 / GRAN; qt -= p0 / ROW_BQ;
    }
    const int q0 = qt * ROW_BQ, r0 = q0 + 32 * wave;
    const int row = r0 + c32, rowc = row < S ? row : S - 1;
    const bool wave_active = r0 < S;
    const size_t rsX = MODE == MODE_FWD ? rsA : rsB, offX = MODE == MODE_FWD ? offA : offB;
    const size_t rsO = MODE == MODE_FWD ? rsB : rsA, offO = MODE == MODE_FWD ? offB : offA;
    const T* X = reinterpret_cast<const T*>(a.X) + offX;
    const T* Y1 = reinterpret_cast<const T*>(a.Y1) + offA;
    const T* Y2 = reinterpret_cast<const T*>(a.Y2) + offA;

    frag xf[NS];
#pragma unroll
    for (int s = 0; s < NS; s++) xf[s] = frag_rowmajor<T>(X + (size_t)rowc * rsX, s, h);

    // granule bases of this head in LDS: a global load inside the main loop would have to be waited for with
    // vmcnt(0), which would also wait for the tile copies in flight
    double* const sG = reinterpret_cast<double*>(smem + Cfg::STAGES_BYTES);
    for (int g = tid; g < NG; g += 256) sG[g] = a.G2[goff + g];
    float crow_base = -0.5f * __log2f((float)D) - a.beta2[poff + rowc];
    float inv_n = 0.f, dbv = 0.f;
    if constexpr (MODE == MODE_DQ) {
        const T* hlo = nullptr;
        if constexpr (STRICT) { if (a.Hin_lo) hlo = reinterpret_cast<const T*>(a.Hin_lo) + (hoff + rowc) * D; }
        row_stats<T, NS>(xf, reinterpret_cast<const T*>(a.Hin) + offH + (size_t)rowc * rsH, h, a.Bin[hoff + rowc], a.M[hoff + rowc], inv_n, dbv, hlo);
        if (row < S && h == 0) { a.inv_n[poff + row] = inv_n; a.db[poff + row] = dbv; }
    }
#pragma unroll
    for (int s = 0; s < NS; s++) pin(xf[s]);
    pin(crow_base); pin(inv_n); pin(dbv);

    f32x16 oacc[NDB];
#pragma unroll
    for (int d = 0; d < NDB; d++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[d][r] = 0.f;
    float bsum = 0.f;

    constexpr bool FAST_TR = R::HALF && Swz<T, D>::CPR >= 16;  // precomputed offsets for the transposing reads
    SwzRowReader<T, D> krd;
    krd.init(lane);
    SwzTransReader<typename std::conditional<FAST_TR, T, __bf16>::type, FAST_TR ? D : 256> vrd;
    if constexpr (FAST_TR) vrd.init(lane);

    const int last_row = (q0 + ROW_BQ - 1 < S - 1) ? q0 + ROW_BQ - 1 : S - 1;
    const int nJ = last_row / GRAN + 1;

#define ST_Y1(st) (reinterpret_cast<T*>(smem + (st) * Cfg::STAGE_BYTES))
#define ST_Y2(st) (ST_Y1(st) + Cfg::TILE_ELEMS)
#define ST_AL(st) (reinterpret_cast<float*>(ST_Y2(st) + Cfg::TILE_ELEMS))
    const float* const alpha_head = a.alpha2 + poff;
    const float* const ek_head = a.ek2 + poff;
    const float* const amax_head = a.amax2 + goff * 2;
    TileDma<T, D, GRAN, 256> tdma;
    tdma.init(tid);
    const auto ra = tdma.rows(tid, (unsigned)(rsA * sizeof(T)));
    RowVec3Dma rvdma;   // alpha, ek (64 per tile) and the two block maxima of a tile (padded arrays: always readable)
    rvdma.init(tid, alpha_head, ek_head, amax_head, 64, 64, 2);
    const int full_tiles = S / GRAN;  // key tiles whose 64 rows all exist
#define ROW_DMA(j, st)                                                                   \
    do {                                                                                 \
        if ((j) < full_tiles) {                                                          \
            tdma.issue(ST_Y1(st), Y1 + (size_t)GRAN * (j) * rsA, ra);                     \
            tdma.issue(ST_Y2(st), Y2 + (size_t)GRAN * (j) * rsA, ra);                     \
        } else {                                                                         \
            tile_dma<T, D, GRAN, 256>(ST_Y1(st), Y1, GRAN * (j), S, tid, rsA);            \
            tile_dma<T, D, GRAN, 256>(ST_Y2(st), Y2, GRAN * (j), S, tid, rsA);            \
        }                                                                                \
        rvdma.issue(ST_AL(st), (j));                                                     \
    } while (0)

    // first product of both 32-key blocks of a tile, S^T (or dC^T) in accumulator layout; the two accumulation
    // chains are interleaved so that consecutive MFMAs never depend on each other
    auto gemm1x2 = [&](const T* y1, f32x16& s0, f32x16& s1, auto&& hook) {
        constexpr int BATCH = NS < 4 ? NS : 4;  // fragments fetched ahead of the MFMAs that consume them
#pragma unroll
        for (int b0 = 0; b0 < NS; b0 += BATCH) {
            hook(b0 / BATCH, NS / BATCH);
            frag k0[BATCH], k1[BATCH];
#pragma unroll
            for (int s = 0; s < BATCH; s++) { k0[s] = krd.read(y1, 0, b0 + s); k1[s] = krd.read(y1, 1, b0 + s); }
#pragma unroll
            for (int s = 0; s < BATCH; s++) {
                if (b0 + s == 0) {
                    const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                    s0 = z; s1 = z;
                }
                R::mma(s0, k0[s], xf[b0 + s]);
                R::mma(s1, k1[s], xf[b0 + s]);
            }
        }
    };
    auto gemm1 = [&](const T* y1, int kb, f32x16& sacc) {
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[r] = 0.f;
#pragma unroll
        for (int s = 0; s < NS; s++) R::mma(sacc, krd.read(y1, kb, s), xf[s]);
    };
    // gate weights; `diag` masks the keys above the diagonal of a diagonal block
    auto weigh = [&](f32x16& sacc, const float* sal, int kb, float crow, bool diag) {
#pragma unroll
        for (int a4 = 0; a4 < 4; a4++) {
            const f32x4 al = *reinterpret_cast<const f32x4*>(sal + 32 * kb + 8 * a4 + 4 * h);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const int r = 4 * a4 + c;
                float e = fast_exp2(al[c] + crow);
                if (diag && (8 * a4 + 4 * h + c > c32)) e = 0.f;
                if constexpr (MODE == MODE_FWD) {
                    const float p = sacc[r] * e;
                    bsum += p;
                    sacc[r] = p;
                } else {
                    sacc[r] = (sacc[r] * inv_n + dbv) * e;
                }
            }
        }
    };
    // gate weights of a block entirely below the diagonal, factorised: exp2(alpha_j - c0) comes from the pre-pass
    // (sek), exp2(c0 - beta_i + dG) is one exponential per lane and block
    auto weigh_fact = [&](f32x16& sacc, const float* sek, int kb, float crow) {
        const float er = fast_exp2(crow + sek[GRAN + kb]);
        float blk = 0.f;
#pragma unroll
        for (int a4 = 0; a4 < 4; a4++) {
            const f32x4 ek = *reinterpret_cast<const f32x4*>(sek + 32 * kb + 8 * a4 + 4 * h);
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const int r = 4 * a4 + c;
                if constexpr (MODE == MODE_FWD) {
                    const float t = sacc[r] * ek[c];
                    blk += t;
                    sacc[r] = t * er;
                } else {
                    sacc[r] = (sacc[r] * inv_n + dbv) * (ek[c] * er);
                }
            }
        }
        if constexpr (MODE == MODE_FWD) bsum += blk * er;
    };
    // second product: accumulate this key block into the output
    auto gemm2 = [&](const T* y2, const f32x16& sacc, int kb, auto&& hook) {
#pragma unroll
        for (int t = 0; t < NSTEP32; t++) {
            hook(kb * NSTEP32 + t, 2 * NSTEP32);
            frag pf, pl;
            if constexpr (STRICT) R::from_acc_split(sacc, t, pf, pl);
            else pf = R::from_acc(sacc, t);
            frag vf[NDB];
#pragma unroll
            for (int d = 0; d < NDB; d++) {
                if constexpr (FAST_TR) vf[d] = vrd.read(y2, 32 * kb + KW * t, d);
                else vf[d] = swz_frag_transposed<T, D>(y2, 32 * kb + KW * t, 32 * d, lane);
            }
#pragma unroll
            for (int d = 0; d < NDB; d++) {
                R::mma(oacc[d], vf[d], pf);
                if constexpr (STRICT) R::mma(oacc[d], vf[d], pl);
            }
        }
    };

    // A whole mask-free tile with the vector work hidden behind the matrix work.  A wave issues in order and an MFMA
    // executes asynchronously, so vector instructions placed between two MFMAs cost nothing while the matrix unit
    // is busy; the tile is therefore walked as
    //     S0 = K0 Q^T | S1 = K1 Q^T with the weighing of S0 between its MFMAs | H += V0^T P0^T with the weighing of S1
    //     between its MFMAs | H += V1^T P1^T
    // and every LDS operand is read a few MFMAs ahead of its use.
    auto tile_overlapped = [&](const T* y1, const T* y2, const float* sek, float crow, auto&& hook1, auto&& hook2) {
      if constexpr (FAST_TR && NSTEP32 == 2) {
        constexpr int AH = NS < 4 ? NS : 4;
        f32x16 s0, s1;
        // one accumulator register of a block below the diagonal: see weigh_fact
        auto weigh_reg = [&](f32x16& sacc, int r, const f32x4 (&ek)[4], float er, float& blk) {
            if constexpr (MODE == MODE_FWD) {
                const float t = sacc[r] * ek[r >> 2][r & 3];
                blk += t;
                sacc[r] = t * er;
            } else {
                sacc[r] = (sacc[r] * inv_n + dbv) * (ek[r >> 2][r & 3] * er);
            }
        };
        f32x4 ek0[4], ek1[4];
#pragma unroll
        for (int a4 = 0; a4 < 4; a4++) {
            ek0[a4] = *reinterpret_cast<const f32x4*>(sek + 8 * a4 + 4 * h);
            ek1[a4] = *reinterpret_cast<const f32x4*>(sek + 32 + 8 * a4 + 4 * h);
        }
        const float er0 = fast_exp2(crow + sek[GRAN]), er1 = fast_exp2(crow + sek[GRAN + 1]);
        float blk0 = 0.f, blk1 = 0.f;
        frag kq[NS];
        // ---- S0
#pragma unroll
        for (int s = 0; s < AH; s++) kq[s] = krd.read(y1, 0, s);
#pragma unroll
        for (int s = 0; s < NS; s++) {
            if (s % 4 == 0) hook1(s / 4, 2 * (NS / 4));
            if (s + AH < NS) kq[s + AH] = krd.read(y1, 0, s + AH);
            if (s == 0) {
                const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                s0 = z; s1 = z;
            }
            R::mma(s0, kq[s], xf[s]);
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- S1, weighing S0 (16 registers over NS MFMAs)
        frag kr[NS];
#pragma unroll
        for (int s = 0; s < AH; s++) kr[s] = krd.read(y1, 1, s);
#pragma unroll
        for (int s = 0; s < NS; s++) {
            if (s % 4 == 0) hook1(NS / 4 + s / 4, 2 * (NS / 4));
            if (s + AH < NS) kr[s + AH] = krd.read(y1, 1, s + AH);
            R::mma(s1, kr[s], xf[s]);
#pragma unroll
            for (int r = s * 16 / NS; r < (s + 1) * 16 / NS; r++) weigh_reg(s0, r, ek0, er0, blk0);
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- H += V^T P^T: groups g = 2*kb + t of 16 keys; the weighing of S1 rides on the groups of key block 0
        frag vf[2][NDB];
#pragma unroll
        for (int d = 0; d < NDB; d++) vf[0][d] = vrd.read(y2, 0, d);
        frag pf, pl;
        auto take_p = [&](const f32x16& sacc, int t) {
            if constexpr (STRICT) R::from_acc_split(sacc, t, pf, pl);
            else pf = R::from_acc(sacc, t);
        };
        take_p(s0, 0);
#pragma unroll
        for (int g = 0; g < 4; g++) {
            hook2(g, 4);
#pragma unroll
            for (int d = 0; d < NDB; d++) {
                if (g + 1 < 4) vf[(g + 1) & 1][d] = vrd.read(y2, KW * (g + 1), d);
                R::mma(oacc[d], vf[g & 1][d], pf);
                if constexpr (STRICT) R::mma(oacc[d], vf[g & 1][d], pl);
                if (g < 2) {
#pragma unroll
                    for (int r = (g * NDB + d) * 16 / (2 * NDB); r < (g * NDB + d + 1) * 16 / (2 * NDB); r++) weigh_reg(s1, r, ek1, er1, blk1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (g == 0) take_p(s0, 1);
            if (g == 1) take_p(s1, 0);
            if (g == 2) take_p(s1, 1);
        }
        if constexpr (MODE == MODE_FWD) bsum += blk0 * er0 + blk1 * er1;
      }
    };

    __syncthreads();  // sG visible; every plain global load above has been waited for (pin)
    const double GI = sG[(wave_active ? r0 : S - 1) / GRAN];
    if (chunk > 0) {
        // ---- what lies before the chunk: the state at the end of the previous chunk, as D/64 tiles of 64 rows in the order
        // in which this product contracts them (mlstm_chunk.hip), hi tile in a stage's Y1 slot and, in split mode, the lo
        // tile in its Y2 slot.  The last state tile sits in stage 1, so that key tile 0 can follow into stage 0 under it.
        constexpr int NTL = D / GRAN, NGRP = GRAN / KW;
        const size_t sbase = ((size_t)bh * a.n_states + chunk - 1) * D * D;
        const T* const Cs = reinterpret_cast<const T*>(a.Cst) + sbase;
        const T* const Cl = STRICT ? reinterpret_cast<const T*>(a.Cst_lo) + sbase : nullptr;
        auto issue_state = [&](int tau) {
            const int stg = (tau + (NTL & 1)) & 1;
            tdma.issue(ST_Y1(stg), Cs + (size_t)GRAN * tau * D);
            if constexpr (STRICT) tdma.issue(ST_Y2(stg), Cl + (size_t)GRAN * tau * D);
        };
        issue_state(0);
        // the rows' decay since the end of the previous chunk: requested now, used behind the tiles
        const float dec = fast_exp2(a.beta2[poff - 1] - a.beta2[poff + rowc] + (float)(a.G2[goff + rowc / GRAN] - a.G2[goff - 1]));
#pragma unroll
        for (int tau = 0; tau < NTL; tau++) {
            const int stg = (tau + (NTL & 1)) & 1;
            dma_wait();
            __syncthreads();   // tile tau has landed; the other stage is free
            if (tau + 1 < NTL) issue_state(tau + 1);
            else ROW_DMA(0, 0);
            const T* th = ST_Y1(stg);
            const T* tl = ST_Y2(stg);
            auto rd = [&](const T* tile, int g, int d) {
                if constexpr (FAST_TR) return vrd.read(tile, KW * g, d);
                else return swz_frag_transposed<T, D>(tile, KW * g, 32 * d, lane);
            };
            frag vf[2][NDB];
#pragma unroll
            for (int d = 0; d < NDB; d++) vf[0][d] = rd(th, 0, d);
#pragma unroll
            for (int g = 0; g < NGRP; g++) {
                frag vl[STRICT ? NDB : 1];
#pragma unroll
                for (int d = 0; d < NDB; d++) {
                    if constexpr (STRICT) vl[d] = rd(tl, g, d);
                    if (g + 1 < NGRP) vf[(g + 1) & 1][d] = rd(th, g + 1, d);
                    R::mma(oacc[d], vf[g & 1][d], xf[NGRP * tau + g]);
                }
                if constexpr (STRICT) {
#pragma unroll
                    for (int d = 0; d < NDB; d++) R::mma(oacc[d], vl[d], xf[NGRP * tau + g]);
                }
            }
        }
        const float* nst = a.Nst + ((size_t)bh * a.n_states + chunk - 1) * D;
        if constexpr (MODE == MODE_FWD) {
            // row sums: decay_i (q_i . n~); the lane's half of the row (the halves meet in the epilogue)
            float part = 0.f;
#pragma unroll
            for (int s2 = 0; s2 < NS; s2++)
#pragma unroll
                for (int e = 0; e < R::EPL; e++) part += to_f32(xf[s2][e]) * nst[KW * s2 + R::EPL * h + e];
            bsum += dec * part;
#pragma unroll
            for (int d = 0; d < NDB; d++)
#pragma unroll
                for (int r = 0; r < 16; r++) oacc[d][r] *= dec;
        } else {
            const float decn = dec * inv_n, rank1 = dec * dbv;
            const T* qrow = reinterpret_cast<const T*>(a.Qrow) + offA + (size_t)rowc * rsA;
            float rp = 0.f;
#pragma unroll
            for (int d = 0; d < NDB; d++)
#pragma unroll
                for (int a4 = 0; a4 < 4; a4++) {
                    const int col = 32 * d + 8 * a4 + 4 * h;
                    const f32x4 nv = *reinterpret_cast<const f32x4*>(nst + col);
                    const f32x4 qv = __builtin_convertvector(*reinterpret_cast<const typename R::vec4*>(qrow + col), f32x4);
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        const float v = oacc[d][4 * a4 + c] * decn + rank1 * nv[c];
                        oacc[d][4 * a4 + c] = v;
                        rp += v * qv[c];
                    }
                }
            // row sums of dD over the keys before the chunk: q_i . dQ_i of what the accumulators hold now
            rp = sum_halves(rp);
            if (row < S && h == 0) a.rowinter[hoff + row] = rp;
        }
    } else {
        if constexpr (MODE == MODE_DQ) {
            if (a.chunk_len > 0 && row < S && h == 0) a.rowinter[hoff + row] = 0.f;
        }
        ROW_DMA(0, 0);
    }
    // Tiles strictly below this wave's rows take the mask-free path; the last one or two tiles of the workgroup are
    // diagonal, or entirely above the diagonal, for this wave.  Two loops with one code path each keep the output
    // accumulators in place (a two-way branch inside one loop makes the register allocator copy them every step).
    // Every wave executes nJ barriers in total, whichever loop it is in.
    const int jfull = wave_active ? (r0 / GRAN < nJ ? r0 / GRAN : nJ) : 0;   // tiles with 64*j + 63 < r0
    auto no_hook = [](int, int) {};
    constexpr int PW = TileDma<T, D, GRAN, 256>::PER_WAVE;
    // Main loop in two parts, each a single code path.  Part 1: the next tile exists and is complete, and its copy
    // is interleaved with this tile's MFMAs (hooks).  Part 2 (at most a step or two): the next tile is the partial
    // last tile of the sequence, or there is none; the copy is issued in one go through the clamping path.
    const int lim = (nJ < full_tiles ? nJ : full_tiles) - 1;
    const int jspread = jfull < lim ? jfull : (lim > 0 ? lim : 0);
    int j = 0;
    for (; j < jspread; j++) {
        dma_wait();
        __syncthreads();  // tile j has landed for every wave and stage (j+1)&1 is free again
        const int jn = j + 1, stn = jn & 1;
        rvdma.issue(ST_AL(stn), jn);
        const T* gy1 = Y1 + (size_t)GRAN * jn * rsA;
        const T* gy2 = Y2 + (size_t)GRAN * jn * rsA;
        T* const ly1 = ST_Y1(stn);
        T* const ly2 = ST_Y2(stn);
        auto hook1 = [&](int idx, int n) { tdma.issue_range(ly1, gy1, idx * PW / n, (idx + 1) * PW / n, ra); };
        auto hook2 = [&](int idx, int n) { tdma.issue_range(ly2, gy2, idx * PW / n, (idx + 1) * PW / n, ra); };
        const T* y1 = ST_Y1(j & 1);
        const T* y2 = ST_Y2(j & 1);
        const float* sal = ST_AL(j & 1);
        const float crow = crow_base + (float)(GI - sG[j]);
        if constexpr (FAST_TR && NSTEP32 == 2) {
            tile_overlapped(y1, y2, sal + GRAN, crow, hook1, hook2);
        } else {
            f32x16 s0, s1;
            gemm1x2(y1, s0, s1, hook1);
            weigh_fact(s0, sal + GRAN, 0, crow);
            gemm2(y2, s0, 0, hook2);
            weigh_fact(s1, sal + GRAN, 1, crow);
            gemm2(y2, s1, 1, hook2);
        }
    }
    for (; j < jfull; j++) {
        dma_wait();
        __syncthreads();
        if (j + 1 < nJ) {
            if (j & 1) ROW_DMA(j + 1, 0); else ROW_DMA(j + 1, 1);
        }
        const T* y1 = ST_Y1(j & 1);
        const T* y2 = ST_Y2(j & 1);
        const float* sal = ST_AL(j & 1);
        const float crow = crow_base + (float)(GI - sG[j]);
        if constexpr (FAST_TR && NSTEP32 == 2) {
            tile_overlapped(y1, y2, sal + GRAN, crow, no_hook, no_hook);
        } else {
            f32x16 s0, s1;
            gemm1x2(y1, s0, s1, no_hook);
            weigh_fact(s0, sal + GRAN, 0, crow);
            gemm2(y2, s0, 0, no_hook);
            weigh_fact(s1, sal + GRAN, 1, crow);
            gemm2(y2, s1, 1, no_hook);
        }
    }
    for (; j < nJ; j++) {
        dma_wait();
        __syncthreads();
        if (j + 1 < nJ) {
            if (j & 1) ROW_DMA(j + 1, 0); else ROW_DMA(j + 1, 1);
        }
        if (!wave_active) continue;
        const T* y1 = ST_Y1(j & 1);
        const T* y2 = ST_Y2(j & 1);
        const float* sal = ST_AL(j & 1);
        const float crow = crow_base + (float)(GI - sG[j]);
#pragma unroll
        for (int kb = 0; kb < 2; kb++) {
            const int kstart = GRAN * j + 32 * kb;
            if (kstart <= r0) {
                f32x16 s0;
                gemm1(y1, kb, s0);
                weigh(s0, sal, kb, crow, kstart == r0);
                gemm2(y2, s0, kb, no_hook);
            }
        }
    }
#undef ROW_DMA
#undef ST_Y1
#undef ST_Y2
#undef ST_AL
    float onorm = 1.0f;
    if constexpr (MODE == MODE_FWD) {
        const float b = sum_halves(bsum);
        const float m = a.M[hoff + rowc];
        const float n = fmaxf(fabsf(b), __expf(-m)) + 1e-6f;
        onorm = 1.0f / n;
        if (row < S && h == 0) a.Bsum[hoff + row] = b;
    }
    if (row < S) {
        T* out = reinterpret_cast<T*>(a.out) + offO + (size_t)row * rsO;
#pragma unroll
        for (int d = 0; d < NDB; d++)
#pragma unroll
            for (int a4 = 0; a4 < 4; a4++) {
                f32x4 v;
#pragma unroll
                for (int c = 0; c < 4; c++) v[c] = oacc[d][4 * a4 + c] * onorm;
                if constexpr (STRICT && MODE == MODE_FWD) {
                    typename R::vec4 hi, lo;
                    R::cvt4_split(v, hi, lo);
                    *reinterpret_cast<typename R::vec4*>(out + 32 * d + 8 * a4 + 4 * h) = hi;
                    if (a.out_lo) *reinterpret_cast<typename R::vec4*>(reinterpret_cast<T*>(a.out_lo) + (hoff + row) * D + 32 * d + 8 * a4 + 4 * h) = lo;
                } else {
                    *reinterpret_cast<typename R::vec4*>(out + 32 * d + 8 * a4 + 4 * h) = R::cvt4(v);
                }
            }
        if constexpr (MODE == MODE_FWD) {
            if (a.O) {  // gated copy from the fp32 accumulators
                const T* og = reinterpret_cast<const T*>(a.O) + offB + (size_t)row * rsB;
                T* outg = reinterpret_cast<T*>(a.out_gated) + offB + (size_t)row * rsB;
#pragma unroll
                for (int d = 0; d < NDB; d++)
#pragma unroll
                    for (int a4 = 0; a4 < 4; a4++) {
                        const int col = 32 * d + 8 * a4 + 4 * h;
                        const f32x4 of = __builtin_convertvector(*reinterpret_cast<const typename R::vec4*>(og + col), f32x4);
                        f32x4 v;
#pragma unroll
                        for (int c = 0; c < 4; c++) v[c] = oacc[d][4 * a4 + c] * onorm * silu(of[c]);
                        *reinterpret_cast<typename R::vec4*>(outg + col) = R::cvt4(v);
                    }
            }
        }
    }
#endif
}

template <typename T, int D, int MODE, bool STRICT>
static int launch_row_ts(const RowArgs& a, hipStream_t st) {
    using Cfg = RowCfg<T, D>;
    auto kern = row_kernel<T, D, MODE, STRICT>;
    static std::once_flag once;
    static hipError_t attr_rc = hipSuccess;
    std::call_once(once, [&] {
        attr_rc = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      (int)(Cfg::STAGES_BYTES + 2048 * sizeof(double)));
    });
    if (attr_rc != hipSuccess) return (int)attr_rc;
    const int nQT = (a.S + ROW_BQ - 1) / ROW_BQ;
    hipLaunchKernelGGL(kern, dim3(a.BH * nQT), dim3(256), Cfg::STAGES_BYTES + (size_t)a.NG * sizeof(double), st, a);
    return (int)hipGetLastError();
}

template <typename T, int D, int MODE>
static int launch_row_t(const RowArgs& a, hipStream_t st) {
    if constexpr (Tr<T>::HALF) {
        if (a.precise) return launch_row_ts<T, D, MODE, true>(a, st);
    }
    return launch_row_ts<T, D, MODE, false>(a, st);
}

template <typename T, int MODE>
static int launch_row_d(int D, const RowArgs& a, hipStream_t st) {
    switch (D) {
        case 64: return launch_row_t<T, 64, MODE>(a, st);
        case 128: return launch_row_t<T, 128, MODE>(a, st);
        case 256:
            if constexpr (Tr<T>::HALF) return launch_row_t<T, 256, MODE>(a, st);
            else return MLSTM_ESHAPE;
    }
    return MLSTM_ESHAPE;
}

int launch_row_kernel(int mode, int dtype, int D, const RowArgs& a, hipStream_t st) {
    if (mode == MODE_FWD) {
        switch (dtype) {
            case MLSTM_F32: return launch_row_d<float, MODE_FWD>(D, a, st);
            case MLSTM_F16: return launch_row_d<_Float16, MODE_FWD>(D, a, st);
            case MLSTM_BF16: return launch_row_d<__bf16, MODE_FWD>(D, a, st);
        }
    } else {
        switch (dtype) {
            case MLSTM_F32: return launch_row_d<float, MODE_DQ>(D, a, st);
            case MLSTM_F16: return launch_row_d<_Float16, MODE_DQ>(D, a, st);
            case MLSTM_BF16: return launch_row_d<__bf16, MODE_DQ>(D, a, st);
        }
    }
    return MLSTM_EINVAL;
}

}  // namespace mlstm
