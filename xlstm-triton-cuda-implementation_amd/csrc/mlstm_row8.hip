// Row-parallel tile kernel for the 16-bit types at D >= 128, eight waves: same math as mlstm_row.hip, but the two
// products of a key tile run in different waves so that the matrix pipe of a SIMD always has work from one wave
// while the other one is in its vector / LDS phase, and every wave works on 64 query rows so that each operand
// fragment read from LDS feeds two MFMAs (with 32 rows per wave the LDS reads of the two products, 256 KB per 64-key
// tile and workgroup, take about as long as the MFMAs themselves).
//
//   producer wave (rg, kh), rg = row group of 64 rows, kh = half of the tile's 64 keys (one wave per SIMD):
//       tile j:  S^T = K_j Q^T (or dC^T = V_j dH^T) for its 32 keys x 64 rows, gate weights, row sums,
//                16-bit P fragments -> LDS
//   consumer wave (rg, dh), dh = half of the D output columns (same SIMDs):
//       tile j:  H^T += V_j^T P_j^T (or dQ^T += K_j^T G_j^T) for 64 rows x D/2 columns, one tile behind the producers
// K and V (Y1, Y2) have two LDS stages each; the consumers' stream runs one tile behind the producers', so the
// four stages hold exactly the tiles in use plus the two being copied.  One s_barrier per tile.  The single P
// buffer of a row group is handed back from its two consumers to its two producers through an LDS counter: a
// consumer copies its fragments into registers first thing after the barrier and bumps the counter; the producers
// check it only when they are about to publish the next tile's P, long after.
// The rows' own operand (Q in the forward, dH in the dQ pass) comes in once per workgroup, as two 64-row tiles through
// stages that are idle at that point, and every wave takes its fragments from there (see x_copy).
// MODE_FWD replaces mlstm_matmul_kernel (mlstm_matmul.py:38-101) and the CUDA kernel mlstm_forward
// (cuda-src/mlstm_forward.cu:14-189); MODE_DQ the dQ loop of mlstm_matmul_kernel_backward (mlstm_matmul.py:239-267).
#include <type_traits>
#include "mlstm_device.h"
#include "mlstm_kernels.h"

namespace mlstm {

constexpr int R8_FWD = 0, R8_DQ = 1;
constexpr int R8_BQ = 128;

template <typename T, int D>
struct Row8Cfg {
    static constexpr size_t TILE_BYTES = (size_t)GRAN * D * sizeof(T);
    static constexpr size_t AUX_BYTES = 3 * GRAN * sizeof(float);                      // alpha, ek, amax of a Y1 stage
    static constexpr size_t PBUF_BYTES = 2 * 2 * 4 * 64 * 16;                          // [row group][row block][16-key group][lane] x 16 B
    // partial row sums [rg][kh][r][32] (forward) or the rows' 1/n and db [rg][r][32][2] (dQ pass), then the counters
    // (and [rg][half][r][32] floats for the row sums of the state part of a chunked dQ pass)
    // and the vector state n~ of the previous chunk (D floats)
    static constexpr size_t MISC_BYTES = 2 * 2 * 2 * 32 * sizeof(float) + 64 + 2 * 2 * 2 * 32 * sizeof(float) + D * sizeof(float);
    static constexpr size_t FIXED_BYTES = 4 * TILE_BYTES + 2 * AUX_BYTES + PBUF_BYTES + MISC_BYTES;  // + NG doubles
};

template <typename T, int D, int MODE, bool DENSE>
__global__ __launch_bounds__(512) void row8_kernel(RowArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
    using R = Tr<T>;
    using Cfg = Row8Cfg<T, D>;
    typedef typename R::frag frag;
    static_assert(R::HALF && D >= 128, "16-bit types, D >= 128");
    constexpr int KW = R::KW, NS = D / KW, NDH = D / 64;   // NDH: 32-column blocks of one consumer's half of D
    // epilogue: a consumer's 64 x D/2 block passes through LDS in rows of RB bytes (16 bytes of padding), CPR 16-byte pieces each
    constexpr int RB = (D / 2) * (int)sizeof(T) + 16, CPR = (D / 2) * (int)sizeof(T) / 16;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    char* const y1s = smem;                                    // 2 stages of Y1
    char* const y2s = smem + 2 * Cfg::TILE_BYTES;              // 2 stages of Y2
    float* const auxs = reinterpret_cast<float*>(smem + 4 * Cfg::TILE_BYTES);   // 2 x (alpha | ek | amax)
    frag* const pbuf = reinterpret_cast<frag*>(smem + 4 * Cfg::TILE_BYTES + 2 * Cfg::AUX_BYTES);
    float* const bex = reinterpret_cast<float*>(smem + 4 * Cfg::TILE_BYTES + 2 * Cfg::AUX_BYTES + Cfg::PBUF_BYTES);
    unsigned* const pcnt = reinterpret_cast<unsigned*>(bex + 2 * 2 * 2 * 32);   // [2] fragments-copied counters
    float* const rix = bex + 2 * 2 * 2 * 32 + 16;
    float* const nvl = rix + 2 * 2 * 2 * 32;   // [D]
    double* const sG = reinterpret_cast<double*>(smem + Cfg::FIXED_BYTES);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, h = lane >> 5, c32 = lane & 31;
    const bool producer = wave < 4;
    const int rg = (wave >> 1) & 1;   // row group: rows 64*rg .. 64*rg+63 of the workgroup's 128
    const int sub = wave & 1;         // producers: key half kh; consumers: column half dh
    const int rtid = tid & 255;       // thread index inside the role (the copies are split over the four waves of a role)
    int S = a.S, NG = a.NG;
    const int nQT = (S + R8_BQ - 1) / R8_BQ;
    int bh, qt;
    {
        const int bid = blockIdx.x;
        if ((a.BH & 7) == 0) {
            // Workgroups go round-robin to the 8 XCDs: XCD x gets the heads x, x + 8, ... and works on them two at a
            // time, heaviest row tiles first (K and V of two heads are 8 MB at S = 4096, D = 256 against 4 MB of L2 per
            // XCD; all heads of an XCD at once measured 1 % slower, one head at a time 7 % slower: its last, light tiles
            // leave CUs idle at every change of head).
            const int rest = bid >> 3, ngrp = a.BH >> 3;
            const int paired = (ngrp >> 1) * 2 * nQT;   // workgroups of this XCD that belong to complete pairs of heads
            if (a.chunk_len > 0) {
                // In chunks a row tile reads the keys of its own chunk and one state, so the L2 holds what many heads
                // need at once, and what counts is the balance: all heads of the XCD together (4.5 % faster than in
                // pairs at D = 256, 4 % at D = 128; one head at a time 5 % slower than in pairs).
                // (By descending position, chunk after chunk -- a sawtooth of heavy and light tiles.  Sorting by weight across
                // the chunks, every chunk's last row tile first, measured 8 % slower: the row tiles of a chunk share its
                // keys and its state in the L2.)
                bh = (rest % ngrp) * 8 + (bid & 7);
                qt = nQT - 1 - rest / ngrp;
            } else if (rest < paired) {
                const int pair = rest / (2 * nQT), rr = rest % (2 * nQT);
                bh = (2 * pair + (rr & 1)) * 8 + (bid & 7);
                qt = nQT - 1 - (rr >> 1);
            } else {   // odd number of heads per XCD: the last one on its own
                bh = (ngrp - 1) * 8 + (bid & 7);
                qt = nQT - 1 - (rest - paired);
            }
        } else {
            bh = bid % a.BH;
            qt = nQT - 1 - bid / a.BH;
        }
    }
    size_t hoff = (size_t)bh * S, poff = (size_t)bh * NG * GRAN, goff = (size_t)bh * NG;
    // The caller's tensors: q, k, v, dq in one layout (la), h, dh, o in another (lb); offA / offB: element offset of the
    // head's first position, rsA / rsB: elements from one position to the next.  X and the output change sides between
    // the forward (Q -> H) and the dQ pass (dH -> dQ).
    // (DENSE: every tensor is a contiguous [BH,S,D]; the strides are then compile-time constants)
    const size_t rsA = DENSE ? (size_t)D : (size_t)a.la.ss, rsB = DENSE ? (size_t)D : (size_t)a.lb.ss;
    size_t offA = DENSE ? hoff * D : a.la.head(bh), offB = DENSE ? hoff * D : a.lb.head(bh);
    size_t rsH = DENSE ? (size_t)D : 0, offH = DENSE ? hoff * D : 0;   // Hin (dQ pass)
    if constexpr (MODE == R8_DQ && !DENSE) { rsH = (size_t)a.lh.ss; offH = a.lh.head(bh); }
    // Long sequences in chunks: the workgroup's rows lie in chunk `chunk` of chunk_len positions.  Everything below addresses
    // positions relative to the chunk's first one (the sequence "starts" there: per-position offsets move forward, S, NG
    // and the row tile index shrink); what lies before the chunk enters through the state of the previous chunk.
    int chunk = 0;
    if (a.chunk_len > 0) {
        chunk = (qt * R8_BQ) / a.chunk_len;
        const int p0 = chunk * a.chunk_len;
        hoff += p0; poff += p0; goff += p0 / GRAN;
        offA += (size_t)p0 * rsA; offB += (size_t)p0 * rsB; offH += (size_t)p0 * rsH;
        S -= p0; NG -= p0 / GRAN; qt -= p0 / R8_BQ;
    }
    const int q0 = qt * R8_BQ, r0 = q0 + 64 * rg;            // r0: first of the wave's 64 rows (a multiple of 64)
    const bool wave_active = r0 < S;
    int rowc[2];
#pragma unroll
    for (int r = 0; r < 2; r++) { const int row = r0 + 32 * r + c32; rowc[r] = row < S ? row : S - 1; }
    const size_t rsX = MODE == R8_FWD ? rsA : rsB, offX = MODE == R8_FWD ? offA : offB;
    const size_t rsO = MODE == R8_FWD ? rsB : rsA, offO = MODE == R8_FWD ? offB : offA;
    const T* Y1 = reinterpret_cast<const T*>(a.Y1) + offA;
    const T* Y2 = reinterpret_cast<const T*>(a.Y2) + offA;
    const int last_row = (q0 + R8_BQ - 1 < S - 1) ? q0 + R8_BQ - 1 : S - 1;
    const int nJ = last_row / GRAN + 1;
    const int full_tiles = S / GRAN;
    // the wave's rows lie in granule r0/64: tiles j < jfull need no mask, tile jlast = jfull is its diagonal tile
    const int jlast = wave_active ? r0 / GRAN : -1;
    const int jfull = wave_active ? r0 / GRAN : 0;

    // Every trip to memory in this prologue costs thousands of cycles, so the independent ones are requested back to back
    // and their values used as late as possible: the granule bases are asked for here and stored to LDS just before the
    // first barrier.
    // (likewise the vector state of the previous chunk, D floats: fetched by the first D threads, read from LDS behind the
    // state tiles and behind the tile loop -- as loads of their own there, each was one more trip to memory in the
    // workgroup's chain of them, and a trip is 2 to 2.5 us with one workgroup per CU)
    const double g_mine = tid < NG ? a.G2[goff + tid] : 0.0;
    const float n_mine = (chunk > 0 && tid < D) ? a.Nst[((size_t)bh * a.n_states + chunk - 1) * D + tid] : 0.f;
    auto store_granule_bases = [&]() {
        if (chunk > 0 && tid < D) nvl[tid] = n_mine;
        if (tid < NG) sG[tid] = g_mine;
        for (int g = tid + 512; g < NG; g += 512) sG[g] = a.G2[goff + g];
    };
    if (tid < 2) pcnt[tid] = 0;

    TileDma<T, D, GRAN, 256> tdma;
    tdma.init(rtid);
    const auto ra = tdma.rows(rtid, (unsigned)(rsA * sizeof(T)));   // Y1, Y2 tiles
    constexpr int PW = TileDma<T, D, GRAN, 256>::PER_WAVE;
    frag* const p_rg = pbuf + rg * (2 * 4 * 64) + lane;        // fragment (r, g) of the row group -> p_rg[(4*r + g) * 64]
    // The workgroup's 128 rows of X (Q in the forward, dH in the dQ pass) are operands of every product here, a fragment per
    // lane and contraction step.  Straight from memory that is 16 bytes of a row per lane, 32 rows per instruction, by four
    // waves per row group for the same rows (knocked out, those loads were 16 us of the forward's 113 and 11 of the dQ pass's
    // 133 at B4 H8 S4096 D256).  The rows come in once instead, as two 64-row tiles in whole lines -- row group 0 by the
    // producers into a Y1 stage, row group 1 by the consumers into a Y2 stage -- and every wave reads its fragments from
    // there behind the first barrier.  Behind the first chunk the FIRST stages serve (the second ones hold state tiles), and
    // the first key tiles follow into them once the first pair of state tiles is done with; in the first chunk, and without
    // chunks, the SECOND stages serve, which the tiles' copies reach only behind a later barrier.
    const int xst = chunk > 0 ? 0 : 1;
    const T* const xtile = reinterpret_cast<const T*>((rg ? y2s : y1s) + xst * Cfg::TILE_BYTES);   // the wave's row group's rows
    auto x_copy = [&]() {   // (this role's tile: producers row group 0, consumers row group 1)
        const T* Xg = reinterpret_cast<const T*>(a.X) + (MODE == R8_FWD ? offA : offB);
        const size_t rs = MODE == R8_FWD ? rsA : rsB;
        const int row0 = q0 + (producer ? 0 : GRAN);
        T* dst = reinterpret_cast<T*>((producer ? y1s : y2s) + xst * Cfg::TILE_BYTES);
        // (the per-lane row offsets of the Y tiles serve when X has their stride)
        if (row0 + GRAN <= S) tdma.issue(dst, Xg + (size_t)row0 * rs, (MODE == R8_FWD || DENSE) ? ra : tdma.rows(rtid, (unsigned)(rs * sizeof(T))));
        else tile_dma_rolled<T, D, GRAN, 256>(dst, Xg, row0 < S ? row0 : S - 1, S, rtid, rs);
    };
    SwzRowReaderX<T, D> xrd;
    xrd.init(lane);

    if (producer) {
        // ------------------------------------------------------------------------------------------ producers
        const int kh = sub;
        x_copy();
        if (chunk == 0) {   // the copy of the first Y1 tile (behind the first chunk it follows the first pair of state tiles)
            T* dst = reinterpret_cast<T*>(y1s);
            if (0 < full_tiles) tdma.issue(dst, Y1, ra);
            else tile_dma_rolled<T, D, GRAN, 256>(dst, Y1, 0, S, rtid, rsA);
        }
        frag xf[2][NS];
        float crow_base[2], inv_n[2] = {0.f, 0.f}, dbv[2] = {0.f, 0.f}, bsum[2] = {0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 2; r++) crow_base[r] = -0.5f * __log2f((float)D) - a.beta2[poff + rowc[r]];
        float dec_rows[2] = {0.f, 0.f};   // forward in chunks: the rows' decay since the end of the previous chunk (for the row sums)
        if (MODE == R8_FWD && chunk > 0) {
#pragma unroll
            for (int r = 0; r < 2; r++)
                dec_rows[r] = fast_exp2(a.beta2[poff - 1] - a.beta2[poff + rowc[r]] + (float)(a.G2[goff + rowc[r] / GRAN] - a.G2[goff - 1]));
        }
        // dQ pass behind the first chunk: this role forms the per-row scalars of the backward (1/n, db: see row_stats) for row
        // block kh of the row group, while the consumers work through the state tiles (which need them only at the end).  The
        // rows of h are requested here; the dot products with dh follow behind the barrier, when the dh fragments are there.
        // (In the first chunk, and without chunks, it is the other way round: this role heads the critical path and the
        // consumers, idle until the first P, form the scalars.)
        frag hfr[NS];
        float b_row = 0.f, m_row = 0.f;
        if (MODE == R8_DQ && chunk > 0) {
            const int rc = rowc[kh];
            const T* hrow = reinterpret_cast<const T*>(a.Hin) + offH + (size_t)rc * rsH;
#pragma unroll
            for (int s = 0; s < NS; s++) hfr[s] = frag_rowmajor<T>(hrow, s, h);
            b_row = a.Bin[hoff + rc];
            m_row = a.M[hoff + rc];
        }
#pragma unroll
        for (int r = 0; r < 2; r++) { pin(crow_base[r]); pin(dec_rows[r]); }
        SwzRowReaderX<T, D> krd;
        krd.init(lane);
        const float* const alpha_head = a.alpha2 + poff;
        const float* const ek_head = a.ek2 + poff;
        const float* const amax_head = a.amax2 + goff * 2;

        RowVec3Dma rvdma;   // alpha, ek (64 per tile) and the two block maxima of a tile (padded arrays: always readable)
        rvdma.init(rtid, alpha_head, ek_head, amax_head, 64, 64, 2);
        auto aux_dma = [&](int j) { rvdma.issue(auxs + (j & 1) * 3 * GRAN, j); };
        auto y1_bulk = [&](int j) {
            T* dst = reinterpret_cast<T*>(y1s + (j & 1) * Cfg::TILE_BYTES);
            if (j < full_tiles) tdma.issue(dst, Y1 + (size_t)GRAN * j * rsA, ra);
            else tile_dma_rolled<T, D, GRAN, 256>(dst, Y1, GRAN * j, S, rtid, rsA);
            aux_dma(j);
        };
        // s_r = (32 keys of this wave) x (row block r); every Y1 fragment feeds both row blocks.  The operand reads run
        // AHEAD contraction steps in front of the MFMAs that consume them (a wave issues in order).
        auto gemm1 = [&](auto ahead_tag, const T* y1, f32x16& s0, f32x16& s1, auto&& hook) {
            constexpr int AHEAD = decltype(ahead_tag)::value;
            const T* y1k = y1 + (size_t)kh * 32 * D;
            frag kf[NS];
#pragma unroll
            for (int s = 0; s < AHEAD; s++) kf[s] = krd.read(y1k, 0, s);
#pragma unroll
            for (int s = 0; s < NS; s++) {
                if (s % AHEAD == 0) hook(s / AHEAD, NS / AHEAD);
                if (s + AHEAD < NS) kf[s + AHEAD] = krd.read(y1k, 0, s + AHEAD);
                if (s == 0) {
                    const f32x16 z = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                    s0 = z; s1 = z;
                }
                R::mma(s0, kf[s], xf[0][s]);
                R::mma(s1, kf[s], xf[1][s]);
                __builtin_amdgcn_sched_barrier(0);
            }
        };
        // mask-free tiles: exp2(alpha_j - beta_i) = ek_j * er_i with one exp2 per row and 32-key block
        auto weigh_fact = [&](f32x16& s0, f32x16& s1, const float* sek, float crow0, float crow1) {
            const float am = sek[GRAN + kh];
            const float er0 = fast_exp2(crow0 + am), er1 = fast_exp2(crow1 + am);
            // dQ pass: (s / n + db) * ek * er = (s * sc + of) * ek with the row factors folded into two scalars
            const float sc0 = inv_n[0] * er0, of0 = dbv[0] * er0, sc1 = inv_n[1] * er1, of1 = dbv[1] * er1;
            float blk0 = 0.f, blk1 = 0.f;
#pragma unroll
            for (int a4 = 0; a4 < 4; a4++) {
                const f32x4 ek = *reinterpret_cast<const f32x4*>(sek + 32 * kh + 8 * a4 + 4 * h);
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const int x = 4 * a4 + c;
                    if constexpr (MODE == R8_FWD) {
                        const float t0 = s0[x] * ek[c], t1 = s1[x] * ek[c];
                        blk0 += t0; blk1 += t1;
                        s0[x] = t0 * er0; s1[x] = t1 * er1;
                    } else {
                        s0[x] = (s0[x] * sc0 + of0) * ek[c];
                        s1[x] = (s1[x] * sc1 + of1) * ek[c];
                    }
                }
            }
            if constexpr (MODE == R8_FWD) { bsum[0] += blk0 * er0; bsum[1] += blk1 * er1; }
        };
        // One 32 x 32 block of a tile that the diagonal crosses.  mode (the same in all lanes) 0: the block lies above the
        // diagonal (P = 0), 1: below it (the factorised weights of weigh_fact), 2: on it (one exp2 per element, masked).
        auto weigh_masked = [&](f32x16& sacc, const float* sal, float crow, int mode, float& bs, float invn, float dbr) {
            if (mode == 0) {
#pragma unroll
                for (int x = 0; x < 16; x++) sacc[x] = 0.f;
                return;
            }
            if (mode == 1) {
                const float* sek = sal + GRAN;
                const float er = fast_exp2(crow + sek[GRAN + kh]);
                const float sc = invn * er, of = dbr * er;
                float blk = 0.f;
#pragma unroll
                for (int a4 = 0; a4 < 4; a4++) {
                    const f32x4 ek = *reinterpret_cast<const f32x4*>(sek + 32 * kh + 8 * a4 + 4 * h);
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        const int x = 4 * a4 + c;
                        if constexpr (MODE == R8_FWD) {
                            const float t = sacc[x] * ek[c];
                            blk += t;
                            sacc[x] = t * er;
                        } else {
                            sacc[x] = (sacc[x] * sc + of) * ek[c];
                        }
                    }
                }
                if constexpr (MODE == R8_FWD) bs += blk * er;
                return;
            }
#pragma unroll
            for (int a4 = 0; a4 < 4; a4++) {
                const f32x4 al = *reinterpret_cast<const f32x4*>(sal + 32 * kh + 8 * a4 + 4 * h);
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const int x = 4 * a4 + c;
                    float e = fast_exp2(al[c] + crow);
                    if (8 * a4 + 4 * h + c > c32) e = 0.f;
                    if constexpr (MODE == R8_FWD) {
                        const float p = sacc[x] * e;
                        bs += p;
                        sacc[x] = p;
                    } else {
                        sacc[x] = (sacc[x] * invn + dbr) * e;
                    }
                }
            }
        };
        // hand the fragments of tile j to the consumers of the same rows; they have copied tile j-1's long ago
        bool expired = false;
        auto publish = [&](const f32x16& s0, const f32x16& s1, int j) {
            frag f00 = R::from_acc(s0, 0), f01 = R::from_acc(s0, 1), f10 = R::from_acc(s1, 0), f11 = R::from_acc(s1, 1);
            if (j > 0) {
                // Bounded: the consumers bump the counter long before it is looked at here, but a miscount must not hang
                // the GPU.  An expired wait is reported through the error word and the kernel runs on (wrong results).
                volatile unsigned* c = pcnt + rg;
                if (a.spin_limit < 0) {   // test aid: every wait counts as expired, without waiting
                    if (lane == 0 && j == 1) atomicOr(a.err, 1);
                } else if (!expired) {    // (once a wait has expired in this wave the later ones are not waited for either:
                    int spins = 0;        //  the results are lost anyway, and the kernel should end soon)
                    while (*c < 2u * (unsigned)j) {
                        if (spins++ >= a.spin_limit) {
                            if (lane == 0) atomicOr(a.err, 1);
                            expired = true;
                            break;
                        }
                        __builtin_amdgcn_s_sleep(1);
                    }
                }
            }
            p_rg[(0 + 2 * kh + 0) * 64] = f00;
            p_rg[(0 + 2 * kh + 1) * 64] = f01;
            p_rg[(4 + 2 * kh + 0) * 64] = f10;
            p_rg[(4 + 2 * kh + 1) * 64] = f11;
        };

        store_granule_bases();
        dma_wait();
        __syncthreads();  // sG, counters visible; the X tiles have landed
        if (MODE == R8_DQ && chunk > 0) {   // (before the wave takes all its X fragments: the rows of h leave their registers first)
            float acc = 0.f;
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const frag xk = xrd.read(xtile, kh, s);
#pragma unroll
                for (int e = 0; e < R::EPL; e++) acc += (float)xk[e] * (float)hfr[s][e];
            }
            float inv = 0.f, dbr = 0.f;
            row_stats_of(sum_halves(acc), b_row, m_row, inv, dbr);
            const int row = r0 + 32 * kh + c32;
            if (h == 0) {
                *reinterpret_cast<float2*>(bex + ((rg * 2 + kh) * 32 + c32) * 2) = make_float2(inv, dbr);
                if (row < S) { a.inv_n[poff + row] = inv; a.db[poff + row] = dbr; }
            }
        }
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int s = 0; s < NS; s++) xf[r][s] = xrd.read(xtile, r, s);
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int s = 0; s < NS; s++) pin(xf[r][s]);
        if (chunk > 0) {   // the consumers work through the state tiles: two barriers per pair of tiles
#pragma unroll
            for (int pp = 0; pp < D / 64; pp += 2) {
                __syncthreads();
                __syncthreads();
                if (pp == 0) {   // every wave is done with the X tiles: the first Y1 tile follows into its stage
                    T* dst = reinterpret_cast<T*>(y1s);
                    if (0 < full_tiles) tdma.issue(dst, Y1, ra);
                    else tile_dma_rolled<T, D, GRAN, 256>(dst, Y1, 0, S, rtid, rsA);
                }
            }
        }
        if constexpr (MODE == R8_DQ) {   // 1/n and db of the wave's rows (written ahead of the last barrier passed, by either role)
#pragma unroll
            for (int r = 0; r < 2; r++) {
                const float2 st = *reinterpret_cast<const float2*>(bex + ((rg * 2 + r) * 32 + c32) * 2);
                inv_n[r] = st.x; dbv[r] = st.y;
            }
        }
        const double GI = sG[(wave_active ? r0 : S - 1) / GRAN];
        aux_dma(0);
        // iteration i: barrier, then produce tile i (if any); the copy of tile i+1 is spread over the MFMA groups
        const int lim = (nJ < full_tiles ? nJ : full_tiles) - 1;           // tiles j < lim have a complete successor
        const int jspread = jfull < lim ? jfull : (lim > 0 ? lim : 0);
        // A mask-free tile whose successor is complete.  In iteration 0 the wave copies its share of tile 1 itself, spread
        // over the MFMA groups; from iteration 1 on the consumer wave of the same SIMD issues that share (same blocks:
        // the split of a tile over the four waves of a role is the same in both roles) before it starts on its own
        // products.  Measured: the products here are the head of the critical path of a tile (the gate arithmetic and
        // the P fragments can only follow them) and ran at 2/3 of their speed while the consumer's MFMAs competed from
        // the first cycle on; a consumer that starts 500-800 cycles late finishes all the same before the gate
        // arithmetic here does.
        auto no_hook = [](int, int) {};
        auto main_tile = [&](int j, auto&& hook) {
            dma_wait();
            __syncthreads();
            aux_dma(j + 1);
            const T* y1 = reinterpret_cast<const T*>(y1s + (j & 1) * Cfg::TILE_BYTES);
            const float* sax = auxs + (j & 1) * 3 * GRAN;
            const float dg = (float)(GI - sG[j]);
            f32x16 s0, s1;
            gemm1(std::integral_constant<int, 4>{}, y1, s0, s1, hook);
            weigh_fact(s0, s1, sax + GRAN, crow_base[0] + dg, crow_base[1] + dg);
            publish(s0, s1, j);
        };
        int j = 0;
        if (jspread > 0) {
            T* const ly1 = reinterpret_cast<T*>(y1s + Cfg::TILE_BYTES);
            const T* gy1 = Y1 + (size_t)GRAN * rsA;
            main_tile(0, [&](int idx, int n) { tdma.issue_range(ly1, gy1, idx * PW / n, (idx + 1) * PW / n, ra); });
            j = 1;
        }
        for (; j < jspread; j++) main_tile(j, no_hook);
        for (; j < nJ; j++) {        // the remaining tiles: masked, skipped, or with a partial successor
            dma_wait();
            __syncthreads();
            if (j + 1 < nJ) y1_bulk(j + 1);
            const T* y1 = reinterpret_cast<const T*>(y1s + (j & 1) * Cfg::TILE_BYTES);
            const float* sax = auxs + (j & 1) * 3 * GRAN;
            f32x16 s0, s1;
            if (j <= jlast) {
                const float dg = (float)(GI - sG[j]);
                gemm1(std::integral_constant<int, 2>{}, y1, s0, s1, no_hook);   // (shallower read-ahead: this loop is short of registers)
                const int k0 = GRAN * j + 32 * kh;
                weigh_masked(s0, sax, crow_base[0] + dg, k0 > r0 ? 0 : (k0 == r0 ? 2 : 1), bsum[0], inv_n[0], dbv[0]);
                weigh_masked(s1, sax, crow_base[1] + dg, k0 > r0 + 32 ? 0 : (k0 == r0 + 32 ? 2 : 1), bsum[1], inv_n[1], dbv[1]);
            } else {
#pragma unroll
                for (int x = 0; x < 16; x++) { s0[x] = 0.f; s1[x] = 0.f; }
            }
            publish(s0, s1, j);
        }
        if constexpr (MODE == R8_FWD) {
            if (chunk > 0) {
                // Row sums: what lies before the chunk contributes decay_i (q_i . n~) with the vector state n~ of the
                // previous chunk (in LDS since the prologue); the two producers of a row group take half of the contraction
                // each.  Done here, behind the tile loop, where this role has time to spare (the consumers are one tile
                // behind).
                const float* nst = nvl + 8 * h;
                float part[2] = {0.f, 0.f};
                auto half_dot = [&](auto first_tag) {   // (the fragment index must be a constant: xf lives in registers)
                    constexpr int S0 = decltype(first_tag)::value;
#pragma unroll
                    for (int s = S0; s < S0 + NS / 2; s++) {
                        const f32x4 n0 = *reinterpret_cast<const f32x4*>(nst + KW * s), n1 = *reinterpret_cast<const f32x4*>(nst + KW * s + 4);
#pragma unroll
                        for (int r = 0; r < 2; r++) {
                            const f32x8 qv = __builtin_convertvector(xf[r][s], f32x8);
#pragma unroll
                            for (int e = 0; e < 4; e++) part[r] += qv[e] * n0[e] + qv[4 + e] * n1[e];
                        }
                    }
                };
                if (kh == 0) half_dot(std::integral_constant<int, 0>{});
                else half_dot(std::integral_constant<int, NS / 2>{});
#pragma unroll
                for (int r = 0; r < 2; r++) bsum[r] += part[r] * dec_rows[r];
            }
        }
        dma_wait();
        // Output gate: this wave is done while the consumer of the same rows still has its last product and the
        // epilogue ahead.  It fetches the gate values of that consumer's 64 x D/2 block now and, once the block lies
        // in LDS, writes the gated copy while the consumer writes the plain one.
        uint4 og[CPR];
        if constexpr (MODE == R8_FWD) {
            if (a.O) {
                const char* const go = reinterpret_cast<const char*>(a.O) + (offB + (size_t)r0 * rsB + (size_t)kh * (D / 2)) * sizeof(T);
#pragma unroll
                for (int x = 0; x < CPR; x++) {
                    const int c = lane + 64 * x, rr = c / CPR, cc = c % CPR;
                    og[x] = r0 + rr < S ? *reinterpret_cast<const uint4*>(go + (size_t)rr * rsB * sizeof(T) + 16 * cc) : uint4{0, 0, 0, 0};
                }
            }
        }
        __syncthreads();   // iteration nJ: the consumers work on the last tile
        if constexpr (MODE == R8_FWD) {
#pragma unroll
            for (int r = 0; r < 2; r++) {
                const float b = sum_halves(bsum[r]);
                if (h == 0) bex[((rg * 2 + kh) * 2 + r) * 32 + c32] = b;
            }
        }
        __syncthreads();   // partial row sums visible to the consumers
        if constexpr (MODE == R8_FWD) {
            if (a.O) {
                __syncthreads();   // the consumers' blocks lie in LDS
                typedef typename R::vec4 V4;
                struct Pair { V4 lo, hi; };
                const char* const stage = smem + wave * 64 * RB;
                char* const gg = reinterpret_cast<char*>(a.out_gated) + (offB + (size_t)r0 * rsB + (size_t)kh * (D / 2)) * sizeof(T);
#pragma unroll
                for (int x = 0; x < CPR; x++) {
                    const int c = lane + 64 * x, rr = c / CPR, cc = c % CPR;
                    const Pair hv = *reinterpret_cast<const Pair*>(stage + rr * RB + 16 * cc);
                    const Pair ov = *reinterpret_cast<const Pair*>(&og[x]);
                    Pair res;
                    res.lo = gate4<T>(hv.lo, ov.lo);
                    res.hi = gate4<T>(hv.hi, ov.hi);
                    if (r0 + rr < S) *reinterpret_cast<Pair*>(gg + (size_t)rr * rsB * sizeof(T) + 16 * cc) = res;
                }
            }
        }
    } else {
        // ------------------------------------------------------------------------------------------ consumers
        const int dh = sub;
        f32x16 oacc[2][NDH];
#pragma unroll
        for (int r = 0; r < 2; r++)
#pragma unroll
            for (int d = 0; d < NDH; d++)
#pragma unroll
                for (int x = 0; x < 16; x++) oacc[r][d][x] = 0.f;
        SwzTransReader<T, D> vrd;
        vrd.init(lane, NDH * dh);
        auto y2_bulk = [&](int j) {
            T* dst = reinterpret_cast<T*>(y2s + (j & 1) * Cfg::TILE_BYTES);
            if (j < full_tiles) tdma.issue(dst, Y2 + (size_t)GRAN * j * rsA, ra);
            else tile_dma_rolled<T, D, GRAN, 256>(dst, Y2, GRAN * j, S, rtid, rsA);
        };
        // fragments of one tile into registers, then tell the producers their buffer is free again
        auto take = [&](frag (&pf)[2][4]) {
#pragma unroll
            for (int r = 0; r < 2; r++)
#pragma unroll
                for (int g = 0; g < 4; g++) pf[r][g] = p_rg[(4 * r + g) * 64];
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (lane == 0) atomicAdd(pcnt + rg, 1u);
        };
        // group g contracts 16 keys; every Y2 fragment feeds both row blocks; the next group's fragments are read while
        // this group's MFMAs run
        auto gemm2 = [&](const T* y2, const frag (&pf)[2][4], auto&& hook) {
            frag vf[2][NDH];
#pragma unroll
            for (int d = 0; d < NDH; d++) vf[0][d] = vrd.read(y2, 0, d);
#pragma unroll
            for (int g = 0; g < 4; g++) {
                if (g < 2) hook(g, 2);  // the whole copy in the first half: it has to land before the barrier that ends the tile
#pragma unroll
                for (int d = 0; d < NDH; d++) {
                    if (g + 1 < 4) vf[(g + 1) & 1][d] = vrd.read(y2, KW * (g + 1), d);
                    R::mma(oacc[0][d], vf[g & 1][d], pf[0][g]);
                    R::mma(oacc[1][d], vf[g & 1][d], pf[1][g]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };

        // (chunks: the first two state tiles travel while this role sets up; their stages are free until the first key
        // tile has been worked on)
        const T* const Cst = chunk > 0 ? reinterpret_cast<const T*>(a.Cst) + ((size_t)bh * a.n_states + chunk - 1) * D * D : nullptr;
        T* const sa = reinterpret_cast<T*>(y1s + Cfg::TILE_BYTES);
        T* const sb = reinterpret_cast<T*>(y2s + Cfg::TILE_BYTES);
        if (chunk > 0) {
            tdma.issue(sa, Cst);
            tdma.issue(sb, Cst + (size_t)GRAN * D);
        }
        // per-row scalars that are only needed late (the rows' decay since the end of the previous chunk; the forward's
        // stabiliser for the normaliser): requested now, so that their trip to memory is not waited for then
        x_copy();
        float dec_pre[2] = {1.f, 1.f}, m_pre[2] = {0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 2; r++) {
            if (chunk > 0)
                dec_pre[r] = fast_exp2(a.beta2[poff - 1] - a.beta2[poff + rowc[r]] + (float)(a.G2[goff + rowc[r] / GRAN] - a.G2[goff - 1]));
            if constexpr (MODE == R8_FWD) m_pre[r] = a.M[hoff + rowc[r]];
        }
        if (chunk == 0) y2_bulk(0);   // (behind the first chunk the first Y2 tile follows the first pair of state tiles)
        if (MODE == R8_DQ && chunk == 0) {
            // Per-row scalars of the backward for row block r = dh of the row group (the producers need them from their
            // first tile on, the column kernel reads them from global memory): this role idles until the first P arrives.
            // (Behind the first chunk the producers compute them: see there.)
            const T* X = reinterpret_cast<const T*>(a.X) + offX;
            const int rc = rowc[dh];
            frag xs[NS];
#pragma unroll
            for (int s = 0; s < NS; s++) xs[s] = frag_rowmajor<T>(X + (size_t)rc * rsX, s, h);
            float inv = 0.f, dbr = 0.f;
            row_stats<T, NS>(xs, reinterpret_cast<const T*>(a.Hin) + offH + (size_t)rc * rsH, h, a.Bin[hoff + rc], a.M[hoff + rc], inv, dbr);
            const int row = r0 + 32 * dh + c32;
            if (h == 0) {
                *reinterpret_cast<float2*>(bex + ((rg * 2 + dh) * 32 + c32) * 2) = make_float2(inv, dbr);
                if (row < S) { a.inv_n[poff + row] = inv; a.db[poff + row] = dbr; }
            }
        }
        const T* const Xc = reinterpret_cast<const T*>(a.X) + offX;
        frag pf0[2][4], pf1[2][4];
        auto load_pf = [&](int pp) {   // the rows' X fragments for the pair of state tiles pp, pp + 1, from memory
#pragma unroll
            for (int r = 0; r < 2; r++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    pf0[r][g] = frag_rowmajor<T>(Xc + (size_t)rowc[r] * rsX, 4 * pp + g, h);
                    pf1[r][g] = frag_rowmajor<T>(Xc + (size_t)rowc[r] * rsX, 4 * pp + 4 + g, h);
                }
        };
        store_granule_bases();
        dma_wait();
        __syncthreads();   // sG, counters visible; the X tiles (and behind the first chunk the first state tiles) have landed
        if (chunk > 0) {   // (the first pair's fragments out of the X tile)
#pragma unroll
            for (int r = 0; r < 2; r++)
#pragma unroll
                for (int g = 0; g < 4; g++) { pf0[r][g] = xrd.read(xtile, r, g); pf1[r][g] = xrd.read(xtile, r, 4 + g); }
        }
        if (chunk > 0) {
            // What lies before the chunk: the state at the end of the previous chunk, D rows of D entries, as D/64 tiles
            // through the second stages of Y1 and Y2 (free until the first key tile has been worked on), two at a time.
            // The other operand of a tile is the rows' own X fragments (Q in the forward, dH in the dQ pass), straight
            // from global memory: the state's rows are stored in the order in which this product contracts them.
            //   forward: H^T += C~^T-tiles x Q^T, then the rows' decay exp(A_e - A_i)
            //   dQ pass: dQ^T += C~-tiles x dH^T, then decay / n; and the rank-one term decay * db_i * n~
            auto none = [](int, int) {};
#pragma unroll 1
            for (int pp = 0; pp < D / 64; pp += 2) {
                if (pp > 0) {
                    tdma.issue(sa, Cst + (size_t)GRAN * pp * D);
                    tdma.issue(sb, Cst + (size_t)GRAN * (pp + 1) * D);
                    if (pp > 2) load_pf(pp);   // (the second pair's fragments came out of the X tile: below)
                }
                dma_wait();
                __syncthreads();
                gemm2(sa, pf0, none);
                gemm2(sb, pf1, none);
                if (pp == 0 && D / 64 > 2) {   // the next pair's fragments, while the X tile is still there
#pragma unroll
                    for (int r = 0; r < 2; r++)
#pragma unroll
                        for (int g = 0; g < 4; g++) { pf0[r][g] = xrd.read(xtile, r, 8 + g); pf1[r][g] = xrd.read(xtile, r, 12 + g); }
#pragma unroll
                    for (int r = 0; r < 2; r++)
#pragma unroll
                        for (int g = 0; g < 4; g++) { pin(pf0[r][g]); pin(pf1[r][g]); }
                }
                __syncthreads();   // both stages are free again
                if (pp == 0) y2_bulk(0);   // (and so are the X tiles' stages: the first Y2 tile follows into its own)
            }
            const float* nst = nvl + dh * (D / 2) + 4 * h;
#pragma unroll
            for (int r = 0; r < 2; r++) {
                float dec = dec_pre[r];
                float rank1 = 0.f;
                if constexpr (MODE == R8_DQ) {
                    const float2 st = *reinterpret_cast<const float2*>(bex + ((rg * 2 + r) * 32 + c32) * 2);   // {1/n, db} of the row
                    rank1 = dec * st.y;
                    dec *= st.x;
                }
#pragma unroll
                for (int d = 0; d < NDH; d++)
#pragma unroll
                    for (int a4 = 0; a4 < 4; a4++) {
                        f32x4 nv = {0.f, 0.f, 0.f, 0.f};
                        if constexpr (MODE == R8_DQ) nv = *reinterpret_cast<const f32x4*>(nst + 32 * d + 8 * a4);
#pragma unroll
                        for (int c = 0; c < 4; c++) oacc[r][d][4 * a4 + c] = oacc[r][d][4 * a4 + c] * dec + rank1 * nv[c];
                    }
            }
            if constexpr (MODE == R8_DQ) {
                // Row sums of dD over the keys before the chunk: q_i . dQ_i of what the accumulators hold now; this wave's
                // half of the columns goes to LDS, the halves meet behind the next barrier
                // The wave's half row is 2 NP pieces of 8 columns; a lane holds four columns of every piece (8 bytes), which as
                // loads of their own were 8 bytes of 32 rows per instruction: the lane half h loads the pieces NP h .. NP h + NP-1
                // whole instead, and one swap per register pair hands each lane its four columns of every piece.  One row block
                // at a time: with both blocks' pieces in flight the kernel spills at D = 256.  (Touching the rows' lines ahead
                // of the state phase, as an L2 prefetch, cost more than it saved: measured.)
                typedef int i32x4 __attribute__((ext_vector_type(4)));
                typedef int i32x2 __attribute__((ext_vector_type(2)));
                constexpr int HRB = (D / 2) * (int)sizeof(T), NP = row8_pieces_per_lane(HRB);
                static_assert(NP == 2 * NDH, "a lane's pieces cover two of its column blocks' groups each");
                const char* Qh = reinterpret_cast<const char*>(reinterpret_cast<const T*>(a.Qrow) + offA + (size_t)dh * (D / 2));
#pragma unroll
                for (int r = 0; r < 2; r++) {
                    float rp = 0.f;
                    i32x4 wq[NP];
#pragma unroll
                    for (int i = 0; i < NP; i++)
                        wq[i] = *reinterpret_cast<const i32x4*>(Qh + (size_t)rowc[r] * rsA * sizeof(T) + row8_piece_offset(i, h, HRB));
#pragma unroll
                    for (int i = 0; i < NP; i++) {
                        // (lanes 32..63 of the first operand change places with lanes 0..31 of the second: result u is piece NP u + i)
                        const auto s0 = __builtin_amdgcn_permlane32_swap(wq[i][0], wq[i][2], false, false);
                        const auto s1 = __builtin_amdgcn_permlane32_swap(wq[i][1], wq[i][3], false, false);
#pragma unroll
                        for (int u = 0; u < 2; u++) {
                            const f32x4 qv = __builtin_convertvector(__builtin_bit_cast(typename R::vec4, i32x2{(int)s0[u], (int)s1[u]}), f32x4);
                            const int pc = NP * u + i, d = pc / 4, a4 = pc % 4;   // column block and group of four registers
#pragma unroll
                            for (int c = 0; c < 4; c++) rp += oacc[r][d][4 * a4 + c] * qv[c];
                        }
                    }
                    rp = sum_halves(rp);
                    if (h == 0) rix[((rg * 2 + dh) * 2 + r) * 32 + c32] = rp;
                }
            }
        }
        dma_wait();
        __syncthreads();   // iteration 0: nothing to consume yet
        if constexpr (MODE == R8_DQ) {
            if (a.chunk_len > 0 && dh == 0 && h == 0) {
#pragma unroll
                for (int r = 0; r < 2; r++) {
                    const int row = r0 + 32 * r + c32;
                    const float v = chunk > 0 ? rix[((rg * 2 + 0) * 2 + r) * 32 + c32] + rix[((rg * 2 + 1) * 2 + r) * 32 + c32] : 0.f;
                    if (row < S) a.rowinter[hoff + row] = v;
                }
            }
        }
        // iteration i (1..nJ): consume tile i-1; the copy of Y2 tile i is spread over its MFMA groups
        const int lim = (nJ < full_tiles ? nJ : full_tiles);               // tiles j < lim are complete
        const int nwork = jlast + 1 < nJ ? jlast + 1 : nJ;                 // tiles 0..nwork-1 reach this wave's rows
        const int ispread = (nwork < lim - 0 ? nwork : lim - 1);           // iterations whose next Y2 tile (index i) is complete
        // iterations 1 .. jspread-1 (jspread as in the producer of the same SIMD, which has the same rows): this wave also
        // issues the producer's share of the copy of Y1 tile i+1, all at once, before its own products
        const int limp = lim - 1;
        const int jspread = jfull < limp ? jfull : (limp > 0 ? limp : 0);
        auto main_tile = [&](int i, auto copy_y1_tag) {
            dma_wait();
            __syncthreads();
            frag pf[2][4];
            take(pf);
            if constexpr (decltype(copy_y1_tag)::value)
                tdma.issue(reinterpret_cast<T*>(y1s + ((i + 1) & 1) * Cfg::TILE_BYTES), Y1 + (size_t)GRAN * (i + 1) * rsA, ra);
            T* const ly2 = reinterpret_cast<T*>(y2s + (i & 1) * Cfg::TILE_BYTES);
            const T* gy2 = Y2 + (size_t)GRAN * i * rsA;
            auto hook = [&](int idx, int n) { tdma.issue_range(ly2, gy2, idx * PW / n, (idx + 1) * PW / n, ra); };
            gemm2(reinterpret_cast<const T*>(y2s + ((i - 1) & 1) * Cfg::TILE_BYTES), pf, hook);
        };
        int i = 1;
        for (; i < jspread; i++) main_tile(i, std::true_type{});
        for (; i <= ispread && i < nJ; i++) main_tile(i, std::false_type{});
        auto no_hook = [](int, int) {};
        for (; i <= nJ; i++) {
            dma_wait();
            __syncthreads();
            frag pf[2][4];
            take(pf);
            if (i < nJ) y2_bulk(i);
            if (i - 1 < nwork) gemm2(reinterpret_cast<const T*>(y2s + ((i - 1) & 1) * Cfg::TILE_BYTES), pf, no_hook);
        }
        __syncthreads();   // partial row sums from the producers
        float onorm[2] = {1.0f, 1.0f};
        if constexpr (MODE == R8_FWD) {
#pragma unroll
            for (int r = 0; r < 2; r++) {
                const float b = bex[((rg * 2 + 0) * 2 + r) * 32 + c32] + bex[((rg * 2 + 1) * 2 + r) * 32 + c32];
                const float m = m_pre[r];
                onorm[r] = 1.0f / (fmaxf(fabsf(b), __expf(-m)) + 1e-6f);
                const int row = r0 + 32 * r + c32;
                if (dh == 0 && h == 0 && row < S) a.Bsum[hoff + row] = b;
            }
        }
        // A lane holds 4 consecutive columns of its row: stored directly that would be 8-byte pieces scattered over 32
        // rows per instruction.  The wave's 64 x D/2 block goes through its own LDS tile (rows padded by 16 bytes; the
        // K / V stages are free: every wave is past the last barrier of the tile loop) and leaves in 16-byte pieces.
        {
            char* const stage = smem + (wave - 4) * 64 * RB;
#pragma unroll
            for (int r = 0; r < 2; r++)
#pragma unroll
                for (int d = 0; d < NDH; d++)
#pragma unroll
                    for (int a4 = 0; a4 < 4; a4++) {
                        f32x4 v;
#pragma unroll
                        for (int c = 0; c < 4; c++) v[c] = oacc[r][d][4 * a4 + c] * onorm[r];
                        *reinterpret_cast<typename R::vec4*>(stage + (32 * r + c32) * RB + (32 * d + 8 * a4 + 4 * h) * (int)sizeof(T)) = R::cvt4(v);
                    }
            // (same wave wrote and reads: no barrier, the compiler's wait for the LDS writes suffices)
            if constexpr (MODE == R8_FWD) {
                if (a.O) __syncthreads();   // with an output gate, the producer of the same rows takes the gated copy from here
            }
            char* const gout = reinterpret_cast<char*>(a.out) + (offO + (size_t)r0 * rsO + (size_t)dh * (D / 2)) * sizeof(T);
#pragma unroll
            for (int i = 0; i < 64 * CPR / 64; i++) {
                const int c = lane + 64 * i, rr = c / CPR, cc = c % CPR;
                if (r0 + rr < S)
                    *reinterpret_cast<uint4*>(gout + (size_t)rr * rsO * sizeof(T) + 16 * cc) = *reinterpret_cast<const uint4*>(stage + rr * RB + 16 * cc);
            }
        }
    }
#endif
}

template <typename T, int D, int MODE, bool DENSE>
static int launch_row8_t(const RowArgs& a, hipStream_t st) {
    using Cfg = Row8Cfg<T, D>;
    auto kern = row8_kernel<T, D, MODE, DENSE>;
    if (hipError_t e = lds_limit_once<row8_kernel<T, D, MODE, DENSE>>(160 * 1024); e != hipSuccess) return (int)e;
    const size_t lds = Cfg::FIXED_BYTES + (size_t)a.NG * sizeof(double);
    if (lds > 160 * 1024) return MLSTM_ESHAPE;  // caller falls back to the four-wave kernel
    const int nQT = (a.S + R8_BQ - 1) / R8_BQ;
    hipLaunchKernelGGL(kern, dim3(a.BH * nQT), dim3(512), lds, st, a);
    return (int)hipGetLastError();
}

template <typename T, bool DENSE>
static int launch_row8_m(int mode, int D, const RowArgs& a, hipStream_t st) {
    if (mode == R8_FWD) {
        if (D == 128) return launch_row8_t<T, 128, R8_FWD, DENSE>(a, st);
        if (D == 256) return launch_row8_t<T, 256, R8_FWD, DENSE>(a, st);
    } else {
        if (D == 128) return launch_row8_t<T, 128, R8_DQ, DENSE>(a, st);
        if (D == 256) return launch_row8_t<T, 256, R8_DQ, DENSE>(a, st);
    }
    return MLSTM_ESHAPE;
}

int launch_row8_kernel(int mode, int dtype, int D, const RowArgs& a, hipStream_t st) {
    const bool dense = is_dense(a.la, a.S, D) && is_dense(a.lb, a.S, D) && (mode == R8_FWD || is_dense(a.lh, a.S, D));
    if (dtype == MLSTM_F16) return dense ? launch_row8_m<_Float16, true>(mode, D, a, st) : launch_row8_m<_Float16, false>(mode, D, a, st);
    if (dtype == MLSTM_BF16) return dense ? launch_row8_m<__bf16, true>(mode, D, a, st) : launch_row8_m<__bf16, false>(mode, D, a, st);
    return MLSTM_ESHAPE;
}

}  // namespace mlstm
