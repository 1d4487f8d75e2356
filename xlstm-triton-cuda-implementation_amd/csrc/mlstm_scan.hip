// Scan (recurrent, chunked) form of the mLSTM forward with the silu(o) output gate, fp32.
// Replaces stabilize_fi / precompute_mlstm_triton_scan / reduce_mlstm_triton / mlstm_triton_scan
// (mlstm_scan.py:48-278) and their host driver mlstm_scan (mlstm_scan.py:281-327).
//
// State per head (mlstm_scan.py:16-26): C_t = f'_t C_{t-1} + i'_t v_t (k_t/sqrt D)^T, n_t likewise, m_t the running
// stabiliser.  With a_j = i_j - Fc_j and A_t = max_{j<=t} a_j (the gate pre-pass) the stabilised state is
//     C~_t = sum_{j<=t} exp(a_j - A_t) v_j k_j^T / sqrt(D),     h_t = C~_t q_t / (max(|n~_t . q_t|, exp(-m_t)) + 1e-6).
// The sequence is cut into chunks of 64 positions (one gate granule).  Kernels, in launch order:
//   scan_intra_kernel   per (head, chunk): P_c[t][j] = [j <= t] exp(a_j - A_t) (q_t . k_j)/sqrt(D) for the pairs inside
//                       the chunk (the only place a q.k product is formed), its row sums, and the chunk's contribution
//                       dn_c = sum_j exp(a_j - A_end) k_j / sqrt(D) to the vector state n~.
//   scan_ncarry_kernel  n~ at every chunk end: n~_c = gamma_c n~_{c-1} + dn_c, in place, coalesced streaming.
//   scan_state_kernel   one workgroup per (head, 32 value columns, key range) walks the chunks in order and keeps its
//                       slice of C~ in MFMA accumulator registers for the whole sequence (the matrix carry never
//                       leaves the chip): per chunk  num = decay_t (Q_c C~^T) + P_c V_c, then C~ = gamma C~ + (w V_c)^T K_c.
//                       With more than one key range per value tile the partial numerators go to separate buffers.
//   scan_finish_kernel  per row: b_t = decay_t (n~_{c-1} . q_t) + rowsum_t(P_c),
//                       h = (sum of partial numerators) / (max(|b|, exp(-m)) + 1e-6) * silu(o)   (mlstm_scan.py:273-277).
// HBM traffic: the compulsory stream of q, k, v, o, h, one round trip of the numerator per key range, q once more.
// The same four kernels evaluate the causal weighted sums of the backward (mlstm_scan_bwd.hip) with other operands in the
// places of q, k and v: ScanArgs::finish_mode 2 leaves the numerator itself, ScanArgs::rev walks the operands from their
// last row, ScanArgs::Epilogue says what rides along (a vector sum) and what the last kernel does with a row.
#include "mlstm_device.h"
#include "mlstm_kernels.h"
#include <type_traits>

namespace mlstm {

__device__ __forceinline__ f32x16 mma_f32(float a, float b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0); }

// ---------------------------------------------------------------------------------------------------------------
// Four workgroups per (head, chunk): three form one 32x32 block of P each (the head dimension split over the four
// waves, summed through LDS), the fourth clears the masked block and forms the chunk's contribution to n~ (mode 2: to the
// vector sum that rides along, over the rows of v, if there is one).
// The products' operands want one row per lane, which from memory would be 32 bytes per row and instruction; so a wave
// fetches its quarter of the head dimension in blocks of FBW columns with whole 128-byte lines per row (four blocks in
// flight), passes them through a piece of LDS of its own (rows padded by four floats: conflict-free both ways) and reads
// the operands from there.
template <int D>
__global__ __launch_bounds__(256) void scan_intra_kernel(ScanArgs a) {
    constexpr int DW = D / 4, FBW = DW < 32 ? DW : 32, NB = DW / FBW;   // columns per wave, per block; blocks
    constexpr int LPR = FBW / 4, RPI = 64 / LPR, NLD = LPR;             // lanes per row, rows per load instruction, loads per block
    constexpr int LST = FBW + 4, PD = NB < 4 ? NB : 4;                  // LDS row stride (floats); blocks in flight
    __shared__ __align__(16) float stage[4][64 * LST];                  // per wave: 32 rows of q, then 32 rows of k
    static_assert(64 * LST >= 16 * 64, "the partial sums reuse a wave's stage");
    auto red_at = [&](int w, int r, int l) -> float& { return stage[w][r * 64 + l]; };
    // Consecutive workgroups go to the eight XCDs in turn; the four roles of a chunk read the same rows of q and k, so
    // they take workgroups of one XCD (eight apart), which share an L2.
    int role, cidx;
    if ((gridDim.x & 31) == 0) {
        const int xcd = blockIdx.x & 7, r = blockIdx.x >> 3;
        role = r & 3; cidx = (r >> 2) * 8 + xcd;
    } else {
        role = blockIdx.x & 3; cidx = blockIdx.x >> 2;
    }
    const int c = cidx % a.NC, bh = cidx / a.NC;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, h = lane >> 5, c32 = lane & 31;
    const int S = a.S;
    const size_t hoff = (size_t)bh * S, poff = (size_t)bh * a.NC * GRAN;
    float* P = a.P + ((size_t)bh * a.NC + c) * GRAN * GRAN;
    const float log2scale = -0.5f * __log2f((float)D);
    auto row_of = [&](int t) { return hoff + (a.rev ? S - 1 - t : t); };   // the row of q, k, v that holds walk position t < S
    const bool mode2 = a.finish_mode == 2, vec = mode2 && a.ep.vec;
    if (role == 3) {
        float* sw = &stage[0][0];
        for (int i = tid; i < 32 * 32; i += 256) P[(i >> 5) * GRAN + 32 + (i & 31)] = 0.f;  // queries 0..31, keys 32..63
        if (mode2 && !vec) return;
        if (tid < GRAN) {
            float w = fast_exp2(a.alpha2[poff + GRAN * c + tid] - a.beta2[poff + GRAN * c + GRAN - 1] + log2scale);
            if (vec && a.col_scale) w *= a.col_scale[row_of(GRAN * c + tid < S ? GRAN * c + tid : S - 1)];
            sw[tid] = w;
        }
        __syncthreads();
        const float* const src = mode2 ? a.v : a.k;
        float* dn = a.Nst + ((size_t)bh * a.NC + c) * D;  // dn[k] = sum_j w_j K[j][k]   (w_j = 0 for padded positions)
        for (int k = tid; k < D; k += 256) {   // (the column's 64 loads are issued together: the loop is bound by their latency)
            float kv[GRAN];
#pragma unroll
            for (int j = 0; j < GRAN; j++) {
                int j0 = GRAN * c + j;
                j0 = j0 < S ? j0 : S - 1;
                kv[j] = src[row_of(j0) * D + k];
            }
            float s0 = 0.f, s1 = 0.f;
#pragma unroll
            for (int j = 0; j < GRAN; j += 2) {
                s0 += sw[j] * kv[j];
                s1 += sw[j + 1] * kv[j + 1];
            }
            dn[k] = s0 + s1;
        }
        return;
    }
    const int tb = role > 0, jb = role > 1;  // 32x32 block: queries 32*tb.., keys 32*jb..
    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    {
        float* const stg = stage[wave];
        const int lrow = lane / LPR, lcol = 4 * (lane % LPR);
        const float* src[NLD];   // this lane's rows: load i covers stage rows RPI*i .. RPI*i + RPI-1 (0..31: q, 32..63: k)
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            const int r = RPI * i + lrow;
            int t = GRAN * c + (r < 32 ? 32 * tb + r : 32 * jb + r - 32);
            t = t < S ? t : S - 1;
            src[i] = (r < 32 ? a.q : a.k) + row_of(t) * D + wave * DW + lcol;
        }
        f32x4 rg[PD][NLD];
#pragma unroll
        for (int b = 0; b < PD; b++)
#pragma unroll
            for (int i = 0; i < NLD; i++) rg[b][i] = *reinterpret_cast<const f32x4*>(src[i] + b * FBW);
#pragma unroll
        for (int b = 0; b < NB; b++) {
#pragma unroll
            for (int i = 0; i < NLD; i++) *reinterpret_cast<f32x4*>(stg + (RPI * i + lrow) * LST + lcol) = rg[b % PD][i];
            if (b + PD < NB) {
#pragma unroll
                for (int i = 0; i < NLD; i++) rg[b % PD][i] = *reinterpret_cast<const f32x4*>(src[i] + (b + PD) * FBW);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int s = 0; s < FBW / 8; s++) {
                const f32x4 qv = *reinterpret_cast<const f32x4*>(stg + c32 * LST + 8 * s + 4 * h);
                const f32x4 kv = *reinterpret_cast<const f32x4*>(stg + (32 + c32) * LST + 8 * s + 4 * h);
#pragma unroll
                for (int e = 0; e < 4; e++) acc = mma_f32(qv[e], kv[e], acc);  // rows = queries, columns = keys
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }
    __syncthreads();   // (every wave is done with its stage: the partial sums go there)
#pragma unroll
    for (int r = 0; r < 16; r++) red_at(wave, r, lane) = acc[r];
    __syncthreads();
    // accumulator: column (key) = 32*jb + c32, rows (queries) 32*tb + 8*(r/4) + 4h + r%4; wave w finishes r = 4w..4w+3
    const int jl = 32 * jb + c32;
    const float alj = a.alpha2[poff + GRAN * c + jl];
    const float cs = !vec ? 0.f : (a.col_scale ? a.col_scale[row_of(GRAN * c + jl < S ? GRAN * c + jl : S - 1)] : 1.0f);
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int r = 4 * wave + e;
        const int tl = 32 * tb + 8 * (r >> 2) + 4 * h + (r & 3);
        float sum = red_at(0, r, lane) + red_at(1, r, lane) + red_at(2, r, lane) + red_at(3, r, lane);
        if (vec) sum += cs * (a.ep.row_scale ? a.ep.row_scale[hoff + (GRAN * c + tl < S ? GRAN * c + tl : S - 1)] : 1.0f);
        float p = sum * fast_exp2(alj - a.beta2[poff + GRAN * c + tl] + log2scale);
        if (jl > tl) p = 0.f;
        P[tl * GRAN + jl] = p;
    }
}

// n~_c = gamma_c n~_{c-1} + dn_c over the chunks of a head, in place.  One thread per column; the decays of 256 chunks at
// a time are formed side by side, and the column's sums are fetched eight chunks ahead of the serial sum.
__global__ __launch_bounds__(256) void scan_ncarry_kernel(ScanArgs a) {
    __shared__ float sgam[256];
    const int bh = blockIdx.y, tid = threadIdx.x, k = blockIdx.x * 256 + tid, NC = a.NC;
    const bool mine = k < a.D;
    const size_t poff = (size_t)bh * NC * GRAN;
    float* n = a.Nst + (size_t)bh * NC * a.D + (mine ? k : 0);
    float run = mine ? n[0] : 0.f;
    for (int c0 = 1; c0 < NC; c0 += 256) {
        __syncthreads();
        if (const int c = c0 + tid; c < NC)
            sgam[tid] = fast_exp2(a.beta2[poff + GRAN * c - 1] - a.beta2[poff + GRAN * c + GRAN - 1] +
                                  (float)(a.G2[(size_t)bh * NC + c] - a.G2[(size_t)bh * NC + c - 1]));
        __syncthreads();
        const int cn = NC - c0 < 256 ? NC - c0 : 256;
        for (int cb = 0; cb < cn && mine; cb += 8) {
            float x[8];
#pragma unroll
            for (int j = 0; j < 8; j++) x[j] = cb + j < cn ? n[(size_t)(c0 + cb + j) * a.D] : 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) {
                run = (cb + j < cn ? sgam[cb + j] : 1.0f) * run + x[j];
                if (cb + j < cn) n[(size_t)(c0 + cb + j) * a.D] = run;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The contraction over the 64 keys of a chunk runs in 32 MFMA steps; step s takes the keys {s, 32 + s} (lane half h
// supplies key 32h + s), so that a lane's P operands and gate weights are contiguous in memory.  A wave's key columns
// are interleaved over its NKB accumulator blocks (row rho of block kb is column kbase + NKB*rho + kb): one vector load
// per key row then feeds all blocks.
// Operands from memory are fetched one phase ahead into registers (one wave per SIMD has 512 of them): K of the chunk
// before the read-out products, Q of the next chunk before the state update products.
template <int N> struct FVec { typedef float type __attribute__((ext_vector_type(N))); };
template <> struct FVec<1> { struct type { float x; __device__ float operator[](int) const { return x; } }; };

// A sequence may also be cut into segments of seg_chunks chunks that run side by side (blockIdx.y), for the cases in
// which heads x value tiles x key ranges alone leave most of the chip idle (one long sequence, small D):
//   STATE_ONLY = true   every segment but the last walks its chunks from a zero state, updates only, and leaves the
//                       state at its end (accumulator registers as they are) in seg_state;
//   scan_segcarry_kernel turns those into the true states at the segment ends (a short serial sum over the segments);
//   STATE_ONLY = false  the walk proper: segment s > 0 starts from the state at the end of segment s - 1.
// REV: q, k and v are walked from their last row (ScanArgs::rev).  A complete chunk's 64 rows then lie in front of the row of
// its first position; the lane parts of the addresses stay non-negative by counting from the chunk's last position.
template <int D, int KS, int NW, bool STATE_ONLY, bool REV>
__global__ __launch_bounds__(NW * 64) void scan_state_kernel(ScanArgs a) {
    constexpr int KPW = D / KS / NW, NKB = KPW / 32, NVT = D / 32;  // key columns per wave, in blocks of 32
    constexpr int SH = 32 / (NW * KS);                              // in-chunk contraction steps per wave
    static_assert(SH >= 1 && NW >= 1 && NW <= 8 && (NKB == 1 || NKB == 2 || NKB == 4) && NKB * 32 == KPW, "32, 64 or 128 key columns per wave");
    using kvec = typename FVec<NKB>::type;
    extern __shared__ __align__(16) float lds[];
    float (*red)[NW][32][64] = reinterpret_cast<float (*)[NW][32][64]>(lds);  // [chunk parity][wave][accumulator register][lane]
    float (*sgate)[2][GRAN] = reinterpret_cast<float (*)[2][GRAN]>(lds + 2 * NW * 32 * 64);  // [chunk mod 3][0: key weights w_j, 1: query decays][position]
    const int bh = blockIdx.x % a.BH;
    const int rest = blockIdx.x / a.BH;
    const int vt = rest % NVT, ks = rest / NVT;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, h = lane >> 5, c32 = lane & 31;
    const int S = a.S, NC = a.NC;
    const int seg = blockIdx.y, c_begin = seg * a.seg_chunks, c_end = c_begin + a.seg_chunks < NC ? c_begin + a.seg_chunks : NC;
    const size_t hoff = (size_t)bh * S, poff = (size_t)bh * NC * GRAN;
    const float* Q = a.q + hoff * D;
    const float* K = a.k + hoff * D;
    const float* V = a.v + hoff * D;
    const double* G2 = a.G2 + (size_t)bh * NC;
    float* out = (ks == 0 ? a.h : a.hpart + (size_t)(ks - 1) * a.BH * S * D) + hoff * D;
    const int kbase = (ks * NW + wave) * KPW, v0 = 32 * vt;
    const float log2scale = -0.5f * __log2f((float)D);
    const int hrow = REV ? 32 * (1 - h) : 32 * h;         // the lane half's first row in a chunk's 64 rows as they lie in memory
    const int v_lofs = hrow * D + v0 + c32;               // lane part of a value address (column v0 + c32)
    const int k_lofs = hrow * D + kbase + NKB * c32;      // lane part of a key address
    auto row_of = [&](int t) { return (size_t)(REV ? S - 1 - t : t); };   // the row that holds walk position t < S

    // Gate vectors of a chunk: weights of its keys, decays of its queries (from the previous chunk end).  The carried
    // state is kept as st = C~ / Gamma with a running power of two Gamma <= 1, so that the per-chunk decay gamma_c
    // multiplies into Gamma (folded into these vectors) and the registers are rescaled only when Gamma gets small.
    constexpr int NI = (2 * GRAN + NW * 64 - 1) / (NW * 64);
    float lg = 0.f;  // log2 Gamma for the read-out of the next chunk to prepare
    struct Gates { float x[NI]; float dec_add, w_add, rescale; };
    auto gates_fetch = [&](int c) {  // the loads, and the scalars (identical in all lanes)
        Gates g;
        const int cp = c > 0 ? c - 1 : 0;
        const float bprev = a.beta2[poff + GRAN * cp + GRAN - 1], bend = a.beta2[poff + GRAN * c + GRAN - 1];
        const float dG = (float)(G2[c] - G2[cp]);
        const float lgam = c > 0 ? bprev - bend + dG : 0.f;
        g.dec_add = c > 0 ? bprev + dG + lg : 0.f;
        float lnew = lg + lgam;
        g.rescale = 0.f;
        if (lnew < -24.f) { g.rescale = lnew; lnew = 0.f; }
        g.w_add = log2scale - bend - lnew;
        lg = lnew;
#pragma unroll
        for (int n = 0; n < NI; n++) {
            const int i = tid + n * NW * 64, pos = i & (GRAN - 1);
            g.x[n] = i < GRAN ? a.alpha2[poff + GRAN * c + pos] : (i < 2 * GRAN ? a.beta2[poff + GRAN * c + pos] : 0.f);
        }
        return g;
    };
    auto gates_store = [&](int c, const Gates& g) {
#pragma unroll
        for (int n = 0; n < NI; n++) {
            const int i = tid + n * NW * 64, pos = i & (GRAN - 1);
            if (i < GRAN) sgate[c % 3][0][pos] = fast_exp2(g.x[n] + g.w_add);
            else if (i < 2 * GRAN) sgate[c % 3][1][pos] = c > 0 ? fast_exp2(g.dec_add - g.x[n]) : 1.0f;
        }
    };

    f32x16 st[NKB];  // st[kb][r] = C~[v = v0 + c32][k = kbase + NKB*(8*(r/4) + 4h + r%4) + kb]
    // a workgroup's state in seg_state: [segment][workgroup][wave][kb][r][lane]
    const size_t seg_stride = (size_t)gridDim.x * NW * NKB * 16 * 64;
    float* const seg_mine = a.seg_state + ((size_t)blockIdx.x * NW + wave) * NKB * 16 * 64 + lane;
#pragma unroll
    for (int kb = 0; kb < NKB; kb++)
#pragma unroll
        for (int r = 0; r < 16; r++) st[kb][r] = (!STATE_ONLY && seg > 0) ? seg_mine[(size_t)(seg - 1) * seg_stride + (kb * 16 + r) * 64] : 0.f;
    kvec qreg[2][4][4];  // [query block][x][e]: Q[t][kbase + NKB*(8x + 4h + e) + 0..NKB-1]
    auto load_q = [&](int c, int tb, int x, int e) {  // (row clamped: the chunk may be the partial one)
        int t = GRAN * c + 32 * tb + c32;
        t = t < S ? t : S - 1;
        qreg[tb][x][e] = *reinterpret_cast<const kvec*>(Q + row_of(t) * D + kbase + 4 * NKB * h + NKB * (8 * x + e));
    };
    if constexpr (!STATE_ONLY) {
#pragma unroll
        for (int i = 0; i < 32; i++) load_q(c_begin, i & 1, i >> 3, (i >> 1) & 3);
    }
    float rescale_cur;
    float lg_done = 0.f;   // log2 Gamma of the last chunk whose update is in st
    {
        const Gates g0 = gates_fetch(c_begin);
        gates_store(c_begin, g0);
        rescale_cur = g0.rescale;
    }
    __syncthreads();

    // One chunk.  The memory operations are spread between the groups of matrix instructions that cover them (a wave
    // issues in order, and four waves share the CU's one address path: a burst of loads would idle the matrix unit):
    // values, pair weights and keys of this chunk during the read-out products, the next chunk's queries during the
    // state update.  LAST: the final chunk of the sequence (possibly partial: rows clamped; no state update follows).
    auto chunk = [&](const int c, auto last_tag) {
        constexpr bool LAST = decltype(last_tag)::value;
        const int t0 = GRAN * c;
        const float* sw = sgate[c % 3][0];
        const float* sdec = sgate[c % 3][1];
        float vraw[32];
        float pa[2][SH];
        float vin[SH];  // this wave's values for the in-chunk products (a register array takes no wave-dependent index)
        kvec kreg[32];
        // uniform: the first of the chunk's 64 rows in memory (REV: the row of its last position; only complete chunks use it)
        const size_t r0 = LAST ? 0 : (REV ? (size_t)(S - GRAN - t0) : (size_t)t0);
        const float* vrow = V + r0 * D;
        const float* krow = K + r0 * D;
        auto load_v = [&](int s) {   // position t0 + 32h + s
            if constexpr (LAST) {
                int j = t0 + 32 * h + s;
                j = j < S ? j : S - 1;
                vraw[s] = V[row_of(j) * D + v0 + c32];
            } else {
                vraw[s] = (vrow + (size_t)(REV ? 31 - s : s) * D)[v_lofs];
            }
        };
        auto load_k = [&](int s) { kreg[s] = *reinterpret_cast<const kvec*>(krow + (size_t)(REV ? 31 - s : s) * D + k_lofs); };
        // ---- read-out of the carried state: acc[tb] = decay_t * Q_c[32 tb.., k-range of this wave] . C~^T
        f32x16 acc[2];
#pragma unroll
        for (int tb = 0; tb < 2; tb++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[tb][r] = 0.f;
        Gates gn;
        lg_done = lg;
        if constexpr (!LAST) gn = gates_fetch(c + 1);
        // the in-chunk products are split over all waves of all key ranges: SH contraction steps each
        const int s0 = (ks * NW + wave) * SH;
        auto load_p = [&]() {
            const float* Pc = a.P + ((size_t)bh * NC + c) * GRAN * GRAN + 32 * h + s0;
            using pvec = typename FVec<(SH < 4 ? SH : 4)>::type;
#pragma unroll
            for (int tb = 0; tb < 2; tb++)
#pragma unroll
                for (int x = 0; x < (SH + 3) / 4; x++) {
                    const pvec pv = *reinterpret_cast<const pvec*>(Pc + (32 * tb + c32) * GRAN + 4 * x);
#pragma unroll
                    for (int e = 0; e < (SH < 4 ? SH : 4); e++) pa[tb][4 * x + e] = pv[e];
                }
        };
        auto load_vin = [&]() {
#pragma unroll
            for (int s = 0; s < SH; s++) {
                int j = t0 + 32 * h + s0 + s;
                if constexpr (LAST) j = j < S ? j : S - 1;
                vin[s] = V[row_of(j) * D + v0 + c32];
            }
        };
#pragma unroll
        for (int g = 0; g < 16; g++) {  // g = 4x + e
            if constexpr (!STATE_ONLY) {
                if (g == 0) load_p();
                if (g == 1) load_vin();
            }
            load_v(2 * g);
            load_v(2 * g + 1);
            if constexpr (!LAST) {
                load_k(2 * g);
                load_k(2 * g + 1);
            }
            if constexpr (!STATE_ONLY) {
#pragma unroll
                for (int kb = 0; kb < NKB; kb++) {
                    acc[0] = mma_f32(qreg[0][g >> 2][g & 3][kb], st[kb][g], acc[0]);
                    acc[1] = mma_f32(qreg[1][g >> 2][g & 3][kb], st[kb][g], acc[1]);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if constexpr (!STATE_ONLY) {
#pragma unroll
            for (int tb = 0; tb < 2; tb++)
#pragma unroll
                for (int x = 0; x < 4; x++) {
                    const f32x4 dec = *reinterpret_cast<const f32x4*>(sdec + 32 * tb + 8 * x + 4 * h);
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[tb][4 * x + e] *= dec[e];
                }
            // ---- pairs inside the chunk: acc += P_c[:, this wave's keys] . V_c
#pragma unroll
            for (int s = 0; s < SH; s++) {
                acc[0] = mma_f32(pa[0][s], vin[s], acc[0]);
                acc[1] = mma_f32(pa[1][s], vin[s], acc[1]);
            }
            // ---- sum the partial numerators of the waves and store them (unnormalised)
#pragma unroll
            for (int tb = 0; tb < 2; tb++)
#pragma unroll
                for (int r = 0; r < 16; r++) red[c & 1][wave][16 * tb + r][lane] = acc[tb][r];
        }
        if constexpr (!LAST) gates_store(c + 1, gn);
        // The only barrier of a chunk.  Between two barriers a wave is in the tail of one chunk or the head of the next:
        // the partial sums alternate between two buffers, the gate vectors (written a chunk ahead) between three.
        __syncthreads();
        auto sum_store = [&](int idx) {  // one accumulator register of the numerator: sum over the waves, store
            float sum = 0.f;
#pragma unroll
            for (int w = 0; w < NW; w++) sum += red[c & 1][w][idx][lane];
            const int tl = 32 * (idx >> 4) + 8 * ((idx & 15) >> 2) + 4 * h + (idx & 3);
            const int t = t0 + tl;
            if (!LAST || t < S) out[(size_t)t * D + v0 + c32] = sum;
        };
        if constexpr (LAST) {
            for (int idx = wave; idx < 32; idx += NW) sum_store(idx);
        } else {
            // ---- state update: st += (w V_c)^T K_c (the weights carry 1/Gamma), rescaled first when Gamma got small
            if (rescale_cur != 0.f) {
                const float f = fast_exp2(rescale_cur);
#pragma unroll
                for (int kb = 0; kb < NKB; kb++)
#pragma unroll
                    for (int r = 0; r < 16; r++) st[kb][r] *= f;
            }
            rescale_cur = gn.rescale;
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int x = 0; x < 8; x++) {
                const f32x4 w4 = *reinterpret_cast<const f32x4*>(sw + 32 * h + 4 * x);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int i = 4 * x + e;
                    if constexpr (!STATE_ONLY) {
                        load_q(c + 1, i & 1, i >> 3, (i >> 1) & 3);
                        if (i < 32 / NW) sum_store(wave + NW * i);
                    }
                    const float wv = vraw[i] * w4[e];
#pragma unroll
                    for (int kb = 0; kb < NKB; kb++) st[kb] = mma_f32(kreg[i][kb], wv, st[kb]);  // rows = k, columns = v
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    };
    if constexpr (STATE_ONLY) {
        // (never the last segment: every chunk is complete and has a successor whose gates the walk fetches ahead)
        for (int c = c_begin; c < c_end; c++) chunk(c, std::false_type{});
        const float f = fast_exp2(lg_done);   // st = C~ / Gamma
#pragma unroll
        for (int kb = 0; kb < NKB; kb++)
#pragma unroll
            for (int r = 0; r < 16; r++) seg_mine[(size_t)seg * seg_stride + (kb * 16 + r) * 64] = st[kb][r] * f;
    } else {
        for (int c = c_begin; c + 1 < c_end; c++) chunk(c, std::false_type{});
        chunk(c_end - 1, std::true_type{});
    }
}

// States at the segment ends from the segments' own sums, in place: x_s = exp(A_{e(s-1)} - A_{e(s)}) x_{s-1} + x_s with
// e(s) the last position of segment s.  One thread per state element; elems = floats per segment, wg_elems = floats per
// workgroup of the state kernel (whose index modulo BH is the head).
__global__ __launch_bounds__(256) void scan_segcarry_kernel(ScanArgs a, size_t elems, int wg_elems) {
    const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= elems) return;
    const int bh = (int)((e / wg_elems) % a.BH);
    const size_t poff = (size_t)bh * a.NC * GRAN;
    float run = a.seg_state[e];
    for (int s = 1; s + 1 < a.nseg; s++) {
        const int c1 = (s + 1) * a.seg_chunks - 1, c0 = s * a.seg_chunks - 1;   // last chunks of segments s and s - 1
        const double A1 = (double)a.beta2[poff + GRAN * c1 + GRAN - 1] - a.G2[(size_t)bh * a.NC + c1];
        const double A0 = (double)a.beta2[poff + GRAN * c0 + GRAN - 1] - a.G2[(size_t)bh * a.NC + c0];
        run = fast_exp2((float)(A0 - A1)) * run + a.seg_state[(size_t)s * elems + e];
        a.seg_state[(size_t)s * elems + e] = run;
    }
}

// ---------------------------------------------------------------------------------------------------------------
// one wave per row: normaliser sum, then the row of h
__global__ __launch_bounds__(256) void scan_finish_kernel(ScanArgs a, int KS) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t rows = (size_t)a.BH * a.S;
    const int D = a.D;
    for (size_t row = (size_t)blockIdx.x * 4 + wave; row < rows; row += (size_t)gridDim.x * 4) {
        const int bh = (int)(row / a.S), t = (int)(row % a.S), c = t / GRAN;
        const size_t poff = (size_t)bh * a.NC * GRAN;
        if (a.finish_mode == 2) {
            const ScanArgs::Epilogue& ep = a.ep;
            const size_t orow = ep.out_rev ? (size_t)bh * a.S + (a.S - 1 - t) : row;
            const bool carried = ep.vec && c > 0;
            // rs_t decay_t, the factor of the vector sum at the end of the chunk before
            const float cf = !carried ? 0.f : (ep.row_scale ? ep.row_scale[row] : 1.0f) *
                                                  fast_exp2(a.beta2[poff + GRAN * c - 1] - a.beta2[poff + t] +
                                                            (float)(a.G2[(size_t)bh * a.NC + c] - a.G2[(size_t)bh * a.NC + c - 1]));
            const float* cr = carried ? a.Nst + ((size_t)bh * a.NC + c - 1) * D : nullptr;
            const float wd = ep.wd_alpha2 ? fast_exp2(ep.wd_alpha2[poff + (orow - (size_t)bh * a.S)] - ep.wd_beta2[poff + (orow - (size_t)bh * a.S)]) : 1.0f;
            float* const dst = (ep.out ? ep.out : a.h) + orow * D;
            float acc = 0.f;
            for (int k = 4 * lane; k < D; k += 256) {
                f32x4 x = *reinterpret_cast<const f32x4*>(a.h + row * D + k);
                for (int p = 1; p < KS; p++) x += *reinterpret_cast<const f32x4*>(a.hpart + ((size_t)(p - 1) * rows + row) * D + k);
                if (carried) {
                    const f32x4 cv = *reinterpret_cast<const f32x4*>(cr + k);
#pragma unroll
                    for (int e = 0; e < 4; e++) x[e] += cf * cv[e];
                }
#pragma unroll
                for (int e = 0; e < 4; e++) x[e] *= wd;
                if (ep.dot_with) {
                    const f32x4 dv = *reinterpret_cast<const f32x4*>(ep.dot_with + orow * D + k);
                    acc += dv[0] * x[0] + dv[1] * x[1] + dv[2] * x[2] + dv[3] * x[3];
                }
                *reinterpret_cast<f32x4*>(dst + k) = x;
            }
            if (ep.dot_with) {
                acc = wave_reduce<OpAdd>(acc);
                if (lane == 0) {
                    ep.dot_out[orow] = acc;
                    if (ep.x_out) ep.x_out[orow] = acc - ep.dot_minus[orow];
                }
            }
            continue;
        }
        float dot = 0.f;
        if (c > 0) {
            const float* n = a.Nst + ((size_t)bh * a.NC + c - 1) * D;
            const float* q = a.q + row * D;
            for (int k = 4 * lane; k < D; k += 256) {
                const f32x4 nv = *reinterpret_cast<const f32x4*>(n + k);
                const f32x4 qv = *reinterpret_cast<const f32x4*>(q + k);
                dot += nv[0] * qv[0] + nv[1] * qv[1] + nv[2] * qv[2] + nv[3] * qv[3];
            }
            dot = wave_reduce<OpAdd>(dot);
            dot *= fast_exp2(a.beta2[poff + GRAN * c - 1] - a.beta2[poff + t] +
                             (float)(a.G2[(size_t)bh * a.NC + c] - a.G2[(size_t)bh * a.NC + c - 1]));
        }
        const float prow = a.P[((size_t)bh * a.NC + c) * GRAN * GRAN + (size_t)(t - GRAN * c) * GRAN + lane];
        const float b = dot + wave_reduce<OpAdd>(prow);
        const float inv = 1.0f / (fmaxf(fabsf(b), __expf(-a.M[row])) + 1e-6f);
        if (a.Bout && lane == 0) a.Bout[row] = b;
        for (int k = 4 * lane; k < D; k += 256) {
            f32x4 x = *reinterpret_cast<const f32x4*>(a.h + row * D + k);
            for (int p = 1; p < KS; p++) {
                const f32x4 y = *reinterpret_cast<const f32x4*>(a.hpart + ((size_t)(p - 1) * rows + row) * D + k);
                x += y;
            }
            if (a.finish_mode == 0) {
                const f32x4 ov = *reinterpret_cast<const f32x4*>(a.o + row * D + k);
#pragma unroll
                for (int e = 0; e < 4; e++) x[e] *= inv;
                if (a.Hun) *reinterpret_cast<f32x4*>(a.Hun + row * D + k) = x;
#pragma unroll
                for (int e = 0; e < 4; e++) x[e] = x[e] * (ov[e] / (1.0f + __expf(-ov[e])));
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) x[e] *= inv;
            }
            *reinterpret_cast<f32x4*>(a.h + row * D + k) = x;
        }
    }
}

template <int D, int KS, int NW, bool REV>
static void launch_state(const ScanArgs& a, hipStream_t st) {
    if constexpr ((D / KS / NW == 32 || D / KS / NW == 64 || D / KS / NW == 128) && NW * KS <= 32) {
        constexpr int lds_bytes = (2 * NW * 32 * 64 + 3 * 2 * GRAN) * 4;
        // (a failure here shows up as a launch error, which the caller reads with hipGetLastError)
        (void)lds_limit_once<scan_state_kernel<D, KS, NW, false, REV>>(lds_bytes);
        const int wgs = a.BH * (D / 32) * KS;
        if (a.nseg > 1) {
            (void)lds_limit_once<scan_state_kernel<D, KS, NW, true, REV>>(lds_bytes);
            hipLaunchKernelGGL((scan_state_kernel<D, KS, NW, true, REV>), dim3(wgs, a.nseg - 1), dim3(NW * 64), lds_bytes, st, a);
            const size_t elems = (size_t)wgs * NW * (D / KS / NW / 32) * 16 * 64;   // = BH * D * D
            hipLaunchKernelGGL(scan_segcarry_kernel, dim3((unsigned)((elems + 255) / 256)), dim3(256), 0, st, a, elems,
                               NW * (D / KS / NW / 32) * 16 * 64);
        }
        hipLaunchKernelGGL((scan_state_kernel<D, KS, NW, false, REV>), dim3(wgs, a.nseg), dim3(NW * 64), lds_bytes, st, a);
    }
}

template <int D, int KS>
static void launch_state_w(const ScanArgs& a, int NW, hipStream_t st) {
    (void)NW;  // scan_plan: two waves per workgroup at D = 64, four above
    if (a.rev) launch_state<D, KS, (D / 32 < 4 ? D / 32 : 4), true>(a, st);
    else launch_state<D, KS, (D / 32 < 4 ? D / 32 : 4), false>(a, st);
}

template <int D>
static int launch_scan_d(const ScanArgs& a, int KS, int NW, hipStream_t st, void (*mark)(int, hipStream_t, bool)) {
    mark(MLSTM_K_SCAN_CARRY, st, true);
    hipLaunchKernelGGL(scan_intra_kernel<D>, dim3(a.BH * a.NC * 4), dim3(256), 0, st, a);
    if (a.finish_mode != 2 || a.ep.vec) hipLaunchKernelGGL(scan_ncarry_kernel, dim3((D + 255) / 256, a.BH), dim3(256), 0, st, a);
    mark(MLSTM_K_SCAN_CARRY, st, false);
    mark(MLSTM_K_SCAN_STATE, st, true);
    if (KS == 8) launch_state_w<D, 8>(a, NW, st);
    else if (KS == 4) launch_state_w<D, 4>(a, NW, st);
    else if (KS == 2) launch_state_w<D, 2>(a, NW, st);
    else launch_state_w<D, 1>(a, NW, st);
    mark(MLSTM_K_SCAN_STATE, st, false);
    mark(MLSTM_K_SCAN_OUT, st, true);
    const size_t rows = (size_t)a.BH * a.S;
    const int blocks = (int)((rows + 3) / 4 < 16384 ? (rows + 3) / 4 : 16384);
    hipLaunchKernelGGL(scan_finish_kernel, dim3(blocks), dim3(256), 0, st, a, KS);
    mark(MLSTM_K_SCAN_OUT, st, false);
    return (int)hipGetLastError();
}

void launch_scan_ncarry(const ScanArgs& a, hipStream_t st) {
    hipLaunchKernelGGL(scan_ncarry_kernel, dim3((a.D + 255) / 256, a.BH), dim3(256), 0, st, a);
}

// Key ranges per value tile and waves per workgroup.
void scan_plan(int BH, int D, int* KS, int* NW) {
    const int nw = D / 32 < 4 ? D / 32 : 4;    // waves per workgroup: one per SIMD (each wants the full register file)
    int ks = D / nw > 128 ? D / nw / 128 : 1;  // at most 128 key columns per wave
    while (D / ks / nw > 32 && BH * (D / 32) * ks < 256) ks *= 2;  // at least one workgroup per CU where D allows
    *KS = ks; *NW = nw;
}
int scan_key_splits(int BH, int D) { int ks, nw; scan_plan(BH, D, &ks, &nw); return ks; }

// Segments of a sequence that run side by side: none while heads x value tiles x key ranges fill the chip; otherwise
// enough for about two workgroups per CU, of at least eight chunks each.
void scan_segments(int BH, int S, int D, int* nseg, int* seg_chunks) {
    const int NC = (S + GRAN - 1) / GRAN, wgs = BH * (D / 32) * scan_key_splits(BH, D);
    int n = 1;
    if (wgs < 256) {
        n = (512 + wgs - 1) / wgs;
        if (n > NC / 8) n = NC / 8;
        if (n < 1) n = 1;
    }
    const int len = (NC + n - 1) / n;
    *seg_chunks = len;
    *nseg = (NC + len - 1) / len;
}
size_t scan_segment_state_bytes(int BH, int S, int D) {
    int n, len; scan_segments(BH, S, D, &n, &len);
    return n > 1 ? (size_t)(n - 1) * BH * D * D * sizeof(float) : 0;
}

int launch_scan(const ScanArgs& a_in, int KS, hipStream_t st, void (*mark)(int, hipStream_t, bool)) {
    ScanArgs a = a_in;
    scan_segments(a.BH, a.S, a.D, &a.nseg, &a.seg_chunks);
    if (a.nseg > 1 && !a.seg_state) return MLSTM_EWORKSPACE;
    if (a.finish_mode != 2 && (a.rev || a.col_scale)) return MLSTM_EINVAL;
    if (a.finish_mode == 2 && ((a.ep.out_rev && (!a.ep.out || a.ep.out == a.h)) ||
                               (a.ep.dot_with && !a.ep.dot_out) || (a.ep.x_out && !(a.ep.dot_with && a.ep.dot_minus)) ||
                               (!a.ep.wd_alpha2 != !a.ep.wd_beta2)))
        return MLSTM_EINVAL;
    int ks, NW; scan_plan(a.BH, a.D, &ks, &NW);
    if (NW != (a.D / 32 < 4 ? a.D / 32 : 4)) return MLSTM_ESHAPE;
    const int kpw = a.D / KS / NW;
    if (kpw * KS * NW != a.D || (kpw != 32 && kpw != 64 && kpw != 128) || NW > 8 || NW * KS > 32) return MLSTM_ESHAPE;
    switch (a.D) {
        case 64: return launch_scan_d<64>(a, KS, NW, st, mark);
        case 128: return launch_scan_d<128>(a, KS, NW, st, mark);
        case 256: return launch_scan_d<256>(a, KS, NW, st, mark);
        case 512: return launch_scan_d<512>(a, KS, NW, st, mark);
        case 1024: return launch_scan_d<1024>(a, KS, NW, st, mark);
    }
    return MLSTM_ESHAPE;
}

}  // namespace mlstm
