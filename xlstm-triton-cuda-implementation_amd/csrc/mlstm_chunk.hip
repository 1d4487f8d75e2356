// Chunk states for the matmul-form forward of long sequences (16-bit types).
//
// The forward of a row i only needs the keys of its own chunk of L positions one by one; everything before the chunk
// enters through the state the scan form carries (mlstm_scan.py:16-26; the two forms are the same function):
//     C~_c = sum_{j <= e_c} exp(a_j - A_{e_c}) k_j v_j^T / sqrt(D),     n~_c likewise with k_j alone,
// with e_c the last position of chunk c, a_j = i_j - Fc_j and A the running maximum of a (the gate pre-pass), so that
//     sum_{j <= e_c} C~_ij v_j = exp(A_{e_c} - A_i) q_i^T C~_c     for every row i behind the chunk (A_i >= A_{e_c}).
// The row kernel then walks the key tiles of the row's own chunk and D/64 "tiles" of the state instead of all the key
// tiles back to position 0: 2 L/64 + D/64 tiles at most, whatever the sequence length.
//
//   chunk_sum_kernel    per (head, chunk, 128 value columns): dC_c = sum_{j in chunk} w_j k_j v_j^T with
//                       w_j = exp(a_j - A_{e_c}) / sqrt(D), as a bf16 / fp16 MFMA product over the chunk's positions (both
//                       operands are contracted over positions: transposing LDS reads; V is scaled by w on its way
//                       into LDS), fp32 result; and dn_c = sum_j w_j k_j.  Eight waves: four multiply, four bring the tiles.
//   chunk_carry_kernel  C~_c = gamma_c C~_{c-1} + dC_c over the chunks of a head (gamma_c = exp(A_{e_{c-1}} - A_{e_c})),
//                       element-wise, written in the element type; n~_c likewise, in place, fp32.
// State rows are stored in the order in which the row kernel's second product contracts them (see PERM16 below).
#include "mlstm_device.h"
#include "mlstm_kernels.h"
#include <type_traits>
#include <utility>

namespace mlstm {

// The row kernel feeds the state tiles to its second product with the lanes' own row-major Q fragments as the other
// operand: the lane of half h holds columns 16 s + 8 h + e (e = 0..7) of step s, while the transposing read of the
// tile hands it rows 16 s + 4 h + e (e < 4) and 16 s + 8 + 4 h + e - 4 (e >= 4).  Tile row u (mod 16) therefore holds
// state row PERM16(u): the two middle groups of four swap places.
__device__ __forceinline__ int perm16(int u) { return (u & ~12) | ((u & 4) << 1) | ((u & 8) >> 1); }
// (fp32 tiles are read one element per lane, in the natural order)
template <typename T>
__device__ __forceinline__ int state_row(int u) { return sizeof(T) == 2 ? ((u & ~15) | perm16(u & 15)) : u; }

// STRICT: split mode, the weighted V rows go to LDS as two tiles, hi and lo (ChunkArgs::precise)
template <typename T, int D, bool STRICT = false>
struct ChunkCfg {
    static constexpr int VW = 128;                                  // value columns per workgroup
    static constexpr int STAGES = 2;                                // LDS stages: the tile worked on and the next one
    static constexpr int RSETS = 3;                                 // register sets: tiles in flight from memory
    static constexpr size_t K_BYTES = (size_t)GRAN * D * sizeof(T), V_TILE = (size_t)GRAN * VW * sizeof(T);
    static constexpr size_t V_BYTES = (STRICT ? 2 : 1) * V_TILE;    // per stage: the hi tile, then the lo tile
    static constexpr size_t TILE_BYTES = STAGES * (K_BYTES + V_BYTES);   // plus one float per position of the chunk
    static constexpr int MAX_L = (int)((160 * 1024 - TILE_BYTES) / (2 * sizeof(float))) / 128 * 128;
};

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// Eight 16-bit elements (four dwords) as floats.  bf16 by hand: one shift or mask per element (the generic vector
// conversion costs several instructions per element, in a kernel that is bound by instruction issue).
template <typename T>
__device__ __forceinline__ void unpack8(const u32x4& d, float (&x)[8]) {
    if constexpr (std::is_same<T, __bf16>::value) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            x[2 * i] = __builtin_bit_cast(float, d[i] << 16);
            x[2 * i + 1] = __builtin_bit_cast(float, d[i] & 0xffff0000u);
        }
    } else {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        const h8 v = __builtin_bit_cast(h8, d);
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = (float)v[e];
    }
}

template <int... I, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) { (f(std::integral_constant<int, I>{}), ...); }
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) { static_for_impl(std::make_integer_sequence<int, N>{}, f); }

// NTT: tiles per chunk as a compile-time constant (the tile loop is then straight-line code), or 0 for any chunk length
template <typename T, int D, int NTT, bool STRICT>
__global__ __launch_bounds__(512) void chunk_sum_kernel(ChunkArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
    using R = Tr<T>;
    using Cfg = ChunkCfg<T, D, STRICT>;
    typedef typename R::frag frag;
    static_assert(R::HALF && (D == 128 || D == 256), "16-bit types, D = 128 or 256");
    constexpr int VW = Cfg::VW, VH = D / VW, MB = D / 128, NB = VW / 32, KW = R::KW, ST = Cfg::STAGES;
    using ZK = Swz<T, D>;
    using ZV = Swz<T, VW>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    char* const ks = smem;
    char* const vs = smem + ST * Cfg::K_BYTES;
    float* const sw = reinterpret_cast<float*>(smem + Cfg::TILE_BYTES);   // [L] position weights of the matrix sum
    float* const sw2 = sw + a.L;                                           // [L] ... of the vector sum

    // Eight waves, two on every SIMD.  Waves 0..3 multiply: operand reads and MFMAs, nothing else.  Waves 4..7 feed them: they
    // load the tiles, scale V, write the LDS stages and add up the vector state from the K pieces they hold anyway.  With
    // four waves doing both in turn the kernel was bound by instruction issue (about 430 other instructions per tile next to
    // 1024 cycles of MFMAs, on a SIMD with nothing else to run); the two kinds of work now overlap.
    const bool feeder = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8) != 0;
    const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6, h = lane >> 5, c32 = lane & 31;
    // Workgroups go round-robin to the 8 XCDs, each with an L2 of its own: the VH workgroups of a (head, chunk), which read
    // the same K, sit 8 apart in the launch order, on one XCD
    int vh, pair;
    if (VH == 2 && (gridDim.x & 15) == 0) { vh = (blockIdx.x >> 3) & 1; pair = (blockIdx.x & 7) | ((blockIdx.x >> 4) << 3); }
    else { vh = blockIdx.x % VH; pair = blockIdx.x / VH; }
    const int cc = pair % a.NCS, bh = pair / a.NCS;
    const int S = a.S, L = a.L, NT = NTT ? NTT : L / GRAN;
    const size_t hoff = (size_t)bh * S, poff = (size_t)bh * a.NG * GRAN, goff = (size_t)bh * a.NG;
    // forward states: sum cc is over chunk cc, relative to its own last position; reverse states (K = Q, V = dH): sum cc
    // is over chunk cc + 1 (the last chunk may be short), relative to the last position of chunk cc
    const int p0 = (a.reverse ? cc + 1 : cc) * L, pe = a.reverse ? p0 - 1 : p0 + L - 1;
    // K and V are the caller's tensors, each in its layout (elements per position rsK / rsV)
    const size_t rsK = (size_t)a.lk.ss, rsV = (size_t)a.lv.ss;
    const T* Kh = reinterpret_cast<const T*>(a.K) + a.lk.head(bh) + (size_t)p0 * rsK;
    const T* Vh = reinterpret_cast<const T*>(a.V) + a.lv.head(bh) + (size_t)p0 * rsV + VW * vh;

    // vector state: a feeder thread's K pieces of a tile are rows pg + NPG it (it < KP) of the eight keys 8 kc .. 8 kc + 7
    const int kc = tid & (D / 8 - 1), pg = tid / (D / 8);
    constexpr int NPG = 256 / (D / 8);

    // The two kinds of waves run code of their own from here on (every value of one kind is dead in the other: the registers
    // of a wave hold either the accumulators or the tiles in flight); both pass the same barriers.
    auto feed = [&]() __attribute__((always_inline)) {
    f32x8 nacc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // Tiles travel memory -> registers -> LDS.  A thread's pieces of a tile: KP 16-byte pieces of K (piece tid + 256 it of
    // the tile's rows of CPR pieces) and four of V (rows tid/16 + 16 it, piece tid%16); tile j uses register set j % 3 and
    // LDS stage j % 2.  Rows past the end of the sequence are clamped (their weights are 0).
    constexpr int KP = GRAN * ZK::CPR / 256, LPT = KP + 4;   // loads per thread and tile
    const int vrow = tid >> 4, vch = tid & 15;
    u32x4 kset[Cfg::RSETS][KP], vset[Cfg::RSETS][4];
    // A thread's pieces lie a fixed number of rows apart (K: 256 / CPR, V: 16): one per-lane element offset each, everything
    // else of an address is the same for all lanes.  Only the last tile of a short last chunk needs its rows clamped.
    constexpr int KROWS = 256 / ZK::CPR;
    const unsigned koff = (unsigned)((tid / ZK::CPR) * rsK + 8 * (tid % ZK::CPR)), voff = (unsigned)(vrow * rsV + 8 * vch);
    auto issue = [&](auto set_tag, int j) __attribute__((always_inline)) {
        constexpr int P = decltype(set_tag)::value;
        if (p0 + GRAN * (j + 1) <= S) {
            const T* kt = Kh + (size_t)GRAN * j * rsK;
            const T* vt = Vh + (size_t)GRAN * j * rsV;
#pragma unroll
            for (int it = 0; it < KP; it++) kset[P][it] = *reinterpret_cast<const u32x4*>(kt + (size_t)(KROWS * it) * rsK + koff);
#pragma unroll
            for (int it = 0; it < 4; it++) vset[P][it] = *reinterpret_cast<const u32x4*>(vt + (size_t)(16 * it) * rsV + voff);
        } else {
#pragma unroll
            for (int it = 0; it < KP; it++) {
                const int pc = tid + 256 * it;
                int pos = GRAN * j + pc / ZK::CPR;
                pos = p0 + pos < S ? pos : S - 1 - p0;
                kset[P][it] = *reinterpret_cast<const u32x4*>(Kh + (size_t)pos * rsK + 8 * (pc % ZK::CPR));
            }
#pragma unroll
            for (int it = 0; it < 4; it++) {
                int pos = GRAN * j + vrow + 16 * it;
                pos = p0 + pos < S ? pos : S - 1 - p0;
                vset[P][it] = *reinterpret_cast<const u32x4*>(Vh + (size_t)pos * rsV + 8 * vch);
            }
        }
        __builtin_amdgcn_sched_barrier(0);   // the loads go out here, not where the scheduler would like them
    };
    // K of tile j as it is, V times the positions' weights, into stage j % 2
    auto commit = [&](auto set_tag, int j) __attribute__((always_inline)) {
        constexpr int P = decltype(set_tag)::value;
        typedef typename R::vec4 V4;
        struct Pair { V4 lo, hi; };
#pragma unroll
        for (int it = 0; it < KP; it++) {
            const int pc = tid + 256 * it;
            *reinterpret_cast<u32x4*>(ks + (j % ST) * Cfg::K_BYTES + ZK::off(pc / ZK::CPR, 8 * (pc % ZK::CPR))) = kset[P][it];
            if (vh == 0) {   // the vector state's share of this piece
                float x[8];
                unpack8<T>(kset[P][it], x);
                const float w2 = sw2[GRAN * j + pc / ZK::CPR];
#pragma unroll
                for (int e = 0; e < 8; e++) nacc[e] += x[e] * w2;
            }
        }
#pragma unroll
        for (int it = 0; it < 4; it++) {
            const int row = vrow + 16 * it;
            const float w = sw[GRAN * j + row];
            float x[8];
            unpack8<T>(vset[P][it], x);
            Pair out;
            if constexpr (STRICT) {   // the weighted row as two terms: what rounding to the element type loses goes to the lo tile
                Pair rest;
                R::cvt4_split(f32x4{x[0] * w, x[1] * w, x[2] * w, x[3] * w}, out.lo, rest.lo);
                R::cvt4_split(f32x4{x[4] * w, x[5] * w, x[6] * w, x[7] * w}, out.hi, rest.hi);
                *reinterpret_cast<Pair*>(vs + (j % ST) * Cfg::V_BYTES + Cfg::V_TILE + ZV::off(row, 8 * vch)) = rest;
            } else {
                out.lo = R::cvt4(f32x4{x[0] * w, x[1] * w, x[2] * w, x[3] * w});
                out.hi = R::cvt4(f32x4{x[4] * w, x[5] * w, x[6] * w, x[7] * w});
            }
            *reinterpret_cast<Pair*>(vs + (j % ST) * Cfg::V_BYTES + ZV::off(row, 8 * vch)) = out;
        }
    };
    // Iteration t, feeders (register set P = t % 3): the loads of tile t + 3 go out into the registers tile t left in the previous
    // iteration; tile t + 1 moves to the LDS stage that tile t - 1 left behind the last barrier.  The others multiply tile t.
    // Two to three tiles are in flight while a tile is worked on.  The loads are ordinary ones, so that the compiler places the counted
    // waits itself; it counts exactly in straight-line code (hence NTT: the default chunk's eight iterations are unrolled)
    // and falls back to waiting for everything across a loop's back edge.  Loads issued by hand -- direct-to-LDS copies of
    // K, or register loads from inline assembly -- gave wrong states now and then at full size as soon as a wait was a
    // counted one: the compiler moves or stashes a register it believes written while the load is still in flight.  With
    // one tile in flight and a wait for everything the kernel waited for memory latency in every iteration.
    auto iteration = [&](auto set_tag, int t) __attribute__((always_inline)) {
        constexpr int P = decltype(set_tag)::value, P1 = (P + 1) % 3;
        if (t + 3 < NT) issue(std::integral_constant<int, P>{}, t + 3);
        if (t + 1 < NT) commit(std::integral_constant<int, P1>{}, t + 1);
        __syncthreads();
    };

    // The positions' weights.  Forward: w_j = exp(a_j - A_e) / sqrt(D) for both sums, e the chunk's last position.
    // Reverse: rho_i = exp(A_e - A_i) / sqrt(D), e the last position BEFORE the chunk, times 1/n_i (matrix sum) or db_i
    // (vector sum), the per-row scalars of the dQ pass.
    const float log2scale = -0.5f * __log2f((float)D);
    if constexpr (NTT > 0) {
        // Their inputs are requested first and used behind the first tile's loads: the waits the compiler places for them
        // then count the tile loads as "behind" and do not wait for those (requested after the tiles, the weights waited
        // for all three tiles: 13 k cycles before the first iteration, measured).  The other two tiles' loads follow one
        // by one, so that the first tile's data is not queued behind theirs.
        {
            constexpr int WPT = NTT * GRAN / 256;   // positions per thread
            float x0[WPT], x1[WPT], x2[WPT];
            double xg[WPT];
            const float bend = a.beta2[poff + pe];
            const double Gend = a.G2[goff + pe / GRAN];
#pragma unroll
            for (int n = 0; n < WPT; n++) {
                int pos = p0 + tid + 256 * n;
                pos = pos < S ? pos : S - 1;
                xg[n] = a.G2[goff + pos / GRAN];
                if (a.reverse) { x0[n] = a.beta2[poff + pos]; x1[n] = a.inv_n[poff + pos]; x2[n] = a.db[poff + pos]; }
                else { x0[n] = a.alpha2[poff + pos]; x1[n] = 0.f; x2[n] = 0.f; }
            }
            __builtin_amdgcn_sched_barrier(0);
            issue(std::integral_constant<int, 0>{}, 0);
#pragma unroll
            for (int n = 0; n < WPT; n++) {
                const int p = tid + 256 * n;
                float w = 0.f, w2 = 0.f;
                if (p0 + p < S) {
                    if (a.reverse) {
                        const float rho = fast_exp2(bend - x0[n] + (float)(xg[n] - Gend) + log2scale);
                        w = rho * x1[n];
                        w2 = rho * x2[n];
                    } else {
                        w = w2 = fast_exp2(x0[n] - bend + (float)(Gend - xg[n]) + log2scale);
                    }
                }
                sw[p] = w;
                sw2[p] = w2;
            }
            __builtin_amdgcn_sched_barrier(0);
            issue(std::integral_constant<int, 1>{}, 1);   // (NT >= 2: a chunk is a multiple of 128 positions)
        }
        __syncthreads();   // the weights are in LDS
        commit(std::integral_constant<int, 0>{}, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (2 < NT) issue(std::integral_constant<int, 2>{}, 2);
        __syncthreads();
    } else {
        {
            issue(std::integral_constant<int, 0>{}, 0);
            issue(std::integral_constant<int, 1>{}, 1);
            if (2 < NT) issue(std::integral_constant<int, 2>{}, 2);
            const float bend = a.beta2[poff + pe];
            const double Gend = a.G2[goff + pe / GRAN];
            for (int p = tid; p < L; p += 256) {
                const int pos = p0 + p;
                float w = 0.f, w2 = 0.f;
                if (pos < S) {
                    if (a.reverse) {
                        const float rho = fast_exp2(bend - a.beta2[poff + pos] + (float)(a.G2[goff + pos / GRAN] - Gend) + log2scale);
                        w = rho * a.inv_n[poff + pos];
                        w2 = rho * a.db[poff + pos];
                    } else {
                        w = w2 = fast_exp2(a.alpha2[poff + pos] - bend + (float)(Gend - a.G2[goff + pos / GRAN]) + log2scale);
                    }
                }
                sw[p] = w;
                sw2[p] = w2;
            }
        }
        __syncthreads();   // the weights are in LDS
        commit(std::integral_constant<int, 0>{}, 0);
        __syncthreads();
    }
    if constexpr (NTT > 0) {
        static_for<NTT>([&](auto tt) __attribute__((always_inline)) { iteration(std::integral_constant<int, decltype(tt)::value % 3>{}, decltype(tt)::value); });
    } else {
        for (int t = 0; t < NT; t += 3) {
            iteration(std::integral_constant<int, 0>{}, t);
            if (t + 1 < NT) iteration(std::integral_constant<int, 1>{}, t + 1);
            if (t + 2 < NT) iteration(std::integral_constant<int, 2>{}, t + 2);
        }
    }
    if (vh == 0) {   // the partial sums (one per group of rows) meet in LDS (the tiles are done with: the last barrier)
        float* red = reinterpret_cast<float*>(smem);   // [NPG][D]
        *reinterpret_cast<f32x8*>(red + pg * D + 8 * kc) = nacc;
        __syncthreads();
        if (tid < D) {
            float sum = 0.f;
#pragma unroll
            for (int g = 0; g < NPG; g++) sum += red[g * D + tid];
            a.Nst[((size_t)bh * a.NCS + cc) * D + tid] = sum;
        }
    }
    };

    auto multiply = [&]() __attribute__((always_inline)) {
    SwzTransReader<T, D> krd;        // per-lane offsets of the transposing reads, computed once
    krd.init(lane, (D / 128) * wave);
    SwzTransReader<T, VW> vrd;
    vrd.init(lane, 0);
    f32x16 acc[MB][NB];
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int x = 0; x < 16; x++) acc[mb][nb][x] = 0.f;
    auto compute = [&](int t) __attribute__((always_inline)) {
        const T* kt = reinterpret_cast<const T*>(ks + (t % ST) * Cfg::K_BYTES);
        const T* vt = reinterpret_cast<const T*>(vs + (t % ST) * Cfg::V_BYTES);
        // the operand reads of a contraction step run one step ahead of its MFMAs (read, wait, multiply in turns left the
        // matrix unit idle for an LDS round trip per step: 3000 cycles per tile for 1024 of MFMAs, measured)
        constexpr int NSTEP = GRAN / KW;
        frag af[2][MB], bf[2][NB], bl[STRICT ? NB : 1];
        const T* vl = reinterpret_cast<const T*>(vs + (t % ST) * Cfg::V_BYTES + Cfg::V_TILE);   // (split mode: the lo tile)
        auto rd = [&](int s) __attribute__((always_inline)) {
#pragma unroll
            for (int mb = 0; mb < MB; mb++) af[s & 1][mb] = krd.read(kt, KW * s, mb);
#pragma unroll
            for (int nb = 0; nb < NB; nb++) bf[s & 1][nb] = vrd.read(vt, KW * s, nb);
        };
        rd(0);
#pragma unroll
        for (int s = 0; s < NSTEP; s++) {
            // (split mode: the lo fragments of this step are single-buffered -- a second set does not fit the registers at
            // D = 256 -- and requested here, behind the MFMAs on the hi fragments)
            if constexpr (STRICT) {
#pragma unroll
                for (int nb = 0; nb < NB; nb++) bl[nb] = vrd.read(vl, KW * s, nb);
            }
            if (s + 1 < NSTEP) rd(s + 1);
#pragma unroll
            for (int mb = 0; mb < MB; mb++)
#pragma unroll
                for (int nb = 0; nb < NB; nb++) R::mma(acc[mb][nb], af[s & 1][mb], bf[s & 1][nb]);
            if constexpr (STRICT) {
#pragma unroll
                for (int mb = 0; mb < MB; mb++)
#pragma unroll
                    for (int nb = 0; nb < NB; nb++) R::mma(acc[mb][nb], af[s & 1][mb], bl[nb]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    __syncthreads();   // (the weights are in LDS)
    __syncthreads();   // (the first tile is)
    if constexpr (NTT > 0) {
        static_for<NTT>([&](auto tt) __attribute__((always_inline)) { compute(decltype(tt)::value); __syncthreads(); });
    } else {
        for (int t = 0; t < NT; t++) { compute(t); __syncthreads(); }
    }
    // accumulator block (mb, nb): column (value) 32 nb + c32, rows (keys) 8 (r / 4) + 4 h + r % 4
    float* out = a.dC + ((size_t)bh * a.NCS + cc) * D * D + VW * vh;
#pragma unroll
    for (int mb = 0; mb < MB; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int k = (D / 4) * wave + 32 * mb + 8 * (r >> 2) + 4 * h + (r & 3);
                out[(size_t)k * D + 32 * nb + c32] = acc[mb][nb][r];
            }
    if (vh == 0) __syncthreads();   // (the feeders' sum of the vector state)
    };

    if (feeder) feed();
    else multiply();
#endif
}

// The chunk sums for the shapes the MFMA kernel above does not serve (fp32 at D = 64 and 128, 16-bit types at D = 64): the
// same sums as plain fp32 multiply-adds out of LDS tiles of 64 positions.  One workgroup per (head, chunk, 64 value
// columns); a thread holds D/16 keys x 4 values.  These shapes are small (the sums are 2 S D^2 flops per head).
template <typename T, int D>
__global__ __launch_bounds__(256) void chunk_sum_small_kernel(ChunkArgs a) {
    constexpr int VW = 64, VH = D / VW, KPT = D / 16;
    __shared__ __attribute__((aligned(16))) float ks[GRAN][D + 4];
    __shared__ __attribute__((aligned(16))) float vs[GRAN][VW + 4];
    __shared__ float sw2[GRAN];
    const int tid = threadIdx.x;
    const int vh = blockIdx.x % VH, pair = blockIdx.x / VH;
    const int cc = pair % a.NCS, bh = pair / a.NCS;
    const int S = a.S, L = a.L;
    const size_t poff = (size_t)bh * a.NG * GRAN, goff = (size_t)bh * a.NG;
    // (the positions and the reference point of a sum: see chunk_sum_kernel)
    const int p0 = (a.reverse ? cc + 1 : cc) * L, pe = a.reverse ? p0 - 1 : p0 + L - 1;
    const size_t rsK = (size_t)a.lk.ss, rsV = (size_t)a.lv.ss;
    const T* Kh = reinterpret_cast<const T*>(a.K) + a.lk.head(bh);
    const T* Vh = reinterpret_cast<const T*>(a.V) + a.lv.head(bh) + VW * vh;
    const float log2scale = -0.5f * __log2f((float)D);
    const float bend = a.beta2[poff + pe];
    const double Gend = a.G2[goff + pe / GRAN];
    const int k0 = KPT * (tid >> 4), v0 = 4 * (tid & 15);
    float acc[KPT][4];
#pragma unroll
    for (int x = 0; x < KPT; x++)
#pragma unroll
        for (int y = 0; y < 4; y++) acc[x][y] = 0.f;
    float nacc = 0.f;
    const int n_pos = (p0 + L <= S ? L : S - p0);
    for (int t0 = 0; t0 < n_pos; t0 += GRAN) {
        __syncthreads();   // (the previous tile has been used)
        // position tid / 4 of the tile, a quarter of its row each: K as it is, V times the position's weight
        {
            const int j = tid >> 2, part = tid & 3;
            const int pos = p0 + t0 + j, pc = pos < S ? pos : S - 1;
            float w = 0.f, w2 = 0.f;
            if (pos < S) {
                if (a.reverse) {
                    const float rho = fast_exp2(bend - a.beta2[poff + pos] + (float)(a.G2[goff + pos / GRAN] - Gend) + log2scale);
                    w = rho * a.inv_n[poff + pos];
                    w2 = rho * a.db[poff + pos];
                } else {
                    w = w2 = fast_exp2(a.alpha2[poff + pos] - bend + (float)(Gend - a.G2[goff + pos / GRAN]) + log2scale);
                }
            }
            if (part == 0) sw2[j] = w2;
            const T* kr = Kh + (size_t)pc * rsK + (D / 4) * part;
            const T* vr = Vh + (size_t)pc * rsV + (VW / 4) * part;
#pragma unroll
            for (int e = 0; e < D / 4; e++) ks[j][(D / 4) * part + e] = (float)kr[e];
#pragma unroll
            for (int e = 0; e < VW / 4; e++) vs[j][(VW / 4) * part + e] = (float)vr[e] * w;
        }
        __syncthreads();
#pragma unroll 4
        for (int j = 0; j < GRAN; j++) {
            const f32x4 vv = *reinterpret_cast<const f32x4*>(&vs[j][v0]);
            float kk[KPT];
#pragma unroll
            for (int x = 0; x < KPT; x += 4) {
                const f32x4 q4 = *reinterpret_cast<const f32x4*>(&ks[j][k0 + x]);
                kk[x] = q4[0]; kk[x + 1] = q4[1]; kk[x + 2] = q4[2]; kk[x + 3] = q4[3];
            }
#pragma unroll
            for (int x = 0; x < KPT; x++)
#pragma unroll
                for (int y = 0; y < 4; y++) acc[x][y] += kk[x] * vv[y];
        }
        if (vh == 0 && tid < D) {
#pragma unroll 8
            for (int j = 0; j < GRAN; j++) nacc += ks[j][tid] * sw2[j];
        }
    }
    float* out = a.dC + ((size_t)bh * a.NCS + cc) * D * D + VW * vh;
#pragma unroll
    for (int x = 0; x < KPT; x++)
        *reinterpret_cast<f32x4*>(out + (size_t)(k0 + x) * D + v0) = f32x4{acc[x][0], acc[x][1], acc[x][2], acc[x][3]};
    if (vh == 0 && tid < D) a.Nst[((size_t)bh * a.NCS + cc) * D + tid] = nacc;
}

// gamma_c = exp(A_{e_{c-1}} - A_{e_c}), e_c the last position of chunk c (c >= 1, both chunks complete): what the state
// at the end of chunk c - 1 decays by until the end of chunk c, and what the reverse state behind chunk c decays by
// until it is seen from the end of chunk c - 1
__device__ __forceinline__ float carry_gamma(const ChunkArgs& a, size_t poff, size_t goff, int c) {
    const int e0 = c * a.L - 1, e1 = e0 + a.L;
    return fast_exp2(a.beta2[poff + e0] - a.beta2[poff + e1] + (float)(a.G2[goff + e1 / GRAN] - a.G2[goff + e0 / GRAN]));
}

template <typename T, int D>
__global__ __launch_bounds__(256) void chunk_carry_kernel(ChunkArgs a) {
    const int bh = blockIdx.y, tid = threadIdx.x;
    const int idx = blockIdx.x * 256 + tid;
    const int k = idx / (D / 8), v8 = (idx % (D / 8)) * 8;
    const size_t poff = (size_t)bh * a.NG * GRAN, goff = (size_t)bh * a.NG;
    const int L = a.L;
    const size_t hbase = (size_t)bh * a.NCS * D * D;
    const float* src = a.dC + hbase + (size_t)k * D + v8;
    const size_t koff = hbase + (size_t)state_row<T>(k) * D + v8;   // key-major: eight values of key k
    float* nst = a.Nst + (size_t)bh * a.NCS * D + tid;
    const bool vec = blockIdx.x == 0 && tid < D;
    f32x4 run0 = {0.f, 0.f, 0.f, 0.f}, run1 = {0.f, 0.f, 0.f, 0.f};
    float nrun = 0.f;
    typedef typename Tr<T>::vec4 V4;
    struct Pair { V4 lo, hi; };
    // The steps depend on each other through the running state only: the chunk sums, the decay factors and the vector
    // sums of four steps are requested together (one memory round trip per four steps; with few heads this kernel is a
    // handful of workgroups waiting for memory, step by step)
    constexpr int AHEAD = 4;
    for (int step0 = 0; step0 < a.NCS; step0 += AHEAD) {
      f32x4 d0s[AHEAD], d1s[AHEAD];
      float gams[AHEAD], nin[AHEAD];
#pragma unroll
      for (int u = 0; u < AHEAD; u++) {
          const int step = step0 + u < a.NCS ? step0 + u : a.NCS - 1;
          const int c = a.reverse ? a.NCS - 1 - step : step;
          gams[u] = step > 0 ? carry_gamma(a, poff, goff, a.reverse ? c + 1 : c) : 0.f;
          d0s[u] = *reinterpret_cast<const f32x4*>(src + (size_t)c * D * D);
          d1s[u] = *reinterpret_cast<const f32x4*>(src + (size_t)c * D * D + 4);
          nin[u] = vec ? nst[(size_t)c * D] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < AHEAD; u++) {
        const int step = step0 + u;
        if (step >= a.NCS) break;
        const int c = a.reverse ? a.NCS - 1 - step : step;
        const float gam = gams[u];
        run0 = run0 * gam + d0s[u];
        run1 = run1 * gam + d1s[u];
#pragma unroll
        for (int e = 0; e < 4; e++) {   // (see chunk_carry_t_kernel: the fp32 value is fixed before any conversion)
            asm volatile("" : "+v"(run0[e]));
            asm volatile("" : "+v"(run1[e]));
        }
        Pair o, rest;
        const bool split = a.Cst_lo || a.CstT_lo;   // split mode: the state as two terms
        if (split) {
            Tr<T>::cvt4_split(run0, o.lo, rest.lo);
            Tr<T>::cvt4_split(run1, o.hi, rest.hi);
        } else {
            o.lo = Tr<T>::cvt4(run0);
            o.hi = Tr<T>::cvt4(run1);
        }
        if (a.Cst) {
            *reinterpret_cast<Pair*>(reinterpret_cast<T*>(a.Cst) + koff + (size_t)c * D * D) = o;
            if (a.Cst_lo) *reinterpret_cast<Pair*>(reinterpret_cast<T*>(a.Cst_lo) + koff + (size_t)c * D * D) = rest;
        }
        if (a.CstT) {
            // value-major copy, element by element (the small shapes only: at D = 128 and 256 in 16 bits
            // chunk_carry_t_kernel turns the blocks round in LDS)
            T* t = reinterpret_cast<T*>(a.CstT) + hbase + (size_t)c * D * D + k;
            T* tl = a.CstT_lo ? reinterpret_cast<T*>(a.CstT_lo) + hbase + (size_t)c * D * D + k : nullptr;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const size_t r = (size_t)state_row<T>(v8 + e) * D;
                t[r] = e < 4 ? o.lo[e & 3] : o.hi[e & 3];
                if (tl) tl[r] = e < 4 ? rest.lo[e & 3] : rest.hi[e & 3];
            }
        }
        if (vec) {
            nrun = nrun * gam + nin[u];
            nst[(size_t)c * D] = nrun;
        }
      }
    }
}

// The same carry with the states written transposed, [value][key], for the dQ pass (which contracts the state over the
// value index): a workgroup takes 64 values x 64 keys, reads the chunk sums along the value index (coalesced), and
// turns the block round in LDS so that the rows leave 128 bytes at a time.  Rows in the contraction order of the row
// kernel, like the untransposed states.
template <typename T, int D, bool DOT, bool KM>
__global__ __launch_bounds__(256, 4) void chunk_carry_t_kernel(ChunkArgs a) {
    __shared__ __attribute__((aligned(16))) T tile[2][64][64 + 8];   // [hi | lo (split mode)]
    const int bh = blockIdx.y, tid = threadIdx.x;
    const bool split = a.CstT_lo != nullptr;
    const int vb = blockIdx.x % (D / 64), kb = blockIdx.x / (D / 64);
    const int vl = tid & 63, kq = tid >> 6;
    const size_t poff = (size_t)bh * a.NG * GRAN, goff = (size_t)bh * a.NG;
    const int L = a.L;
    const int orow = tid >> 2, opiece = tid & 3;
    const int vrow = 64 * vb + orow;
    T* dst = reinterpret_cast<T*>(a.CstT) + (size_t)bh * a.NCS * D * D + (size_t)((vrow & ~15) | perm16(vrow & 15)) * D + 64 * kb + 16 * opiece;
    f32x8 run[2];
#pragma unroll
    for (int g = 0; g < 2; g++)
#pragma unroll
        for (int e = 0; e < 8; e++) run[g][e] = 0.f;
    float* nst = a.Nst + (size_t)bh * a.NCS * D + tid;   // the vector states, in place, by the first workgroup of a head
    const bool vec = blockIdx.x == 0 && tid < D;
    float nrun = 0.f;
    __shared__ float red[4];
    const int lane = tid & 63, wave = tid >> 6;
    // (the kernel moves 4 bytes in and 2 to 4 out per element and runs at memory speed: nothing to gain from requesting a
    // step's chunk sums ahead of time)
    for (int step = 0; step < a.NCS; step++) {
        const int c = a.reverse ? a.NCS - 1 - step : step;
        const float gam = step > 0 ? carry_gamma(a, poff, goff, a.reverse ? c + 1 : c) : 0.f;
        if (vec) {
            nrun = nrun * gam + nst[(size_t)c * D];
            nst[(size_t)c * D] = nrun;
        }
        const float* src = a.dC + ((size_t)bh * a.NCS + c) * D * D + 64 * vb + vl;
        typedef typename Tr<T>::frag V8;
#pragma unroll
        for (int g = 0; g < 2; g++) {
            f32x8 d;
#pragma unroll
            for (int e = 0; e < 8; e++) d[e] = src[(size_t)(64 * kb + 8 * (kq + 4 * g) + e) * D];
            run[g] = run[g] * gam + d;
            // (the fp32 value is fixed here: left to itself the compiler may fold this multiply-add into a conversion to
            // fp16 further down -- one rounding instead of two -- in one kernel and not in its twin, and the two carries
            // must give the same bits)
#pragma unroll
            for (int e = 0; e < 8; e++) asm volatile("" : "+v"(run[g][e]));
            if constexpr (KM) {   // key-major copy: lanes of a wave hold consecutive values of one key, 128 bytes per store
                const size_t koff = ((size_t)bh * a.NCS + c) * D * D + 64 * vb + vl;
                T* kd = reinterpret_cast<T*>(a.Cst) + koff;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int k = 64 * kb + 8 * (kq + 4 * g) + e;
                    const T hi = (T)run[g][e];
                    kd[(size_t)((k & ~15) | perm16(k & 15)) * D] = hi;
                    if (a.Cst_lo) (reinterpret_cast<T*>(a.Cst_lo) + koff)[(size_t)((k & ~15) | perm16(k & 15)) * D] = (T)(run[g][e] - (float)hi);
                }
            }
            typedef typename Tr<T>::vec4 V4;
            struct Pair { V4 lo, hi; };
            Pair o;
            if (split) {   // the state as two terms: the second holds what rounding to the element type loses
                Pair rest;
                Tr<T>::cvt4_split(__builtin_shufflevector(run[g], run[g], 0, 1, 2, 3), o.lo, rest.lo);
                Tr<T>::cvt4_split(__builtin_shufflevector(run[g], run[g], 4, 5, 6, 7), o.hi, rest.hi);
                *reinterpret_cast<Pair*>(&tile[1][vl][8 * (kq + 4 * g)]) = rest;
            } else {
                o.lo = Tr<T>::cvt4(__builtin_shufflevector(run[g], run[g], 0, 1, 2, 3));
                o.hi = Tr<T>::cvt4(__builtin_shufflevector(run[g], run[g], 4, 5, 6, 7));
            }
            *reinterpret_cast<Pair*>(&tile[0][vl][8 * (kq + 4 * g)]) = o;
        }
        __syncthreads();
        const uint4 p0 = *reinterpret_cast<const uint4*>(&tile[0][orow][16 * opiece]), p1 = *reinterpret_cast<const uint4*>(&tile[0][orow][16 * opiece + 8]);
        *reinterpret_cast<uint4*>(dst + (size_t)c * D * D) = p0;
        *reinterpret_cast<uint4*>(dst + (size_t)c * D * D + 8) = p1;
        if constexpr (DOT) {   // <state c as it is written (the sum of its terms in split mode), the other set's state c>
            f32x8 x0 = __builtin_convertvector(__builtin_bit_cast(V8, p0), f32x8), x1 = __builtin_convertvector(__builtin_bit_cast(V8, p1), f32x8);
            // the other set's state c at the places this thread has just written (four workgroups share a CU: their
            // steps hide this round trip)
            const size_t doff = (size_t)(dst - reinterpret_cast<T*>(a.CstT)) + (size_t)c * D * D;
            const T* other = reinterpret_cast<const T*>(a.dot_with) + doff;
            f32x8 y0 = __builtin_convertvector(*reinterpret_cast<const V8*>(other), f32x8);
            f32x8 y1 = __builtin_convertvector(*reinterpret_cast<const V8*>(other + 8), f32x8);
            if (split) {
                x0 += __builtin_convertvector(*reinterpret_cast<const V8*>(&tile[1][orow][16 * opiece]), f32x8);
                x1 += __builtin_convertvector(*reinterpret_cast<const V8*>(&tile[1][orow][16 * opiece + 8]), f32x8);
            }
            if (a.dot_with_lo) {
                const T* other_lo = reinterpret_cast<const T*>(a.dot_with_lo) + doff;
                y0 += __builtin_convertvector(*reinterpret_cast<const V8*>(other_lo), f32x8);
                y1 += __builtin_convertvector(*reinterpret_cast<const V8*>(other_lo + 8), f32x8);
            }
            const f32x8 pr = x0 * y0 + x1 * y1;
            float dot = ((pr[0] + pr[1]) + (pr[2] + pr[3])) + ((pr[4] + pr[5]) + (pr[6] + pr[7]));
            dot = wave_scan_inclusive<OpAdd>(dot);
            if (lane == 63) red[wave] = dot;
        }
        if (split) {
            T* dlo = reinterpret_cast<T*>(a.CstT_lo) + (dst - reinterpret_cast<T*>(a.CstT));
            *reinterpret_cast<uint4*>(dlo + (size_t)c * D * D) = *reinterpret_cast<const uint4*>(&tile[1][orow][16 * opiece]);
            *reinterpret_cast<uint4*>(dlo + (size_t)c * D * D + 8) = *reinterpret_cast<const uint4*>(&tile[1][orow][16 * opiece + 8]);
        }
        __syncthreads();
        if (DOT && tid == 0)   // (the waves' sums were written between the two barriers; the next ones follow the next barrier)
            a.dot_part[((size_t)bh * a.NCS + c) * gridDim.x + blockIdx.x] = (red[0] + red[1]) + (red[2] + red[3]);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// The same states in ONE pass: a workgroup owns a 64 x D/2 block of a head's state (64 keys x D/2 values) and walks the
// head's chunks in their order (forward: first to last; reverse: last to first), the running state in its accumulators:
// at a chunk's end the block is written in the element type (either layout, the accumulator's own rounding being the
// only one), decays by gamma, and takes the next chunk's products.  No fp32 chunk sums travel through memory (4 + 4
// bytes per state element in the two-kernel form above), no second launch.  (D/64) * 2 workgroups per head: for
// launches with enough heads to fill the chip (launch_chunk_states decides); not in split mode.
//
// Eight waves.  Waves 4..7 bring the tiles (64 positions: K's 64 columns, V's D/2 columns, and the positions' gate
// rows) by direct global->LDS copies, PF tiles ahead, into NS = PF + 1 stages; one tile ahead of the product they
// leave the positions' weights in LDS and add up the vector state from K.  Waves 0..3 multiply straight out of the
// stages -- the weights go onto the K^T fragments in registers, eight products per fragment (a weighted copy of a
// tile in LDS costs every wave a chain of LDS round trips per tile, and those chains, not the copies or the MFMAs, set
// the pace: measured) -- write the states and own every global store.  One barrier per tile.  The copies are counted
// by hand: a feeder wave issues exactly NI direct loads per tile and no other vector memory operation after the
// prologue, and waits with vmcnt((PF - 2) * NI) -- everything but the newest PF - 2 tiles -- before the barrier that
// hands a tile on; the launch is refused if the compiled kernel uses scratch memory.
template <typename T, int D>
struct SeqCfg {
    static constexpr int KR = 64, VW = D / 2;
    static constexpr int VP = GRAN * VW * (int)sizeof(T) / 16 / 256;   // direct loads of V per feeder wave and tile
    static constexpr int NI = 2 + VP + 1;                              // direct loads per feeder wave and tile: K, V, one gate row
    static constexpr int MAX_STEPS = 256;                              // chunk states per head
    static constexpr size_t K_BYTES = (size_t)GRAN * KR * sizeof(T), V_BYTES = (size_t)GRAN * VW * sizeof(T), AUX_BYTES = 4 * GRAN * sizeof(float);
    static constexpr size_t STAGE_BYTES = K_BYTES + V_BYTES + AUX_BYTES;
    static constexpr size_t TABLE_BYTES = MAX_STEPS * (sizeof(double) + 2 * sizeof(float));
    static constexpr size_t RED_BYTES = 32 * KR * sizeof(float) + 64;
    static constexpr size_t SW_BYTES = 8 * GRAN * sizeof(float);
    // tiles requested ahead: as many stages as LDS holds
    static constexpr int NS = (int)((160 * 1024 - TABLE_BYTES - RED_BYTES - SW_BYTES) / STAGE_BYTES) < 8
                                  ? (int)((160 * 1024 - TABLE_BYTES - RED_BYTES - SW_BYTES) / STAGE_BYTES) : 8;
    static constexpr int PF = NS - 1;
    static_assert(PF >= 3 && (PF - 1) * NI < 64, "the counted wait must fit vmcnt's six bits");
    static constexpr size_t LDS_BYTES = NS * STAGE_BYTES + SW_BYTES + TABLE_BYTES + RED_BYTES;
    static constexpr int WPH = (D / KR) * 2;                           // workgroups per head
};

// cycle stamps of the one-pass kernel's two kinds of waves (a measurement build only: -DMLSTM_SEQ_PROF; the sums go to
// the unused chunk-sum scratch, 16 floats per workgroup)
#if defined(MLSTM_SEQ_PROF)
#define SQ_DECL float prof_[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}; long long last_ = (long long)__builtin_amdgcn_s_memtime()
#define SQ_STAMP(k) do { const long long now_ = (long long)__builtin_amdgcn_s_memtime(); prof_[k] += (float)(now_ - last_); last_ = now_; } while (0)
#define SQ_DUMP(kind) do { if ((threadIdx.x & 255) == 0) for (int z_ = 0; z_ < 8; z_++) a.dC[(size_t)blockIdx.x * 16 + 8 * (kind) + z_] = prof_[z_]; } while (0)
#else
#define SQ_DECL do {} while (0)
#define SQ_STAMP(k) do {} while (0)
#define SQ_DUMP(kind) do {} while (0)
#endif

template <int N> __device__ __forceinline__ void dma_wait_all_but() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }

template <typename T, int D, bool DOT>
__global__ __launch_bounds__(512) void chunk_seq_kernel(ChunkArgs a) {
#if defined(__HIP_DEVICE_COMPILE__)
    using R = Tr<T>;
    using Cfg = SeqCfg<T, D>;
    typedef typename R::frag frag;
    static_assert(R::HALF && (D == 128 || D == 256), "16-bit types, D = 128 or 256");
    constexpr int VW = Cfg::VW, NB = VW / 64, KW = R::KW, NS = Cfg::NS, PF = Cfg::PF, NI = Cfg::NI, VP = Cfg::VP;
    using ZK = Swz<T, 64>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    float* const sw = reinterpret_cast<float*>(smem + NS * Cfg::STAGE_BYTES);   // [4][2][64]: the weights of two tiles, a copy per multiplying wave
    double* const tGend = reinterpret_cast<double*>(sw + 8 * GRAN);
    float* const tbend = reinterpret_cast<float*>(tGend + Cfg::MAX_STEPS);
    float* const tgam = tbend + Cfg::MAX_STEPS;
    float* const red = tgam + Cfg::MAX_STEPS;     // [32][64]: the feeders' partial vector sums of a chunk
    float* const dotred = red + 32 * 64;          // [4]
    auto stage_k = [&](int st) { return reinterpret_cast<T*>(smem + st * Cfg::STAGE_BYTES); };
    auto stage_v = [&](int st) { return reinterpret_cast<T*>(smem + st * Cfg::STAGE_BYTES + Cfg::K_BYTES); };
    auto stage_aux = [&](int st) { return reinterpret_cast<float*>(smem + st * Cfg::STAGE_BYTES + Cfg::K_BYTES + Cfg::V_BYTES); };

    const bool feeder = __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 8) != 0;
    const int tid = threadIdx.x & 255, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), h = lane >> 5, c32 = lane & 31;
    // the workgroups of a head on one XCD (they read the same K and V columns), heads dealt round the eight XCDs
    int w, bh;
    if ((a.BH & 7) == 0) { const int q = blockIdx.x >> 3; w = q % Cfg::WPH; bh = (blockIdx.x & 7) + 8 * (q / Cfg::WPH); }
    else { w = blockIdx.x % Cfg::WPH; bh = blockIdx.x / Cfg::WPH; }
    const int kq = w >> 1, vh = w & 1;
    const int S = a.S, L = a.L, NT = L / GRAN, NCS = a.NCS;
    const size_t poff = (size_t)bh * a.NG * GRAN, goff = (size_t)bh * a.NG;
    const bool rev = a.reverse != 0;
    // step s of the walk: forward chunk s (state s); reverse the positions of chunk NCS - s (state NCS - 1 - s), of which
    // the first, the sequence's last chunk, may be short
    const int NT0 = rev ? (S - NCS * L + GRAN - 1) / GRAN : NT;
    const int NTOT = NT0 + (NCS - 1) * NT;
    auto step_base = [&](int s) { return rev ? (NCS - s) * L : s * L; };
    auto step_tiles = [&](int s) { return s == 0 ? NT0 : NT; };
    struct Cur {   // a tile of the walk
        int s, tt;
    };
    auto advance = [&](Cur& c) { if (++c.tt == step_tiles(c.s)) { c.tt = 0; c.s++; } };

    // per-step tables, by everybody: reference exponent of the step's weights and the decay between steps
    for (int s = threadIdx.x; s < NCS; s += 512) {
        const int c = rev ? NCS - 1 - s : s;
        const int pe = (c + 1) * L - 1;   // forward: the chunk's last position; reverse: the last position before the chunk
        tbend[s] = a.beta2[poff + pe];
        tGend[s] = a.G2[goff + pe / GRAN];
        tgam[s] = s > 0 ? carry_gamma(a, poff, goff, rev ? c + 1 : c) : 0.f;
    }
    const float log2scale = -0.5f * __log2f((float)D);
    const size_t rsK = (size_t)a.lk.ss, rsV = (size_t)a.lv.ss;
    const T* Kh = reinterpret_cast<const T*>(a.K) + a.lk.head(bh) + 64 * kq;
    const T* Vh = reinterpret_cast<const T*>(a.V) + a.lv.head(bh) + VW * vh;
    dma_wait();        // (the last plain loads of the feeder waves: from here on their vmcnt counts direct loads only)
    __syncthreads();

    if (feeder) {
        TileDma<T, 64, GRAN, 256> kdma;
        TileDma<T, VW, GRAN, 256> vdma;
        kdma.init(tid);
        vdma.init(tid);
        const auto krows = kdma.rows(tid, (unsigned)(rsK * sizeof(T)));
        const auto vrows = vdma.rows(tid, (unsigned)(rsV * sizeof(T)));
        static_assert(TileDma<T, 64, GRAN, 256>::PER_WAVE == 2 && TileDma<T, VW, GRAN, 256>::PER_WAVE == VP, "direct loads per tile");
        // gate rows of a tile: wave 0 alpha (forward) or beta (reverse), waves 1 and 2 the dQ pass's 1/n and db (reverse; the
        // forward repeats alpha), wave 3 the granule's G (two dwords; the other lanes read them again)
        const float* auxsrc;
        if (wave == 3) auxsrc = reinterpret_cast<const float*>(a.G2 + goff) + (lane & 1);
        else if (!rev || wave == 0) auxsrc = (rev ? a.beta2 : a.alpha2) + poff + lane;
        else auxsrc = (wave == 1 ? a.inv_n : a.db) + poff + lane;
        const int auxstep = wave == 3 ? 2 : GRAN;   // floats per tile
        auto issue = [&](const Cur& c, int st) __attribute__((always_inline)) {
            const int pos0 = step_base(c.s) + GRAN * c.tt;
            if (pos0 + GRAN <= S) {
                kdma.issue(stage_k(st), Kh + (size_t)pos0 * rsK, krows);
                vdma.issue(stage_v(st), Vh + (size_t)pos0 * rsV, vrows);
            } else {   // the sequence's last tile: rows past the end are clamped (their weights are 0)
                tile_dma<T, 64, GRAN, 256>(stage_k(st), Kh, pos0, S, tid, rsK);
                tile_dma<T, VW, GRAN, 256>(stage_v(st), Vh, pos0, S, tid, rsV);
            }
            dma4(auxsrc + (size_t)(pos0 / GRAN) * auxstep, __builtin_amdgcn_readfirstlane(lds_offset_of(stage_aux(st))) + wave * 256);
        };
        // Tile c (landed in stage st, published by a barrier): the vector sum from K, two 16-byte pieces per thread (rows
        // tid / 8 and tid / 8 + 32), in the workgroups that own it
        f32x8 nacc = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        const int prow = tid / ZK::CPR, pch = tid % ZK::CPR;
        auto prepare = [&](const Cur& c, int st) __attribute__((always_inline)) {
            if (vh != 0) return;
            const float* ax = stage_aux(st);
            const int pos0 = step_base(c.s) + GRAN * c.tt;
            const float bend = tbend[c.s];
            const float dG = (float)(rev ? *reinterpret_cast<const double*>(ax + 3 * GRAN) - tGend[c.s]
                                         : tGend[c.s] - *reinterpret_cast<const double*>(ax + 3 * GRAN));
            u32x4 raw[2];
            if (vh == 0) {
#pragma unroll
                for (int it = 0; it < 2; it++) raw[it] = *reinterpret_cast<const u32x4*>(reinterpret_cast<const char*>(stage_k(st)) + ZK::off(prow + 32 * it, 8 * pch));
            }
#pragma unroll
            for (int it = 0; it < 2; it++) {
                const int row = prow + 32 * it;
                const float e = rev ? bend - ax[row] : ax[row] - bend;
                float rho = fast_exp2(e + dG + log2scale);
                if (pos0 + row >= S) rho = 0.f;
                const float w2 = rev ? rho * ax[2 * GRAN + row] : rho;
                {
                    float x[8];
                    unpack8<T>(raw[it], x);
#pragma unroll
                    for (int e8 = 0; e8 < 8; e8++) nacc[e8] += x[e8] * w2;
                }
            }
            if (vh == 0 && c.tt == step_tiles(c.s) - 1) {   // the step's last tile: the partial sums go to the multiplying waves
                *reinterpret_cast<f32x8*>(red + prow * 64 + 8 * pch) = nacc;
#pragma unroll
                for (int e8 = 0; e8 < 8; e8++) nacc[e8] = 0.f;
            }
        };
        Cur ci{0, 0}, ct{0, 0};   // the next tile to request, the next one to prepare
#pragma unroll
        for (int p = 0; p < PF; p++)
            if (p < NTOT) { issue(ci, p % NS); advance(ci); }
        if (NTOT >= PF) dma_wait_all_but<(PF - 1) * NI>(); else dma_wait();
        __syncthreads();   // tile 0 has landed
        prepare(ct, 0);
        advance(ct);
        if (NTOT >= PF) dma_wait_all_but<(PF - 2) * NI>(); else dma_wait();
        __syncthreads();   // tile 1 has landed
        SQ_DECL;
        for (int t = 0; t < NTOT; t++) {
            if (t + PF < NTOT) { issue(ci, (t + PF) % NS); advance(ci); }
            SQ_STAMP(0);
            if (t + 1 < NTOT) { prepare(ct, (t + 1) % NS); advance(ct); }
            SQ_STAMP(1);
            if (t + PF < NTOT) dma_wait_all_but<(PF - 2) * NI>(); else dma_wait();
            SQ_STAMP(2);
            __syncthreads();
            SQ_STAMP(3);
        }
        SQ_DUMP(0);
    } else {
        const int wk = wave & 1, wv = wave >> 1;
        f32x16 acc[NB];
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
            for (int x = 0; x < 16; x++) acc[nb][x] = 0.f;
        float nrun = 0.f;
        Cur cm{0, 0};
        __syncthreads();
        __syncthreads();
        int pending_dot = -1;   // state whose contraction's parts lie in dotred
        // per-lane byte offsets of the transposing reads (see swz_frag_transposed), contraction step s4 = 0: K block wk and
        // V blocks NB wv + nb; a step further lies 16 tile rows on (the swizzle key has a period of 16 rows)
        const int tj = lane & 15, tsub = (lane >> 4) & 1;
        int koff[2], voff[NB][2];
#pragma unroll
        for (int hi = 0; hi < 2; hi++) {
            koff[hi] = ZK::off(4 * h + (tj >> 2) + 8 * hi, 32 * wk + 16 * tsub + 4 * (tj & 3));
#pragma unroll
            for (int nb = 0; nb < NB; nb++) voff[nb][hi] = Swz<T, VW>::off(4 * h + (tj >> 2) + 8 * hi, 32 * (NB * wv + nb) + 16 * tsub + 4 * (tj & 3));
        }
        auto read_tr = [&](const T* tile, const int (&off)[2], int row_bytes, int s4) __attribute__((always_inline)) {
            const char* base = reinterpret_cast<const char*>(tile) + KW * s4 * row_bytes;
            s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(base + off[0]));
            s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(base + off[1]));
            return __builtin_bit_cast(frag, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
        };
        float* const wt = sw + wave * 2 * GRAN;   // this wave's copies of two tiles' weights
        // the weight of position `lane` of tile c (in stage st) into the wave's copy wb: written and read in program order
        auto weigh = [&](const Cur& c, int st, int wb) __attribute__((always_inline)) {
            const float* ax = stage_aux(st);
            const int pos0 = step_base(c.s) + GRAN * c.tt;
            const float dG = (float)(rev ? *reinterpret_cast<const double*>(ax + 3 * GRAN) - tGend[c.s]
                                         : tGend[c.s] - *reinterpret_cast<const double*>(ax + 3 * GRAN));
            const float e = rev ? tbend[c.s] - ax[lane] : ax[lane] - tbend[c.s];
            float rho = fast_exp2(e + dG + log2scale);
            if (pos0 + lane >= S) rho = 0.f;
            wt[wb * GRAN + lane] = rev ? rho * ax[GRAN + lane] : rho;
        };
        constexpr int NSTEP = GRAN / KW;
        frag af[2], bf[2][NB];
        f32x4 w0[2], w1[2];
        // fragment s4 of K^T holds, for the lane's key, positions 16 s4 + 4 h + (0..3) and 16 s4 + 8 + 4 h + (0..3)
        auto rd = [&](int tile, int s4) __attribute__((always_inline)) {
            const T* kt = stage_k(tile % NS);
            const T* vt = stage_v(tile % NS);
            const float* wv4 = wt + (tile & 1) * GRAN + KW * s4;
            af[s4 & 1] = read_tr(kt, koff, ZK::ROW_BYTES, s4);
            w0[s4 & 1] = *reinterpret_cast<const f32x4*>(wv4 + 4 * h);
            w1[s4 & 1] = *reinterpret_cast<const f32x4*>(wv4 + 8 + 4 * h);
#pragma unroll
            for (int nb = 0; nb < NB; nb++) bf[s4 & 1][nb] = read_tr(vt, voff[nb], Swz<T, VW>::ROW_BYTES, s4);
        };
        // The reads of a tile's first step, and its weights, are requested during the tile before it (both tiles are
        // published by then): a tile's product is a chain of LDS round trips, and with one barrier per tile nothing else
        // would cover them.
        Cur cn{0, 0};   // the tile whose weights are formed next
        weigh(cn, 0, 0);
        advance(cn);
        rd(0, 0);
        SQ_DECL;
        for (int t = 0; t < NTOT; t++) {
            if (t + 1 < NTOT) { weigh(cn, (t + 1) % NS, (t + 1) & 1); advance(cn); }
            if (DOT && pending_dot >= 0 && tid == 0) {
                a.dot_part[((size_t)bh * NCS + pending_dot) * Cfg::WPH + w] = (dotred[0] + dotred[1]) + (dotred[2] + dotred[3]);
            }
            pending_dot = -1;
#pragma unroll
            for (int s4 = 0; s4 < NSTEP; s4++) {
                if (s4 + 1 < NSTEP) rd(t, s4 + 1);
                else if (t + 1 < NTOT) rd(t + 1, 0);
                float x[8];
                unpack8<T>(__builtin_bit_cast(u32x4, af[s4 & 1]), x);
                const f32x4 lo = f32x4{x[0], x[1], x[2], x[3]} * w0[s4 & 1], hi = f32x4{x[4], x[5], x[6], x[7]} * w1[s4 & 1];
                typedef typename R::vec4 V4;
                struct Pair { V4 lo, hi; } wa{R::cvt4(lo), R::cvt4(hi)};
                const frag aw = __builtin_bit_cast(frag, wa);
#pragma unroll
                for (int nb = 0; nb < NB; nb++) R::mma(acc[nb], aw, bf[s4 & 1][nb]);
            }
            SQ_STAMP(0);
            if (cm.tt == step_tiles(cm.s) - 1) {   // the step's last tile: state c leaves, the running state decays
                const int c = rev ? NCS - 1 - cm.s : cm.s;
                const size_t sbase = ((size_t)bh * NCS + c) * D * D;
                float dot = 0.f;
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    const int vg = VW * vh + 32 * (NB * wv + nb) + c32;
                    const size_t vrow_off = sbase + (size_t)state_row<T>(vg) * D;
#pragma unroll
                    for (int g4 = 0; g4 < 4; g4++) {
                        const int kg = 64 * kq + 32 * wk + 8 * g4 + 4 * h;
                        const typename R::vec4 hi = R::cvt4(f32x4{acc[nb][4 * g4], acc[nb][4 * g4 + 1], acc[nb][4 * g4 + 2], acc[nb][4 * g4 + 3]});
                        if (a.CstT) *reinterpret_cast<typename R::vec4*>(reinterpret_cast<T*>(a.CstT) + vrow_off + kg) = hi;
                        if (a.Cst) {
#pragma unroll
                            for (int e = 0; e < 4; e++) reinterpret_cast<T*>(a.Cst)[sbase + (size_t)state_row<T>(kg + e) * D + vg] = hi[e];
                        }
                        if constexpr (DOT) {
                            const f32x4 o = __builtin_convertvector(*reinterpret_cast<const typename R::vec4*>(reinterpret_cast<const T*>(a.dot_with) + vrow_off + kg), f32x4);
                            const f32x4 x = __builtin_convertvector(hi, f32x4);
                            dot += (x[0] * o[0] + x[1] * o[1]) + (x[2] * o[2] + x[3] * o[3]);
                        }
                    }
                }
                if constexpr (DOT) {
                    dot = wave_scan_inclusive<OpAdd>(dot);
                    if (lane == 63) dotred[wave] = dot;
                    pending_dot = c;
                }
                if (vh == 0 && wave == 0) {   // the vector state: the feeders' partial sums of this step, carried like the matrix
                    float sum = 0.f;
#pragma unroll 8
                    for (int g = 0; g < 32; g++) sum += red[g * 64 + lane];
                    nrun = nrun * tgam[cm.s] + sum;
                    a.Nst[((size_t)bh * NCS + c) * D + 64 * kq + lane] = nrun;
                }
                if (cm.s + 1 < NCS) {
                    const float gam = tgam[cm.s + 1];
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
#pragma unroll
                        for (int x = 0; x < 16; x++) acc[nb][x] *= gam;
                }
            }
            advance(cm);
            SQ_STAMP(1);
            __syncthreads();
            SQ_STAMP(3);
        }
        SQ_DUMP(1);
        if (DOT && pending_dot >= 0 && tid == 0)
            a.dot_part[((size_t)bh * NCS + pending_dot) * Cfg::WPH + w] = (dotred[0] + dotred[1]) + (dotred[2] + dotred[3]);
    }
#endif
}

// Whether the one-pass kernel serves a launch: on request only (set_state_kernel(2)), a table's worth of states, no split
// mode.  Measured at B4 H8 S4096 D256 and B2 H32 S16384 D128 (256 workgroups each) it takes the same 68 / 234 us per
// direction as the two kernels above (69 / 231 us): it moves half the bytes, but with one workgroup per CU and one
// barrier per tile each of its waves spends 1500 to 2000 cycles per tile on some 150 instructions (cycle stamps: direct
// loads 700, vector sum 600, products 1500, state write-out 400 per tile on average), so the launch stays with the two
// kernels until that per-tile cost is halved (two workgroups per CU, or two tiles per barrier).
int g_state_kernel = 0;   // 0 and 1 = chunk sums + carry, 2 = one pass where it can serve
template <typename T, int D>
static bool chunk_seq_serves(const ChunkArgs& a) {
    using Cfg = SeqCfg<T, D>;
    if (a.precise || a.NCS > Cfg::MAX_STEPS || (a.Cst && a.dot_part)) return false;
    return g_state_kernel == 2;
}
template <typename T, int D>
static int launch_chunk_seq(const ChunkArgs& a, hipStream_t st) {
    using Cfg = SeqCfg<T, D>;
    const dim3 grid(a.BH * Cfg::WPH);
    if (a.dot_part) {
        if (!a.dot_with || a.dot_with_lo) return MLSTM_EINVAL;
        if (int rc = no_scratch_once<chunk_seq_kernel<T, D, true>>()) return rc;
        if (hipError_t e = lds_limit_once<chunk_seq_kernel<T, D, true>>(160 * 1024); e != hipSuccess) return (int)e;
        hipLaunchKernelGGL((chunk_seq_kernel<T, D, true>), grid, dim3(512), Cfg::LDS_BYTES, st, a);
    } else {
        if (int rc = no_scratch_once<chunk_seq_kernel<T, D, false>>()) return rc;
        if (hipError_t e = lds_limit_once<chunk_seq_kernel<T, D, false>>(160 * 1024); e != hipSuccess) return (int)e;
        hipLaunchKernelGGL((chunk_seq_kernel<T, D, false>), grid, dim3(512), Cfg::LDS_BYTES, st, a);
    }
    return (int)hipGetLastError();
}

template <typename T, int D, bool STRICT>
static int launch_chunk_sum(const ChunkArgs& a, hipStream_t st) {
    using Cfg = ChunkCfg<T, D, STRICT>;
    if (a.L > Cfg::MAX_L) return MLSTM_ESHAPE;
    const dim3 grid(a.BH * a.NCS * (D / Cfg::VW));
    const size_t lds = Cfg::TILE_BYTES + 2 * (size_t)a.L * sizeof(float);
    // (the unrolled variant of split mode at D = 256 does not fit the 256 registers of a wave and would spill)
    constexpr bool UNROLLED_FITS = !(STRICT && D == 256);
    if (UNROLLED_FITS && a.L == 8 * GRAN) {   // the default chunk length
        constexpr int NTT = UNROLLED_FITS ? 8 : 0;
        if (hipError_t e = lds_limit_once<chunk_sum_kernel<T, D, NTT, STRICT>>(160 * 1024); e != hipSuccess) return (int)e;
        hipLaunchKernelGGL((chunk_sum_kernel<T, D, NTT, STRICT>), grid, dim3(512), lds, st, a);
    } else {
        if (hipError_t e = lds_limit_once<chunk_sum_kernel<T, D, 0, STRICT>>(160 * 1024); e != hipSuccess) return (int)e;
        hipLaunchKernelGGL((chunk_sum_kernel<T, D, 0, STRICT>), grid, dim3(512), lds, st, a);
    }
    return 0;
}

template <typename T, int D>
static int launch_chunk_t(const ChunkArgs& a, hipStream_t st) {
    if (a.precise && ((a.Cst && !a.Cst_lo) || (a.CstT && !a.CstT_lo))) return MLSTM_EINVAL;
    if (chunk_seq_serves<T, D>(a)) return launch_chunk_seq<T, D>(a, st);
    if (int rc = a.precise ? launch_chunk_sum<T, D, true>(a, st) : launch_chunk_sum<T, D, false>(a, st)) return rc;
    // one carry kernel: the value-major one writes both layouts and the vector states
    if (a.dot_part && !(a.CstT && a.dot_with)) return MLSTM_EINVAL;
    // (the variants of the value-major carry: with the contraction, with the key-major copy, with neither; both at once do
    // not fit the registers of four workgroups per CU, and nothing asks for both)
    const dim3 cgrid((D / 64) * (D / 64), a.BH);
    if (a.CstT && a.dot_part && a.Cst) return MLSTM_EINVAL;
    else if (a.CstT && a.dot_part) hipLaunchKernelGGL((chunk_carry_t_kernel<T, D, true, false>), cgrid, dim3(256), 0, st, a);
    else if (a.CstT && a.Cst) hipLaunchKernelGGL((chunk_carry_t_kernel<T, D, false, true>), cgrid, dim3(256), 0, st, a);
    else if (a.CstT) hipLaunchKernelGGL((chunk_carry_t_kernel<T, D, false, false>), cgrid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL((chunk_carry_kernel<T, D>), dim3(D * D / 8 / 256, a.BH), dim3(256), 0, st, a);
    return (int)hipGetLastError();
}

// the small shapes: plain multiply-adds for the sums, one element-wise carry for both layouts
template <typename T, int D>
static int launch_chunk_small(const ChunkArgs& a, hipStream_t st) {
    if (a.precise && ((a.Cst && !a.Cst_lo) || (a.CstT && !a.CstT_lo))) return MLSTM_EINVAL;
    if (!a.precise && (a.Cst_lo || a.CstT_lo)) return MLSTM_EINVAL;
    if (a.dot_part) return MLSTM_EINVAL;   // (launch_anchor serves these shapes)
    hipLaunchKernelGGL((chunk_sum_small_kernel<T, D>), dim3(a.BH * a.NCS * (D / 64)), dim3(256), 0, st, a);
    hipLaunchKernelGGL((chunk_carry_kernel<T, D>), dim3(D * D / 8 / 256, a.BH), dim3(256), 0, st, a);
    return (int)hipGetLastError();
}

// Sum of dD over all pairs (query behind the end of chunk c, key up to it): the forward state at that boundary
// contracted with the reverse state, <C~_c, E_c> + n~_c . g_c.  Rounding errors of the two matrices' 16-bit entries
// average out over the D^2 products.
template <typename T>
__global__ __launch_bounds__(1024) void anchor_kernel(const T* __restrict__ A, const T* __restrict__ B, const T* __restrict__ Al,
                                                     const T* __restrict__ Bl, const float* __restrict__ va, const float* __restrict__ vb,
                                                     float* __restrict__ anchor, int D, int NCS) {
    __shared__ float part[16];
    const int c = blockIdx.x, bh = blockIdx.y, tid = threadIdx.x;
    const size_t base = ((size_t)bh * NCS + c) * D * D;
    typedef T V8 __attribute__((ext_vector_type(8)));
    float acc = 0.f;
    for (int e = 8 * tid; e < D * D; e += 8 * 1024) {
        f32x8 x = __builtin_convertvector(*reinterpret_cast<const V8*>(A + base + e), f32x8);
        f32x8 y = __builtin_convertvector(*reinterpret_cast<const V8*>(B + base + e), f32x8);
        if (Al) {   // split mode: both states as hi + lo (the sums are exact in fp32: 8 + 8 significant bits at most)
            x += __builtin_convertvector(*reinterpret_cast<const V8*>(Al + base + e), f32x8);
            y += __builtin_convertvector(*reinterpret_cast<const V8*>(Bl + base + e), f32x8);
        }
        acc += ((x[0] * y[0] + x[1] * y[1]) + (x[2] * y[2] + x[3] * y[3])) + ((x[4] * y[4] + x[5] * y[5]) + (x[6] * y[6] + x[7] * y[7]));
    }
    if (tid < D) acc += va[((size_t)bh * NCS + c) * D + tid] * vb[((size_t)bh * NCS + c) * D + tid];
    acc = wave_scan_inclusive<OpAdd>(acc);
    if ((tid & 63) == 63) part[tid >> 6] = acc;
    __syncthreads();
    // (both states carry the factor 1 / sqrt(D) of the scores; dD has it once)
    if (tid == 0) {
        float sum = 0.f;
#pragma unroll
        for (int w = 0; w < 16; w++) sum += part[w];
        anchor[(size_t)bh * NCS + c] = sum * sqrtf((float)D);
    }
}

int launch_anchor(int dtype, int D, const void* A, const void* B, const void* A_lo, const void* B_lo, const float* va, const float* vb,
                  float* anchor, int BH, int NCS, hipStream_t st) {
    if ((A_lo == nullptr) != (B_lo == nullptr)) return MLSTM_EINVAL;
    if (dtype == MLSTM_BF16)
        hipLaunchKernelGGL(anchor_kernel<__bf16>, dim3(NCS, BH), dim3(1024), 0, st, (const __bf16*)A, (const __bf16*)B, (const __bf16*)A_lo,
                           (const __bf16*)B_lo, va, vb, anchor, D, NCS);
    else if (dtype == MLSTM_F16)
        hipLaunchKernelGGL(anchor_kernel<_Float16>, dim3(NCS, BH), dim3(1024), 0, st, (const _Float16*)A, (const _Float16*)B,
                           (const _Float16*)A_lo, (const _Float16*)B_lo, va, vb, anchor, D, NCS);
    else if (dtype == MLSTM_F32)
        hipLaunchKernelGGL(anchor_kernel<float>, dim3(NCS, BH), dim3(1024), 0, st, (const float*)A, (const float*)B, (const float*)A_lo,
                           (const float*)B_lo, va, vb, anchor, D, NCS);
    else return MLSTM_ESHAPE;
    return (int)hipGetLastError();
}

int launch_chunk_states(int dtype, int D, const ChunkArgs& a, hipStream_t st) {
    // NCS complete chunks, and at least one position behind them
    if (a.NCS <= 0 || a.L % 128 != 0 || (size_t)a.L * a.NCS >= (size_t)a.S || (size_t)a.L * (a.NCS + 1) < (size_t)a.S) return MLSTM_EINVAL;
    if (dtype == MLSTM_BF16 && D == 128) return launch_chunk_t<__bf16, 128>(a, st);
    if (dtype == MLSTM_BF16 && D == 256) return launch_chunk_t<__bf16, 256>(a, st);
    if (dtype == MLSTM_F16 && D == 128) return launch_chunk_t<_Float16, 128>(a, st);
    if (dtype == MLSTM_F16 && D == 256) return launch_chunk_t<_Float16, 256>(a, st);
    if (dtype == MLSTM_BF16 && D == 64) return launch_chunk_small<__bf16, 64>(a, st);
    if (dtype == MLSTM_F16 && D == 64) return launch_chunk_small<_Float16, 64>(a, st);
    if (dtype == MLSTM_F32 && D == 64) return launch_chunk_small<float, 64>(a, st);
    if (dtype == MLSTM_F32 && D == 128) return launch_chunk_small<float, 128>(a, st);
    return MLSTM_ESHAPE;
}

bool chunk_states_fused_dot(int dtype, int D) { return dtype != MLSTM_F32 && (D == 128 || D == 256); }

int chunk_states_dot_parts(int dtype, int D, const ChunkArgs& a) {
    bool seq = false;
    if (dtype == MLSTM_BF16 && D == 128) seq = chunk_seq_serves<__bf16, 128>(a);
    if (dtype == MLSTM_BF16 && D == 256) seq = chunk_seq_serves<__bf16, 256>(a);
    if (dtype == MLSTM_F16 && D == 128) seq = chunk_seq_serves<_Float16, 128>(a);
    if (dtype == MLSTM_F16 && D == 256) seq = chunk_seq_serves<_Float16, 256>(a);
    return seq ? (D / 64) * 2 : (D / 64) * (D / 64);
}

int set_state_kernel(int variant) {
    if (variant < 0 || variant > 2) return MLSTM_EINVAL;
    g_state_kernel = variant;
    return 0;
}

}  // namespace mlstm
