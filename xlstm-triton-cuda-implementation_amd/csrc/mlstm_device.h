// Shared device helpers for the gfx950 (CDNA4) mLSTM kernels: MFMA wrappers for bf16 / fp16 / fp32
// operands, LDS fragment loaders (row-major and transposing), wave64 DPP scans and reductions.
//
// Lane conventions, measured on MI355X hardware and used everywhere below (l = lane id, h = l / 32):
//   v_mfma_f32_32x32x16_{bf16,f16}: A holds row l%32, k = 8h..8h+7; B holds column l%32, k = 8h..8h+7;
//   the 16 accumulator registers r of a lane are column l%32, row 8*(r/4) + 4h + r%4.
//   v_mfma_f32_32x32x2_f32: A row l%32, k = h; B column l%32, k = h; same accumulator layout.
//   ds_read_b64_tr_b16: inside a block of 16 lanes, lanes 4r..4r+3 address "row r" (4 elements each);
//   lane j of the block receives element j of rows 0..3.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlstm {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(8))) float f32x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

constexpr float LOG2E = 1.4426950408889634f;
constexpr double LOG2E_D = 1.4426950408889634074;
constexpr int GRAN = 64;  // positions per gate granule == keys per key tile

#define LDS_PTR(T) T __attribute__((address_space(3)))*

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// ---------------------------------------------------------------------------------------------
// Per-element-type traits.  A "macro step" contracts KW elements: one 32x32x16 MFMA for the 16-bit
// types, four 32x32x2 MFMAs for fp32.  A fragment is the 16 bytes one lane contributes to it.
// ---------------------------------------------------------------------------------------------
template <typename T> struct Tr;

template <> struct Tr<__bf16> {
    static constexpr int EPL = 8, KW = 16;
    static constexpr bool HALF = true;
    typedef bf16x8 frag;
    typedef bf16x4 vec4;
    static __device__ __forceinline__ void mma(f32x16& c, frag a, frag b) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    // fragment for macro step t of a 32-row accumulator block: registers 8t..8t+7
    static __device__ __forceinline__ frag from_acc(const f32x16& c, int t) {
        f32x8 x;
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = c[8 * t + e];
        return __builtin_convertvector(x, frag);
    }
    static __device__ __forceinline__ vec4 cvt4(f32x4 x) { return __builtin_convertvector(x, vec4); }
    // Two-term split x = hi + lo with hi = x rounded to the element type and lo = the rounded remainder: a second MFMA on
    // lo gives the product of a weight operand about 16 significant bits instead of 8 (bf16) / 11 (fp16).
    static __device__ __forceinline__ void from_acc_split(const f32x16& c, int t, frag& hi, frag& lo) {
        f32x8 x;
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = c[8 * t + e];
        hi = __builtin_convertvector(x, frag);
        lo = __builtin_convertvector(x - __builtin_convertvector(hi, f32x8), frag);
    }
    static __device__ __forceinline__ void cvt4_split(f32x4 x, vec4& hi, vec4& lo) {
        hi = __builtin_convertvector(x, vec4);
        lo = __builtin_convertvector(x - __builtin_convertvector(hi, f32x4), vec4);
    }
};

template <> struct Tr<_Float16> {
    static constexpr int EPL = 8, KW = 16;
    static constexpr bool HALF = true;
    typedef f16x8 frag;
    typedef f16x4 vec4;
    static __device__ __forceinline__ void mma(f32x16& c, frag a, frag b) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ frag from_acc(const f32x16& c, int t) {
        f32x8 x;
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = c[8 * t + e];
        return __builtin_convertvector(x, frag);
    }
    static __device__ __forceinline__ vec4 cvt4(f32x4 x) { return __builtin_convertvector(x, vec4); }
    // Two-term split x = hi + lo with hi = x rounded to the element type and lo = the rounded remainder: a second MFMA on
    // lo gives the product of a weight operand about 16 significant bits instead of 8 (bf16) / 11 (fp16).
    static __device__ __forceinline__ void from_acc_split(const f32x16& c, int t, frag& hi, frag& lo) {
        f32x8 x;
#pragma unroll
        for (int e = 0; e < 8; e++) x[e] = c[8 * t + e];
        hi = __builtin_convertvector(x, frag);
        lo = __builtin_convertvector(x - __builtin_convertvector(hi, f32x8), frag);
    }
    static __device__ __forceinline__ void cvt4_split(f32x4 x, vec4& hi, vec4& lo) {
        hi = __builtin_convertvector(x, vec4);
        lo = __builtin_convertvector(x - __builtin_convertvector(hi, f32x4), vec4);
    }
};

template <> struct Tr<float> {
    static constexpr int EPL = 4, KW = 8;
    static constexpr bool HALF = false;
    typedef f32x4 frag;
    typedef f32x4 vec4;
    static __device__ __forceinline__ void mma(f32x16& c, frag a, frag b) {
#pragma unroll
        for (int e = 0; e < 4; e++) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], c, 0, 0, 0);
    }
    static __device__ __forceinline__ frag from_acc(const f32x16& c, int t) {
        frag x;
#pragma unroll
        for (int e = 0; e < 4; e++) x[e] = c[4 * t + e];
        return x;
    }
    static __device__ __forceinline__ vec4 cvt4(f32x4 x) { return x; }
    // (fp32 operands are exact: there is no split mode; these keep the shared templates well-formed)
    static __device__ __forceinline__ void from_acc_split(const f32x16& c, int t, frag& hi, frag& lo) { hi = from_acc(c, t); lo = frag{0.f, 0.f, 0.f, 0.f}; }
    static __device__ __forceinline__ void cvt4_split(f32x4 x, vec4& hi, vec4& lo) { hi = x; lo = vec4{0.f, 0.f, 0.f, 0.f}; }
};

// Output gate of the scan form (mlstm_scan.py:277): silu(o) * h on four packed elements, in fp32.
__device__ __forceinline__ float silu(float x) { return x / (1.0f + __expf(-x)); }
template <typename T>
__device__ __forceinline__ typename Tr<T>::vec4 gate4(typename Tr<T>::vec4 h, typename Tr<T>::vec4 o) {
    const f32x4 hf = __builtin_convertvector(h, f32x4), of = __builtin_convertvector(o, f32x4);
    f32x4 r;
#pragma unroll
    for (int c = 0; c < 4; c++) r[c] = hf[c] * silu(of[c]);
    return Tr<T>::cvt4(r);
}

// Row-major fragment: the contraction index runs along a tile row.  `row` points at the first element of
// the lane's row (row index l%32 of the block), macro step s.  Element e of the fragment is column
// KW*s + EPL*h + e.
template <typename T>
__device__ __forceinline__ typename Tr<T>::frag frag_rowmajor(const T* row, int s, int h) {
    return *reinterpret_cast<const typename Tr<T>::frag*>(row + Tr<T>::KW * s + Tr<T>::EPL * h);
}

// Transposed fragment out of an LDS tile stored row-major [contraction index][column], row stride ldt:
// the lane receives column cb + l%32 for the contraction indices of one macro step starting at row kr.
// 16-bit: element e = 4x + e' is row kr + 8x + 4h + e'; fp32: element e is row kr + 4h + e.  Both match
// Tr<T>::from_acc, so an accumulator block can be the other operand without any lane exchange.
template <typename T>
__device__ __forceinline__ typename Tr<T>::frag frag_transposed(const T* tile, int ldt, int kr, int cb, int lane) {
    const int h = lane >> 5;
    if constexpr (Tr<T>::HALF) {
        const int j = lane & 15, sub = (lane >> 4) & 1;
        const T* p0 = tile + (kr + 4 * h + (j >> 2)) * ldt + cb + 16 * sub + 4 * (j & 3);
        const T* p1 = p0 + 8 * ldt;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(p0));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(p1));
        s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(typename Tr<T>::frag, both);
    } else {
        const T* p = tile + (kr + 4 * h) * ldt + cb + (lane & 31);
        typename Tr<T>::frag f;
#pragma unroll
        for (int e = 0; e < 4; e++) f[e] = p[e * ldt];
        return f;
    }
}

// Cooperative copy of a ROWS x D tile (rows row0.. of a [S, D] matrix) into LDS with row stride LDT, split in two
// halves so that the global loads of the next tile can be in flight while the current one is being consumed:
// fetch() issues the 16-byte loads into registers, commit() writes them to LDS.
// Rows past S-1 are clamped to S-1 (their products are masked or never stored).
template <typename T, int D, int ROWS, int LDT, int NT>
struct TileCopy {
    static constexpr int EPC = 16 / sizeof(T);  // elements per 16-byte chunk
    static constexpr int CPR = D / EPC;         // chunks per row
    static constexpr int N = ROWS * CPR / NT;   // chunks per thread
    static_assert((ROWS * CPR) % NT == 0, "tile must divide evenly over the block");
    uint4 v[N];
    __device__ __forceinline__ void fetch(const T* g, int row0, int S, int tid) {
#pragma unroll
        for (int it = 0; it < N; it++) {
            int c = tid + it * NT;
            int r = c / CPR, cc = c % CPR;
            int gr = row0 + r;
            gr = gr < S ? gr : S - 1;
            v[it] = *reinterpret_cast<const uint4*>(g + (size_t)gr * D + cc * EPC);
        }
    }
    __device__ __forceinline__ void commit(T* lds, int tid) const {
#pragma unroll
        for (int it = 0; it < N; it++) {
            int c = tid + it * NT;
            int r = c / CPR, cc = c % CPR;
            *reinterpret_cast<uint4*>(lds + r * LDT + cc * EPC) = v[it];
        }
    }
};

// ---------------------------------------------------------------------------------------------
// Swizzled LDS tiles filled by direct global->LDS loads (global_load_lds_dwordx4: the data never passes through
// VGPRs and the copy is asynchronous, tracked by vmcnt; __syncthreads() waits for it).
//
// A tile is ROWS x D elements, rows contiguous (no padding: one wave instruction deposits 64 consecutive 16-byte
// chunks).  Chunk c of row r sits at chunk position c ^ key(r).  The key spreads (a) the same chunk of 16
// consecutive rows over all 64 banks, for the row-major ds_read_b128 where a lane owns a row, and (b) four
// consecutive rows over the four 64-byte bank windows, for the transposing reads that gather 4 rows x 64 bytes.
// ---------------------------------------------------------------------------------------------
template <typename T, int D>
struct Swz {
    static constexpr int EPC = 16 / sizeof(T);   // elements per chunk
    static constexpr int CPR = D / EPC;          // chunks per row
    static constexpr int ROW_BYTES = D * sizeof(T);
    static_assert(CPR >= 8 && (CPR & (CPR - 1)) == 0, "row must be a power-of-two number of chunks, at least 128 bytes");
    static __host__ __device__ __forceinline__ int key(int r) {
        if constexpr (CPR >= 16) return ((r & 3) << 2) | ((r >> 2) & 3);
        else return (r >> 1) & 7;
    }
    // byte offset of element column `col` (a multiple of the access width) of row r
    static __host__ __device__ __forceinline__ int off(int r, int col) {
        const int c = col / EPC, w = col % EPC;
        return r * ROW_BYTES + (((c ^ key(r))) << 4) + w * (int)sizeof(T);
    }
};

// One direct global->LDS load: every lane fetches 16 (or 4) bytes from its own global address and the wave's data
// lands at LDS byte offset lds_off + lane * 16 (or * 4).  Issued through inline assembly on purpose: the compiler's
// wait-count pass makes every later LDS read it cannot disambiguate (all transposing reads) wait for vmcnt(0) when
// it knows of a direct load in flight, which would serialise the copy of the next tile with the work on the current
// one.  The kernels wait explicitly (dma_wait) before the barrier that publishes a tile.
__device__ __forceinline__ void dma16(const void* g, unsigned lds_off) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_off) : "memory", "m0");
}
__device__ __forceinline__ void dma4(const void* g, unsigned lds_off) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(g), "s"(lds_off) : "memory", "m0");
}
__device__ __forceinline__ void dma_wait() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// The compiler does not know about the direct loads in flight, so a wait it places inside the main loop for a value
// that was loaded from global memory before the loop would, every iteration, also wait for the tile copy just
// issued.  pin() makes a prologue value "used" at the point of the call, which moves that wait out of the loop.
template <typename V> __device__ __forceinline__ void pin(V& v) { asm volatile("" : "+v"(v)); }
// LDS byte offset of a (non-null) pointer into LDS: the low half of its flat address.  The address-space cast would
// give the same value plus a null check, three scalar instructions per use.
__device__ __forceinline__ unsigned lds_offset_of(const void* p) {
    return (unsigned)(size_t)p;
}

// Asynchronous copy of rows row0..row0+ROWS-1 of a [S, D] matrix into a swizzled tile.  `tile` must be the same for
// all lanes of the wave.  Rows past S-1 are clamped (their products are masked or never stored).
template <typename T, int D, int ROWS, int NT>
__device__ __forceinline__ void tile_dma(T* tile, const T* g, int row0, int S, int tid, size_t row_stride = D) {
    using Z = Swz<T, D>;   // (row_stride: elements between the matrix' rows in memory)
    constexpr int NW = NT / 64, BLOCKS = ROWS * Z::CPR / 64;
    static_assert(BLOCKS % NW == 0, "tile must divide evenly over the waves");
    const int wave = tid >> 6, lane = tid & 63;
    const unsigned base = lds_offset_of(tile);
#pragma unroll
    for (int it = 0; it < BLOCKS / NW; it++) {
        const int blk = it * NW + wave;
        const int p = blk * 64 + lane;
        const int r = p / Z::CPR, pc = p % Z::CPR;
        const int c = pc ^ Z::key(r);
        int gr = row0 + r;
        gr = gr < S ? gr : S - 1;
        dma16(g + (size_t)gr * row_stride + c * Z::EPC, __builtin_amdgcn_readfirstlane(base + blk * 1024));
    }
}

// The same copy as a loop that stays a loop, for the places where it rarely runs (a sequence's last, partial tile) but would
// otherwise keep one 64-bit address per block alive across code that needs every register.
template <typename T, int D, int ROWS, int NT>
__device__ __forceinline__ void tile_dma_rolled(T* tile, const T* g, int row0, int S, int tid, size_t row_stride = D) {
    using Z = Swz<T, D>;
    constexpr int NW = NT / 64, BLOCKS = ROWS * Z::CPR / 64;
    static_assert(BLOCKS % NW == 0, "tile must divide evenly over the waves");
    const int wave = tid >> 6, lane = tid & 63;
    const unsigned base = lds_offset_of(tile);
#pragma unroll 1
    for (int it = 0; it < BLOCKS / NW; it++) {
        const int blk = it * NW + wave;
        const int p = blk * 64 + lane;
        const int r = p / Z::CPR, pc = p % Z::CPR;
        const int c = pc ^ Z::key(r);
        int gr = row0 + r;
        gr = gr < S ? gr : S - 1;
        dma16(g + (size_t)gr * row_stride + c * Z::EPC, __builtin_amdgcn_readfirstlane(base + blk * 1024));
    }
}

// Same copy with everything that does not change from tile to tile hoisted out of the loop: the per-lane byte offsets
// inside a tile are computed once (init), a tile is addressed by a scalar base pointer, and the LDS destinations are
// scalar arithmetic on the wave index.  A tile then costs no vector ALU work at all: per 1 KB block one s_mov to M0
// and one global_load_lds with "scalar base + lane offset" addressing.  Only valid for tiles whose ROWS rows all
// exist (row0 + ROWS <= S); the last, partial tile of a sequence goes through tile_dma, which clamps.
// No "memory" clobber here: the copy targets the LDS stage nobody reads in this step, and a clobber would pin every
// LDS read of the surrounding MFMA groups in place (one read, one wait, one MFMA: no prefetch depth at all).
__device__ __forceinline__ void dma16_s(const void* sbase, unsigned voff, unsigned lds_base, unsigned lds_blk) {
    asm volatile("s_add_u32 m0, %2, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(sbase), "s"(lds_base), "s"(lds_blk)
                 : "m0", "scc");
}
template <typename T, int D, int ROWS, int NT>
struct TileDma {
    using Z = Swz<T, D>;
    static constexpr int NW = NT / 64, BLOCKS = ROWS * Z::CPR / 64, PER_WAVE = BLOCKS / NW;
    static_assert(BLOCKS % NW == 0, "tile must divide evenly over the waves");
    // A wave's successive blocks lie RSTEP rows apart and the swizzle key has a period of 16 rows, so the per-lane
    // offsets repeat (shifted by whole rows) after PERIOD blocks: only those are kept in registers, the shift goes
    // into the scalar base address.
    static_assert((NW * 64) % Z::CPR == 0, "a wave's blocks must start at the same column");
    static constexpr int RSTEP = NW * 64 / Z::CPR;
    static_assert(RSTEP >= 16 ? RSTEP % 16 == 0 : 16 % RSTEP == 0, "row step and swizzle period must nest");
    static constexpr int PERIOD_RAW = RSTEP >= 16 ? 1 : 16 / RSTEP;
    static constexpr int PERIOD = PERIOD_RAW < PER_WAVE ? PERIOD_RAW : PER_WAVE;
    static constexpr int GROUP_BYTES = PERIOD * RSTEP * Z::ROW_BYTES;   // global and LDS distance of blocks it and it + PERIOD
    unsigned voff[PERIOD];
    int wave_s;  // wave index as a scalar
    // Byte offset, from the tile's first row in memory, of the 16 bytes lane `lane` of wave `wave` fetches in its block
    // `it` (rows `row_bytes` apart); the data lands at byte (it * NW + wave) * 1024 + 16 * lane of the LDS tile.  The
    // kernels keep lane_source(it) for it < PERIOD only and add (it / PERIOD) * group_bytes(row_bytes) for the others;
    // a host-side check (tests/harness/tile_bounds.hip) walks every block of every tile shape and asserts that the two
    // agree, that every 16-byte piece of the tile is fetched exactly once, and that no fetch ends beyond the tile's last row.
    static __host__ __device__ __forceinline__ unsigned lane_source(int it, int wave, int lane, unsigned row_bytes) {
        const int p = (it * NW + wave) * 64 + lane;
        const int r = p / Z::CPR, pc = p % Z::CPR;
        return (unsigned)r * row_bytes + (unsigned)((pc ^ Z::key(r)) << 4);
    }
    static __host__ __device__ __forceinline__ unsigned group_bytes(unsigned row_bytes) { return (unsigned)(PERIOD * RSTEP) * row_bytes; }
    __device__ __forceinline__ void init(int tid) {
        wave_s = __builtin_amdgcn_readfirstlane(tid >> 6);
        const int lane = tid & 63;
#pragma unroll
        for (int it = 0; it < PERIOD; it++) voff[it] = lane_source(it, wave_s, lane, Z::ROW_BYTES);
    }
    // g_tile: first row of the tile (the same for all lanes); tile: LDS destination
    // Blocks [first, last) of this wave only: the kernels spread a tile's copy over the matrix work of the previous
    // tile, a block or two between groups of MFMAs.  A wave that issues all its loads back to back sits in the
    // memory pipeline's queue (64 lanes x 16 bytes take 16 cycles each, and four waves share it) and cannot issue
    // the MFMAs behind them in program order.
    __device__ __forceinline__ void issue_range(T* tile, const T* g_tile_v, int first, int last) const {
        const unsigned base = __builtin_amdgcn_readfirstlane(lds_offset_of(tile));
        const unsigned long long gv = (unsigned long long)(size_t)g_tile_v;
        const unsigned long long gs = ((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(gv >> 32)) << 32) |
                                      (unsigned)__builtin_amdgcn_readfirstlane((int)gv);
        const void* g_tile = (const void*)(size_t)gs;
#pragma unroll
        for (int it = 0; it < PER_WAVE; it++)
            if (it >= first && it < last)
                dma16_s(reinterpret_cast<const char*>(g_tile) + (it / PERIOD) * GROUP_BYTES, voff[it % PERIOD], base, (it * NW + wave_s) * 1024);
    }
    __device__ __forceinline__ void issue(T* tile, const T* g_tile_v) const {
        const unsigned base = __builtin_amdgcn_readfirstlane(lds_offset_of(tile));
        // force the (wave-uniform) tile address into a scalar register pair
        const unsigned long long gv = (unsigned long long)(size_t)g_tile_v;
        const unsigned long long gs = ((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(gv >> 32)) << 32) |
                                      (unsigned)__builtin_amdgcn_readfirstlane((int)gv);
        const void* g_tile = (const void*)(size_t)gs;
#pragma unroll
        for (int it = 0; it < PER_WAVE; it++)
            dma16_s(reinterpret_cast<const char*>(g_tile) + (it / PERIOD) * GROUP_BYTES, voff[it % PERIOD], base, (it * NW + wave_s) * 1024);
    }
    // The same copies from a matrix whose rows lie `row_bytes` apart in memory (a tensor of the caller's in a layout of
    // its own; init's offsets serve matrices with D elements per row, such as the chunk states).  rows() after init().
    struct Rows { unsigned voff[PERIOD]; unsigned group_bytes; };
    __device__ __forceinline__ Rows rows(int tid, unsigned row_bytes) const {
        Rows o;
        const int lane = tid & 63;
#pragma unroll
        for (int it = 0; it < PERIOD; it++) o.voff[it] = lane_source(it, wave_s, lane, row_bytes);
        o.group_bytes = group_bytes(row_bytes);
        return o;
    }
    __device__ __forceinline__ void issue_range(T* tile, const T* g_tile_v, int first, int last, const Rows& o) const {
        const unsigned base = __builtin_amdgcn_readfirstlane(lds_offset_of(tile));
        const unsigned long long gv = (unsigned long long)(size_t)g_tile_v;
        const unsigned long long gs = ((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(gv >> 32)) << 32) |
                                      (unsigned)__builtin_amdgcn_readfirstlane((int)gv);
        const void* g_tile = (const void*)(size_t)gs;
        const unsigned gb = __builtin_amdgcn_readfirstlane(o.group_bytes);
#pragma unroll
        for (int it = 0; it < PER_WAVE; it++)
            if (it >= first && it < last)
                dma16_s(reinterpret_cast<const char*>(g_tile) + (size_t)((it / PERIOD) * gb), o.voff[it % PERIOD], base, (it * NW + wave_s) * 1024);
    }
    __device__ __forceinline__ void issue(T* tile, const T* g_tile_v, const Rows& o) const { issue_range(tile, g_tile_v, 0, PER_WAVE, o); }
};

// The 16-byte pieces that the two lanes (h = 0, 1) of a row load of their wave's half row for the row sums q . dQ of the
// eight-wave row kernel: a half row of `half_row_bytes` has half_row_bytes / 16 pieces, lane h takes the pieces
// NP h .. NP h + NP - 1 with NP = half of them.  Shared with the host-side bounds check.
__host__ __device__ constexpr int row8_pieces_per_lane(int half_row_bytes) { return half_row_bytes / 32; }
__host__ __device__ constexpr int row8_piece_offset(int i, int h, int half_row_bytes) { return 16 * (row8_pieces_per_lane(half_row_bytes) * h + i); }

// 64 floats (one per key of a tile) by the first wave
__device__ __forceinline__ void vec64_dma(float* dst, const float* src, int tid) {
    if (tid < 64) dma4(src + tid, __builtin_amdgcn_readfirstlane(lds_offset_of(dst)));
}
// n <= 64 floats by wave `w`
__device__ __forceinline__ void vecn_dma(float* dst, const float* src, int n, int tid, int w) {
    if ((tid >> 6) == w && (tid & 63) < n) dma4(src + (tid & 63), __builtin_amdgcn_readfirstlane(lds_offset_of(dst)));
}

// Three per-tile vectors (64 floats each in LDS), copied by a four-wave group without any branch: every wave issues one
// direct load of 64 floats per tile; waves 0..2 take one vector each, the fourth repeats the first wave's (the same
// data to the same place).  Vector k advances by step_k floats per tile; a vector with fewer than 64 values per tile
// (step < 64) must stay readable 64 floats past its last tile's first element.  A wave of a kernel that keeps one wave
// per SIMD issues an instruction every four cycles or so, and the masked variant (three `if (wave == k)` blocks) costs
// some forty of them per tile.
struct RowVec3Dma {
    const float* src;    // this wave's vector + lane
    unsigned slot_off;   // byte offset of this wave's vector inside the destination area [3][64] floats
    int step;            // floats per tile of this wave's vector
    __device__ __forceinline__ void init(int tid, const float* p0, const float* p1, const float* p2, int step0 = 64, int step1 = 64,
                                         int step2 = 64) {
        const int w = __builtin_amdgcn_readfirstlane(tid >> 6) & 3;
        const int k = w == 3 ? 0 : w;
        src = (k == 0 ? p0 : (k == 1 ? p1 : p2)) + (tid & 63);
        step = k == 0 ? step0 : (k == 1 ? step1 : step2);
        slot_off = (unsigned)k * 64u * 4u;
    }
    // dst: the [3][64] float area of a stage; tile: index of the tile
    __device__ __forceinline__ void issue(const float* dst, int tile) const {
        dma4(src + tile * step, __builtin_amdgcn_readfirstlane(lds_offset_of(dst)) + slot_off);
    }
};

// Row-major fragment of a swizzled tile: lane owns row r, macro step s (columns KW*s + EPL*h ..).
template <typename T, int D>
__device__ __forceinline__ typename Tr<T>::frag swz_frag_rowmajor(const T* tile, int r, int s, int h) {
    const char* base = reinterpret_cast<const char*>(tile);
    return *reinterpret_cast<const typename Tr<T>::frag*>(base + Swz<T, D>::off(r, Tr<T>::KW * s + Tr<T>::EPL * h));
}

// Transposed fragment of a swizzled tile (see frag_transposed for the element order).
template <typename T, int D>
__device__ __forceinline__ typename Tr<T>::frag swz_frag_transposed(const T* tile, int kr, int cb, int lane) {
    using Z = Swz<T, D>;
    const char* base = reinterpret_cast<const char*>(tile);
    const int h = lane >> 5;
    if constexpr (Tr<T>::HALF) {
        const int j = lane & 15, sub = (lane >> 4) & 1;
        const int row = kr + 4 * h + (j >> 2), col = cb + 16 * sub + 4 * (j & 3);
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(base + Z::off(row, col)));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(base + Z::off(row + 8, col)));
        s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(typename Tr<T>::frag, both);
    } else {
        typename Tr<T>::frag f;
#pragma unroll
        for (int e = 0; e < 4; e++) f[e] = *reinterpret_cast<const float*>(base + Z::off(kr + 4 * h + e, cb + (lane & 31)));
        return f;
    }
}

// Per-lane byte offsets for the two fragment kinds of a swizzled tile, precomputed once per kernel so that every
// read in the unrolled loops is "one address register + immediate".  XOR swizzling is not affine in the chunk index,
// but the key only touches chunk bits 0..3, and it only depends on the row modulo 16:
//   row-major reads: chunk = 2s + h, so macro steps s and s + 8 differ by 256 bytes and rows r and r + 32 by 32 rows;
//   transposed reads (16-bit): column block d and d + 4 differ by 256 bytes, rows kr and kr + 16 by 16 rows.
template <typename T, int D>
struct SwzRowReader {
    static constexpr int NS = D / Tr<T>::KW, KO = NS < 8 ? NS : 8;
    int off[KO];
    __device__ __forceinline__ void init(int lane) {
#pragma unroll
        for (int s = 0; s < KO; s++) off[s] = Swz<T, D>::off(lane & 31, Tr<T>::KW * s + Tr<T>::EPL * (lane >> 5));
    }
    // fragment of row 32*rb + (lane & 31), macro step s
    __device__ __forceinline__ typename Tr<T>::frag read(const T* tile, int rb, int s) const {
        const char* base = reinterpret_cast<const char*>(tile);
        return *reinterpret_cast<const typename Tr<T>::frag*>(base + off[s % KO] + (s / KO) * 256 + rb * 32 * Swz<T, D>::ROW_BYTES);
    }
};

// The same row-major reads from ONE per-lane offset: the chunk index 2s + h only meets the key in an XOR, so
// off(s) = off(0) ^ (s << 5) for s < 8; one vector ALU instruction per read instead of eight address registers.
template <typename T, int D>
struct SwzRowReaderX {
    static_assert(Tr<T>::HALF && Swz<T, D>::CPR >= 16, "16-bit tiles of at least 256 bytes per row");
    int off0;
    __device__ __forceinline__ void init(int lane) { off0 = Swz<T, D>::off(lane & 31, Tr<T>::EPL * (lane >> 5)); }
    __device__ __forceinline__ typename Tr<T>::frag read(const T* tile, int rb, int s) const {
        const char* base = reinterpret_cast<const char*>(tile);
        return *reinterpret_cast<const typename Tr<T>::frag*>(base + (off0 ^ ((s % 8) << 5)) + (s / 8) * 256 + rb * 32 * Swz<T, D>::ROW_BYTES);
    }
};

template <typename T, int D>
struct SwzTransReader {
    static constexpr int NDB = D / 32, VO = NDB < 4 ? NDB : 4;
    static_assert(Tr<T>::HALF && Swz<T, D>::CPR >= 16, "16-bit tiles of at least 256 bytes per row");
    int off[2][VO];
    // cb0: first 32-column block this reader serves (a multiple of VO when more than VO blocks are read)
    __device__ __forceinline__ void init(int lane, int cb0 = 0) {
        const int h = lane >> 5, j = lane & 15, sub = (lane >> 4) & 1;
#pragma unroll
        for (int hi = 0; hi < 2; hi++)
#pragma unroll
            for (int d = 0; d < VO; d++)
                off[hi][d] = Swz<T, D>::off(4 * h + (j >> 2) + 8 * hi, 32 * (cb0 + d) + 16 * sub + 4 * (j & 3));
    }
    // contraction rows kr..kr+15 (kr a multiple of 16), column block cb0 + d
    __device__ __forceinline__ typename Tr<T>::frag read(const T* tile, int kr, int d) const {
        const char* base = reinterpret_cast<const char*>(tile) + kr * Swz<T, D>::ROW_BYTES + (d / VO) * 256;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(base + off[0][d % VO]));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_PTR(s16x4))(base + off[1][d % VO]));
        s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(typename Tr<T>::frag, both);
    }
};

// ---------------------------------------------------------------------------------------------
// wave64 scans and reductions (DPP row shifts + row broadcasts, no LDS)
// ---------------------------------------------------------------------------------------------
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, bool BOUND = false>
__device__ __forceinline__ float dpp_f(float old, float src) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, src),
                                                                 CTRL, ROW_MASK, BANK_MASK, BOUND));
}

struct OpAdd { static __device__ __forceinline__ float id() { return 0.0f; } static __device__ __forceinline__ float f(float a, float b) { return a + b; } };
struct OpMax { static __device__ __forceinline__ float id() { return -INFINITY; } static __device__ __forceinline__ float f(float a, float b) { return fmaxf(a, b); } };

// Inclusive scan across the 64 lanes of a wave.
template <typename Op>
__device__ __forceinline__ float wave_scan_inclusive(float v) {
    // within rows of 16 lanes: row_shr:1,2,4,8 (0x111, 0x112, 0x114, 0x118); lanes shifted in from outside keep `old`
    v = Op::f(v, dpp_f<0x111>(Op::id(), v));
    v = Op::f(v, dpp_f<0x112>(Op::id(), v));
    v = Op::f(v, dpp_f<0x114>(Op::id(), v));
    v = Op::f(v, dpp_f<0x118>(Op::id(), v));
    // carry across rows with lane reads of each row's last element
    const int lane = __lane_id();
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 15));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 31));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 47));
    float c = Op::id();
    if (lane >= 16) c = r0;
    if (lane >= 32) c = Op::f(r0, r1);
    if (lane >= 48) c = Op::f(Op::f(r0, r1), r2);
    return Op::f(c, v);
}

template <typename Op>
__device__ __forceinline__ float wave_reduce(float v) {
    v = Op::f(v, dpp_f<0x111>(Op::id(), v));
    v = Op::f(v, dpp_f<0x112>(Op::id(), v));
    v = Op::f(v, dpp_f<0x114>(Op::id(), v));
    v = Op::f(v, dpp_f<0x118>(Op::id(), v));
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 15));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 31));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 47));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
    return Op::f(Op::f(r0, r1), Op::f(r2, r3));
}

// maxima over lanes 0..31 and over lanes 32..63
__device__ __forceinline__ void wave_half_max(float v, float& lo, float& hi) {
    v = fmaxf(v, dpp_f<0x111>(-INFINITY, v));
    v = fmaxf(v, dpp_f<0x112>(-INFINITY, v));
    v = fmaxf(v, dpp_f<0x114>(-INFINITY, v));
    v = fmaxf(v, dpp_f<0x118>(-INFINITY, v));
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 15));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 31));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 47));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
    lo = fmaxf(r0, r1);
    hi = fmaxf(r2, r3);
}

// v(l) + v(l ^ 32): lanes l and l^32 share an accumulator column.  v_permlane32_swap hands each lane its
// own value in one result and the partner's in the other, so the sum needs no select.
__device__ __forceinline__ float sum_halves(float v) {
    int x = __builtin_bit_cast(int, v);
    auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
    return __builtin_bit_cast(float, (int)r[0]) + __builtin_bit_cast(float, (int)r[1]);
}

template <typename T> __device__ __forceinline__ float to_f32(T x) { return (float)x; }

// Per-row scalars of the backward, computed by the lanes that already hold the row's dh fragments (xf):
//   n = max(|b|, exp(-m)) + 1e-6,  dn = -(dh . h) / n,  db = sign(b) dn [|b| > exp(-m)].
// The reference obtains dn from a full tile loop (mlstm_matmul_kernel_backward_db, mlstm_matmul.py:133-197); because
// sum_j C~_ij (dh_i . v_j) = n_i (dh_i . h_i) it collapses to one dot product per row.
// hrow_lo (may be null): the remainder h - (h rounded to the element type), left by a forward in split mode; with it
// the dot product sees h to about 16 significant bits.
// 1/n and db of a row from delta = dh . h, the normaliser sum b and the stabiliser m (mlstm_matmul.py:194-196)
__device__ __forceinline__ void row_stats_of(float delta, float b, float m, float& inv_n, float& db) {
    const float em = __expf(-m);
    inv_n = 1.0f / (fmaxf(fabsf(b), em) + 1e-6f);
    const float dn = -delta * inv_n;
    const float sg = (b > 0.f) ? 1.f : ((b < 0.f) ? -1.f : 0.f);
    db = (fabsf(b) > em) ? sg * dn : 0.f;
}

template <typename T, int NS>
__device__ __forceinline__ void row_stats(const typename Tr<T>::frag (&xf)[NS], const T* hrow, int h, float b, float m, float& inv_n,
                                          float& db, const T* hrow_lo = nullptr) {
    float acc = 0.f;
#pragma unroll
    for (int s = 0; s < NS; s++) {
        const typename Tr<T>::frag hf = frag_rowmajor<T>(hrow, s, h);
#pragma unroll
        for (int e = 0; e < Tr<T>::EPL; e++) acc += (float)xf[s][e] * (float)hf[e];
    }
    if (hrow_lo) {
        float acc_lo = 0.f;
#pragma unroll
        for (int s = 0; s < NS; s++) {
            const typename Tr<T>::frag hf = frag_rowmajor<T>(hrow_lo, s, h);
#pragma unroll
            for (int e = 0; e < Tr<T>::EPL; e++) acc_lo += (float)xf[s][e] * (float)hf[e];
        }
        acc += acc_lo;
    }
    row_stats_of(sum_halves(acc), b, m, inv_n, db);
}

__device__ __forceinline__ float log_sigmoid(float x) {
    // log(sigmoid(x)) = min(x, 0) - log1p(exp(-|x|))
    return fminf(x, 0.0f) - log1pf(__expf(-fabsf(x)));
}

}  // namespace mlstm
