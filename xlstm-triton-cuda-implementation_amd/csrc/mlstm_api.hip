// C ABI of libmlstm_hip.so: argument checks, workspace carving and the launch sequences.
#include <hip/hip_runtime.h>
#include <mutex>
#include <utility>
#include <vector>
#include "mlstm_kernels.h"

using namespace mlstm;

namespace mlstm {
bool g_force_generic = false;  // see mlstm_force_generic_kernels
int g_col_variant = 0;         // see mlstm_set_column_kernel
}

namespace {

// Optional per-kernel timing with HIP events on the launch stream (off by default; see mlstm_timing_enable).
struct TimingState {
    bool on = false;
    unsigned mask = ~0u;       // kernels that are timed while `on` (bit = kernel id)
    int every = 1;             // of a selected kernel's launches, every `every`-th is timed
    int seen[32] = {};
    std::mutex mu;
    struct Rec { int id; hipEvent_t a, b; };
    std::vector<Rec> recs;
} g_timing;

struct Timed {
    int id; hipStream_t st; hipEvent_t a = nullptr, b = nullptr;
    Timed(int id_, hipStream_t st_) : id(id_), st(st_) {
        if (!g_timing.on) return;
        {
            std::lock_guard<std::mutex> lk(g_timing.mu);   // (callers on several threads share the launch counters)
            if (!((g_timing.mask >> (id & 31)) & 1u)) return;
            if (g_timing.seen[id & 31]++ % g_timing.every != 0) return;
        }
        if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) { a = nullptr; return; }
        (void)hipEventRecord(a, st);
    }
    ~Timed() {
        if (!a) return;
        (void)hipEventRecord(b, st);
        std::lock_guard<std::mutex> lk(g_timing.mu);
        g_timing.recs.push_back({id, a, b});
    }
};

inline size_t up256(size_t x) { return (x + 255) & ~(size_t)255; }

struct Carver {
    char* base; size_t off;
    template <typename T> T* take(size_t n) { T* p = reinterpret_cast<T*>(base + off); off += up256(n * sizeof(T)); return p; }
};

// Chunk length of the chunked forward for this shape, 0 = walk all the keys.  The eight-wave row kernel serves the
// 16-bit types at D >= 128; a chunk pays D/64 state tiles per row tile and saves the key tiles before the chunk, and the
// states cost 2 S D^2 flops per head whatever the length.
int g_chunk_override = 0;   // test aid: > 0 forces this length, < 0 switches chunking off
int chunk_len_for(int dtype, int D, size_t S) {
    // (the chunk states are formed by 16-bit MFMA products at D = 128 and 256 and by plain multiply-adds at the smaller
    // shapes; every tile kernel knows chunks, the four-wave ones of fp32, of split mode and of the test switch included)
    const bool shape_ok = dtype == MLSTM_F32 ? (D == 64 || D == 128) : (D == 64 || D == 128 || D == 256);
    if (!shape_ok || g_chunk_override < 0) return 0;
    if (g_chunk_override > 0) return S > (size_t)g_chunk_override ? g_chunk_override : 0;
    if (S < 1024) return 0;   // (below two full chunks of 512 the state pass costs more than the skipped key tiles)
    // fp32 products run at a sixteenth of the 16-bit rate, so the key tiles a chunk saves weigh more against the states: the
    // shortest chunk wins there (B1 H4 S2048 D64: 0.47 ms unchunked, 0.24 / 0.16 / 0.13 ms at 512 / 256 / 128; D = 128
    // likewise); at D = 64 in 16 bits 256 is the measured best (B4 H8 S4096: 0.48 unchunked, 0.24 / 0.22 / 0.25 ms)
    if (dtype == MLSTM_F32) return 128;
    return D == 64 ? 256 : 512;
}

// What mlstm_forward_save_* writes at the head of `saved` and mlstm_backward_saved_* checks on the device (no host
// round trip): shape, types and the process-wide settings the two calls must agree on.
constexpr size_t SAVED_HEADER_BYTES = 256;
// The eight words: magic, BH, S, D, dtype argument, chunk length, kernel switch, states per head.  The forward's gate
// pre-pass writes them and the backward's last kernel compares them (mlstm::SavedStamp): no launch of their own.
constexpr int SAVED_MAGIC = 0x4d4c5356;   // "MLSV"

struct Sizes {
    size_t BH, S, D, NG, el;
    size_t gates() const { return 3 * up256(BH * NG * 64 * 4) + up256(BH * NG * 8) + up256((BH * NG * 2 + 64) * 4); }
    size_t stats() const { return 2 * up256(BH * S * 4); }                       // m, b
    // chunked forward: per-chunk sums (fp32), matrix states (element type), vector states
    size_t n_states(int L) const { return L > 0 && S > (size_t)L ? (S - 1) / L : 0; }
    size_t chunk_states(int dtype) const {
        const size_t n = n_states(chunk_len_for(dtype, (int)D, S));
        return up256(BH * n * D * D * 4) + up256(BH * n * D * D * el * parts()) + up256(BH * n * D * 4);
    }
    int dtype_code = MLSTM_F32;
    // layouts of the caller's tensors (dense unless an _lx entry point says otherwise): q, k, v and their gradients;
    // h and dh; the gates and their gradients; and what f holds
    Lay la{}, lb{}, lg{};
    int gate_form = MLSTM_GATE_RAW;
    bool precise = false;   // split mode (MLSTM_PRECISE): states as two terms, and the low-order part of h travels to the backward
    size_t parts() const { return precise ? 2 : 1; }   // terms per matrix state: hi, and lo directly behind it
    int chunk_len() const { return chunk_len_for(dtype_code, (int)D, S); }
    size_t state_elems() const { return BH * n_states(chunk_len()) * D * D; }             // one term of one set of states
    size_t states_t() const { return up256(state_elems() * el * parts()); }               // value-major copy for the dQ pass
    size_t saved_vec() const { return up256(BH * n_states(chunk_len()) * D * 4); }
    size_t h_lo() const { return precise ? up256(BH * S * D * el) : 0; }
    // the column kernel runs in chunks too, for lengths at which the row kernel, which leaves the far row sums, is sure to
    // have run in chunks
    bool col_chunks() const { return n_states(chunk_len()) > 0 && NG <= 1024; }
    // row partials of dD per position: one per key tile at or before it, in chunks one per key tile of its own chunk
    size_t row_slices() const { return col_chunks() ? (size_t)chunk_len() / 64 : NG; }
    // what the backward reuses of the forward: a header, in chunks the value-major states, the vector states and the gate
    // pre-pass; in split mode h - (h rounded to the element type)
    size_t saved_chunk() const { return n_states(chunk_len()) ? states_t() + saved_vec() + gates() : 0; }
    size_t saved() const { return saved_chunk() + h_lo() > 0 ? SAVED_HEADER_BYTES + saved_chunk() + h_lo() : 0; }
    // fp32 at head dimensions of 256 and more: the matmul form's entry points run on the scan form's kernels (the same
    // function; the tile kernels' accumulators and LDS stages end at D = 128 in fp32)
    bool scan_engine() const { return dtype_code == MLSTM_F32 && D >= 256; }
    // scan form: gates, m, row sums, in-chunk pairs, vector states, partial numerators of the other key ranges
    size_t scan_fwd() const {
        return gates() + stats() + up256(BH * NG * 64 * 64 * 4) + up256(BH * NG * D * 4) +
               (size_t)(scan_key_splits((int)BH, (int)D) - 1) * up256(BH * S * D * 4) +
               up256(scan_segment_state_bytes((int)BH, (int)S, (int)D));
    }
    size_t fwd() const { return scan_engine() ? scan_fwd() : gates() + stats() + chunk_states(dtype_code); }
    size_t anchor_parts() const { return D >= 64 ? (D / 64) * (D / 64) : 1; }   // workgroups per head of the value-major carry
    size_t fwd_fixed() const { return gates() + stats(); }   // offset of the chunk states inside fwd()
    size_t bwd() const {
        if (scan_engine()) return scan_backward_workspace_bytes((int)BH, (int)S, (int)D);
        return fwd() + up256(BH * S * D * el)                                      // recomputed h
               + 2 * up256(BH * NG * 64 * 4) + states_t()                          // inv_n, db; transposed chunk states
               + states_t() + saved_vec() + up256(BH * S * 4)                      // reverse states (value-major, vector); far row sums
               + up256(BH * n_states(chunk_len()) * anchor_parts() * 4)            // dF anchors (in parts)
               + up256(BH * S * 4) + up256(BH * row_slices() * S * 4)              // colsum, rowpart
               + h_lo();                                                           // split mode: low-order part of a recomputed h
    }
    // gated backward: the ungated upstream gradient, and (h, m, b) when the caller does not bring them
    size_t bwd_gated() const { return bwd() + 2 * up256(BH * S * D * el) + stats(); }
};

// begin/end marks for groups of scan kernels (the scan translation unit has no access to Timed)
thread_local Timed* g_scan_mark[16] = {};
void scan_mark(int id, hipStream_t st, bool begin) {
    if (begin) g_scan_mark[id] = new Timed(id, st);
    else { delete g_scan_mark[id]; g_scan_mark[id] = nullptr; }
}

bool good_dtype(int dt) { return dt == MLSTM_F32 || dt == MLSTM_F16 || dt == MLSTM_BF16; }
// element type code as the caller passes it: one of the three types, optionally with MLSTM_PRECISE
bool good_dtype_arg(int dt) { return dt >= 0 && good_dtype(dt & ~MLSTM_PRECISE); }
// (fp32 operands are exact: the flag is accepted and has no effect there)
bool precise_of(int dt) { return (dt & MLSTM_PRECISE) != 0 && (dt & ~MLSTM_PRECISE) != MLSTM_F32; }
Sizes sizes_of(int B, int NH, int S, int D, int dtype_arg) {
    const int dt = dtype_arg & ~MLSTM_PRECISE;
    Sizes z{(size_t)B * NH, (size_t)S, (size_t)D, (size_t)(S + GATE_GRANULE - 1) / GATE_GRANULE, dtype_size(dt), dt};
    z.precise = precise_of(dtype_arg);
    z.la = z.lb = dense_layout(NH, S, D);
    z.lg = dense_layout(NH, S, 1);
    return z;
}
bool good_shape(int D, int dtype) { return D == 64 || D == 128 || D == 256 || (dtype == MLSTM_F32 && (D == 512 || D == 1024)); }

// Do the elements of a [B,NH,S] grid of rows of `row` elements each stay apart under these strides?  (Sufficient test:
// taken in the order of their strides, every dimension must step over everything the smaller ones span.)  A tensor the
// library WRITES must pass it: with an expanded view (a zero stride) or any other overlap several workgroups would
// write one address and the last writer would win.
bool non_overlapping(long long B, long long NH, long long S, long long sb, long long sh, long long ss, long long row) {
    long long n[3] = {B, NH, S}, st[3] = {sb, sh, ss};
    for (int a = 0; a < 3; a++)
        for (int b = a + 1; b < 3; b++)
            if (st[b] < st[a]) { std::swap(st[a], st[b]); std::swap(n[a], n[b]); }
    long long extent = row;
    for (int a = 0; a < 3; a++) {
        if (n[a] <= 1) continue;
        if (st[a] < extent) return false;
        extent += (n[a] - 1) * st[a];
    }
    return true;
}

// The caller's layout into z (null: everything dense).  Rows of q, k, v, h must start on 16-byte boundaries, and the
// tile copies address a tile's 64 rows with 32-bit byte offsets.  written_qkv / written_out / written_gates: the call
// writes tensors in that layout (gradients, h), which must then not overlap themselves.
int apply_layout(Sizes& z, const mlstm_layout* L, int NH, int gate_dtype, std::initializer_list<const void*> row_tensors, bool written_qkv,
                 bool written_out, bool written_gates) {
    if (!L) return 0;
    const long long el = (long long)z.el;
    auto good = [&](long long b, long long h, long long s) {
        return b >= 0 && h >= 0 && s >= (long long)z.D && (b * el) % 16 == 0 && (h * el) % 16 == 0 && (s * el) % 16 == 0 && s * el <= (1ll << 24);
    };
    if (!good(L->qkv_stride_b, L->qkv_stride_h, L->qkv_stride_s) || !good(L->out_stride_b, L->out_stride_h, L->out_stride_s)) return MLSTM_EINVAL;
    if (L->gate_stride_b < 0 || L->gate_stride_h < 0 || L->gate_stride_s < 1) return MLSTM_EINVAL;
    if (L->gate_form != MLSTM_GATE_RAW && L->gate_form != MLSTM_GATE_LOGSIGMOID && L->gate_form != MLSTM_GATE_CUMSUM) return MLSTM_EINVAL;
    if (L->gate_form == MLSTM_GATE_CUMSUM && gate_dtype != MLSTM_F32) return MLSTM_EINVAL;
    const long long B = (long long)z.BH / NH, S = (long long)z.S, D = (long long)z.D;
    if (written_qkv && !non_overlapping(B, NH, S, L->qkv_stride_b, L->qkv_stride_h, L->qkv_stride_s, D)) return MLSTM_EINVAL;
    if (written_out && !non_overlapping(B, NH, S, L->out_stride_b, L->out_stride_h, L->out_stride_s, D)) return MLSTM_EINVAL;
    if (written_gates && !non_overlapping(B, NH, S, L->gate_stride_b, L->gate_stride_h, L->gate_stride_s, 1)) return MLSTM_EINVAL;
    for (const void* p : row_tensors)
        if (p && (reinterpret_cast<size_t>(p) & 15)) return MLSTM_EINVAL;
    z.la = Lay{L->qkv_stride_b, L->qkv_stride_h, L->qkv_stride_s, NH};
    z.lb = Lay{L->out_stride_b, L->out_stride_h, L->out_stride_s, NH};
    z.lg = Lay{L->gate_stride_b, L->gate_stride_h, L->gate_stride_s, NH};
    z.gate_form = L->gate_form;
    return 0;
}

// RAII for a stream-ordered scratch allocation when the caller brings no workspace
struct Scratch {
    void* p = nullptr; hipStream_t st; bool owned = false;
    int get(void* user, size_t user_bytes, size_t need, hipStream_t s) {
        st = s;
        if (user) { if (user_bytes < need) return MLSTM_EWORKSPACE; p = user; return 0; }
        hipError_t e = hipMallocAsync(&p, need, s);
        if (e != hipSuccess) return (int)e;
        owned = true;
        return 0;
    }
    ~Scratch() { if (owned && p) (void)hipFreeAsync(p, st); }
};

// Scratch of mlstm_forward_noalloc_ex: the forward's workspace as a file-scope device array, for callers that cannot
// allocate.  Every GPU the library runs on holds its own copy at its own address until the process ends; in host code
// the array's name is only a handle for hipGetSymbolAddress, never a device address, so the address is looked up once
// per device (with that device current) and everything after that -- kernel arguments included -- uses the pointer.
constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)MLSTM_NOALLOC_MAX_WORKSPACE;
static __device__ __align__(256) unsigned char scratch[NOALLOC_SCRATCH_BYTES];
// Error word of the kernels' bounded waits (mlstm_kernel_error): one int per GPU, zero when the library is loaded, only
// ever or-ed into by kernels and cleared by mlstm_kernel_error.
static __device__ int kernel_error_word;
constexpr int NOALLOC_MAX_DEVICES = 64;
void* g_scratch_ptr[NOALLOC_MAX_DEVICES] = {};
int* g_err_ptr[NOALLOC_MAX_DEVICES] = {};
std::mutex g_scratch_mu;
int symbols_of_current_device(char** scratch_out, int** err_out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= NOALLOC_MAX_DEVICES) return MLSTM_EINVAL;
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void *p = nullptr, *pe = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e == hipSuccess) e = hipGetSymbolAddress(&pe, HIP_SYMBOL(kernel_error_word));
        if (e != hipSuccess) return (int)e;
        if (!p || !pe) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = p;
        g_err_ptr[dev] = static_cast<int*>(pe);
    }
    if (scratch_out) *scratch_out = static_cast<char*>(g_scratch_ptr[dev]);
    if (err_out) *err_out = g_err_ptr[dev];
    return 0;
}
int g_spin_limit = 0;   // test aid (mlstm_set_spin_limit): 0 = the default bound
constexpr int DEFAULT_SPIN_LIMIT = 1 << 22;   // iterations of 64 cycles and an LDS read each: a fraction of a second
// error word and wait bound of the eight-wave row kernel
int arm_row_args(RowArgs& a) {
    if (int rc = symbols_of_current_device(nullptr, &a.err)) return rc;
    a.spin_limit = g_spin_limit == 0 ? DEFAULT_SPIN_LIMIT : g_spin_limit;
    return 0;
}

// the first Sizes::fwd() bytes of every workspace
struct FwdWs {
    double* G2; float *alpha2, *beta2, *ek2, *amax2, *mw, *bw;
    int L; size_t ncs; float* dC; char* Cst; char* Cst_lo; float* Nst;
    FwdWs(char* ws, const Sizes& z, int dtype, int D) {
        Carver c{ws, 0};
        G2 = c.take<double>(z.BH * z.NG);
        alpha2 = c.take<float>(z.BH * z.NG * 64);
        beta2 = c.take<float>(z.BH * z.NG * 64);
        ek2 = c.take<float>(z.BH * z.NG * 64);
        amax2 = c.take<float>(z.BH * z.NG * 2 + 64);   // (+64: the row kernels copy 64 floats from each tile's pair on)
        mw = c.take<float>(z.BH * z.S);
        bw = c.take<float>(z.BH * z.S);
        L = z.chunk_len();
        ncs = z.n_states(L);
        dC = c.take<float>(z.BH * ncs * z.D * z.D);
        Cst = c.take<char>(z.BH * ncs * z.D * z.D * z.el * z.parts());
        Cst_lo = z.precise ? Cst + z.BH * ncs * z.D * z.D * z.el : nullptr;
        Nst = c.take<float>(z.BH * ncs * z.D);
    }
    // the gate pre-pass in a buffer of its own (Sizes::gates() bytes) instead of the workspace
    void gates_at(char* p, const Sizes& z) {
        Carver c{p, 0};
        G2 = c.take<double>(z.BH * z.NG);
        alpha2 = c.take<float>(z.BH * z.NG * 64);
        beta2 = c.take<float>(z.BH * z.NG * 64);
        ek2 = c.take<float>(z.BH * z.NG * 64);
        amax2 = c.take<float>(z.BH * z.NG * 2 + 64);
    }
};

// The parts of a `saved` buffer (Sizes::saved() bytes)
struct SavedView {
    int* header; char* CstT = nullptr; float* Nst = nullptr; char* gates = nullptr; char* h_lo = nullptr;
    SavedView(char* sv, const Sizes& z) {
        header = reinterpret_cast<int*>(sv);
        char* p = sv + SAVED_HEADER_BYTES;
        if (z.saved_chunk() > 0) {
            CstT = p; p += z.states_t();
            Nst = reinterpret_cast<float*>(p); p += z.saved_vec();
            gates = p; p += z.gates();
        }
        if (z.precise) h_lo = p;
    }
};
SavedStamp saved_stamp_of(const Sizes& z) {
    SavedStamp s;
    const int v[8] = {SAVED_MAGIC, (int)z.BH, (int)z.S, (int)z.D, z.dtype_code | (z.precise ? MLSTM_PRECISE : 0), z.chunk_len(),
                      mlstm::g_force_generic ? 1 : 0, (int)z.n_states(z.chunk_len())};
    for (int t = 0; t < 8; t++) s.v[t] = v[t];
    return s;
}

// states at the chunk ends of a long sequence (both layouts when CstT is given; split mode: each as two terms, the
// second directly behind the first)
int chunk_states_impl(const void* k, const void* v, const FwdWs& w, bool key_major, void* CstT, float* Nst, const Sizes& z, int D, int dtype,
                      hipStream_t st) {
    ChunkArgs ca{k, v, w.alpha2, w.beta2, w.G2, w.dC, Nst, key_major ? w.Cst : nullptr, CstT, (int)z.BH, (int)z.S, (int)z.NG, w.L, (int)w.ncs,
                 0, nullptr, nullptr};
    ca.lk = ca.lv = z.la;
    ca.precise = z.precise ? 1 : 0;
    if (z.precise) {
        ca.Cst_lo = key_major ? w.Cst_lo : nullptr;
        ca.CstT_lo = CstT ? static_cast<char*>(CstT) + z.state_elems() * z.el : nullptr;
    }
    Timed t(MLSTM_K_CHUNK_STATES, st);
    return launch_chunk_states(dtype, D, ca, st);
}

// The scan form's pipeline on a workspace of Sizes::scan_fwd() bytes: gate pre-pass, in-chunk pairs and vector carry,
// matrix state walk, finish.  finish_mode as in ScanArgs; m_out / b_out (may be null) receive the stabiliser and the
// normaliser sums.
int scan_forward_impl(const void* q, const void* k, const void* v, const void* f, const void* i, const void* o, void* h, float* m_out,
                      float* b_out, const Sizes& z, int gate_dtype, int finish_mode, char* ws, hipStream_t st, float* h_ungated = nullptr) {
    Carver c{ws, 0};
    double* G2 = c.take<double>(z.BH * z.NG);
    float* alpha2 = c.take<float>(z.BH * z.NG * 64);
    float* beta2 = c.take<float>(z.BH * z.NG * 64);
    float* ek2 = c.take<float>(z.BH * z.NG * 64);
    float* amax2 = c.take<float>(z.BH * z.NG * 2 + 64);   // (+64: the row kernels copy 64 floats from each tile's pair on)
    float* m = c.take<float>(z.BH * z.S);
    float* bw = c.take<float>(z.BH * z.S);
    float* P = c.take<float>(z.BH * z.NG * 64 * 64);
    float* Nst = c.take<float>(z.BH * z.NG * z.D);
    const int KS = scan_key_splits((int)z.BH, (int)z.D);
    float* hpart = nullptr;
    for (int p = 1; p < KS; p++) { float* x = c.take<float>(z.BH * z.S * z.D); if (p == 1) hpart = x; }
    float* seg_state = c.take<float>(scan_segment_state_bytes((int)z.BH, (int)z.S, (int)z.D) / 4);
    if (m_out) m = m_out;
    (void)bw;
    {
        Timed t(MLSTM_K_GATES, st);
        hipError_t e = launch_gates(gate_dtype, f, i, alpha2, beta2, G2, m, ek2, amax2, (int)z.BH, (int)z.S, st, z.lg, z.gate_form);
        if (e != hipSuccess) return (int)e;
    }
    ScanArgs a{};
    a.q = (const float*)q; a.k = (const float*)k; a.v = (const float*)v; a.o = (const float*)o; a.h = (float*)h;
    a.alpha2 = alpha2; a.beta2 = beta2; a.G2 = G2; a.M = m; a.P = P; a.Nst = Nst; a.hpart = hpart;
    a.BH = (int)z.BH; a.S = (int)z.S; a.D = (int)z.D; a.NC = (int)z.NG;
    a.finish_mode = finish_mode; a.Bout = b_out; a.Hun = h_ungated; a.seg_state = seg_state;
    return launch_scan(a, KS, st, scan_mark);
}

int forward_impl(const void* q, const void* k, const void* v, const void* f, const void* i, void* h, float* m, float* b,
                 const Sizes& z, int D, int dtype, int gate_dtype, char* ws, hipStream_t st, float** alpha_out = nullptr,
                 float** beta_out = nullptr, double** g_out = nullptr, float** m_out = nullptr, float** b_out = nullptr,
                 float** ek_out = nullptr, float** amax_out = nullptr, const void* o = nullptr, void* h_gated = nullptr,
                 void* CstT = nullptr, float* Nst_ext = nullptr, char* gates_ext = nullptr, void* h_lo = nullptr,
                 const SavedStamp* stamp = nullptr) {
    if (z.scan_engine()) {
        // dense tensors only, no fused gate copy (mlstm_scan_forward_ex is the gated form of these kernels)
        if (o || h_gated || !is_dense(z.la, (long long)z.S, (long long)z.D) || !is_dense(z.lb, (long long)z.S, (long long)z.D)) return MLSTM_ESHAPE;
        return scan_forward_impl(q, k, v, f, i, nullptr, h, m, b, z, gate_dtype, 1, ws, st);
    }
    FwdWs w(ws, z, dtype, D);
    if (gates_ext) w.gates_at(gates_ext, z);
    double* G2 = w.G2; float *alpha2 = w.alpha2, *beta2 = w.beta2, *ek2 = w.ek2, *amax2 = w.amax2;
    const size_t ncs = w.ncs;
    if (!m) m = w.mw;
    if (!b) b = w.bw;
    {
        Timed t(MLSTM_K_GATES, st);
        hipError_t e = launch_gates(gate_dtype, f, i, alpha2, beta2, G2, m, ek2, amax2, (int)z.BH, (int)z.S, st, z.lg, z.gate_form, stamp);
        if (e != hipSuccess) return (int)e;
    }
    RowArgs a{};
    a.la = z.la; a.lb = z.lb; a.lh = z.lb;
    a.X = q; a.Y1 = k; a.Y2 = v; a.out = h; a.alpha2 = alpha2; a.beta2 = beta2; a.G2 = G2; a.M = m; a.Bsum = b;
    a.ek2 = ek2; a.amax2 = amax2; a.O = o; a.out_gated = h_gated;
    a.BH = (int)z.BH; a.S = (int)z.S; a.NG = (int)z.NG;
    a.precise = z.precise ? 1 : 0; a.out_lo = h_lo;
    if (int rc = arm_row_args(a)) return rc;
    if (ncs > 0) {   // long sequence: the states at the chunk ends first, then every row tile stays inside its chunk
        float* Nst = Nst_ext ? Nst_ext : w.Nst;
        if (int e = chunk_states_impl(k, v, w, true, CstT, Nst, z, D, dtype, st)) return e;
        a.chunk_len = w.L; a.n_states = (int)ncs; a.Cst = w.Cst; a.Cst_lo = w.Cst_lo; a.Nst = Nst;
    }
    int rc;
    {
        Timed t(MLSTM_K_ROW_FWD, st);
        rc = launch_row_best(0, dtype, D, a, st);
    }
    if (alpha_out) { *alpha_out = alpha2; *beta_out = beta2; *g_out = G2; *m_out = m; *b_out = b; *ek_out = ek2; *amax_out = amax2; }
    return rc;
}

}  // namespace

extern "C" {

const char* mlstm_version(void) { return "mlstm_hip 0.1 gfx950"; }

int mlstm_force_generic_kernels(int on) {
    const int before = mlstm::g_force_generic ? 1 : 0;
    mlstm::g_force_generic = on != 0;
    return before;
}

int mlstm_set_column_kernel(int variant) {
    if (variant < 0 || variant > 3) return MLSTM_EINVAL;
    mlstm::g_col_variant = variant;
    return 0;
}

int mlstm_chunk_length_for(int S, int D, int dtype) {
    if (S <= 0 || D <= 0 || !good_dtype_arg(dtype)) return 0;
    return chunk_len_for(dtype & ~MLSTM_PRECISE, D, (size_t)S);
}

int mlstm_set_state_kernel(int variant) { return mlstm::set_state_kernel(variant); }

int mlstm_set_chunk_length(int length) {
    if (length > 0 && length % 128 != 0) return MLSTM_EINVAL;
    g_chunk_override = length;
    return 0;
}

int mlstm_set_spin_limit(int limit) {
    g_spin_limit = limit;
    return 0;
}

int mlstm_init(void) { return symbols_of_current_device(nullptr, nullptr); }

int mlstm_kernel_error(void) {
    int* word = nullptr;
    if (int rc = symbols_of_current_device(nullptr, &word)) return rc;
    // Every stream of the device, the non-blocking ones included (a plain copy on the null stream waits for the
    // blocking streams only); with the device idle the read and the clear below cannot lose an error in between.
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return (int)e;
    int value = 0;
    e = hipMemcpy(&value, word, sizeof(int), hipMemcpyDeviceToHost);
    if (e != hipSuccess) return (int)e;
    if (value != 0) {
        const int zero = 0;
        e = hipMemcpy(word, &zero, sizeof(int), hipMemcpyHostToDevice);
        if (e != hipSuccess) return (int)e;
        return (value & 1) ? MLSTM_EKERNEL : MLSTM_ESAVED;
    }
    return 0;
}

int mlstm_timing_enable(int on) {
    std::lock_guard<std::mutex> lk(g_timing.mu);
    g_timing.on = on != 0;
    return 0;
}

int mlstm_timing_select(unsigned mask, int every) {
    if (every < 1) return MLSTM_EINVAL;
    std::lock_guard<std::mutex> lk(g_timing.mu);
    g_timing.mask = mask;
    g_timing.every = every;
    for (int& c : g_timing.seen) c = 0;
    return 0;
}

int mlstm_timing_read(int kernel, double* total_ms, int* launches) {
    if (!total_ms || !launches) return MLSTM_EINVAL;
    std::lock_guard<std::mutex> lk(g_timing.mu);
    double tot = 0.0; int n = 0;
    std::vector<TimingState::Rec> keep;
    for (auto& r : g_timing.recs) {
        if (r.id != kernel) { keep.push_back(r); continue; }
        float ms = 0.f;
        hipError_t e = hipEventSynchronize(r.b);
        if (e == hipSuccess) e = hipEventElapsedTime(&ms, r.a, r.b);
        (void)hipEventDestroy(r.a); (void)hipEventDestroy(r.b);
        if (e != hipSuccess) return (int)e;
        tot += ms; n++;
    }
    g_timing.recs.swap(keep);
    *total_ms = tot; *launches = n;
    return 0;
}

size_t mlstm_workspace_bytes(int op, int B, int NH, int S, int D, int dtype) {
    if (B <= 0 || NH <= 0 || S <= 0 || D <= 0 || !good_dtype_arg(dtype)) return 0;
    const Sizes z = sizes_of(B, NH, S, D, dtype);
    switch (op) {
        case MLSTM_OP_FORWARD: return z.fwd();
        case MLSTM_OP_BACKWARD: return z.bwd();
        case MLSTM_OP_FORWARD_GATED: return z.fwd();
        case MLSTM_OP_BACKWARD_GATED: return z.bwd_gated();
        case MLSTM_OP_SCAN_FORWARD: return z.scan_fwd();
        case MLSTM_OP_SCAN_BACKWARD:
            return (D % 64 == 0 && D >= 64) ? scan_backward_workspace_bytes((int)z.BH, S, D) : 0;
    }
    return 0;
}

int mlstm_forward_ex(const void* q, const void* k, const void* v, const void* f, const void* i, void* h, float* m, float* b,
                     int B, int NH, int S, int D, int dtype, int gate_dtype, void* workspace, size_t workspace_bytes,
                     void* stream) {
    return mlstm_forward_lx(q, k, v, f, i, h, m, b, B, NH, S, D, dtype, gate_dtype, nullptr, workspace, workspace_bytes, stream);
}

int mlstm_forward_lx(const void* q, const void* k, const void* v, const void* f, const void* i, void* h, float* m, float* b,
                     int B, int NH, int S, int D, int dtype, int gate_dtype, const mlstm_layout* layout, void* workspace,
                     size_t workspace_bytes, void* stream) {
    if (!q || !k || !v || !f || !i || !h || B <= 0 || NH <= 0 || S <= 0 || !good_dtype_arg(dtype) || !good_dtype(gate_dtype))
        return MLSTM_EINVAL;
    const int dtype_arg = dtype;
    dtype &= ~MLSTM_PRECISE;
    if (!good_shape(D, dtype) || S > 131072) return MLSTM_ESHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    Sizes z = sizes_of(B, NH, S, D, dtype_arg);
    if (int rc = apply_layout(z, layout, NH, gate_dtype, {q, k, v, h}, false, true, false)) return rc;
    Scratch sc;
    if (int rc = sc.get(workspace, workspace_bytes, z.fwd(), st)) return rc;
    return forward_impl(q, k, v, f, i, h, m, b, z, D, dtype, gate_dtype, (char*)sc.p, st);
}

int mlstm_forward_noalloc_ex(const void* q, const void* k, const void* v, const void* f, const void* i, void* h, float* m, float* b,
                             int B, int NH, int S, int D, int dtype, int gate_dtype, void* stream) {
    if (!q || !k || !v || !f || !i || !h || B <= 0 || NH <= 0 || S <= 0 || !good_dtype_arg(dtype) || !good_dtype(gate_dtype))
        return MLSTM_EINVAL;
    const int dtype_arg = dtype;
    dtype &= ~MLSTM_PRECISE;
    if (!good_shape(D, dtype) || S > 131072) return MLSTM_ESHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const Sizes z = sizes_of(B, NH, S, D, dtype_arg);
    if (z.fwd() > NOALLOC_SCRATCH_BYTES) return MLSTM_EWORKSPACE;   // the shape needs more scratch than the array holds
    char* ws = nullptr;
    if (int rc = symbols_of_current_device(&ws, nullptr)) return rc;
    // Nothing in the workspace has to start at zero: the gate pre-pass writes every element the tile kernels read,
    // padding included, and the states are written before they are read; what the previous call left is overwritten.
    return forward_impl(q, k, v, f, i, h, m, b, z, D, dtype, gate_dtype, ws, st);
}

size_t mlstm_saved_state_bytes(int B, int NH, int S, int D, int dtype) {
    if (B <= 0 || NH <= 0 || S <= 0 || D <= 0 || !good_dtype_arg(dtype)) return 0;
    const Sizes z = sizes_of(B, NH, S, D, dtype);
    return z.saved();
}

int mlstm_forward_save_ex(const void* q, const void* k, const void* v, const void* f, const void* i, void* h, float* m, float* b,
                          void* saved, size_t saved_bytes, int B, int NH, int S, int D, int dtype, int gate_dtype, void* workspace,
                          size_t workspace_bytes, void* stream) {
    return mlstm_forward_save_lx(q, k, v, f, i, h, m, b, saved, saved_bytes, B, NH, S, D, dtype, gate_dtype, nullptr, workspace,
                                 workspace_bytes, stream);
}

int mlstm_forward_save_lx(const void* q, const void* k, const void* v, const void* f, const void* i, void* h, float* m, float* b,
                          void* saved, size_t saved_bytes, int B, int NH, int S, int D, int dtype, int gate_dtype,
                          const mlstm_layout* layout, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k || !v || !f || !i || !h || B <= 0 || NH <= 0 || S <= 0 || !good_dtype_arg(dtype) || !good_dtype(gate_dtype))
        return MLSTM_EINVAL;
    const int dtype_arg = dtype;
    dtype &= ~MLSTM_PRECISE;
    if (!good_shape(D, dtype) || S > 131072) return MLSTM_ESHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    Sizes z = sizes_of(B, NH, S, D, dtype_arg);
    if (int rc = apply_layout(z, layout, NH, gate_dtype, {q, k, v, h}, false, true, false)) return rc;
    if (z.saved() > 0 && (!saved || saved_bytes != z.saved())) return MLSTM_EWORKSPACE;
    Scratch sc;
    if (int rc = sc.get(workspace, workspace_bytes, z.fwd(), st)) return rc;
    if (z.saved() == 0) return forward_impl(q, k, v, f, i, h, m, b, z, D, dtype, gate_dtype, (char*)sc.p, st);
    SavedView sv((char*)saved, z);
    SavedStamp stamp = saved_stamp_of(z);
    stamp.dst = sv.header;
    return forward_impl(q, k, v, f, i, h, m, b, z, D, dtype, gate_dtype, (char*)sc.p, st, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                        nullptr, nullptr, nullptr, sv.CstT, sv.Nst, sv.gates, sv.h_lo, &stamp);
}

int mlstm_forward_gated_ex(const void* q, const void* k, const void* v, const void* f, const void* i, const void* o, void* h,
                           void* h_gated, float* m, float* b, int B, int NH, int S, int D, int dtype, int gate_dtype, void* workspace,
                           size_t workspace_bytes, void* stream) {
    return mlstm_forward_gated_lx(q, k, v, f, i, o, h, h_gated, m, b, B, NH, S, D, dtype, gate_dtype, nullptr, workspace, workspace_bytes, stream);
}

int mlstm_forward_gated_lx(const void* q, const void* k, const void* v, const void* f, const void* i, const void* o, void* h,
                           void* h_gated, float* m, float* b, int B, int NH, int S, int D, int dtype, int gate_dtype,
                           const mlstm_layout* layout, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k || !v || !f || !i || !o || !h || !h_gated || B <= 0 || NH <= 0 || S <= 0 || !good_dtype_arg(dtype) || !good_dtype(gate_dtype))
        return MLSTM_EINVAL;
    const int dtype_arg = dtype;
    dtype &= ~MLSTM_PRECISE;
    if (!good_shape(D, dtype) || S > 131072) return MLSTM_ESHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    Sizes z = sizes_of(B, NH, S, D, dtype_arg);
    if (layout && z.scan_engine()) return MLSTM_ESHAPE;
    if (int rc = apply_layout(z, layout, NH, gate_dtype, {q, k, v, o, h, h_gated}, false, true, false)) return rc;   // (o, h, h_gated: the layout of h)
    Scratch sc;
    if (int rc = sc.get(workspace, workspace_bytes, z.fwd(), st)) return rc;
    return forward_impl(q, k, v, f, i, h, m, b, z, D, dtype, gate_dtype, (char*)sc.p, st, nullptr, nullptr, nullptr, nullptr, nullptr,
                        nullptr, nullptr, o, h_gated);
}

}  // extern "C"

namespace {

// the backward on a workspace of Sizes::bwd() bytes; arguments already validated
int backward_impl(const void* dh, const void* q, const void* k, const void* v, const void* f, const void* i, const void* h, const float* m,
                  const float* b, void* dq, void* dk, void* dv, void* df, void* di, const Sizes& z, int D, int dtype, int gate_dtype,
                  char* ws, hipStream_t st, const char* saved = nullptr, const Lay* h_layout = nullptr) {
    if (z.scan_engine()) {   // (recomputes the forward it needs; h, m, b are not read)
        if (!is_dense(z.la, (long long)z.S, (long long)z.D) || !is_dense(z.lb, (long long)z.S, (long long)z.D) ||
            !is_dense(z.lg, (long long)z.S, 1) || z.gate_form != MLSTM_GATE_RAW || gate_dtype != MLSTM_F32)
            return MLSTM_ESHAPE;
        ScanBwdArgs a{};
        a.dhg = (const float*)dh; a.q = (const float*)q; a.k = (const float*)k; a.v = (const float*)v;
        a.f = (const float*)f; a.i = (const float*)i; a.o = nullptr;
        a.dq = (float*)dq; a.dk = (float*)dk; a.dv = (float*)dv; a.df = (float*)df; a.di = (float*)di; a.d_o = nullptr;
        a.BH = (int)z.BH; a.S = (int)z.S; a.D = D;
        return launch_scan_backward(a, ws, st, scan_mark);
    }
    Carver c{ws, z.fwd()};
    char* hbuf = c.take<char>(z.BH * z.S * z.D * z.el);
    float* inv_n = c.take<float>(z.BH * z.NG * 64);
    float* dbuf = c.take<float>(z.BH * z.NG * 64);
    float* colsum = c.take<float>(z.BH * z.S);
    float* rowpart = c.take<float>(z.BH * z.row_slices() * z.S);
    FwdWs w(ws, z, dtype, D);
    char* CstT = c.take<char>(z.state_elems() * z.el * z.parts());
    const float* Nst = w.Nst;
    const bool reuse = saved && w.ncs > 0;
    const void* h_lo = nullptr;   // split mode: the low-order part of h, from the forward (saved) or from a recomputation
    SavedStamp stamp;
    if (saved) {
        SavedView sv(const_cast<char*>(saved), z);
        // the header is compared on the device (by the last kernel of this pass): a buffer written for another shape,
        // type or setting (chunk length, kernel switch) sets bit 1 of the error word, which mlstm_kernel_error reports
        stamp = saved_stamp_of(z);
        stamp.src = sv.header;
        if (int rc = symbols_of_current_device(nullptr, &stamp.err)) return rc;
        if (reuse) {   // the forward's states (value-major matrices, then the vectors) and its gate pre-pass
            CstT = sv.CstT;
            Nst = sv.Nst;
            w.gates_at(sv.gates, z);
        }
        h_lo = sv.h_lo;
    }
    char* Ev = c.take<char>(z.state_elems() * z.el * z.parts());    // reverse states, value-major
    float* gvec = c.take<float>(z.BH * w.ncs * z.D);
    float* rowinter = c.take<float>(z.BH * z.S);
    float* anchor = c.take<float>(z.BH * w.ncs * z.anchor_parts());
    int anchor_parts = 0;
    // (the one-kernel dF pass adds the parts up; see DfArgs)
    const bool fused_anchor = w.L <= 1024 && mlstm::chunk_states_fused_dot(dtype, D);
    char* hlo_buf = c.take<char>(z.precise ? z.BH * z.S * z.D * z.el : 0);
    const size_t lo_off = z.state_elems() * z.el;   // split mode: a set of states is [hi | lo]
    const bool col_chunks = z.col_chunks();

    float *alpha2, *beta2, *mm, *bb, *ek2, *amax2; double* G2;
    // Split mode needs h beyond the element type's precision for dh . h: either the forward left the low-order part
    // (saved), or the forward is run again here
    const bool have_fwd = h && m && b && (!z.precise || h_lo);
    Lay lh = h_layout ? *h_layout : z.lb;   // layout of the forward output the dQ pass reads (dh's, unless the caller says otherwise)
    if (have_fwd) {
        // gates only: alpha, beta, G (and m again, into the workspace) are cheap to rebuild; so are the chunk states
        G2 = w.G2; alpha2 = w.alpha2; beta2 = w.beta2; ek2 = w.ek2; amax2 = w.amax2; mm = w.mw;
        if (reuse) {
            mm = const_cast<float*>(m);
        } else {
            Timed t(MLSTM_K_GATES, st);
            hipError_t e = launch_gates(gate_dtype, f, i, alpha2, beta2, G2, mm, ek2, amax2, (int)z.BH, (int)z.S, st, z.lg, z.gate_form);
            if (e != hipSuccess) return (int)e;
        }
        bb = const_cast<float*>(b);
        if (w.ncs > 0 && !saved)
            if (int e = chunk_states_impl(k, v, w, false, CstT, w.Nst, z, D, dtype, st)) return e;   // (the dQ pass wants them value-major only)
    } else {
        Sizes zf = z;            // (the recomputed h is the library's own, dense)
        zf.lb = lh = dense_layout(z.la.NH, (long long)z.S, (long long)z.D);
        int rc = forward_impl(q, k, v, f, i, hbuf, nullptr, nullptr, zf, D, dtype, gate_dtype, ws, st, &alpha2, &beta2, &G2, &mm, &bb, &ek2, &amax2,
                              nullptr, nullptr, CstT, nullptr, nullptr, z.precise ? hlo_buf : nullptr);
        Nst = w.Nst;
        if (rc) return rc;
        h = hbuf;
        if (z.precise) h_lo = hlo_buf;
    }
    // dQ first: it derives 1/n and db per row from (dh, h, m, b) and leaves them for the column kernel
    RowArgs ra{};
    ra.la = z.la; ra.lb = z.lb; ra.lh = lh;
    ra.X = dh; ra.Y1 = v; ra.Y2 = k; ra.out = dq; ra.alpha2 = alpha2; ra.beta2 = beta2; ra.G2 = G2; ra.inv_n = inv_n; ra.db = dbuf;
    ra.ek2 = ek2; ra.amax2 = amax2; ra.Hin = h; ra.Bin = bb; ra.M = mm;
    ra.BH = (int)z.BH; ra.S = (int)z.S; ra.NG = (int)z.NG;
    ra.precise = z.precise ? 1 : 0; ra.Hin_lo = h_lo;
    if (int rc = arm_row_args(ra)) return rc;
    if (w.ncs > 0) {
        ra.chunk_len = w.L; ra.n_states = (int)w.ncs; ra.Cst = CstT; ra.Cst_lo = z.precise ? CstT + lo_off : nullptr; ra.Nst = Nst; ra.Qrow = q;
        ra.rowinter = rowinter;
    }
    {
        Timed t(MLSTM_K_ROW_DQ, st);
        if (int rc = launch_row_best(1, dtype, D, ra, st)) return rc;
    }

    if (col_chunks) {
        // reverse states from (Q, dH) and the dQ pass's per-row scalars (the column kernel applies them to its keys
        // itself), and the dF anchors at the chunk boundaries
        Timed t(MLSTM_K_CHUNK_STATES, st);
        ChunkArgs ra2{q, dh, alpha2, beta2, G2, w.dC, gvec, nullptr, Ev, (int)z.BH, (int)z.S, (int)z.NG, w.L, (int)w.ncs, 1, inv_n, dbuf};
        ra2.lk = z.la; ra2.lv = z.lb;
        ra2.precise = z.precise ? 1 : 0;
        ra2.CstT_lo = z.precise ? Ev + lo_off : nullptr;
        if (fused_anchor) {
            ra2.dot_with = CstT; ra2.dot_with_lo = z.precise ? CstT + lo_off : nullptr; ra2.dot_part = anchor;
            anchor_parts = mlstm::chunk_states_dot_parts(dtype, D, ra2);
        }
        if (int e = launch_chunk_states(dtype, D, ra2, st)) return e;
        if (fused_anchor) {
        } else if (int e = launch_anchor(dtype, D, CstT, Ev, z.precise ? CstT + lo_off : nullptr, z.precise ? Ev + lo_off : nullptr, Nst, gvec, anchor,
                                  (int)z.BH, (int)w.ncs, st))
            return e;   // (both value-major)
    }
    ColArgs ca{};
    ca.la = z.la; ca.lb = z.lb;
    ca.Q = q; ca.K = k; ca.V = v; ca.dH = dh; ca.dK = dk; ca.dV = dv; ca.colsum = colsum; ca.rowpart = rowpart;
    ca.alpha2 = alpha2; ca.beta2 = beta2; ca.G2 = G2; ca.inv_n = inv_n; ca.db = dbuf;
    ca.BH = (int)z.BH; ca.S = (int)z.S; ca.NG = (int)z.NG;
    ca.precise = z.precise ? 1 : 0; ca.RS = (int)z.row_slices();
    if (col_chunks) { ca.chunk_len = w.L; ca.n_states = (int)w.ncs; ca.Ev = Ev; ca.Ev_lo = z.precise ? Ev + lo_off : nullptr; ca.gvec = gvec; }
    {
        Timed t(MLSTM_K_COL, st);
        if (int rc = launch_col_best(dtype, D, ca, st)) return rc;
    }

    DfArgs da{f, colsum, rowpart, df, di, (int)z.BH, (int)z.S, (int)z.NG, (int)z.row_slices(), col_chunks ? w.L : 0, rowinter, anchor, (int)w.ncs};
    da.lg = z.lg; da.gate_form = z.gate_form; da.stamp = stamp;
    if (col_chunks && fused_anchor) {
        da.anchor = nullptr; da.anchor_part = anchor; da.anchor_parts = anchor_parts; da.anchor_va = Nst; da.anchor_vb = gvec; da.D = D;
    }
    Timed t(MLSTM_K_DF, st);
    return launch_df(gate_dtype, da, st);
}

}  // namespace

extern "C" {

int mlstm_backward_ex(const void* dh, const void* q, const void* k, const void* v, const void* f, const void* i, const void* h,
                      const float* m, const float* b, void* dq, void* dk, void* dv, void* df, void* di, int B, int NH, int S,
                      int D, int dtype, int gate_dtype, void* workspace, size_t workspace_bytes, void* stream) {
    return mlstm_backward_lx(dh, q, k, v, f, i, h, m, b, dq, dk, dv, df, di, B, NH, S, D, dtype, gate_dtype, nullptr, workspace, workspace_bytes,
                             stream);
}

int mlstm_backward_lx(const void* dh, const void* q, const void* k, const void* v, const void* f, const void* i, const void* h,
                      const float* m, const float* b, void* dq, void* dk, void* dv, void* df, void* di, int B, int NH, int S,
                      int D, int dtype, int gate_dtype, const mlstm_layout* layout, void* workspace, size_t workspace_bytes, void* stream) {
    if (!dh || !q || !k || !v || !f || !i || !dq || !dk || !dv || !df || !di || B <= 0 || NH <= 0 || S <= 0 || !good_dtype_arg(dtype) ||
        !good_dtype(gate_dtype))
        return MLSTM_EINVAL;
    const int dtype_arg = dtype;
    dtype &= ~MLSTM_PRECISE;
    if (!good_shape(D, dtype) || S > 131072) return MLSTM_ESHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    Sizes z = sizes_of(B, NH, S, D, dtype_arg);
    if (int rc = apply_layout(z, layout, NH, gate_dtype, {dh, q, k, v, h, dq, dk, dv}, true, false, true)) return rc;
    Scratch sc;
    if (int rc = sc.get(workspace, workspace_bytes, z.bwd(), st)) return rc;
    return backward_impl(dh, q, k, v, f, i, h, m, b, dq, dk, dv, df, di, z, D, dtype, gate_dtype, (char*)sc.p, st);
}

int mlstm_backward_saved_ex(const void* dh, const void* q, const void* k, const void* v, const void* f, const void* i, const void* h,
                            const float* m, const float* b, const void* saved, size_t saved_bytes, void* dq, void* dk, void* dv, void* df,
                            void* di, int B, int NH, int S, int D, int dtype, int gate_dtype, void* workspace, size_t workspace_bytes,
                            void* stream) {
    return mlstm_backward_saved_lx(dh, q, k, v, f, i, h, m, b, saved, saved_bytes, dq, dk, dv, df, di, B, NH, S, D, dtype, gate_dtype, nullptr,
                                   workspace, workspace_bytes, stream);
}

int mlstm_backward_saved_lx(const void* dh, const void* q, const void* k, const void* v, const void* f, const void* i, const void* h,
                            const float* m, const float* b, const void* saved, size_t saved_bytes, void* dq, void* dk, void* dv, void* df,
                            void* di, int B, int NH, int S, int D, int dtype, int gate_dtype, const mlstm_layout* layout, void* workspace,
                            size_t workspace_bytes, void* stream) {
    if (!dh || !q || !k || !v || !f || !i || !h || !m || !b || !dq || !dk || !dv || !df || !di || B <= 0 || NH <= 0 || S <= 0 ||
        !good_dtype_arg(dtype) || !good_dtype(gate_dtype))
        return MLSTM_EINVAL;
    const int dtype_arg = dtype;
    dtype &= ~MLSTM_PRECISE;
    if (!good_shape(D, dtype) || S > 131072) return MLSTM_ESHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    Sizes z = sizes_of(B, NH, S, D, dtype_arg);
    if (int rc = apply_layout(z, layout, NH, gate_dtype, {dh, q, k, v, h, dq, dk, dv}, true, false, true)) return rc;
    if (z.saved() > 0 && (!saved || saved_bytes != z.saved())) return MLSTM_EWORKSPACE;
    Scratch sc;
    if (int rc = sc.get(workspace, workspace_bytes, z.bwd(), st)) return rc;
    return backward_impl(dh, q, k, v, f, i, h, m, b, dq, dk, dv, df, di, z, D, dtype, gate_dtype, (char*)sc.p, st,
                         z.saved() > 0 ? (const char*)saved : nullptr);
}

int mlstm_backward_gated_ex(const void* dh_gated, const void* q, const void* k, const void* v, const void* f, const void* i, const void* o,
                            const void* h, const float* m, const float* b, void* dq, void* dk, void* dv, void* df, void* di, void* d_o,
                            int B, int NH, int S, int D, int dtype, int gate_dtype, void* workspace, size_t workspace_bytes, void* stream) {
    return mlstm_backward_gated_lx(dh_gated, q, k, v, f, i, o, h, m, b, dq, dk, dv, df, di, d_o, B, NH, S, D, dtype, gate_dtype, nullptr, workspace,
                                   workspace_bytes, stream);
}

int mlstm_backward_gated_lx(const void* dh_gated, const void* q, const void* k, const void* v, const void* f, const void* i, const void* o,
                            const void* h, const float* m, const float* b, void* dq, void* dk, void* dv, void* df, void* di, void* d_o,
                            int B, int NH, int S, int D, int dtype, int gate_dtype, const mlstm_layout* layout, void* workspace,
                            size_t workspace_bytes, void* stream) {
    if (!dh_gated || !q || !k || !v || !f || !i || !o || !dq || !dk || !dv || !df || !di || !d_o || B <= 0 || NH <= 0 || S <= 0 ||
        !good_dtype_arg(dtype) || !good_dtype(gate_dtype))
        return MLSTM_EINVAL;
    const int dtype_arg = dtype;
    dtype &= ~MLSTM_PRECISE;
    if (!good_shape(D, dtype) || S > 131072) return MLSTM_ESHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    Sizes z = sizes_of(B, NH, S, D, dtype_arg);
    if (layout && z.scan_engine()) return MLSTM_ESHAPE;
    // dh_gated, o, h and d_o in the layout of h; q, k, v and their gradients, the gates and theirs as in mlstm_backward_lx
    if (int rc = apply_layout(z, layout, NH, gate_dtype, {dh_gated, q, k, v, o, h, dq, dk, dv, d_o}, true, true, true)) return rc;
    Scratch sc;
    if (int rc = sc.get(workspace, workspace_bytes, z.bwd_gated(), st)) return rc;
    char* ws = (char*)sc.p;
    Carver c{ws, z.bwd()};
    char* dh = c.take<char>(z.BH * z.S * z.D * z.el);
    char* hown = c.take<char>(z.BH * z.S * z.D * z.el);
    float* mown = c.take<float>(z.BH * z.S);
    float* bown = c.take<float>(z.BH * z.S);
    const Lay dense = dense_layout(NH, (long long)z.S, (long long)z.D);
    Lay lh = z.lb;
    if (!(h && m && b)) {  // the ungated h is an input of the gate's own backward: rebuild it (and m, b) first, dense
        Sizes zf = z;
        zf.lb = dense;
        if (int rc = forward_impl(q, k, v, f, i, hown, mown, bown, zf, D, dtype, gate_dtype, ws, st)) return rc;
        h = hown; m = mown; b = bown;
        lh = dense;
    }
    {
        Timed t(MLSTM_K_GATE_BWD, st);
        if (!layout) {
            if (int rc = launch_gate_backward(dtype, dh_gated, o, h, dh, d_o, z.BH * z.S * z.D, st)) return rc;
        } else if (int rc = launch_gate_backward_rows(dtype, dh_gated, o, h, dh, d_o, (int)z.BH, (int)z.S, (int)z.D, z.lb, lh, dense, st)) {
            return rc;
        }
    }
    // the ungated upstream gradient is the library's own, dense; h stays where it is
    Sizes zb = z;
    zb.lb = dense;
    return backward_impl(dh, q, k, v, f, i, h, m, b, dq, dk, dv, df, di, zb, D, dtype, gate_dtype, ws, st, nullptr, &lh);
}

int mlstm_forward(const void* Q, const void* K, const void* V, const void* F, const void* I, void* H, unsigned S) {
    return mlstm_forward_ex(Q, K, V, F, I, H, nullptr, nullptr, 1, 1, (int)S, 128, MLSTM_F16, MLSTM_F16, nullptr, 0, nullptr);
}

int mlstm_backward(const void* dH, const void* Q, const void* K, const void* V, const void* F, const void* I, const void* M,
                   const void* B, void* dQ, void* dK, void* dV, void* dF, void* dI, unsigned S) {
    (void)M; (void)B;
    return mlstm_backward_ex(dH, Q, K, V, F, I, nullptr, nullptr, nullptr, dQ, dK, dV, dF, dI, 1, 1, (int)S, 128, MLSTM_F16,
                             MLSTM_F16, nullptr, 0, nullptr);
}

int mlstm_scan_forward_ex(const void* q, const void* k, const void* v, const void* f, const void* i, const void* o, void* h, int B,
                          int NH, int S, int D, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
    if (!q || !k || !v || !f || !i || !o || !h || B <= 0 || NH <= 0 || S <= 0) return MLSTM_EINVAL;
    if (dtype != MLSTM_F32) return MLSTM_ESHAPE;  // the scan form is fp32, like the reference's
    if (!(D == 64 || D == 128 || D == 256 || D == 512 || D == 1024) || S > 131072) return MLSTM_ESHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const Sizes z = sizes_of(B, NH, S, D, MLSTM_F32);
    Scratch sc;
    if (int rc = sc.get(workspace, workspace_bytes, z.scan_fwd(), st)) return rc;
    return scan_forward_impl(q, k, v, f, i, o, h, nullptr, nullptr, z, MLSTM_F32, 0, (char*)sc.p, st);
}

int mlstm_scan_forward_save_ex(const void* q, const void* k, const void* v, const void* f, const void* i, const void* o, void* h,
                               void* h_ungated, float* b, int B, int NH, int S, int D, int dtype, void* workspace,
                               size_t workspace_bytes, void* stream) {
    if (!q || !k || !v || !f || !i || !o || !h || !h_ungated || !b || B <= 0 || NH <= 0 || S <= 0) return MLSTM_EINVAL;
    if (dtype != MLSTM_F32) return MLSTM_ESHAPE;
    if (!(D == 64 || D == 128 || D == 256 || D == 512 || D == 1024) || S > 131072) return MLSTM_ESHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const Sizes z = sizes_of(B, NH, S, D, MLSTM_F32);
    Scratch sc;
    if (int rc = sc.get(workspace, workspace_bytes, z.scan_fwd(), st)) return rc;
    return scan_forward_impl(q, k, v, f, i, o, h, nullptr, b, z, MLSTM_F32, 0, (char*)sc.p, st, (float*)h_ungated);
}

int mlstm_scan_backward_ex(const void* dh_gated, const void* q, const void* k, const void* v, const void* f, const void* i,
                           const void* o, void* dq, void* dk, void* dv, void* df, void* di, void* d_o, int B, int NH, int S, int D,
                           int dtype, void* workspace, size_t workspace_bytes, void* stream) {
    return mlstm_scan_backward_saved_ex(dh_gated, q, k, v, f, i, o, nullptr, nullptr, dq, dk, dv, df, di, d_o, B, NH, S, D, dtype,
                                        workspace, workspace_bytes, stream);
}

int mlstm_scan_backward_saved_ex(const void* dh_gated, const void* q, const void* k, const void* v, const void* f, const void* i,
                                 const void* o, const void* h_ungated, const float* b, void* dq, void* dk, void* dv, void* df,
                                 void* di, void* d_o, int B, int NH, int S, int D, int dtype, void* workspace,
                                 size_t workspace_bytes, void* stream) {
    if (!dh_gated || !q || !k || !v || !f || !i || !o || !dq || !dk || !dv || !df || !di || !d_o || B <= 0 || NH <= 0 || S <= 0)
        return MLSTM_EINVAL;
    if ((h_ungated == nullptr) != (b == nullptr)) return MLSTM_EINVAL;   // both kept, or neither
    if (dtype != MLSTM_F32) return MLSTM_ESHAPE;
    if (!(D == 64 || D == 128 || D == 256 || D == 512 || D == 1024) || S > 131072) return MLSTM_ESHAPE;
    hipStream_t st = reinterpret_cast<hipStream_t>(stream);
    const size_t need = scan_backward_workspace_bytes(B * NH, S, D);
    Scratch sc;
    if (int rc = sc.get(workspace, workspace_bytes, need, st)) return rc;
    ScanBwdArgs a{};
    a.dhg = (const float*)dh_gated; a.q = (const float*)q; a.k = (const float*)k; a.v = (const float*)v;
    a.f = (const float*)f; a.i = (const float*)i; a.o = (const float*)o;
    a.dq = (float*)dq; a.dk = (float*)dk; a.dv = (float*)dv; a.df = (float*)df; a.di = (float*)di; a.d_o = (float*)d_o;
    a.BH = B * NH; a.S = S; a.D = D;
    a.h_kept = (const float*)h_ungated; a.b_kept = b;
    return launch_scan_backward(a, (char*)sc.p, st, scan_mark);
}

}  // extern "C"
