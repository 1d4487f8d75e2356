"""ctypes binding of libmlstm_hip.so (declared in include/mlstm_hip.h)."""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmlstm_hip.so")

F32, F16, BF16 = 0, 1, 2
PRECISE = 0x100   # MLSTM_PRECISE, or-ed into the dtype code: split mode of the 16-bit kernels
OP_FORWARD, OP_BACKWARD, OP_SCAN_FORWARD, OP_FORWARD_GATED, OP_BACKWARD_GATED, OP_SCAN_BACKWARD = 0, 1, 2, 3, 4, 5
NOALLOC_MAX_WORKSPACE = 8 << 20   # MLSTM_NOALLOC_MAX_WORKSPACE
_DTYPES = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}
_ERRORS = {-1: "invalid argument (null pointer, non-positive size or unknown dtype)",
           -2: "unsupported shape (head dimension / sequence length)",
           -3: "workspace (or saved buffer) too small or of the wrong size",
           -4: "a kernel's bounded wait expired",
           -5: "a backward was given a saved buffer written for another shape or setting",
           -6: "a kernel with hand-counted memory waits was compiled with register spills"}

GATE_FORMS = {"raw": 0, "logsigmoid": 1, "cumsum": 2}   # MLSTM_GATE_RAW / _LOGSIGMOID / _CUMSUM


class Layout(ctypes.Structure):
    """struct mlstm_layout: element strides (batch, head, position) of q/k/v, of h/dh and of the gates; what f holds."""
    _fields_ = [(n, ctypes.c_longlong) for n in ("qkv_b", "qkv_h", "qkv_s", "out_b", "out_h", "out_s", "gate_b", "gate_h", "gate_s")] + \
               [("gate_form", ctypes.c_int)]


_lib = None


def lib():
    """The loaded library.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
                "(or __graft_entry__.build()); the mLSTM operators have no fallback implementation")
        L = ctypes.CDLL(LIB_PATH)
        vp, ci, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
        L.mlstm_version.restype = ctypes.c_char_p
        L.mlstm_workspace_bytes.restype = sz
        L.mlstm_workspace_bytes.argtypes = [ci] * 6
        L.mlstm_forward.restype = ci
        L.mlstm_forward.argtypes = [vp] * 6 + [ctypes.c_uint]
        L.mlstm_backward.restype = ci
        L.mlstm_backward.argtypes = [vp] * 13 + [ctypes.c_uint]
        L.mlstm_forward_ex.restype = ci
        L.mlstm_forward_ex.argtypes = [vp] * 8 + [ci] * 6 + [vp, sz, vp]
        L.mlstm_forward_noalloc_ex.restype = ci
        L.mlstm_forward_noalloc_ex.argtypes = [vp] * 8 + [ci] * 6 + [vp]
        L.mlstm_backward_ex.restype = ci
        L.mlstm_backward_ex.argtypes = [vp] * 14 + [ci] * 6 + [vp, sz, vp]
        L.mlstm_saved_state_bytes.restype = sz
        L.mlstm_saved_state_bytes.argtypes = [ci] * 5
        L.mlstm_forward_save_ex.restype = ci
        L.mlstm_forward_save_ex.argtypes = [vp] * 9 + [sz] + [ci] * 6 + [vp, sz, vp]
        L.mlstm_backward_saved_ex.restype = ci
        L.mlstm_backward_saved_ex.argtypes = [vp] * 10 + [sz] + [vp] * 5 + [ci] * 6 + [vp, sz, vp]
        L.mlstm_forward_gated_ex.restype = ci
        L.mlstm_forward_gated_ex.argtypes = [vp] * 10 + [ci] * 6 + [vp, sz, vp]
        L.mlstm_backward_gated_ex.restype = ci
        L.mlstm_backward_gated_ex.argtypes = [vp] * 16 + [ci] * 6 + [vp, sz, vp]
        lp = ctypes.POINTER(Layout)
        L.mlstm_forward_lx.restype = ci
        L.mlstm_forward_lx.argtypes = [vp] * 8 + [ci] * 6 + [lp, vp, sz, vp]
        L.mlstm_backward_lx.restype = ci
        L.mlstm_backward_lx.argtypes = [vp] * 14 + [ci] * 6 + [lp, vp, sz, vp]
        L.mlstm_forward_gated_lx.restype = ci
        L.mlstm_forward_gated_lx.argtypes = [vp] * 10 + [ci] * 6 + [lp, vp, sz, vp]
        L.mlstm_backward_gated_lx.restype = ci
        L.mlstm_backward_gated_lx.argtypes = [vp] * 16 + [ci] * 6 + [lp, vp, sz, vp]
        L.mlstm_forward_save_lx.restype = ci
        L.mlstm_forward_save_lx.argtypes = [vp] * 9 + [sz] + [ci] * 6 + [lp, vp, sz, vp]
        L.mlstm_backward_saved_lx.restype = ci
        L.mlstm_backward_saved_lx.argtypes = [vp] * 10 + [sz] + [vp] * 5 + [ci] * 6 + [lp, vp, sz, vp]
        fp = ctypes.c_void_p
        L.slstm_saved_bytes.restype = sz
        L.slstm_saved_bytes.argtypes = [ci] * 4
        L.slstm_workspace_bytes.restype = sz
        L.slstm_workspace_bytes.argtypes = [ci] * 4
        L.slstm_forward_ex.restype = ci
        L.slstm_forward_ex.argtypes = [fp] * 5 + [ci] * 5 + [vp]
        L.slstm_backward_ex.restype = ci
        L.slstm_backward_ex.argtypes = [fp] * 7 + [ci] * 5 + [vp, sz, vp]
        L.mlstm_scan_forward_ex.restype = ci
        L.mlstm_scan_forward_ex.argtypes = [vp] * 7 + [ci] * 5 + [vp, sz, vp]
        L.mlstm_scan_backward_ex.restype = ci
        L.mlstm_scan_backward_ex.argtypes = [vp] * 13 + [ci] * 5 + [vp, sz, vp]
        L.mlstm_scan_forward_save_ex.restype = ci
        L.mlstm_scan_forward_save_ex.argtypes = [vp] * 8 + [fp] + [ci] * 5 + [vp, sz, vp]
        L.mlstm_scan_backward_saved_ex.restype = ci
        L.mlstm_scan_backward_saved_ex.argtypes = [vp] * 8 + [fp] + [vp] * 6 + [ci] * 5 + [vp, sz, vp]
        L.mlstm_timing_enable.restype = ci
        L.mlstm_timing_enable.argtypes = [ci]
        L.mlstm_timing_select.restype = ci
        L.mlstm_timing_select.argtypes = [ctypes.c_uint, ci]
        L.mlstm_set_chunk_length.restype = ci
        L.mlstm_set_chunk_length.argtypes = [ci]
        L.mlstm_chunk_length_for.restype = ci
        L.mlstm_chunk_length_for.argtypes = [ci] * 3
        L.mlstm_kernel_error.restype = ci
        L.mlstm_kernel_error.argtypes = []
        L.mlstm_init.restype = ci
        L.mlstm_init.argtypes = []
        L.mlstm_set_column_kernel.restype = ci
        L.mlstm_set_column_kernel.argtypes = [ci]
        L.mlstm_set_state_kernel.restype = ci
        L.mlstm_set_state_kernel.argtypes = [ci]
        L.mlstm_set_spin_limit.restype = ci
        L.mlstm_set_spin_limit.argtypes = [ci]
        L.mlstm_force_generic_kernels.restype = ci
        L.mlstm_force_generic_kernels.argtypes = [ci]
        L.mlstm_timing_read.restype = ci
        L.mlstm_timing_read.argtypes = [ci, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ci)]
        _lib = L
    return _lib


def exported_symbols():
    return ["mlstm_forward", "mlstm_backward", "mlstm_forward_ex", "mlstm_forward_noalloc_ex", "mlstm_backward_ex", "mlstm_scan_forward_ex",
            "mlstm_scan_backward_ex", "mlstm_scan_forward_save_ex", "mlstm_scan_backward_saved_ex", "slstm_saved_bytes", "slstm_workspace_bytes", "slstm_forward_ex", "slstm_backward_ex", "mlstm_forward_lx", "mlstm_backward_lx", "mlstm_forward_save_lx", "mlstm_backward_saved_lx",
            "mlstm_forward_gated_ex", "mlstm_backward_gated_ex", "mlstm_forward_gated_lx", "mlstm_backward_gated_lx", "mlstm_set_chunk_length", "mlstm_chunk_length_for",
            "mlstm_saved_state_bytes", "mlstm_forward_save_ex", "mlstm_backward_saved_ex",
            "mlstm_workspace_bytes", "mlstm_version", "mlstm_timing_enable", "mlstm_timing_select", "mlstm_timing_read",
            "mlstm_force_generic_kernels", "mlstm_kernel_error", "mlstm_set_spin_limit", "mlstm_init", "mlstm_set_column_kernel",
            "mlstm_set_state_kernel"]


KERNELS = {"gates": 0, "row_fwd": 1, "col": 3, "row_dq": 4, "df": 5, "scan_state": 6, "scan_carry": 7,
           "scan_out": 8, "gate_bwd": 9, "chunk_states": 10, "scan_glue": 11}


def force_generic_kernels(on):
    """Test aid: route every shape through the generic four-wave kernels; returns the previous setting."""
    return bool(lib().mlstm_force_generic_kernels(1 if on else 0))


def set_column_kernel(variant):
    """Measurement and test aid: 0 = the library's choice, 1 = col16_kernel, 2 = cold_kernel, 3 = col_kernel."""
    check_rc(lib().mlstm_set_column_kernel(int(variant)), "mlstm_set_column_kernel")


def set_state_kernel(variant):
    """Measurement and test aid: 0 = the library's choice, 1 = chunk sums + carry, 2 = the one-pass kernel."""
    check_rc(lib().mlstm_set_state_kernel(int(variant)), "mlstm_set_state_kernel")


def set_chunk_length(length):
    """Test aid: chunk length of the chunked forward (> 0 forces it, < 0 switches chunking off, 0 = default)."""
    check_rc(lib().mlstm_set_chunk_length(int(length)), "mlstm_set_chunk_length")


def timing_enable(on):
    lib().mlstm_timing_enable(1 if on else 0)


def timing_select(kernels=None, every=1):
    """Narrow the timing to the named kernels (None: all of them) and to every `every`-th of their launches."""
    mask = 0xFFFFFFFF if kernels is None else sum(1 << KERNELS[k] for k in kernels)
    check_rc(lib().mlstm_timing_select(mask, every), "mlstm_timing_select")


def timing_read(kernel):
    """(total milliseconds, launches) of one kernel since the last read; waits for the recorded launches."""
    ms, n = ctypes.c_double(0.0), ctypes.c_int(0)
    check_rc(lib().mlstm_timing_read(KERNELS[kernel], ctypes.byref(ms), ctypes.byref(n)), "mlstm_timing_read")
    return ms.value, n.value


def dtype_code(dt, precise=False):
    try:
        return _DTYPES[dt] | (PRECISE if precise and dt != torch.float32 else 0)
    except KeyError:
        raise TypeError(f"unsupported dtype {dt}; expected float32, float16 or bfloat16") from None


def check_rc(rc, what):
    if rc == 0:
        return
    if rc < 0:
        raise ValueError(f"{what}: {_ERRORS.get(rc, 'error')} (code {rc})")
    raise RuntimeError(f"{what}: HIP error {rc}")


def require(t, name, shape=None):
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got device {t.device})")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} has shape {tuple(t.shape)}, expected {tuple(shape)}")


def require_rows(t, name, shape=None, like=None):
    """A GPU tensor whose last dimension is contiguous (any strides elsewhere: the kernels address rows through them)."""
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (got device {t.device})")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} has shape {tuple(t.shape)}, expected {tuple(shape)}")
    if t.dim() == 4 and t.stride(-1) != 1 and t.shape[-1] > 1:
        raise ValueError(f"{name}: the head dimension must be contiguous (strides {t.stride()})")
    if like is not None and tuple(t.stride()) != tuple(like.stride()):
        raise ValueError(f"{name} must have the layout of its companion (strides {t.stride()} against {like.stride()})")


def overlaps(t):
    """Does the view address one element more than once (an expanded tensor, stride 0, or any other self-overlap)?
    Sufficient test, the one the library applies to tensors it writes: in the order of their strides every dimension
    must step over everything the smaller ones span."""
    extent = 1
    for n, s in sorted(((n, s) for n, s in zip(t.shape, t.stride()) if n > 1), key=lambda p: p[1]):
        if s < extent:
            return True
        extent += (n - 1) * s
    return False


def dense_unless_disjoint(*ts):
    """The tensors as they are, or, if any of them overlaps itself, contiguous copies of all of them.  Gradients are
    laid out like their tensors: for an expanded input (``f.expand(...)`` to share gates over heads) that layout would
    make several workgroups write one address.  With a dense copy autograd's own backward of the expansion does the sum."""
    if any(overlaps(t) for t in ts):
        return tuple(t.contiguous() for t in ts)
    return ts


def dense_in_order_of(t):
    """A new tensor of t's shape, contiguous in the order of t's dimensions in memory (for a [B,NH,S,D] view of
    [B,S,NH,D] activations that is again such a view)."""
    order = sorted(range(t.dim()), key=lambda d: (t.stride(d), -d if t.shape[d] == 1 else 0), reverse=True)
    if t.dim() == 4:
        order = [d for d in order if d != 3] + [3]
    buf = torch.empty([t.shape[d] for d in order], dtype=t.dtype, device=t.device)
    inverse = [order.index(d) for d in range(t.dim())]
    return buf.permute(inverse)


def span(t):
    return 1 + sum((n - 1) * s for n, s in zip(t.shape, t.stride())) if t.numel() else 0


def strided_like(t, count=1):
    """`count` new tensors with exactly t's shape and strides."""
    if t.is_contiguous() or torch._prims_common.is_non_overlapping_and_dense(t):
        return [torch.empty_strided(t.shape, t.stride(), dtype=t.dtype, device=t.device) for _ in range(count)]
    n = span(t)
    return [torch.empty(n, dtype=t.dtype, device=t.device).as_strided(t.shape, t.stride()) for _ in range(count)]


def layout(q, h, f, gate_form="raw"):
    """struct mlstm_layout for q (and k, v, dq, dk, dv), h (and dh) and f (and i, df, di), all [B,NH,S(,D)] views."""
    if gate_form not in GATE_FORMS:
        raise ValueError(f"gate_form must be one of {sorted(GATE_FORMS)}, got {gate_form!r}")
    return Layout(q.stride(0), q.stride(1), q.stride(2), h.stride(0), h.stride(1), h.stride(2),
                  f.stride(0), f.stride(1), f.stride(2), GATE_FORMS[gate_form])


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def workspace(op, B, NH, S, D, dt, device):
    n = lib().mlstm_workspace_bytes(op, B, NH, S, D, dt)
    return torch.empty(max(int(n), 1), dtype=torch.uint8, device=device), int(n)
