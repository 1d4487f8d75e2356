"""Matmul (parallel) form of the mLSTM: forward and backward on hand-written gfx950 kernels.

Mirror of the reference module mlstm_matmul.py: ``Triton_mLSTM.apply(q, k, v, f, i, SB, NUM_WARPS)``
(:368-405) and ``mlstm_matmul(q, k, v, f, i, SB, num_warps)`` (:121-129), same positional order and defaults.
``SB`` and ``num_warps`` are accepted and ignored: tiling is fixed by the kernels and results do not depend on it.
Outputs follow the inputs: h and dq, dk, dv have q's dtype (fp32 for fp32 inputs, as in the reference),
df and di have f's dtype, the saved m and b are fp32.
"""
import torch

from . import _ffi


def _check_inputs(q, k, v, f, i, precise=False):
    if q.dim() != 4:
        raise ValueError(f"q must be [B, NH, S, D], got {tuple(q.shape)}")
    B, NH, S, D = q.shape
    _ffi.require(q, "q")
    _ffi.require(k, "k", q.shape)
    _ffi.require(v, "v", q.shape)
    _ffi.require(f, "f", (B, NH, S))
    _ffi.require(i, "i", (B, NH, S))
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("q, k, v must share one dtype")
    if i.dtype != f.dtype:
        raise TypeError("f and i must share one dtype")
    return B, NH, S, D, _ffi.dtype_code(q.dtype, precise), _ffi.dtype_code(f.dtype)


def mlstm_forward_hip(q, k, v, f, i, precise=False):
    """Returns (h, m, b): h [B,NH,S,D] in q's dtype, m and b [B,NH,S] fp32 (reference mlstm_matmul.py:373-378)."""
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i, precise)
    h = torch.empty_like(q)
    m = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    b = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    ws, n = _ffi.workspace(_ffi.OP_FORWARD, B, NH, S, D, dt, q.device)
    rc = _ffi.lib().mlstm_forward_ex(_ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(h), _ffi.ptr(m),
                                     _ffi.ptr(b), B, NH, S, D, dt, gdt, _ffi.ptr(ws), n, _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_forward_ex")
    return h, m, b


def mlstm_backward_hip(dh, q, k, v, f, i, h=None, m=None, b=None, precise=False):
    """Returns (dq, dk, dv, df, di) (reference mlstm_matmul.py:384-405).  h, m, b: the forward's outputs, or None
    to have them recomputed."""
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i, precise)
    _ffi.require(dh, "dh", q.shape)
    if dh.dtype != q.dtype:
        raise TypeError("dh must have q's dtype")
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    df, di = torch.empty_like(f), torch.empty_like(i)
    ws, n = _ffi.workspace(_ffi.OP_BACKWARD, B, NH, S, D, dt, q.device)
    if h is None or m is None or b is None:
        h = m = b = None
    rc = _ffi.lib().mlstm_backward_ex(_ffi.ptr(dh), _ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(h),
                                      _ffi.ptr(m), _ffi.ptr(b), _ffi.ptr(dq), _ffi.ptr(dk), _ffi.ptr(dv), _ffi.ptr(df),
                                      _ffi.ptr(di), B, NH, S, D, dt, gdt, _ffi.ptr(ws), n, _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_backward_ex")
    return dq, dk, dv, df, di


def mlstm_forward_save_hip(q, k, v, f, i, precise=False):
    """Forward of a training step.  Returns (h, m, b, saved): as mlstm_forward_hip, plus what the backward can reuse (the
    states at the chunk ends of a long 16-bit sequence; None for shapes that do not run in chunks)."""
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i, precise)
    h = torch.empty_like(q)
    m = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    b = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    nsaved = int(_ffi.lib().mlstm_saved_state_bytes(B, NH, S, D, dt))
    saved = torch.empty(nsaved, dtype=torch.uint8, device=q.device) if nsaved else None
    ws, n = _ffi.workspace(_ffi.OP_FORWARD, B, NH, S, D, dt, q.device)
    rc = _ffi.lib().mlstm_forward_save_ex(_ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(h), _ffi.ptr(m),
                                          _ffi.ptr(b), _ffi.ptr(saved), nsaved, B, NH, S, D, dt, gdt, _ffi.ptr(ws), n,
                                          _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_forward_save_ex")
    return h, m, b, saved


def mlstm_backward_saved_hip(dh, q, k, v, f, i, h, m, b, saved, precise=False):
    """Backward of a training step with the forward's outputs and its saved states (mlstm_forward_save_hip)."""
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i, precise)
    _ffi.require(dh, "dh", q.shape)
    if dh.dtype != q.dtype:
        raise TypeError("dh must have q's dtype")
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    df, di = torch.empty_like(f), torch.empty_like(i)
    ws, n = _ffi.workspace(_ffi.OP_BACKWARD, B, NH, S, D, dt, q.device)
    nsaved = 0 if saved is None else saved.numel()
    rc = _ffi.lib().mlstm_backward_saved_ex(_ffi.ptr(dh), _ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(h),
                                            _ffi.ptr(m), _ffi.ptr(b), _ffi.ptr(saved), nsaved, _ffi.ptr(dq), _ffi.ptr(dk), _ffi.ptr(dv),
                                            _ffi.ptr(df), _ffi.ptr(di), B, NH, S, D, dt, gdt, _ffi.ptr(ws), n, _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_backward_saved_ex")
    return dq, dk, dv, df, di


def mlstm_matmul(q, k, v, f, i, SB=16, num_warps=8):
    """Forward only, no autograd (reference mlstm_matmul.py:121-129)."""
    return mlstm_forward_hip(q, k, v, f, i)[0]


class Triton_mLSTM(torch.autograd.Function):
    """Drop-in for the reference's autograd function of the same name (mlstm_matmul.py:368-405)."""

    @staticmethod
    def forward(ctx, q, k, v, f, i, SB=16, num_warps=8):
        h, m, b, saved = mlstm_forward_save_hip(q, k, v, f, i)
        ctx.save_for_backward(q, k, v, f, i, m, b, h, saved)
        ctx.sb = SB
        return h

    @staticmethod
    def backward(ctx, dh):
        assert dh.is_contiguous()
        q, k, v, f, i, m, b, h, saved = ctx.saved_tensors
        dq, dk, dv, df, di = mlstm_backward_saved_hip(dh, q, k, v, f, i, h, m, b, saved)
        return dq, dk, dv, df, di, None, None


HIP_mLSTM = Triton_mLSTM


class Triton_mLSTM_precise(torch.autograd.Function):
    """Triton_mLSTM in split mode (no counterpart in the reference, whose kernels are fp32): for fp16 / bf16 inputs the
    weights of every second product enter it as two terms, so that results and gradients agree with an fp32
    evaluation of the reference's formulas element by element at rtol 2e-2 / atol 2e-3.  Slower: no chunking, half as
    many MFMAs again.  Same call signature."""

    @staticmethod
    def forward(ctx, q, k, v, f, i, SB=16, num_warps=8):
        h, m, b, saved = mlstm_forward_save_hip(q, k, v, f, i, precise=True)
        ctx.save_for_backward(q, k, v, f, i, m, b, h, saved)
        ctx.sb = SB
        return h

    @staticmethod
    def backward(ctx, dh):
        assert dh.is_contiguous()
        q, k, v, f, i, m, b, h, saved = ctx.saved_tensors
        dq, dk, dv, df, di = mlstm_backward_saved_hip(dh, q, k, v, f, i, h, m, b, saved, precise=True)
        return dq, dk, dv, df, di, None, None


# ---------------------------------------------------------------------------------------------------------------
# Matmul form with the scan form's output gate, h_gated = silu(o) * h.  The reference leaves this open for its
# matmul kernels ("Integrate o", mlstm_matmul.py:36); its scan form applies the gate at mlstm_scan.py:277 and has no
# backward.  With the gate fused here, mlstm_matmul_gated(q, k, v, f, i, o) == mlstm_scan(q, k, v, f, i, o), and
# Triton_mLSTM_gated gives that function a backward.
# ---------------------------------------------------------------------------------------------------------------
def mlstm_forward_gated_hip(q, k, v, f, i, o):
    """Returns (h_gated, h, m, b); h is the ungated output, which the backward needs."""
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i)
    _ffi.require(o, "o", q.shape)
    if o.dtype != q.dtype:
        raise TypeError("o must have q's dtype")
    h, hg = torch.empty_like(q), torch.empty_like(q)
    m = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    b = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    ws, n = _ffi.workspace(_ffi.OP_FORWARD_GATED, B, NH, S, D, dt, q.device)
    rc = _ffi.lib().mlstm_forward_gated_ex(_ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(o), _ffi.ptr(h),
                                           _ffi.ptr(hg), _ffi.ptr(m), _ffi.ptr(b), B, NH, S, D, dt, gdt, _ffi.ptr(ws), n,
                                           _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_forward_gated_ex")
    return hg, h, m, b


def mlstm_backward_gated_hip(dhg, q, k, v, f, i, o, h=None, m=None, b=None):
    """Returns (dq, dk, dv, df, di, do) for the gradient dhg of the gated output."""
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i)
    _ffi.require(o, "o", q.shape)
    _ffi.require(dhg, "dh", q.shape)
    if dhg.dtype != q.dtype or o.dtype != q.dtype:
        raise TypeError("dh and o must have q's dtype")
    dq, dk, dv, do = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v), torch.empty_like(o)
    df, di = torch.empty_like(f), torch.empty_like(i)
    ws, n = _ffi.workspace(_ffi.OP_BACKWARD_GATED, B, NH, S, D, dt, q.device)
    if h is None or m is None or b is None:
        h = m = b = None
    rc = _ffi.lib().mlstm_backward_gated_ex(_ffi.ptr(dhg), _ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(o),
                                            _ffi.ptr(h), _ffi.ptr(m), _ffi.ptr(b), _ffi.ptr(dq), _ffi.ptr(dk), _ffi.ptr(dv),
                                            _ffi.ptr(df), _ffi.ptr(di), _ffi.ptr(do), B, NH, S, D, dt, gdt, _ffi.ptr(ws), n,
                                            _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_backward_gated_ex")
    return dq, dk, dv, df, di, do


def mlstm_matmul_gated(q, k, v, f, i, o, SB=16, num_warps=8):
    """Forward only, no autograd: the value mlstm_scan(q, k, v, f, i, o) returns, computed in the matmul form."""
    return mlstm_forward_gated_hip(q, k, v, f, i, o)[0]


class Triton_mLSTM_gated(torch.autograd.Function):
    """``Triton_mLSTM_gated.apply(q, k, v, f, i, o, SB, NUM_WARPS)``: Triton_mLSTM followed by the silu(o) gate."""

    @staticmethod
    def forward(ctx, q, k, v, f, i, o, SB=16, num_warps=8):
        hg, h, m, b = mlstm_forward_gated_hip(q, k, v, f, i, o)
        ctx.save_for_backward(q, k, v, f, i, o, m, b, h)
        ctx.sb = SB
        return hg

    @staticmethod
    def backward(ctx, dhg):
        assert dhg.is_contiguous()
        q, k, v, f, i, o, m, b, h = ctx.saved_tensors
        dq, dk, dv, df, di, do = mlstm_backward_gated_hip(dhg, q, k, v, f, i, o, h, m, b)
        return dq, dk, dv, df, di, do, None, None


HIP_mLSTM_gated = Triton_mLSTM_gated
