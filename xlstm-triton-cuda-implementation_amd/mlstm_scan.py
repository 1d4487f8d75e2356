"""Scan (recurrent) form of the mLSTM forward with the silu(o) output gate, on hand-written gfx950 kernels.

Mirror of the reference module mlstm_scan.py: ``mlstm_scan(q, k, v, f, i, o, reduce_block_size=4,
value_block_size=4, num_warps=8)`` (:281-327), same positional order and defaults; fp32 in, fp32 out.  The three
tuning arguments are accepted and ignored: the kernels fix their own tiling (chunks of 64 positions, 32 value columns
per workgroup) and the result does not depend on them.

The reference's kernel path is forward only (its differentiable counterpart is the PyTorch loop mlstm_scan_pytorch,
mlstm_scan.py:343-372).  Here ``mlstm_scan`` is differentiable: called on tensors that require a gradient it records
``Scan_mLSTM``, whose backward (``mlstm_scan_backward_hip``) evaluates the gradients of mlstm_matmul.py:150-333
behind the silu(o) gate with the scan kernels, at every head dimension the forward takes.
"""
import torch

from . import _ffi


def _check(q, k, v, f, i, o):
    if q.dim() != 4:
        raise ValueError(f"q must be [B, NH, S, D], got {tuple(q.shape)}")
    B, NH, S, D = q.shape
    _ffi.require(q, "q")
    for name, t in (("k", k), ("v", v), ("o", o)):
        _ffi.require(t, name, q.shape)
    _ffi.require(f, "f", (B, NH, S))
    _ffi.require(i, "i", (B, NH, S))
    for name, t in (("q", q), ("k", k), ("v", v), ("f", f), ("i", i), ("o", o)):
        if t.dtype != torch.float32:
            raise TypeError(f"{name} must be float32 (the scan form is fp32, like the reference's)")
    return B, NH, S, D


def _dense(*ts):
    """The scan kernels take dense [B,NH,S,D] / [B,NH,S] tensors: views in another layout ([B,S,NH,D] activations, slices
    of a fused projection) are copied once, here (the matmul form's entry points address such views in place instead)."""
    return [t if (t is None or t.is_contiguous()) else t.contiguous() for t in ts]


def mlstm_scan_forward_hip(q, k, v, f, i, o):
    q, k, v, f, i, o = _dense(q, k, v, f, i, o)
    B, NH, S, D = _check(q, k, v, f, i, o)
    h = torch.empty_like(q)
    ws, n = _ffi.workspace(_ffi.OP_SCAN_FORWARD, B, NH, S, D, _ffi.F32, q.device)
    rc = _ffi.lib().mlstm_scan_forward_ex(_ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(o),
                                          _ffi.ptr(h), B, NH, S, D, _ffi.F32, _ffi.ptr(ws), n, _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_scan_forward_ex")
    return h


def mlstm_scan_forward_save_hip(q, k, v, f, i, o):
    """The forward of a training step: (h, h_ungated, b), the last two (the output before silu(o), the normaliser sums) kept
    for ``mlstm_scan_backward_hip`` so that it does not form them again."""
    q, k, v, f, i, o = _dense(q, k, v, f, i, o)
    B, NH, S, D = _check(q, k, v, f, i, o)
    h, h_ungated = torch.empty_like(q), torch.empty_like(q)
    b = torch.empty((B, NH, S), dtype=torch.float32, device=q.device)
    ws, n = _ffi.workspace(_ffi.OP_SCAN_FORWARD, B, NH, S, D, _ffi.F32, q.device)
    rc = _ffi.lib().mlstm_scan_forward_save_ex(_ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(o),
                                               _ffi.ptr(h), _ffi.ptr(h_ungated), _ffi.ptr(b), B, NH, S, D, _ffi.F32, _ffi.ptr(ws), n,
                                               _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_scan_forward_save_ex")
    return h, h_ungated, b


def mlstm_scan_backward_hip(dh, q, k, v, f, i, o, h_ungated=None, b=None):
    """Gradients (dq, dk, dv, df, di, do) of ``mlstm_scan`` for the output gradient ``dh``; df[..., 0] = 0 as in
    mlstm_matmul.py:320-333.  Nothing but the inputs is needed: the forward is run again inside, unless ``h_ungated`` and
    ``b`` of ``mlstm_scan_forward_save_hip`` are handed over (the same bits either way)."""
    dh, q, k, v, f, i, o, h_ungated, b = _dense(dh, q, k, v, f, i, o, h_ungated, b)
    B, NH, S, D = _check(q, k, v, f, i, o)
    _ffi.require(dh, "dh", q.shape)
    if dh.dtype != torch.float32:
        raise TypeError("dh must be float32")
    if (h_ungated is None) != (b is None):
        raise ValueError("h_ungated and b go together")
    if h_ungated is not None:
        _ffi.require(h_ungated, "h_ungated", q.shape)
        _ffi.require(b, "b", (B, NH, S))
        if h_ungated.dtype != torch.float32 or b.dtype != torch.float32:
            raise TypeError("h_ungated and b must be float32")
    dq, dk, dv, do = (torch.empty_like(q) for _ in range(4))
    df, di = torch.empty_like(f), torch.empty_like(i)
    ws, n = _ffi.workspace(_ffi.OP_SCAN_BACKWARD, B, NH, S, D, _ffi.F32, q.device)
    rc = _ffi.lib().mlstm_scan_backward_saved_ex(_ffi.ptr(dh), _ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i),
                                                 _ffi.ptr(o), _ffi.ptr(h_ungated), _ffi.ptr(b), _ffi.ptr(dq), _ffi.ptr(dk),
                                                 _ffi.ptr(dv), _ffi.ptr(df), _ffi.ptr(di), _ffi.ptr(do), B, NH, S, D, _ffi.F32,
                                                 _ffi.ptr(ws), n, _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_scan_backward_saved_ex")
    return dq, dk, dv, df, di, do


class Scan_mLSTM(torch.autograd.Function):
    """``Scan_mLSTM.apply(q, k, v, f, i, o)``: the scan form with a backward (no counterpart in the reference)."""

    @staticmethod
    def forward(ctx, q, k, v, f, i, o):
        h, h_ungated, b = mlstm_scan_forward_save_hip(q, k, v, f, i, o)
        ctx.save_for_backward(q, k, v, f, i, o, h_ungated, b)
        return h

    @staticmethod
    def backward(ctx, dh):
        return mlstm_scan_backward_hip(dh, *ctx.saved_tensors)


def mlstm_scan(q, k, v, f, i, o, reduce_block_size=4, value_block_size=4, num_warps=8):
    if torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v, f, i, o)):
        return Scan_mLSTM.apply(q, k, v, f, i, o)
    return mlstm_scan_forward_hip(q, k, v, f, i, o)
