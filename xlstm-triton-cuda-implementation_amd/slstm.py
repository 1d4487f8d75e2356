"""sLSTM cell on hand-written gfx950 kernels: ``slstm(wx, r, b)`` with a backward.

The reference lists the sLSTM as an open item (README.md:9) and has no code or interface for it; this module follows the
conventions of its neighbours (``mlstm_scan``: tensors in, tensor out, fp32).  ``wx`` holds the input projections of the
four gates, [B,S,4,NH,DH] in the order i, f, z, o (one GEMM of the caller's over the layer input); ``r`` the block-diagonal
recurrent matrices, [NH,4,DH,DH]; ``b`` the biases, [NH,4,DH].  Returns h [B,S,NH,DH].  The cell is the published one
(Beck et al., arXiv:2405.04517, section 2.2 / appendix A.2) with exponential input gate, exponential or sigmoid forget
gate and the stabiliser state; see include/mlstm_hip.h.
"""
import torch

from . import _ffi


def _check(wx, r, b):
    if wx.dim() != 5 or wx.shape[2] != 4:
        raise ValueError(f"wx must be [B, S, 4, NH, DH], got {tuple(wx.shape)}")
    B, S, _, NH, DH = wx.shape
    _ffi.require(wx, "wx")
    _ffi.require(r, "r", (NH, 4, DH, DH))
    _ffi.require(b, "b", (NH, 4, DH))
    for name, t in (("wx", wx), ("r", r), ("b", b)):
        if t.dtype != torch.float32:
            raise TypeError(f"{name} must be float32")
    return B, NH, S, DH


def slstm_forward_hip(wx, r, b, forget_sigmoid=False, save=True):
    """Returns (h, saved): saved carries the pre-activations and cell states to the backward (None with save=False)."""
    B, NH, S, DH = _check(wx, r, b)
    h = torch.empty((B, S, NH, DH), device=wx.device, dtype=torch.float32)
    n = int(_ffi.lib().slstm_saved_bytes(B, NH, S, DH))
    if n == 0:
        raise ValueError(f"unsupported head dimension {DH}: the sLSTM kernels take 32, 64 or 128")
    saved = torch.empty(n, dtype=torch.uint8, device=wx.device) if save else None
    rc = _ffi.lib().slstm_forward_ex(_ffi.ptr(wx), _ffi.ptr(r), _ffi.ptr(b), _ffi.ptr(h), _ffi.ptr(saved), B, NH, S, DH,
                                     1 if forget_sigmoid else 0, _ffi.stream_ptr())
    _ffi.check_rc(rc, "slstm_forward_ex")
    return h, saved


def slstm_backward_hip(dh, h, r, saved, forget_sigmoid=False):
    """Returns (dwx, dr, db) for the output gradient dh [B,S,NH,DH]."""
    B, S, NH, DH = h.shape
    _ffi.require(dh, "dh", h.shape)
    _ffi.require(h, "h")
    _ffi.require(r, "r", (NH, 4, DH, DH))
    if dh.dtype != torch.float32:
        raise TypeError("dh must be float32")
    dwx = torch.empty((B, S, 4, NH, DH), device=h.device, dtype=torch.float32)
    dr = torch.empty_like(r)
    db = torch.empty((NH, 4, DH), device=h.device, dtype=torch.float32)
    n = int(_ffi.lib().slstm_workspace_bytes(B, NH, S, DH))
    ws = torch.empty(max(n, 1), dtype=torch.uint8, device=h.device)
    rc = _ffi.lib().slstm_backward_ex(_ffi.ptr(dh), _ffi.ptr(h), _ffi.ptr(r), _ffi.ptr(saved), _ffi.ptr(dwx), _ffi.ptr(dr), _ffi.ptr(db),
                                      B, NH, S, DH, 1 if forget_sigmoid else 0, _ffi.ptr(ws), n, _ffi.stream_ptr())
    _ffi.check_rc(rc, "slstm_backward_ex")
    return dwx, dr, db


class HIP_sLSTM(torch.autograd.Function):
    """``HIP_sLSTM.apply(wx, r, b, forget_sigmoid)``"""

    @staticmethod
    def forward(ctx, wx, r, b, forget_sigmoid=False):
        h, saved = slstm_forward_hip(wx, r, b, forget_sigmoid)
        ctx.save_for_backward(h, r, saved)
        ctx.forget_sigmoid = forget_sigmoid
        return h

    @staticmethod
    def backward(ctx, dh):
        h, r, saved = ctx.saved_tensors
        dwx, dr, db = slstm_backward_hip(dh.contiguous(), h, r, saved, ctx.forget_sigmoid)
        return dwx, dr, db, None


def slstm(wx, r, b, forget_sigmoid=False):
    if torch.is_grad_enabled() and any(t.requires_grad for t in (wx, r, b)):
        return HIP_sLSTM.apply(wx, r, b, forget_sigmoid)
    return slstm_forward_hip(wx, r, b, forget_sigmoid, save=False)[0]
