"""Matmul (parallel) form of the mLSTM: forward and backward on hand-written gfx950 kernels.

Mirror of the reference module mlstm_matmul.py: ``Triton_mLSTM.apply(q, k, v, f, i, SB, NUM_WARPS)``
(:368-405) and ``mlstm_matmul(q, k, v, f, i, SB, num_warps)`` (:121-129), same positional order and defaults.
``SB`` and ``num_warps`` are accepted and ignored: tiling is fixed by the kernels and results do not depend on it.
Outputs follow the inputs: h and dq, dk, dv have q's dtype (fp32 for fp32 inputs, as in the reference),
df and di have f's dtype, the saved m and b are fp32.

Beyond the reference: q, k, v need not be contiguous [B,NH,S,D].  Any [B,NH,S,D] view whose head dimension is
contiguous is taken as it is (``x.view(B, S, NH, D).transpose(1, 2)`` of a projection's output, or the three slices of
a fused q/k/v projection), h comes back in the same dimension order and every gradient in the layout of its tensor;
``gate_form`` lets f arrive as its log-sigmoid or as the cumulative sum of that (the step the reference's
cutlass-src-hopper/mlstm_forward.cu:201 suggests fusing into the projection).  The gated variants take the same views
(o, the gated output and its gradient in h's layout).
"""
import torch

from . import _ffi


def _check_inputs(q, k, v, f, i, precise=False):
    """Shapes, dtypes and layouts.  q, k, v: [B,NH,S,D] with a contiguous head dimension and one common layout
    otherwise (a [B,S,NH,D] projection viewed through transpose(1, 2), slices of a fused q/k/v projection, or plain
    contiguous tensors: the kernels address rows through the strides, nothing is copied); f, i: [B,NH,S], any strides."""
    if q.dim() != 4:
        raise ValueError(f"q must be [B, NH, S, D], got {tuple(q.shape)}")
    B, NH, S, D = q.shape
    _ffi.require_rows(q, "q")
    _ffi.require_rows(k, "k", q.shape, like=q)
    _ffi.require_rows(v, "v", q.shape, like=q)
    _ffi.require_rows(f, "f", (B, NH, S))
    _ffi.require_rows(i, "i", (B, NH, S), like=f)
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise TypeError("q, k, v must share one dtype")
    if i.dtype != f.dtype:
        raise TypeError("f and i must share one dtype")
    return B, NH, S, D, _ffi.dtype_code(q.dtype, precise), _ffi.dtype_code(f.dtype)


# Head dimensions below the kernels' smallest tile (64) run zero-padded: the padded columns of q, k, v add nothing to a
# score or to h, and q is scaled by sqrt(padded D / D) so that the kernels' 1 / sqrt(padded D) gives the scores their
# 1 / sqrt(D).  The padded size is four times D: the factor is 2, exact in every type (padding 32 to 64 would round a
# 16-bit q once more, by sqrt 2, and the row sums b would show it).
_PADDED_D = {16: 64, 32: 128}


def _pads(q):
    return q.dim() == 4 and q.shape[-1] in _PADDED_D


def _pad_last(x, Dp):
    return None if x is None else torch.nn.functional.pad(x, (0, Dp - x.shape[-1]))


def _pad_qkv(q, k, v):
    D = q.shape[-1]
    Dp = _PADDED_D[D]
    s = (Dp / D) ** 0.5
    return _pad_last((q.float() * s).to(q.dtype), Dp), _pad_last(k, Dp), _pad_last(v, Dp), D, s


def _unpad_grads(grads, q, D, s):
    dq, dk, dv, df, di = grads
    return (dq[..., :D].float() * s).to(q.dtype), dk[..., :D].contiguous(), dv[..., :D].contiguous(), df, di


# 16-bit tensors at head dimensions beyond the 16-bit tile kernels (512, 1024) run on the fp32 path (the scan form's
# kernels behind the same entry points): inputs widened, outputs and gradients rounded back to the callers' types.
_WIDENED_D = (512, 1024)


def _widens(q):
    return q.dim() == 4 and q.shape[-1] in _WIDENED_D and q.dtype in (torch.float16, torch.bfloat16)


def _wide(*xs):
    return [None if x is None else x.float().contiguous() for x in xs]


def _dh_like(dh, h):
    """dh in h's layout (the kernels read h and dh through one set of strides)."""
    if tuple(dh.stride()) == tuple(h.stride()):
        return dh
    out = _ffi.strided_like(h)[0]
    out.copy_(dh)
    return out


def mlstm_forward_hip(q, k, v, f, i, precise=False, gate_form="raw"):
    """Returns (h, m, b): h [B,NH,S,D] in q's dtype and dimension order in memory, m and b [B,NH,S] fp32 (reference
    mlstm_matmul.py:373-378).  gate_form: what f holds ("raw" pre-activations as in the reference, "logsigmoid", or
    "cumsum" of the log-sigmoid over the positions; fp32 gates only for the last)."""
    if _pads(q):
        qp, kp, vp, D, _ = _pad_qkv(q, k, v)
        h, m, b = mlstm_forward_hip(qp, kp, vp, f, i, precise, gate_form)
        return h[..., :D].contiguous(), m, b
    if _widens(q):
        h, m, b = mlstm_forward_hip(*_wide(q, k, v, f, i), False, gate_form)
        return h.to(q.dtype), m, b
    q, k, v = _ffi.dense_unless_disjoint(q, k, v)   # (expanded views: see there)
    f, i = _ffi.dense_unless_disjoint(f, i)
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i, precise)
    h = _ffi.dense_in_order_of(q)
    m = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    b = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    lay = _ffi.layout(q, h, f, gate_form)
    ws, n = _ffi.workspace(_ffi.OP_FORWARD, B, NH, S, D, dt, q.device)
    rc = _ffi.lib().mlstm_forward_lx(_ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(h), _ffi.ptr(m),
                                     _ffi.ptr(b), B, NH, S, D, dt, gdt, lay, _ffi.ptr(ws), n, _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_forward_lx")
    return h, m, b


def mlstm_backward_hip(dh, q, k, v, f, i, h=None, m=None, b=None, precise=False, gate_form="raw"):
    """Returns (dq, dk, dv, df, di) (reference mlstm_matmul.py:384-405), each in the layout of the tensor it is the
    gradient of; df is the gradient of whatever f held (gate_form).  h, m, b: the forward's outputs, or None to have
    them recomputed."""
    if _pads(q):
        qp, kp, vp, D, s = _pad_qkv(q, k, v)
        have = h is not None and m is not None and b is not None
        grads = mlstm_backward_hip(_pad_last(dh, qp.shape[-1]), qp, kp, vp, f, i, _pad_last(h, qp.shape[-1]) if have else None,
                                   m if have else None, b if have else None, precise, gate_form)
        return _unpad_grads(grads, q, D, s)
    if _widens(q):   # (the fp32 path recomputes the forward it needs)
        dq, dk, dv, df, di = mlstm_backward_hip(*_wide(dh, q, k, v, f, i), None, None, None, False, gate_form)
        return dq.to(q.dtype), dk.to(q.dtype), dv.to(q.dtype), df.to(f.dtype), di.to(f.dtype)
    q, k, v = _ffi.dense_unless_disjoint(q, k, v)   # (expanded views: see there)
    f, i = _ffi.dense_unless_disjoint(f, i)
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i, precise)
    if not dh.is_cuda or tuple(dh.shape) != tuple(q.shape):
        raise ValueError(f"dh must be a GPU tensor of q's shape, got {tuple(dh.shape)} on {dh.device}")
    if dh.dtype != q.dtype:
        raise TypeError("dh must have q's dtype")
    if h is None or m is None or b is None:
        h = m = b = None
        if dh.stride(-1) != 1 and D > 1:   # (an expanded or transposed gradient: one copy, into q's dimension order)
            dh = _dh_like(dh, _ffi.dense_in_order_of(q))
        out_like = dh   # (the recomputed h is the library's own; dh is read through its own strides)
    else:
        _ffi.require_rows(h, "h", q.shape)
        dh = _dh_like(dh, h)
        out_like = h
    dq, dk, dv = _ffi.strided_like(q, 3)
    df, di = _ffi.strided_like(f, 2)
    lay = _ffi.layout(q, out_like, f, gate_form)
    ws, n = _ffi.workspace(_ffi.OP_BACKWARD, B, NH, S, D, dt, q.device)
    rc = _ffi.lib().mlstm_backward_lx(_ffi.ptr(dh), _ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(h),
                                      _ffi.ptr(m), _ffi.ptr(b), _ffi.ptr(dq), _ffi.ptr(dk), _ffi.ptr(dv), _ffi.ptr(df),
                                      _ffi.ptr(di), B, NH, S, D, dt, gdt, lay, _ffi.ptr(ws), n, _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_backward_lx")
    return dq, dk, dv, df, di


def mlstm_forward_save_hip(q, k, v, f, i, precise=False, gate_form="raw"):
    """Forward of a training step.  Returns (h, m, b, saved): as mlstm_forward_hip, plus what the backward can reuse (the
    states at the chunk ends of a long sequence; None for shapes that do not run in chunks)."""
    if _pads(q):
        qp, kp, vp, D, _ = _pad_qkv(q, k, v)
        h, m, b, saved = mlstm_forward_save_hip(qp, kp, vp, f, i, precise, gate_form)
        return h[..., :D].contiguous(), m, b, saved
    if _widens(q):
        return (*mlstm_forward_hip(q, k, v, f, i, precise, gate_form), None)
    q, k, v = _ffi.dense_unless_disjoint(q, k, v)   # (expanded views: see there)
    f, i = _ffi.dense_unless_disjoint(f, i)
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i, precise)
    h = _ffi.dense_in_order_of(q)
    m = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    b = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    nsaved = int(_ffi.lib().mlstm_saved_state_bytes(B, NH, S, D, dt))
    saved = torch.empty(nsaved, dtype=torch.uint8, device=q.device) if nsaved else None
    lay = _ffi.layout(q, h, f, gate_form)
    ws, n = _ffi.workspace(_ffi.OP_FORWARD, B, NH, S, D, dt, q.device)
    rc = _ffi.lib().mlstm_forward_save_lx(_ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(h), _ffi.ptr(m),
                                          _ffi.ptr(b), _ffi.ptr(saved), nsaved, B, NH, S, D, dt, gdt, lay, _ffi.ptr(ws), n,
                                          _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_forward_save_lx")
    return h, m, b, saved


def mlstm_backward_saved_hip(dh, q, k, v, f, i, h, m, b, saved, precise=False, gate_form="raw"):
    """Backward of a training step with the forward's outputs and its saved states (mlstm_forward_save_hip)."""
    if _pads(q):
        qp, kp, vp, D, s = _pad_qkv(q, k, v)
        Dp = qp.shape[-1]
        grads = mlstm_backward_saved_hip(_pad_last(dh, Dp), qp, kp, vp, f, i, _pad_last(h, Dp), m, b, saved, precise, gate_form)
        return _unpad_grads(grads, q, D, s)
    if _widens(q):
        return mlstm_backward_hip(dh, q, k, v, f, i, None, None, None, precise, gate_form)
    q, k, v = _ffi.dense_unless_disjoint(q, k, v)   # (expanded views: see there)
    f, i = _ffi.dense_unless_disjoint(f, i)
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i, precise)
    if not dh.is_cuda or tuple(dh.shape) != tuple(q.shape):
        raise ValueError(f"dh must be a GPU tensor of q's shape, got {tuple(dh.shape)} on {dh.device}")
    _ffi.require_rows(h, "h", q.shape)
    if dh.dtype != q.dtype:
        raise TypeError("dh must have q's dtype")
    dh = _dh_like(dh, h)
    dq, dk, dv = _ffi.strided_like(q, 3)
    df, di = _ffi.strided_like(f, 2)
    lay = _ffi.layout(q, h, f, gate_form)
    ws, n = _ffi.workspace(_ffi.OP_BACKWARD, B, NH, S, D, dt, q.device)
    nsaved = 0 if saved is None else saved.numel()
    rc = _ffi.lib().mlstm_backward_saved_lx(_ffi.ptr(dh), _ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(h),
                                            _ffi.ptr(m), _ffi.ptr(b), _ffi.ptr(saved), nsaved, _ffi.ptr(dq), _ffi.ptr(dk), _ffi.ptr(dv),
                                            _ffi.ptr(df), _ffi.ptr(di), B, NH, S, D, dt, gdt, lay, _ffi.ptr(ws), n, _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_backward_saved_lx")
    return dq, dk, dv, df, di


def mlstm_matmul(q, k, v, f, i, SB=16, num_warps=8):
    """Forward only, no autograd (reference mlstm_matmul.py:121-129)."""
    return mlstm_forward_hip(q, k, v, f, i)[0]


class Triton_mLSTM(torch.autograd.Function):
    """Drop-in for the reference's autograd function of the same name (mlstm_matmul.py:368-405)."""

    @staticmethod
    def forward(ctx, q, k, v, f, i, SB=16, num_warps=8, gate_form="raw"):
        h, m, b, saved = mlstm_forward_save_hip(q, k, v, f, i, gate_form=gate_form)
        ctx.save_for_backward(q, k, v, f, i, m, b, h, saved)
        ctx.sb = SB
        ctx.gate_form = gate_form
        return h

    @staticmethod
    def backward(ctx, dh):
        # (the reference asserts dh.is_contiguous(), mlstm_matmul.py:385; here every layout with a contiguous head
        # dimension is taken as it is, e.g. the gradient of a [B,S,NH,D] view)
        assert dh.stride(-1) == 1 or dh.shape[-1] == 1
        q, k, v, f, i, m, b, h, saved = ctx.saved_tensors
        dq, dk, dv, df, di = mlstm_backward_saved_hip(dh, q, k, v, f, i, h, m, b, saved, gate_form=ctx.gate_form)
        return dq, dk, dv, df, di, None, None, None


HIP_mLSTM = Triton_mLSTM


class Triton_mLSTM_precise(torch.autograd.Function):
    """Triton_mLSTM in split mode (no counterpart in the reference, whose kernels are fp32): for fp16 / bf16 inputs the
    weights of every second product enter it as two terms, so that results and gradients agree with an fp32
    evaluation of the reference's formulas element by element at rtol 2e-2 / atol 2e-3.  Slower: no chunking, half as
    many MFMAs again.  Same call signature."""

    @staticmethod
    def forward(ctx, q, k, v, f, i, SB=16, num_warps=8, gate_form="raw"):
        h, m, b, saved = mlstm_forward_save_hip(q, k, v, f, i, precise=True, gate_form=gate_form)
        ctx.save_for_backward(q, k, v, f, i, m, b, h, saved)
        ctx.sb = SB
        ctx.gate_form = gate_form
        return h

    @staticmethod
    def backward(ctx, dh):
        # (the reference asserts dh.is_contiguous(), mlstm_matmul.py:385; here every layout with a contiguous head
        # dimension is taken as it is, e.g. the gradient of a [B,S,NH,D] view)
        assert dh.stride(-1) == 1 or dh.shape[-1] == 1
        q, k, v, f, i, m, b, h, saved = ctx.saved_tensors
        dq, dk, dv, df, di = mlstm_backward_saved_hip(dh, q, k, v, f, i, h, m, b, saved, precise=True, gate_form=ctx.gate_form)
        return dq, dk, dv, df, di, None, None, None


# ---------------------------------------------------------------------------------------------------------------
# Matmul form with the scan form's output gate, h_gated = silu(o) * h.  The reference leaves this open for its
# matmul kernels ("Integrate o", mlstm_matmul.py:36); its scan form applies the gate at mlstm_scan.py:277 and has no
# backward.  With the gate fused here, mlstm_matmul_gated(q, k, v, f, i, o) == mlstm_scan(q, k, v, f, i, o), and
# Triton_mLSTM_gated gives that function a backward.
# ---------------------------------------------------------------------------------------------------------------
def mlstm_forward_gated_hip(q, k, v, f, i, o):
    """Returns (h_gated, h, m, b); h is the ungated output, which the backward needs.  q, k, v in one layout (as for
    mlstm_forward_hip); o is taken in the layout h is written in (q's dimension order, dense), or copied into it."""
    q, k, v = _ffi.dense_unless_disjoint(q, k, v)
    f, i = _ffi.dense_unless_disjoint(f, i)
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i)
    if not o.is_cuda or tuple(o.shape) != tuple(q.shape):
        raise ValueError(f"o must be a GPU tensor of q's shape, got {tuple(o.shape)} on {o.device}")
    if o.dtype != q.dtype:
        raise TypeError("o must have q's dtype")
    h = _ffi.dense_in_order_of(q)
    hg = _ffi.strided_like(h)[0]
    o = _dh_like(o, h)
    m = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    b = torch.empty((B, NH, S), device=q.device, dtype=torch.float32)
    lay = _ffi.layout(q, h, f)
    ws, n = _ffi.workspace(_ffi.OP_FORWARD_GATED, B, NH, S, D, dt, q.device)
    rc = _ffi.lib().mlstm_forward_gated_lx(_ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(o), _ffi.ptr(h),
                                           _ffi.ptr(hg), _ffi.ptr(m), _ffi.ptr(b), B, NH, S, D, dt, gdt, lay, _ffi.ptr(ws), n,
                                           _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_forward_gated_lx")
    return hg, h, m, b


def mlstm_backward_gated_hip(dhg, q, k, v, f, i, o, h=None, m=None, b=None):
    """Returns (dq, dk, dv, df, di, do) for the gradient dhg of the gated output, each in the layout of its tensor (do in
    the layout the kernels read o in: h's when h is given, else q's dimension order, dense)."""
    q, k, v = _ffi.dense_unless_disjoint(q, k, v)
    f, i = _ffi.dense_unless_disjoint(f, i)
    B, NH, S, D, dt, gdt = _check_inputs(q, k, v, f, i)
    for name, t in (("o", o), ("dh", dhg)):
        if not t.is_cuda or tuple(t.shape) != tuple(q.shape):
            raise ValueError(f"{name} must be a GPU tensor of q's shape, got {tuple(t.shape)} on {t.device}")
    if dhg.dtype != q.dtype or o.dtype != q.dtype:
        raise TypeError("dh and o must have q's dtype")
    if h is None or m is None or b is None:
        h = m = b = None
        like = _ffi.dense_in_order_of(q)
    else:
        _ffi.require_rows(h, "h", q.shape)
        like = h
    o, dhg = _dh_like(o, like), _dh_like(dhg, like)
    dq, dk, dv = _ffi.strided_like(q, 3)
    do = _ffi.strided_like(like)[0]
    df, di = _ffi.strided_like(f, 2)
    lay = _ffi.layout(q, like, f)
    ws, n = _ffi.workspace(_ffi.OP_BACKWARD_GATED, B, NH, S, D, dt, q.device)
    rc = _ffi.lib().mlstm_backward_gated_lx(_ffi.ptr(dhg), _ffi.ptr(q), _ffi.ptr(k), _ffi.ptr(v), _ffi.ptr(f), _ffi.ptr(i), _ffi.ptr(o),
                                            _ffi.ptr(h), _ffi.ptr(m), _ffi.ptr(b), _ffi.ptr(dq), _ffi.ptr(dk), _ffi.ptr(dv),
                                            _ffi.ptr(df), _ffi.ptr(di), _ffi.ptr(do), B, NH, S, D, dt, gdt, lay, _ffi.ptr(ws), n,
                                            _ffi.stream_ptr())
    _ffi.check_rc(rc, "mlstm_backward_gated_lx")
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
        assert dhg.stride(-1) == 1 or dhg.shape[-1] == 1, "dh must have a contiguous head dimension"
        q, k, v, f, i, o, m, b, h = ctx.saved_tensors
        dq, dk, dv, df, di, do = mlstm_backward_gated_hip(dhg, q, k, v, f, i, o, h, m, b)
        return dq, dk, dv, df, di, do, None, None


HIP_mLSTM_gated = Triton_mLSTM_gated
