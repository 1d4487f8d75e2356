"""The matmul form on tensors in the caller's own layout ([B,S,NH,D] activations, slices of a fused q/k/v projection,
strided gates) and with the forget gate handed over as its log-sigmoid or cumulative sum.

The kernels address rows through the strides and change nothing else, so a run on strided views must equal a run on
dense copies bit for bit; that is what these tests assert (the dense path is the one checked against the oracle
everywhere else).  The gate forms change what is computed on the device (no log-sigmoid, no sum), so they are checked
against the oracle under the usual bound.
"""
import pytest
import torch

from oracle import mlstm_oracle as O
from tests.helpers import GRAD_NAMES, assert_close, literal_violations

pytestmark = pytest.mark.gpu


def bshd(x):
    """[B,NH,S,D] -> the same values stored [B,S,NH,D], viewed as [B,NH,S,D] again."""
    return x.transpose(1, 2).contiguous().transpose(1, 2)


def bsh(x):
    return x.transpose(1, 2).contiguous().transpose(1, 2)


def run_both(dtype, B, NH, S, D, seed, make_views, precise=False):
    from mlstm_matmul import mlstm_backward_saved_hip, mlstm_forward_save_hip
    q, k, v, f, i, dh = (x.cuda() for x in O.make_inputs(B, NH, S, D, dtype, seed=seed))
    qs, ks, vs, fs, is_, dhs = make_views(q, k, v, f, i, dh)
    for a, b_ in ((q, qs), (k, ks), (f, fs), (dh, dhs)):
        assert torch.equal(a, b_)
    h0, m0, b0, sv0 = mlstm_forward_save_hip(q, k, v, f, i, precise=precise)
    g0 = mlstm_backward_saved_hip(dh, q, k, v, f, i, h0, m0, b0, sv0, precise=precise)
    h1, m1, b1, sv1 = mlstm_forward_save_hip(qs, ks, vs, fs, is_, precise=precise)
    g1 = mlstm_backward_saved_hip(dhs, qs, ks, vs, fs, is_, h1, m1, b1, sv1, precise=precise)
    assert torch.equal(h0, h1) and torch.equal(m0, m1) and torch.equal(b0, b1), "forward differs"
    for name, x0, x1 in zip(GRAD_NAMES, g0, g1):
        assert torch.equal(x0, x1), name
    return (qs, ks, vs, fs, is_), h1, g1


CASES = [(torch.bfloat16, 2, 4, 1536, 256), (torch.bfloat16, 1, 3, 1100, 128), (torch.float16, 2, 2, 200, 128),
         (torch.bfloat16, 1, 2, 300, 64), (torch.float32, 2, 2, 330, 64), (torch.float32, 1, 2, 130, 128)]


@pytest.mark.parametrize("dtype,B,NH,S,D", CASES)
def test_projection_layout_equals_dense(dtype, B, NH, S, D):
    # every [.., D] tensor stored [B,S,NH,D], the gates [B,S,NH]: eight-wave and 16x16 kernels in chunks and without,
    # the generic kernels (D = 64, fp32), a ragged last tile
    views, h, grads = run_both(dtype, B, NH, S, D, 31, lambda q, k, v, f, i, dh: (bshd(q), bshd(k), bshd(v), bsh(f), bsh(i), bshd(dh)))
    q = views[0]
    assert q.stride() == (S * NH * D, D, NH * D, 1)
    assert h.stride() == q.stride() and h.transpose(1, 2).is_contiguous()        # h is a [B,S,NH,D] tensor again
    for g in grads[:3]:
        assert g.stride() == q.stride()
    assert grads[3].stride() == views[3].stride() == (S * NH, 1, NH)


@pytest.mark.parametrize("dtype,B,NH,S,D", [CASES[0], CASES[4]])
def test_fused_projection_slices_equal_dense(dtype, B, NH, S, D):
    # q, k, v as slices of one [B,S,3,NH,D] buffer: position stride 3*NH*D, gaps between the rows of one tensor
    def views(q, k, v, f, i, dh):
        qkv = torch.stack([x.transpose(1, 2) for x in (q, k, v)], dim=2).contiguous()      # [B,S,3,NH,D]
        return (qkv[:, :, 0].transpose(1, 2), qkv[:, :, 1].transpose(1, 2), qkv[:, :, 2].transpose(1, 2), f, i, dh)
    vws, h, grads = run_both(dtype, B, NH, S, D, 32, views)
    assert vws[0].stride() == (S * 3 * NH * D, D, 3 * NH * D, 1)
    assert h.stride() == (S * NH * D, D, NH * D, 1)
    assert grads[0].stride() == vws[0].stride()


def test_split_mode_in_projection_layout():
    run_both(torch.bfloat16, 1, 2, 700, 128, 33, lambda q, k, v, f, i, dh: (bshd(q), bshd(k), bshd(v), bsh(f), bsh(i), bshd(dh)), precise=True)


def test_backward_without_saved_forward_in_projection_layout():
    # mlstm_backward_hip recomputes the forward into a buffer of its own (dense) while dh, q, k, v stay strided
    from mlstm_matmul import mlstm_backward_hip
    q, k, v, f, i, dh = (x.cuda() for x in O.make_inputs(1, 4, 1280, 128, torch.bfloat16, seed=34))
    g0 = mlstm_backward_hip(dh, q, k, v, f, i)
    g1 = mlstm_backward_hip(bshd(dh), bshd(q), bshd(k), bshd(v), bsh(f), bsh(i))
    for name, x0, x1 in zip(GRAD_NAMES, g0, g1):
        assert torch.equal(x0, x1), name


def test_autograd_from_a_projection_without_copies():
    from mlstm_matmul import Triton_mLSTM
    B, NH, S, D = 2, 4, 1088, 128
    q, k, v, f, i, dh = (x.cuda() for x in O.make_inputs(B, NH, S, D, torch.bfloat16, seed=35))
    dense = [x.clone().requires_grad_(True) for x in (q, k, v, f, i)]
    Triton_mLSTM.apply(*dense).backward(dh)
    # the same numbers as a module would hold them: activations [B,S,NH*D], gate pre-activations [B,S,NH]
    acts = [x.transpose(1, 2).reshape(B, S, NH * D).clone().requires_grad_(True) for x in (q, k, v)]
    gates = [x.transpose(1, 2).contiguous().clone().requires_grad_(True) for x in (f, i)]
    h = Triton_mLSTM.apply(*(a.view(B, S, NH, D).transpose(1, 2) for a in acts), *(g.transpose(1, 2) for g in gates))
    out = h.transpose(1, 2).reshape(B, S, NH * D)
    assert out.data_ptr() == h.data_ptr()                    # a view: the output projection reads h as it lies
    out.backward(dh.transpose(1, 2).reshape(B, S, NH * D))
    for d, a in zip(dense[:3], acts):
        assert torch.equal(d.grad, a.grad.view(B, S, NH, D).transpose(1, 2))
    for d, g in zip(dense[3:], gates):
        assert torch.equal(d.grad, g.grad.transpose(1, 2))


def gate_form_reference(dh, q, k, v, f, i):
    """Oracle gradients with respect to lf = logsigmoid(f) and Fc = cumsum(lf), from the gradient of f itself."""
    ref = O.mlstm_backward_dense(dh, q, k, v, f, i, zero_first_df=True)
    dlf = ref[3] / torch.sigmoid(-f.double())                  # d/df = sigmoid(-f) d/dlf; entry 0 is 0 either way
    dfc = dlf - torch.cat([dlf[..., 1:], torch.zeros_like(dlf[..., :1])], dim=-1)
    return ref, dlf, dfc


@pytest.mark.parametrize("S,D", [(200, 64), (1300, 128)])
def test_gate_forms_against_oracle_fp32(S, D):
    from mlstm_matmul import mlstm_backward_hip, mlstm_forward_hip
    q, k, v, f, i, dh = O.make_inputs(1, 2, S, D, torch.float32, seed=36)
    ref, dlf, dfc = gate_form_reference(dh, q, k, v, f, i)
    href, mref, bref = O.mlstm_forward_dense(q, k, v, f, i)
    lf = torch.nn.functional.logsigmoid(f.double())
    forms = {"logsigmoid": (lf.float(), dlf), "cumsum": (torch.cumsum(lf, -1).float(), dfc)}
    dev = [x.cuda() for x in (q, k, v, i, dh)]
    for form, (fin, dfin) in forms.items():
        # the oracle sees the gate exactly as the kernel does: the fp32 values handed over, differenced for "cumsum"
        h, m, b = mlstm_forward_hip(dev[0], dev[1], dev[2], fin.cuda(), dev[3], gate_form=form)
        assert_close(h, href, torch.float32, form + " h")
        assert_close(m, mref, torch.float32, form + " m")
        g = mlstm_backward_hip(dev[4], dev[0], dev[1], dev[2], fin.cuda(), dev[3], gate_form=form)
        for name, got, want in zip(GRAD_NAMES, g, (ref[0], ref[1], ref[2], dfin, ref[4])):
            assert_close(got, want, torch.float32, form + " " + name)


def test_logsigmoid_form_matches_raw_form_bf16():
    # 16-bit tensors, fp32 gates, in chunks: handing over logsigmoid(f) changes nothing but who computes it
    from mlstm_matmul import mlstm_backward_hip, mlstm_forward_hip
    q, k, v, f, i, dh = (x.cuda() for x in O.make_inputs(1, 2, 1536, 128, torch.bfloat16, seed=37))
    f, i = f.float(), i.float()
    h0, m0, b0 = mlstm_forward_hip(q, k, v, f, i)
    g0 = mlstm_backward_hip(dh, q, k, v, f, i, h0, m0, b0)
    lf = torch.nn.functional.logsigmoid(f)
    h1, m1, b1 = mlstm_forward_hip(q, k, v, lf, i, gate_form="logsigmoid")
    g1 = mlstm_backward_hip(dh, q, k, v, lf, i, h1, m1, b1, gate_form="logsigmoid")
    assert literal_violations(h1, h0)[0] == 0.0
    for name, x0, x1 in zip(GRAD_NAMES, g0, g1):
        if name == "df":
            x0 = x0 / torch.sigmoid(-f)
        bad, rms = literal_violations(x1, x0)
        assert bad == 0.0 and rms < 2e-3, (name, bad, rms)


def test_layouts_the_kernels_cannot_take_are_rejected():
    from mlstm_matmul import mlstm_forward_hip
    q, k, v, f, i, _ = (x.cuda() for x in O.make_inputs(1, 2, 128, 64, torch.bfloat16, seed=1))
    with pytest.raises(ValueError):      # head dimension not contiguous
        mlstm_forward_hip(q.transpose(2, 3).contiguous().transpose(2, 3), k, v, f, i)
    with pytest.raises(ValueError):      # k in another layout than q
        mlstm_forward_hip(bshd(q), k, v, f, i)
    pad = torch.zeros(1, 2, 128, 68, dtype=torch.bfloat16, device="cuda")   # rows 136 bytes apart: not 16-byte aligned
    with pytest.raises(ValueError):
        mlstm_forward_hip(pad[..., :64], pad[..., :64], pad[..., :64], f, i)
    with pytest.raises(ValueError):      # the cumulative sum needs fp32 gates
        mlstm_forward_hip(q, k, v, f, i, gate_form="cumsum")
    with pytest.raises(ValueError):
        mlstm_forward_hip(q, k, v, f, i, gate_form="sigmoid")


def test_expanded_inputs_get_the_summed_gradient():
    """Gates shared over the heads (f.expand) and a query shared over the batch (q.expand): the gradient with respect to
    the unexpanded tensor is the sum over the copies, as with dense inputs; gradient buffers never alias."""
    from mlstm_matmul import Triton_mLSTM
    B, NH, S, D = 2, 3, 200, 64
    q, k, v, f, i, dh = (x.cuda() for x in O.make_inputs(B, NH, S, D, torch.float32, seed=41))
    f1, i1, q1 = f[:, :1].clone().requires_grad_(True), i[:, :1].clone().requires_grad_(True), q[:1].clone().requires_grad_(True)
    k1, v1 = k.clone().requires_grad_(True), v.clone().requires_grad_(True)
    Triton_mLSTM.apply(q1.expand(B, NH, S, D), k1, v1, f1.expand(B, NH, S), i1.expand(B, NH, S)).backward(dh)
    dense = [q1.detach().expand(B, NH, S, D).contiguous().requires_grad_(True), k.clone().requires_grad_(True), v.clone().requires_grad_(True),
             f1.detach().expand(B, NH, S).contiguous().requires_grad_(True), i1.detach().expand(B, NH, S).contiguous().requires_grad_(True)]
    Triton_mLSTM.apply(*dense).backward(dh)
    assert_close(q1.grad, dense[0].grad.sum(0, keepdim=True), torch.float32, "dq of the shared query")
    assert_close(f1.grad, dense[3].grad.sum(1, keepdim=True), torch.float32, "df of the shared gates")
    assert_close(i1.grad, dense[4].grad.sum(1, keepdim=True), torch.float32, "di of the shared gates")
    assert torch.equal(k1.grad, dense[1].grad) and torch.equal(v1.grad, dense[2].grad)


def test_library_refuses_overlapping_layouts_for_tensors_it_writes():
    from _mlstm_pkg import submodule
    ffi = submodule("_ffi")
    B, NH, S, D = 2, 2, 128, 64
    q, k, v, f, i, dh = (x.cuda() for x in O.make_inputs(B, NH, S, D, torch.float32, seed=42))
    h = torch.empty_like(q)
    g = [torch.empty_like(q) for _ in range(3)] + [torch.empty_like(f) for _ in range(2)]
    L = ffi.lib()
    ws, n = ffi.workspace(ffi.OP_BACKWARD, B, NH, S, D, ffi.F32, q.device)

    def backward(lay):
        return L.mlstm_backward_lx(ffi.ptr(dh), ffi.ptr(q), ffi.ptr(k), ffi.ptr(v), ffi.ptr(f), ffi.ptr(i), None, None, None, *[ffi.ptr(x) for x in g],
                                   B, NH, S, D, ffi.F32, ffi.F32, lay, ffi.ptr(ws), n, ffi.stream_ptr())

    good = ffi.layout(q, h, f)
    assert backward(good) == 0
    shared_gates = ffi.Layout(*[getattr(good, n_) for n_, _ in ffi.Layout._fields_])
    shared_gates.gate_h = 0                       # gates shared over the heads: df, di would alias
    assert backward(shared_gates) == -1
    shared_q = ffi.Layout(*[getattr(good, n_) for n_, _ in ffi.Layout._fields_])
    shared_q.qkv_b = 0                            # q, k, v shared over the batch: dq, dk, dv would alias
    assert backward(shared_q) == -1
    # the forward only reads q, k, v and the gates: the same layouts are fine there, an overlapping h is not
    ws2, n2 = ffi.workspace(ffi.OP_FORWARD, B, NH, S, D, ffi.F32, q.device)
    fwd = lambda lay: L.mlstm_forward_lx(ffi.ptr(q), ffi.ptr(k), ffi.ptr(v), ffi.ptr(f), ffi.ptr(i), ffi.ptr(h), None, None, B, NH, S, D,
                                         ffi.F32, ffi.F32, lay, ffi.ptr(ws2), n2, ffi.stream_ptr())
    assert fwd(shared_gates) == 0 and fwd(shared_q) == 0
    shared_h = ffi.Layout(*[getattr(good, n_) for n_, _ in ffi.Layout._fields_])
    shared_h.out_h = 0
    assert fwd(shared_h) == -1
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype,B,NH,S,D", [CASES[0], CASES[1], CASES[3], CASES[4]])
def test_gated_entry_points_in_projection_layout(dtype, B, NH, S, D):
    # the matmul form with the output gate on [B,S,NH,D] activations: o, the gated output and its gradient travel in h's
    # layout, and every result equals the run on dense copies bit for bit (forward, backward with the forward's outputs,
    # backward that recomputes them, autograd)
    from mlstm_matmul import Triton_mLSTM_gated, mlstm_backward_gated_hip, mlstm_forward_gated_hip
    q, k, v, f, i, dh, o = (x.cuda() for x in O.make_inputs(B, NH, S, D, dtype, seed=77, with_o=True))
    qs, ks, vs, os_, dhs, fs, is_ = bshd(q), bshd(k), bshd(v), bshd(o), bshd(dh), bsh(f), bsh(i)
    hg0, h0, m0, b0 = mlstm_forward_gated_hip(q, k, v, f, i, o)
    hg1, h1, m1, b1 = mlstm_forward_gated_hip(qs, ks, vs, fs, is_, os_)
    assert torch.equal(hg0, hg1) and torch.equal(h0, h1) and torch.equal(m0, m1) and torch.equal(b0, b1)
    assert hg1.stride() == qs.stride() and h1.stride() == qs.stride()
    g0 = mlstm_backward_gated_hip(dh, q, k, v, f, i, o, h0, m0, b0)
    g1 = mlstm_backward_gated_hip(dhs, qs, ks, vs, fs, is_, os_, h1, m1, b1)
    g2 = mlstm_backward_gated_hip(dhs, qs, ks, vs, fs, is_, os_)               # recomputes h, m, b
    for name, x0, x1, x2 in zip(list(GRAD_NAMES) + ["do"], g0, g1, g2):
        assert torch.equal(x0, x1), name
        assert torch.equal(x0, x2), name + " (recomputed forward)"
    assert g1[0].stride() == qs.stride() and g1[5].stride() == qs.stride() and g1[3].stride() == fs.stride()
    ins = [x.clone().requires_grad_(True) for x in (qs, ks, vs, fs, is_, os_)]
    Triton_mLSTM_gated.apply(*ins).backward(dhs)
    for name, x, g in zip(list(GRAD_NAMES) + ["do"], [ins[0], ins[1], ins[2], ins[3], ins[4], ins[5]], g0):
        assert torch.equal(x.grad, g), name


def test_scan_form_takes_views_through_one_copy():
    # the scan kernels are dense; the wrapper copies views once, so a [B,S,NH,D] view gives the dense run's bits
    from mlstm_scan import mlstm_scan
    B, NH, S, D = 2, 2, 200, 128
    q, k, v, f, i, dh, o = (x.cuda() for x in O.make_inputs(B, NH, S, D, torch.float32, seed=5, with_o=True))
    dense = [x.clone().requires_grad_(True) for x in (q, k, v, f, i, o)]
    views = [x.clone().requires_grad_(True) for x in (bshd(q), bshd(k), bshd(v), bsh(f), bsh(i), bshd(o))]
    assert not views[0].is_contiguous()
    h0 = mlstm_scan(*dense)
    h1 = mlstm_scan(*views)
    assert torch.equal(h0, h1)
    h0.backward(dh)
    h1.backward(bshd(dh))
    for a, b_ in zip(dense, views):
        assert torch.equal(a.grad, b_.grad)
