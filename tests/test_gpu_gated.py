"""Parity of the matmul form with the output gate h_gated = silu(o) * h (forward and backward) against the CPU
oracle, through the C ABI, and its agreement with the scan form, which computes the same function."""
import pytest
import torch

from _mlstm_pkg import submodule
from oracle import mlstm_oracle as O
from tests.helpers import assert_close, assert_matches_oracle, rounding_noise

pytestmark = pytest.mark.gpu

ffi = submodule("_ffi")
mm = submodule("mlstm_matmul")
ms = submodule("mlstm_scan")

DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
GRADS = ["dq", "dk", "dv", "df", "di", "do"]


def dev(*xs):
    return [x.cuda() for x in xs]


@pytest.mark.parametrize("S", [1, 33, 100, 257])
@pytest.mark.parametrize("D", [64, 128])
def test_gated_forward_fp32(S, D):
    q, k, v, f, i, _, o = O.make_inputs(1, 2, S, D, torch.float32, seed=S + D, with_o=True)
    hg, h, m, b = mm.mlstm_forward_gated_hip(*dev(q, k, v, f, i, o))
    assert_close(hg, O.mlstm_scan_dense(q, k, v, f, i, o), torch.float32, "h_gated")
    # the ungated outputs are those of the plain forward, bit for bit (same kernel, same accumulators)
    h0, m0, b0 = mm.mlstm_forward_hip(*dev(q, k, v, f, i))
    assert torch.equal(h, h0) and torch.equal(m, m0) and torch.equal(b, b0)


@pytest.mark.parametrize("generic", [False, True])
@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("S,D", [(200, 64), (512, 128), (130, 256), (384, 256)])
def test_gated_forward_half(dt, S, D, generic):
    dtype = DT[dt]
    q, k, v, f, i, _, o = O.make_inputs(2, 2, S, D, dtype, seed=7 * S + D, with_o=True)
    before = ffi.force_generic_kernels(generic)
    try:
        hg, h, _, _ = mm.mlstm_forward_gated_hip(*dev(q, k, v, f, i, o))
    finally:
        ffi.force_generic_kernels(before)
    assert hg.dtype == dtype
    sig = rounding_noise(torch.zeros_like(q), q, k, v, f, i, dtype)
    assert_close(hg, O.mlstm_scan_dense(q, k, v, f, i, o), dtype, "h_gated", sig["h"] * torch.nn.functional.silu(o.double()).abs())
    assert_close(h, O.mlstm_forward_dense(q, k, v, f, i)[0], dtype, "h", sig["h"])


def test_gated_matmul_form_equals_scan_form():
    q, k, v, f, i, _, o = O.make_inputs(1, 2, 512, 128, torch.float32, seed=21, with_o=True)
    args = dev(q, k, v, f, i, o)
    a = mm.mlstm_matmul_gated(*args)
    b = ms.mlstm_scan(*args)
    assert_close(a, b, torch.float32, "matmul form vs scan form")


@pytest.mark.parametrize("S,D", [(1, 64), (40, 64), (129, 64), (256, 128)])
@pytest.mark.parametrize("with_fwd", [True, False])
def test_gated_backward_fp32(S, D, with_fwd):
    q, k, v, f, i, dhg, o = O.make_inputs(1, 2, S, D, torch.float32, seed=3 * S + D, with_o=True)
    args = dev(q, k, v, f, i, o)
    fwd = mm.mlstm_forward_gated_hip(*args)[1:] if with_fwd else ()
    got = mm.mlstm_backward_gated_hip(dhg.cuda(), *args, *fwd)
    ref = O.mlstm_gated_backward_dense(dhg, q, k, v, f, i, o, zero_first_df=True)
    for name, g, r in zip(GRADS, got, ref):
        assert_close(g, r, torch.float32, name)
    assert float(got[3][..., 0].abs().max()) == 0.0


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("S,D", [(64, 64), (200, 128), (320, 256)])
def test_gated_backward_half(dt, S, D):
    dtype = DT[dt]
    q, k, v, f, i, dhg, o = O.make_inputs(1, 2, S, D, dtype, seed=5 * S + D, f_mean=2.0, with_o=True)
    args = dev(q, k, v, f, i, o)
    fwd = mm.mlstm_forward_gated_hip(*args)[1:]
    got = mm.mlstm_backward_gated_hip(dhg.cuda(), *args, *fwd)
    # The kernels see the ungated upstream gradient dhg * silu(o) rounded to the 16-bit type: it is an MFMA operand like
    # every other input.  The oracle gets the same rounded operand, so that the comparison is about the arithmetic and
    # not about the storage format of this one intermediate (d_o does not go through it).
    dh = (dhg.double() * torch.nn.functional.silu(o.double())).to(dtype)
    ref = list(O.mlstm_backward_dense(dh, q, k, v, f, i, zero_first_df=True))
    ref.append(O.mlstm_gated_backward_dense(dhg, q, k, v, f, i, o)[5])
    sig = rounding_noise(dh, q, k, v, f, i, dtype)
    # d_o = dhg * h * silu'(o) is formed from the stored (rounded, noisy) h
    so = torch.sigmoid(o.double())
    sig["do"] = (dhg.double() * so * (1.0 + o.double() * (1.0 - so))).abs() * sig["h"]
    for name, g, r in zip(GRADS, got, ref):
        assert g.dtype == dtype
        assert_close(g, r, dtype, name, sig[name])


def test_gated_autograd_function():
    q, k, v, f, i, dhg, o = O.make_inputs(1, 2, 96, 64, torch.float32, seed=4, with_o=True)
    ins = [x.cuda().requires_grad_(True) for x in (q, k, v, f, i, o)]
    hg = mm.Triton_mLSTM_gated.apply(*ins, 16, 8)
    hg.backward(dhg.cuda())
    ref = O.mlstm_gated_backward_dense(dhg, q, k, v, f, i, o, zero_first_df=True)
    for name, x, r in zip(GRADS, ins, ref):
        assert x.grad is not None and x.grad.shape == x.shape
        assert_close(x.grad, r, torch.float32, name)
    # results do not depend on the tuning hints, and the default arguments work
    hg2 = mm.Triton_mLSTM_gated.apply(*[x.detach() for x in ins])
    assert torch.equal(hg2, hg.detach())


def test_gated_headline_shape_properties():
    """B4 H8 S4096 D256 bf16 is beyond the CPU oracle: there the gate is checked through what fixes it, the ungated
    result of the same launch (h_gated = silu(o) h up to one rounding of h) and the ungated backward run on
    dh = dhg silu(o) formed by torch (gradients equal up to the rounding of dh and the fast exponential)."""
    dtype = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(5)
    B, NH, S, D = 4, 8, 4096, 256
    mk = lambda *s: torch.randn(s, generator=g, device="cuda", dtype=torch.float32)
    q, k, v, o, dhg = (mk(B, NH, S, D).to(dtype) for _ in range(5))
    f, i = (mk(B, NH, S) + 3.0).to(dtype), mk(B, NH, S).to(dtype)
    hg, h, m, b = mm.mlstm_forward_gated_hip(q, k, v, f, i, o)
    want = h.float() * torch.nn.functional.silu(o.float())
    err = (hg.float() - want).abs()
    assert bool((err <= 2.0 ** -7 * want.abs() + 1e-30).all())   # two bf16 roundings (h, then the product)
    got = mm.mlstm_backward_gated_hip(dhg, q, k, v, f, i, o, h, m, b)
    dh = (dhg.float() * torch.nn.functional.silu(o.float())).to(dtype)
    ref = mm.mlstm_backward_hip(dh, q, k, v, f, i, h, m, b)
    for name, a, r in zip(GRADS[:5], got[:5], ref):
        d = (a.float() - r.float()).pow(2).mean().sqrt() / r.float().pow(2).mean().sqrt()
        assert float(d) < 2e-3, (name, float(d))   # a few elements of dh round the other way
    so = torch.sigmoid(o.float())
    do_ref = dhg.float() * h.float() * so * (1.0 + o.float() * (1.0 - so))
    assert_close(got[5], do_ref, dtype, "do")   # (both sides use the same stored h: plain 16-bit rounding of the result)
