"""Parity of the scan form's backward (HIP) against the dense oracle's gated backward, fp32 bound (tests/helpers.py)."""
import pytest
import torch

from oracle import mlstm_oracle as O
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

NAMES = ["dq", "dk", "dv", "df", "di", "do"]


def run_backward(dh, q, k, v, f, i, o):
    from mlstm_scan import mlstm_scan_backward_hip
    return mlstm_scan_backward_hip(*(x.cuda() for x in (dh, q, k, v, f, i, o)))


def check(grads, dh, q, k, v, f, i, o, tag=""):
    ref = O.mlstm_gated_backward_dense(dh, q, k, v, f, i, o, zero_first_df=True)
    for name, g, r in zip(NAMES, grads, ref):
        assert g.dtype == torch.float32
        assert_close(g, r, torch.float32, tag + name)


def test_scan_backward_single_position():
    # S = 1: where |b| > exp(-m) the output is v * sign(b), so dq, dk (and di = k . dk) are the residue of two terms
    # that cancel (1e-7 against terms of 1e-1): those are held to an absolute 1e-6, the rest to the usual bound
    q, k, v, f, i, dh, o = O.make_inputs(1, 2, 1, 64, torch.float32, seed=65, with_o=True)
    got = run_backward(dh, q, k, v, f, i, o)
    ref = O.mlstm_gated_backward_dense(dh, q, k, v, f, i, o, zero_first_df=True)
    for name, g, r in zip(NAMES, got, ref):
        if name in ("dq", "dk", "di"):
            assert float((g.cpu().double() - r).abs().max()) <= 1e-6, name
        else:
            assert_close(g, r, torch.float32, name)


@pytest.mark.parametrize("S,D", [(16, 64), (64, 64), (65, 64), (100, 128), (192, 128), (130, 256), (256, 512), (200, 1024)])
def test_scan_backward_small(S, D):
    # one position, less than a chunk, whole chunks, a ragged last chunk (the reversed pass then starts inside a chunk)
    q, k, v, f, i, dh, o = O.make_inputs(1, 2, S, D, torch.float32, seed=S + D, with_o=True)
    check(run_backward(dh, q, k, v, f, i, o), dh, q, k, v, f, i, o)


@pytest.mark.parametrize("f_mean,i_mean", [(-3.0, 0.0), (0.0, 2.0), (8.0, -1.0), (3.0, -4.0)])
def test_scan_backward_gate_regimes(f_mean, i_mean):
    # strong forgetting, input-dominated, almost no forgetting, and rows whose normaliser is the exp(-m) branch
    q, k, v, f, i, dh, o = O.make_inputs(1, 2, 640, 128, torch.float32, seed=21, f_mean=f_mean, i_mean=i_mean, with_o=True)
    check(run_backward(dh, q, k, v, f, i, o), dh, q, k, v, f, i, o)


def test_scan_backward_many_heads():
    q, k, v, f, i, dh, o = O.make_inputs(4, 4, 200, 256, torch.float32, seed=22, with_o=True)
    check(run_backward(dh, q, k, v, f, i, o), dh, q, k, v, f, i, o)


def test_scan_autograd_path():
    # mlstm_scan on tensors that require a gradient records the backward; .backward() fills every input's .grad
    from mlstm_scan import mlstm_scan
    q, k, v, f, i, dh, o = O.make_inputs(2, 2, 150, 128, torch.float32, seed=23, with_o=True)
    leaves = [x.cuda().requires_grad_(True) for x in (q, k, v, f, i, o)]
    h = mlstm_scan(*leaves)
    assert_close(h, O.mlstm_scan_dense(q, k, v, f, i, o), torch.float32, "h")
    h.backward(dh.cuda())
    check([x.grad for x in leaves], dh, q, k, v, f, i, o, "autograd ")
    with torch.no_grad():
        assert not mlstm_scan(*leaves).requires_grad


def test_scan_backward_equals_gated_matmul_backward():
    # both backward paths on the GPU, at a head dimension both serve in fp32
    from mlstm_matmul import mlstm_backward_gated_hip, mlstm_forward_gated_hip
    q, k, v, f, i, dh, o = (x.cuda() for x in O.make_inputs(2, 2, 320, 128, torch.float32, seed=24, with_o=True))
    got = run_backward(dh, q, k, v, f, i, o)
    _, h, m, b = mlstm_forward_gated_hip(q, k, v, f, i, o)
    ref = mlstm_backward_gated_hip(dh, q, k, v, f, i, o, h, m, b)
    for name, g, r in zip(NAMES, got, ref):
        assert_close(g, r, torch.float32, name)


@pytest.mark.parametrize("S,D", [(100, 64), (192, 128), (700, 256), (300, 1024)])
def test_kept_forward_gives_the_same_bits(S, D):
    # the forward of a training step keeps its ungated output and normaliser sums; the backward that is handed them
    # skips its own forward pass and must return what the recomputing backward returns, bit for bit
    from mlstm_scan import mlstm_scan_backward_hip, mlstm_scan_forward_hip, mlstm_scan_forward_save_hip
    q, k, v, f, i, dh, o = O.make_inputs(1, 3, S, D, torch.float32, seed=S + D, with_o=True)
    dev = [x.cuda() for x in (dh, q, k, v, f, i, o)]
    h, h_ungated, b = mlstm_scan_forward_save_hip(*dev[1:])
    assert torch.equal(h, mlstm_scan_forward_hip(*dev[1:]))
    hu_ref, _, b_ref = O.mlstm_forward_dense(q, k, v, f, i)      # (the scan form without its gate is the matmul form)
    assert_close(h_ungated, hu_ref, torch.float32, "h_ungated")
    assert_close(b, b_ref, torch.float32, "b")
    kept = mlstm_scan_backward_hip(*dev, h_ungated, b)
    plain = mlstm_scan_backward_hip(*dev)
    for name, x, y in zip(NAMES, kept, plain):
        assert torch.equal(x, y), name
    check(kept, dh, q, k, v, f, i, o)
    with pytest.raises(ValueError):
        mlstm_scan_backward_hip(*dev, h_ungated, None)


def test_scan_backward_is_repeatable():
    q, k, v, f, i, dh, o = (x.cuda() for x in O.make_inputs(1, 4, 300, 256, torch.float32, seed=25, with_o=True))
    a = run_backward(dh, q, k, v, f, i, o)
    b = run_backward(dh, q, k, v, f, i, o)
    for name, x, y in zip(NAMES, a, b):
        assert torch.equal(x, y), name


def test_config3_scan_backward():
    # B1 H4 S2048 D1024 fp32: the scan form's own configuration (mlstm_scan.py:375-394)
    q, k, v, f, i, dh, o = O.make_inputs(1, 4, 2048, 1024, torch.float32, seed=0, with_o=True)
    check(run_backward(dh, q, k, v, f, i, o), dh, q, k, v, f, i, o)


def test_scan_backward_rejects_what_it_cannot_serve():
    from mlstm_scan import mlstm_scan_backward_hip
    q, k, v, f, i, dh, o = (x.cuda() for x in O.make_inputs(1, 1, 64, 64, torch.float32, seed=1, with_o=True))
    with pytest.raises(TypeError):
        mlstm_scan_backward_hip(dh.half(), q, k, v, f, i, o)
    with pytest.raises(ValueError):
        mlstm_scan_backward_hip(dh[:, :, :32], q, k, v, f, i, o)
    x96 = [t.cuda() for t in O.make_inputs(1, 1, 64, 96, torch.float32, seed=1, with_o=True)]
    with pytest.raises(ValueError):   # a head dimension the scan kernels are not built for
        mlstm_scan_backward_hip(x96[5], x96[0], x96[1], x96[2], x96[3], x96[4], x96[6])


@pytest.mark.parametrize("S,D", [(300, 256), (200, 512), (130, 1024)])
def test_matmul_form_fp32_at_large_head_dimensions(S, D):
    # fp32 at D >= 256: the matmul form's entry points (forward with m and b, backward, the autograd function) run on
    # the scan kernels; checked against the dense oracle of the matmul form
    from mlstm_matmul import Triton_mLSTM, mlstm_backward_hip, mlstm_forward_hip
    q, k, v, f, i, dh = O.make_inputs(1, 2, S, D, torch.float32, seed=S + D)
    dev = [x.cuda() for x in (q, k, v, f, i)]
    h, m, b = mlstm_forward_hip(*dev)
    hr, mr, br = O.mlstm_forward_dense(q, k, v, f, i)
    assert_close(h, hr, torch.float32, "h")
    assert_close(m, mr, torch.float32, "m")
    assert_close(b, br, torch.float32, "b")
    ref = O.mlstm_backward_dense(dh, q, k, v, f, i, zero_first_df=True)
    for name, g, r in zip(NAMES, mlstm_backward_hip(dh.cuda(), *dev), ref):
        assert_close(g, r, torch.float32, name)
    leaves = [x.clone().requires_grad_(True) for x in dev]
    Triton_mLSTM.apply(*leaves).backward(dh.cuda())
    for name, x, r in zip(NAMES, leaves, ref):
        assert_close(x.grad, r, torch.float32, "autograd " + name)


def test_matmul_form_fp32_large_head_dimension_limits():
    from mlstm_matmul import mlstm_forward_hip
    q, k, v, f, i, _ = (x.cuda() for x in O.make_inputs(1, 2, 128, 256, torch.float32, seed=2))
    with pytest.raises(ValueError):      # a layout of the caller's: dense tensors only at these sizes
        mlstm_forward_hip(*(x.transpose(1, 2).contiguous().transpose(1, 2) for x in (q, k, v)), f, i)


@pytest.mark.parametrize("S,D", [(4096, 128), (2500, 64)])
def test_scan_backward_one_long_sequence(S, D):
    # one head: every pass of the state kernel runs in segments (two of them from the end of the sequence backwards)
    q, k, v, f, i, dh, o = O.make_inputs(1, 1, S, D, torch.float32, seed=S + D, with_o=True)
    check(run_backward(dh, q, k, v, f, i, o), dh, q, k, v, f, i, o)
