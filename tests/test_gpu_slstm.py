"""Parity of the sLSTM kernels against the CPU oracle (oracle/slstm_oracle.py), fp32 bound of tests/helpers.py."""
import pytest
import torch

from oracle import slstm_oracle as SO
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu


def gpu(*xs):
    return [x.cuda() for x in xs]


@pytest.mark.parametrize("forget_sigmoid", [False, True])
@pytest.mark.parametrize("B,NH,S,DH", [(1, 1, 1, 32), (2, 2, 17, 32), (2, 3, 130, 64), (1, 2, 96, 128)])
def test_forward_and_backward_against_oracle(B, NH, S, DH, forget_sigmoid):
    from slstm import slstm_backward_hip, slstm_forward_hip
    wx, r, b, dh = SO.make_inputs(B, NH, S, DH, seed=B + S + DH)
    h, saved = slstm_forward_hip(*gpu(wx, r, b), forget_sigmoid=forget_sigmoid)
    assert_close(h, SO.slstm_forward(wx, r, b, forget_sigmoid), torch.float32, "h")
    dwx, dr, db = slstm_backward_hip(dh.cuda(), h, r.cuda(), saved, forget_sigmoid=forget_sigmoid)
    rwx, rr, rb = SO.slstm_backward(dh, wx, r, b, forget_sigmoid)
    assert_close(dwx, rwx, torch.float32, "dwx")
    assert_close(dr, rr, torch.float32, "dr")
    assert_close(db, rb, torch.float32, "db")


@pytest.mark.parametrize("B,NH,S,DH", [(1, 1, 7, 32), (1, 2, 8, 64), (2, 1, 9, 128), (1, 1, 16, 32), (3, 2, 23, 64)])
def test_sequences_around_the_prefetch_depth(B, NH, S, DH):
    # the kernels keep eight steps of inputs under way: sequences shorter than, equal to and just past that depth
    from slstm import slstm_backward_hip, slstm_forward_hip
    wx, r, b, dh = SO.make_inputs(B, NH, S, DH, seed=100 + S)
    want = SO.slstm_forward(wx, r, b, True)
    h, saved = slstm_forward_hip(*gpu(wx, r, b), forget_sigmoid=True)
    assert_close(h, want, torch.float32, "h")
    h_only, none = slstm_forward_hip(*gpu(wx, r, b), forget_sigmoid=True, save=False)
    assert none is None and torch.equal(h_only, h)      # the variant that keeps nothing for a backward: the same bits
    got = slstm_backward_hip(dh.cuda(), h, r.cuda(), saved, forget_sigmoid=True)
    for name, g, w in zip(("dwx", "dr", "db"), got, SO.slstm_backward(dh, wx, r, b, True)):
        assert_close(g, w, torch.float32, name)


def test_benchmark_shape_twice():
    # B16 NH4 S2048 DH64: two runs give the same bits (nothing depends on when a load lands), and match the oracle
    # (dR and db at a long sequence: test_long_sequence_and_many_heads)
    from slstm import slstm_backward_hip, slstm_forward_hip
    wx, r, b, dh = SO.make_inputs(16, 4, 2048, 64, seed=11, f_mean=2.0)
    dev = gpu(wx, r, b)
    h, saved = slstm_forward_hip(*dev, forget_sigmoid=True)
    got = slstm_backward_hip(dh.cuda(), h, dev[1], saved, forget_sigmoid=True)
    # the second run shares the memory system with a stream of large copies on another (default-priority) stream: the
    # kernels' inputs arrive several steps ahead of their use, later or earlier than before, and nothing may change
    side = torch.cuda.Stream()
    big = torch.empty(64 * 1024 * 1024, device="cuda")
    other = torch.empty_like(big)
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(40):
            other.copy_(big)
    h2, saved2 = slstm_forward_hip(*dev, forget_sigmoid=True)
    got2 = slstm_backward_hip(dh.cuda(), h2, dev[1], saved2, forget_sigmoid=True)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert torch.equal(h, h2) and torch.equal(saved, saved2)
    for x, y in zip(got, got2):
        assert torch.equal(x, y)
    # (the oracle on one sequence of the batch: h and dwx of a sequence depend on no other)
    assert_close(h[3:4], SO.slstm_forward(wx[3:4], r, b, True), torch.float32, "h")
    assert_close(got[0][3:4], SO.slstm_backward(dh[3:4], wx[3:4], r, b, True)[0], torch.float32, "dwx")


def test_long_sequence_and_many_heads():
    from slstm import slstm_backward_hip, slstm_forward_hip
    wx, r, b, dh = SO.make_inputs(4, 4, 1024, 64, seed=5, f_mean=1.0)
    h, saved = slstm_forward_hip(*gpu(wx, r, b), forget_sigmoid=True)
    assert_close(h, SO.slstm_forward(wx, r, b, True), torch.float32, "h")
    got = slstm_backward_hip(dh.cuda(), h, r.cuda(), saved, forget_sigmoid=True)
    for name, g, w in zip(("dwx", "dr", "db"), got, SO.slstm_backward(dh, wx, r, b, True)):
        assert_close(g, w, torch.float32, name)


def test_gates_far_from_zero_stay_finite():
    # the stabiliser at work: input gates of e^80, forget gates of e^(+-60) in turn
    from slstm import slstm_forward_hip
    wx, r, b, _ = SO.make_inputs(1, 2, 200, 32, seed=6)
    wx[:, :, 0] += 80.0
    wx[:, ::3, 1] += 60.0
    wx[:, 1::3, 1] -= 60.0
    h, _ = slstm_forward_hip(*gpu(wx, r, b))
    assert bool(torch.isfinite(h).all())
    assert_close(h, SO.slstm_forward(wx, r, b), torch.float32, "h")


def test_autograd_function_and_repeatability():
    from slstm import slstm
    wx, r, b, dh = SO.make_inputs(2, 2, 64, 64, seed=7)
    leaves = [x.cuda().requires_grad_(True) for x in (wx, r, b)]
    h = slstm(*leaves)
    h.backward(dh.cuda())
    for name, x, w in zip(("dwx", "dr", "db"), leaves, SO.slstm_backward(dh, wx, r, b)):
        assert_close(x.grad, w, torch.float32, name)
    again = [x.detach().clone().requires_grad_(True) for x in leaves]
    slstm(*again).backward(dh.cuda())
    for x, y in zip(leaves, again):
        assert torch.equal(x.grad, y.grad)          # the slices of dR and db are added in a fixed order
    with torch.no_grad():
        assert torch.equal(slstm(*leaves), h)


def test_rejects_what_it_cannot_serve():
    from slstm import slstm_forward_hip
    wx, r, b, _ = SO.make_inputs(1, 1, 8, 48, seed=1)
    with pytest.raises(ValueError):
        slstm_forward_hip(*gpu(wx, r, b))
    wx, r, b, _ = SO.make_inputs(1, 1, 8, 32, seed=1)
    with pytest.raises(TypeError):
        slstm_forward_hip(wx.cuda().half(), r.cuda(), b.cuda())
    with pytest.raises(ValueError):
        slstm_forward_hip(wx.cuda(), r.cuda()[:, :3], b.cuda())
