"""Pins of the sLSTM oracle (oracle/slstm_oracle.py), on the CPU.  The reference holds no sLSTM code or vectors (README.md:9
lists the cell as open), so the oracle is anchored on what the published equations fix: a closed form where the recurrence
is switched off, the paper's unstabilised statement of the cell, invariances, and finite differences for the gradients."""
import pytest
import torch

from oracle import slstm_oracle as SO


def test_without_recurrence_is_a_gated_running_average():
    # r = 0, b = 0, exponential forget gate: c_t / n_t = sum_j w_tj tanh(z_j) / sum_j w_tj with
    # w_tj = exp(i_j + sum_{s=j+1..t} f_s) -- the decay matrix of the mLSTM, per unit
    wx, r, b, _ = SO.make_inputs(2, 2, 40, 8, seed=1, dtype=torch.float64)
    h = SO.slstm_forward(wx, torch.zeros_like(r), torch.zeros_like(b))
    i, f, z, o = (wx[:, :, g] for g in range(4))                       # [B,S,NH,DH]
    F = torch.cumsum(f, dim=1)
    D = i[:, None, :] + F[:, :, None] - F[:, None, :]                  # [B,t,j,NH,DH]
    mask = torch.tril(torch.ones(40, 40, dtype=torch.bool))[None, :, :, None, None]
    w = torch.softmax(D.masked_fill(~mask, float("-inf")), dim=2)
    ref = torch.sigmoid(o) * (w * torch.tanh(z)[:, None]).sum(2)
    assert torch.allclose(h, ref, rtol=1e-10, atol=1e-12)


@pytest.mark.parametrize("forget_sigmoid", [False, True])
def test_stabilised_equals_the_papers_plain_recurrence(forget_sigmoid):
    wx, r, b, _ = SO.make_inputs(2, 3, 24, 16, seed=2, dtype=torch.float64)
    a = SO.slstm_forward(wx, r, b, forget_sigmoid)
    p = SO.slstm_unstabilised(wx, r, b, forget_sigmoid)
    assert torch.allclose(a, p, rtol=1e-9, atol=1e-12)


def test_input_gate_shift_changes_nothing_and_extreme_gates_stay_finite():
    wx, r, b, _ = SO.make_inputs(1, 2, 30, 8, seed=3, dtype=torch.float64)
    h = SO.slstm_forward(wx, r, b)
    shifted = wx.clone()
    shifted[:, :, 0] += 7.5        # every input gate times e^7.5: c and n scale alike
    assert torch.allclose(SO.slstm_forward(shifted, r, b), h, rtol=1e-9, atol=1e-12)
    wild = wx.clone()
    wild[:, :, 0] += 300.0
    wild[:, ::3, 1] += 500.0
    wild[:, 1::3, 1] -= 500.0
    out, c, n, m = SO.slstm_forward(wild, r, b, return_states=True)
    assert bool(torch.isfinite(out).all()) and bool(torch.isfinite(c).all()) and bool((n > 0).all())
    assert float(out.abs().max()) <= 1.0 + 1e-12      # |tanh| <= 1 averaged, times a sigmoid


@pytest.mark.parametrize("forget_sigmoid", [False, True])
def test_gradients_against_finite_differences(forget_sigmoid):
    wx, r, b, dh = SO.make_inputs(1, 2, 6, 4, seed=4, dtype=torch.float64)
    dwx, dr, db = SO.slstm_backward(dh, wx, r, b, forget_sigmoid)
    loss = lambda wx_, r_, b_: float((SO.slstm_forward(wx_, r_, b_, forget_sigmoid) * dh).sum())
    eps = 1e-6
    g = torch.Generator().manual_seed(0)
    for name, t, grad in (("wx", wx, dwx), ("r", r, dr), ("b", b, db)):
        for _ in range(12):
            idx = tuple(int(torch.randint(0, n_, (1,), generator=g)) for n_ in t.shape)
            up, dn = t.clone(), t.clone()
            up[idx] += eps
            dn[idx] -= eps
            args = {"wx": (up, r, b), "r": (wx, up, b), "b": (wx, r, up)}[name], {"wx": (dn, r, b), "r": (wx, dn, b), "b": (wx, r, dn)}[name]
            fd = (loss(*args[0]) - loss(*args[1])) / (2 * eps)
            assert abs(fd - float(grad[idx])) <= 1e-6 * max(1.0, abs(fd)), (name, idx, fd, float(grad[idx]))
