"""Pins for oracle/mlstm_oracle.py: each check is chosen so that a plausible mistake in the
restatement (dropped term, wrong sign or index, transposed operand) fails it.  None of
them re-types the oracle's own formula."""
import math

import pytest
import torch

from oracle import mlstm_oracle as O

torch.manual_seed(0)
F64 = torch.float64


def rnd(*shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=F64)


def small(B=2, NH=2, S=24, D=8, seed=0):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: torch.randn(s, generator=g, dtype=F64)
    return mk(B, NH, S, D), mk(B, NH, S, D), mk(B, NH, S, D), mk(B, NH, S), mk(B, NH, S), mk(B, NH, S, D), mk(B, NH, S, D)


def test_forward_s1_closed_form():
    # S = 1: h = (q.k/sqrt d) v / (max(|q.k/sqrt d|, exp(-i)) + 1e-6), m = i, b = q.k/sqrt d
    q, k, v, f, i, _, _ = small(S=1, D=8)
    h, m, b = O.mlstm_forward_dense(q, k, v, f, i)
    s = (q * k).sum(-1) / math.sqrt(8)
    n = torch.maximum(s.abs(), torch.exp(-i)) + 1e-6
    assert torch.allclose(m, i)
    assert torch.allclose(b, s)
    assert torch.allclose(h, s[..., None] * v / n[..., None], rtol=1e-12, atol=1e-14)


def test_forward_saturated_gates_is_tril_matmul():
    # f -> +inf (logsigmoid = 0), i = 0: D~ = 0 on/below the diagonal, m = 0,
    # h = tril(QK^T/sqrt d) V / (max(|rowsum|, 1) + 1e-6)
    q, k, v, _, _, _, _ = small(S=16, D=4)
    f = torch.full(q.shape[:3], 80.0, dtype=F64)
    i = torch.zeros(q.shape[:3], dtype=F64)
    h, m, b = O.mlstm_forward_dense(q, k, v, f, i)
    s = torch.tril(q @ k.transpose(-1, -2) / 2.0)
    n = torch.clamp(s.sum(-1).abs(), min=1.0) + 1e-6
    assert torch.allclose(m, torch.zeros_like(m), atol=1e-12)
    assert torch.allclose(h, (s @ v) / n[..., None], rtol=1e-10, atol=1e-12)


def test_dense_equals_recurrence():
    # two independent formulations: dense parallel form vs. step-by-step state recurrence
    q, k, v, f, i, _, o = small(S=40, D=6, seed=3)
    h, _, _ = O.mlstm_forward_dense(q, k, v, f, i)
    hr = O.mlstm_recurrent(q, k, v, f, i, None)
    assert torch.allclose(h, hr, rtol=1e-9, atol=1e-11)
    hs = O.mlstm_scan_dense(q, k, v, f, i, o)
    hro = O.mlstm_recurrent(q, k, v, f, i, o)
    assert torch.allclose(hs, hro, rtol=1e-9, atol=1e-11)
    # silu(x) = x * sigmoid(x)
    assert torch.allclose(hro, hr * o * torch.sigmoid(o), rtol=1e-12, atol=1e-14)


def test_unstabilised_definition():
    # h = (C V) / max(|sum_j C_ij|, 1) with C = (QK^T/sqrt d) * exp(D~) (no stabiliser), up to eps
    q, k, v, f, i, _, _ = small(S=20, D=4, seed=5)
    i = 0.3 * i
    lf = torch.nn.functional.logsigmoid(f)
    S = 20
    C = torch.zeros(2, 2, S, S, dtype=F64)
    for a in range(S):
        for c in range(a + 1):
            C[:, :, a, c] = (q[:, :, a] * k[:, :, c]).sum(-1) / 2.0 * torch.exp(lf[:, :, c + 1:a + 1].sum(-1) + i[:, :, c])
    n = torch.clamp(C.sum(-1).abs(), min=1.0)
    h_def = (C @ v) / n[..., None]
    h, m, b = O.mlstm_forward_dense(q, k, v, f, i)
    assert torch.allclose(h, h_def, rtol=1e-4, atol=1e-5)  # differs only by the 1e-6 eps
    assert torch.allclose(b * torch.exp(m), C.sum(-1), rtol=1e-10)


def test_causality_and_m_recurrence():
    q, k, v, f, i, _, _ = small(S=32, D=4, seed=7)
    h, m, _ = O.mlstm_forward_dense(q, k, v, f, i)
    q2, k2, v2, f2, i2 = (x.clone() for x in (q, k, v, f, i))
    for x in (q2, k2, v2, f2, i2):
        x[:, :, 20:] += 1.0
    h2, m2, _ = O.mlstm_forward_dense(q2, k2, v2, f2, i2)
    assert torch.equal(h[:, :, :20], h2[:, :, :20])
    ms, fst, ist = O.stabilizer_scan(f, i)
    assert torch.allclose(m, ms, rtol=1e-12, atol=1e-12)
    lf = torch.nn.functional.logsigmoid(f)
    assert torch.allclose(ist, torch.exp(i - m))
    assert torch.allclose(fst[..., 1:], torch.exp(lf[..., 1:] - m[..., 1:] + m[..., :-1]))
    assert torch.allclose(fst[..., 0], torch.exp(lf[..., 0] - m[..., 0]))


def test_input_gate_shift():
    # i += c  =>  m += c, C~ and b unchanged
    q, k, v, f, i, _, _ = small(S=16, D=4, seed=9)
    _, m, b = O.mlstm_forward_dense(q, k, v, f, i)
    _, m2, b2 = O.mlstm_forward_dense(q, k, v, f, i + 1.5)
    assert torch.allclose(m2, m + 1.5)
    assert torch.allclose(b2, b, rtol=1e-10)


def _autograd_forward(q, k, v, f, i):
    """Independent differentiable forward (explicit double loop free, built from the
    definition with cumsum differences), m detached."""
    S, D = q.shape[-2:]
    lf = torch.nn.functional.logsigmoid(f)
    fc = torch.cumsum(lf, -1)
    dmat = fc[..., :, None] - fc[..., None, :] + i[..., None, :]
    mask = torch.tril(torch.ones(S, S, dtype=torch.bool))
    dmat = dmat.masked_fill(~mask, -float("inf"))
    m = dmat.max(-1)[0].detach()
    c = (q @ k.transpose(-1, -2)) / math.sqrt(D) * torch.exp(dmat - m[..., None])
    n = torch.maximum(c.sum(-1).abs(), torch.exp(-m)) + 1e-6
    return (c @ v) / n[..., None]


def test_backward_vs_autograd_and_finite_differences():
    q, k, v, f, i, dh, _ = small(B=1, NH=2, S=12, D=4, seed=11)
    ins = [x.clone().requires_grad_(True) for x in (q, k, v, f, i)]
    h = _autograd_forward(*ins)
    grads = torch.autograd.grad(h, ins, dh)
    mine = O.mlstm_backward_dense(dh, q, k, v, f, i)
    for name, g, gm in zip("qkvfi", grads, mine):
        if name == "f":
            # index 0: the reference's roll gives round-off there; autograd gives exactly 0
            assert torch.allclose(g[..., 1:], gm[..., 1:], rtol=1e-8, atol=1e-10), name
            assert gm[..., 0].abs().max() < 1e-12
        else:
            assert torch.allclose(g, gm, rtol=1e-8, atol=1e-10), name
    # central finite differences on the oracle forward itself (ties forward and backward)
    eps = 1e-6
    base = (q, k, v, f, i)
    for idx, name in enumerate("qkvfi"):
        x = base[idx]
        flat = x.reshape(-1)
        for pos in (0, flat.numel() // 2, flat.numel() - 1):
            xp, xm = flat.clone(), flat.clone()
            xp[pos] += eps
            xm[pos] -= eps
            ap = list(base); ap[idx] = xp.reshape(x.shape)
            am = list(base); am[idx] = xm.reshape(x.shape)
            hp, _, _ = O.mlstm_forward_dense(*ap)
            hm, _, _ = O.mlstm_forward_dense(*am)
            fd = ((hp - hm) * dh).sum() / (2 * eps)
            an = mine[idx].reshape(-1)[pos]
            assert abs(fd - an) <= 1e-5 * max(1.0, abs(an)), (name, pos, float(fd), float(an))


def test_gated_backward_vs_autograd_and_finite_differences():
    q, k, v, f, i, dhg, o = small(B=1, NH=2, S=10, D=4, seed=13)
    ins = [x.clone().requires_grad_(True) for x in (q, k, v, f, i, o)]
    hg = _autograd_forward(*ins[:5]) * (ins[5] * torch.sigmoid(ins[5]))
    assert torch.allclose(hg.detach(), O.mlstm_recurrent(q, k, v, f, i, o), rtol=1e-9, atol=1e-11)   # the gated forward itself
    grads = torch.autograd.grad(hg, ins, dhg)
    mine = O.mlstm_gated_backward_dense(dhg, q, k, v, f, i, o)
    for name, g, gm in zip(["q", "k", "v", "f", "i", "o"], grads, mine):
        if name == "f":
            assert torch.allclose(g[..., 1:], gm[..., 1:], rtol=1e-8, atol=1e-10), name
            assert gm[..., 0].abs().max() < 1e-12
        else:
            assert torch.allclose(g, gm, rtol=1e-8, atol=1e-10), name
    # the gate alone, against its definition by finite differences
    eps = 1e-6
    flat = o.reshape(-1)
    for pos in (0, flat.numel() // 3, flat.numel() - 1):
        op, om = flat.clone(), flat.clone()
        op[pos] += eps
        om[pos] -= eps
        hp = O.mlstm_scan_dense(q, k, v, f, i, op.reshape(o.shape))
        hm = O.mlstm_scan_dense(q, k, v, f, i, om.reshape(o.shape))
        fd = ((hp - hm) * dhg).sum() / (2 * eps)
        an = mine[5].reshape(-1)[pos]
        assert abs(fd - an) <= 1e-6 * max(1.0, abs(an)), (pos, float(fd), float(an))


def test_backward_invariants():
    q, k, v, f, i, dh, _ = small(B=1, NH=1, S=20, D=4, seed=13)
    dq, dk, dv, df, di = O.mlstm_backward_dense(dh, q, k, v, f, i)
    # dI_j = k_j . dK_j and row_i = q_i . dQ_i ; sum_t(row_t - col_t) = 0
    col = (k * dk).sum(-1)
    row = (q * dq).sum(-1)
    assert torch.allclose(di, col, rtol=1e-9, atol=1e-12)
    assert abs(float((row - col).sum())) < 1e-10
    # dF_t = sigmoid(-f_t) * sum_{s<t}(col_s - row_s)
    g = torch.cumsum(col - row, -1)
    assert torch.allclose(df[..., 1:], torch.sigmoid(-f[..., 1:]) * g[..., :-1], rtol=1e-9, atol=1e-12)
    df0 = O.mlstm_backward_dense(dh, q, k, v, f, i, zero_first_df=True)[3]
    assert torch.equal(df0[..., 0], torch.zeros_like(df0[..., 0]))
    assert torch.equal(df0[..., 1:], df[..., 1:])


def test_row_identities_used_by_the_kernels():
    # dn_i = -(dh_i . h_i)/n_i ; row_i = dh_i . h_i + db_i b_i
    q, k, v, f, i, dh, _ = small(B=1, NH=1, S=20, D=4, seed=17)
    h, m, b = O.mlstm_forward_dense(q, k, v, f, i)
    dq = O.mlstm_backward_dense(dh, q, k, v, f, i)[0]
    n = torch.maximum(b.abs(), torch.exp(-m)) + 1e-6
    delta = (dh * h).sum(-1)
    dn = -delta / n
    db = torch.sign(b) * dn * (b.abs() > torch.exp(-m))
    row = (q * dq).sum(-1)
    assert torch.allclose(row, delta + db * b, rtol=1e-9, atol=1e-12)


def test_check_comparator(capsys):
    a = torch.ones(4)
    assert O.check(a, a + 1e-3, name="X")
    assert not O.check(a, a + 1.0, name="Y")
    out = capsys.readouterr().out
    assert "X -- EQUAL" in out and "Percentage non-matching" in out


# ---------------------------------------------------------------------------------------------------------------
# 16-bit weights: the CPU restatement of what a 16-bit kernel computes, and the predicted size of its rounding noise
# ---------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rounded_weights_restate_the_same_function(dtype):
    """With the weights as hi + lo the 16-bit algorithm is the fp64 oracle to a few 2^-16; with plain rounding it stays
    within the unit roundoff of the weights, relative to the size of an element's terms."""
    q, k, v, f, i, dh = O.make_inputs(1, 2, 96, 32, dtype, seed=3, f_mean=1.0)
    exact = [O.mlstm_forward_dense(q, k, v, f, i)[0], *O.mlstm_backward_dense(dh, q, k, v, f, i, zero_first_df=True)]
    split = O.mlstm_rounded_weights_dense(dh, q, k, v, f, i, dtype, terms=2)
    plain = O.mlstm_rounded_weights_dense(dh, q, k, v, f, i, dtype, terms=1)
    u = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}[dtype]
    for name, e, s2, s1 in zip(["h", "dq", "dk", "dv", "df", "di"], exact, split, plain):
        scale = float(e.abs().max())
        assert float((s2 - e).abs().max()) <= 64 * u * u * scale + 1e-12, name
        assert 0 < float((s1 - e).abs().max()) <= 8 * u * scale or name in ("df", "di"), name
    assert float(split[4][..., 0].abs().max()) == 0.0


@pytest.mark.parametrize("dtype,S,D,f_mean", [(torch.bfloat16, 200, 64, 3.0), (torch.float16, 130, 32, 0.0), (torch.bfloat16, 160, 32, -4.0)])
def test_rounding_noise_model_against_the_emulation(dtype, S, D, f_mean):
    """The predicted standard deviation must describe the emulated 16-bit algorithm's actual error: rms of error / sigma
    between 0.5 and 1.1 (the model takes the rounding unit at its largest), and no element beyond 5 sigma."""
    worst, ratio = {}, {}
    names = ["h", "dq", "dk", "dv", "df", "di"]
    for seed in range(3):
        q, k, v, f, i, dh = O.make_inputs(1, 1, S, D, dtype, seed=seed, f_mean=f_mean, i_mean=2.0 if f_mean < 0 else 0.0)
        exact = [O.mlstm_forward_dense(q, k, v, f, i)[0], *O.mlstm_backward_dense(dh, q, k, v, f, i, zero_first_df=True)]
        emu = O.mlstm_rounded_weights_dense(dh, q, k, v, f, i, dtype)
        sig = O.mlstm_rounding_noise(dh, q, k, v, f, i, dtype)
        for name, e, g, s in zip(names, exact, emu, sig):
            err = (g - e).abs()
            live = s > 1e-12 * float(s.max())
            worst[name] = max(worst.get(name, 0.0), float((err[live] / s[live]).max()))
            ratio[name] = ratio.get(name, 0.0) + float(err.pow(2).mean().sqrt() / s.pow(2).mean().sqrt()) / 3
    for name in names:
        assert worst[name] < 5.0, (name, worst[name])
        assert 0.5 < ratio[name] < 1.1, (name, ratio[name])


def test_rounding_noise_in_chunks_only_adds():
    q, k, v, f, i, dh = O.make_inputs(1, 1, 300, 32, torch.bfloat16, seed=1, f_mean=4.0)
    plain = O.mlstm_rounding_noise(dh, q, k, v, f, i, torch.bfloat16)
    chunks = O.mlstm_rounding_noise(dh, q, k, v, f, i, torch.bfloat16, chunk_len=128)
    for a, c in zip(plain, chunks):
        assert bool((c >= a * (1 - 1e-12)).all())
    assert float(chunks[0][0, 0, 128:].sum()) > float(plain[0][0, 0, 128:].sum())     # rows behind the first chunk read a state
    assert torch.equal(chunks[0][0, 0, :128], plain[0][0, 0, :128])                  # the first chunk reads none
