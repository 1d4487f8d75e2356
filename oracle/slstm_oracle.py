"""CPU oracle of the sLSTM cell (test infrastructure only: nothing the product ships may import this).

The reference repository lists the sLSTM as an open item (README.md:9) and holds no code for it, so this restates the
published cell, Beck et al., "xLSTM: Extended Long Short-Term Memory" (arXiv:2405.04517), section 2.2 with the
stabilised exponential gating of its appendix A.2, per head (the recurrent matrices are block-diagonal):

    i~, f~, z~, o~ = Wx_t[g] + R_g h_{t-1} + b_g            g in (i, f, z, o)
    m_t  = max(log f_t + m_{t-1}, i~)                       log f_t = f~ (exponential) or logsigmoid(f~)
    i'_t = exp(i~ - m_t),   f'_t = exp(log f_t + m_{t-1} - m_t)
    c_t  = f'_t c_{t-1} + i'_t tanh(z~),   n_t = f'_t n_{t-1} + i'_t,   h_t = sigmoid(o~) c_t / n_t

with c_0 = n_0 = h_0 = m_0 = 0.  Plain torch loops in float64; the backward is autograd through them.
tests/test_slstm_oracle.py pins it: closed form without recurrence, invariance under the stabiliser, the paper's
unstabilised recurrence on short sequences, finite differences for the gradients.
"""
import torch

GATES = ("i", "f", "z", "o")


def slstm_forward(wx, r, b, forget_sigmoid=False, dtype=torch.float64, return_states=False):
    """wx: [B,S,4,NH,DH] input pre-activations (gate order i, f, z, o); r: [NH,4,DH,DH] (r[h,g,j,k]: unit j from unit k);
    b: [NH,4,DH].  Returns h [B,S,NH,DH] (and, with return_states, the per-step c, n, m)."""
    wx, r, b = wx.to(dtype), r.to(dtype), b.to(dtype)
    B, S, _, NH, DH = wx.shape
    h = torch.zeros(B, NH, DH, dtype=dtype)
    c = torch.zeros_like(h)
    n = torch.zeros_like(h)
    m = torch.zeros_like(h)
    hs, cs, ns, ms = [], [], [], []
    for t in range(S):
        rec = torch.einsum("hgjk,bhk->bghj", r, h)                      # [B,4,NH,DH]
        pre = wx[:, t] + rec + b.permute(1, 0, 2)[None]
        it, ft, zt, ot = pre[:, 0], pre[:, 1], pre[:, 2], pre[:, 3]
        logf = torch.nn.functional.logsigmoid(ft) if forget_sigmoid else ft
        m_new = torch.maximum(logf + m, it)
        ip = torch.exp(it - m_new)
        fp = torch.exp(logf + m - m_new)
        c = fp * c + ip * torch.tanh(zt)
        n = fp * n + ip
        m = m_new
        h = torch.sigmoid(ot) * c / n
        hs.append(h); cs.append(c); ns.append(n); ms.append(m)
    out = torch.stack(hs, dim=1)
    if return_states:
        return out, torch.stack(cs, 1), torch.stack(ns, 1), torch.stack(ms, 1)
    return out


def slstm_backward(dh, wx, r, b, forget_sigmoid=False, dtype=torch.float64):
    """Gradients (dwx, dr, db) of sum(h * dh), by autograd through the loop above."""
    wx = wx.to(dtype).clone().requires_grad_(True)
    r = r.to(dtype).clone().requires_grad_(True)
    b = b.to(dtype).clone().requires_grad_(True)
    h = slstm_forward(wx, r, b, forget_sigmoid, dtype)
    (h * dh.to(dtype)).sum().backward()
    return wx.grad, r.grad, b.grad


def slstm_unstabilised(wx, r, b, forget_sigmoid=False, dtype=torch.float64):
    """The cell as the paper first states it (equations 8-14), without the stabiliser state: only for short sequences
    with moderate gates, where exp does not overflow."""
    wx, r, b = wx.to(dtype), r.to(dtype), b.to(dtype)
    B, S, _, NH, DH = wx.shape
    h = torch.zeros(B, NH, DH, dtype=dtype)
    c = torch.zeros_like(h)
    n = torch.zeros_like(h)
    hs = []
    for t in range(S):
        pre = wx[:, t] + torch.einsum("hgjk,bhk->bghj", r, h) + b.permute(1, 0, 2)[None]
        i = torch.exp(pre[:, 0])
        f = torch.sigmoid(pre[:, 1]) if forget_sigmoid else torch.exp(pre[:, 1])
        c = f * c + i * torch.tanh(pre[:, 2])
        n = f * n + i
        h = torch.sigmoid(pre[:, 3]) * c / n
        hs.append(h)
    return torch.stack(hs, dim=1)


def make_inputs(B, NH, S, DH, seed=0, r_scale=None, f_mean=0.0, dtype=torch.float32):
    """Seeded inputs: wx ~ N(0,1) (forget pre-activations shifted by f_mean), r ~ N(0, r_scale^2) with r_scale = 1/sqrt(DH)
    by default, b ~ N(0, 0.1^2), dh ~ N(0,1); one CPU generator, drawn in that order."""
    g = torch.Generator().manual_seed(seed)
    wx = torch.randn((B, S, 4, NH, DH), generator=g)
    wx[:, :, 1] += f_mean
    r = torch.randn((NH, 4, DH, DH), generator=g) * (DH ** -0.5 if r_scale is None else r_scale)
    b = torch.randn((NH, 4, DH), generator=g) * 0.1
    dh = torch.randn((B, S, NH, DH), generator=g)
    return [x.to(dtype) for x in (wx, r, b, dh)]
