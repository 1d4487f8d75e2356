"""CPU oracle for the mLSTM hot path.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain dense torch (float64 by default), the algorithms of the
reference's own CPU/PyTorch oracles.  It is the checker for the HIP kernels: only the
test-suite, the smoke check and the benchmark's ``cpu_baseline`` leg may import it.  The
product path (the C-ABI library and the Python operator wrappers) never does.

Reference code each function follows (paths relative to the reference checkout):

* ``mlstm_forward_dense``   -> ``mlstm_matmul.py:104-118``  (``mlstm_matmul_pytorch``), plus the
  m / b side outputs the kernel ``mlstm_matmul.py:38-101`` stores (lines 95-101).
* ``mlstm_backward_dense``  -> ``mlstm_matmul.py:336-365``  (``mlstm_matmul_backward_pytorch``).
* ``mlstm_recurrent``       -> ``mlstm_scan.py:343-372``    (``mlstm_scan_pytorch``) with the
  associative operators of ``mlstm_scan.py:330-339``.
* ``stabilizer_scan``       -> ``mlstm_scan.py:48-69``      (``stabilize_fi``).
* ``check``                 -> ``utils.py:4-15``.

How the oracle is pinned (see ``tests/test_oracle_pins.py``): closed forms for S=1 and
for saturated gates, equality of the two independent formulations (dense parallel form
vs. step-by-step recurrence), causality, the un-stabilised definition evaluated in
float64, autograd of the forward and central finite differences for the backward, and the
invariants ``sum_t(row_t - col_t) = 0``, ``dI = column sums``.  Every function has such a
pin; none is "parity unpinned".

Conventions shared by all functions: q, k, v, dh, o are ``[B, NH, S, D]``; f, i, m, b are
``[B, NH, S]``.  Inputs of any floating dtype are up-cast to ``dtype`` (float64 unless
stated) before any arithmetic, so a bf16/fp16 test evaluates the exact math on the
rounded inputs.
"""
import math

import torch

EPS = 1e-6


def _up(x, dtype):
    return x.detach().to(device="cpu", dtype=dtype)


def _decay_matrix(f, i):
    """log-decay matrix D~ and its row maximum for one head.  f, i: [S].

    mlstm_matmul.py:106-112: fc = cumsum(logsigmoid(f)); D~_ij = fc_i - fc_j + i_j for
    j <= i, -inf above the diagonal; m_i = max_j D~_ij.
    """
    S = f.shape[0]
    fc = torch.cumsum(torch.nn.functional.logsigmoid(f), 0)
    d = fc[:, None] - fc[None, :]
    mask = torch.tril(torch.ones((S, S), dtype=torch.bool))
    d = torch.where(mask, d, torch.full_like(d, -float("inf")))
    d = d + i[None, :]
    m = torch.max(d, -1)[0]
    return d, m


def mlstm_forward_dense(q, k, v, f, i, dtype=torch.float64):
    """Dense parallel-form forward.  Returns (h, m, b) in ``dtype``.

    mlstm_matmul.py:104-118.  m and b are what the kernel stores at mlstm_matmul.py:100-101:
    m_i = row max of D~, b_i = sum_j C~_ij with C~ = (q k^T / sqrt(D)) * exp(D~ - m).
    n_i = max(|b_i|, exp(-m_i)) + 1e-6, h = (C~ / n) v.
    """
    q, k, v, f, i = (_up(x, dtype) for x in (q, k, v, f, i))
    B, NH, S, D = q.shape
    h = torch.empty_like(q)
    m = torch.empty_like(f)
    b = torch.empty_like(f)
    for bi in range(B):
        for hi in range(NH):
            d, mm = _decay_matrix(f[bi, hi], i[bi, hi])
            dp = torch.exp(d - mm[:, None])
            c = (q[bi, hi] @ (k[bi, hi].T / math.sqrt(D))) * dp
            bb = c.sum(-1)
            n = torch.maximum(bb.abs(), torch.exp(-mm)) + EPS
            h[bi, hi] = (c / n[:, None]) @ v[bi, hi]
            m[bi, hi] = mm
            b[bi, hi] = bb
    return h, m, b


def mlstm_backward_dense(dh, q, k, v, f, i, dtype=torch.float64, zero_first_df=False):
    """Dense manual backward.  Returns (dq, dk, dv, df, di) in ``dtype``.

    mlstm_matmul.py:336-365.  ``zero_first_df`` selects the kernels' convention
    dF[..., 0] = 0 exactly (mlstm_matmul.py:316 never writes index 0) instead of the
    rolled cumsum's wrap-around value (mlstm_matmul.py:364), which is round-off.
    """
    dh, q, k, v, f, i = (_up(x, dtype) for x in (dh, q, k, v, f, i))
    B, NH, S, D = q.shape
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    df, di = torch.empty_like(f), torch.empty_like(f)
    sc = 1.0 / math.sqrt(D)
    for bi in range(B):
        for hi in range(NH):
            Q, K, V, dH = q[bi, hi], k[bi, hi], v[bi, hi], dh[bi, hi]
            d, m = _decay_matrix(f[bi, hi], i[bi, hi])
            dp = torch.exp(d - m[:, None])
            dC = dH @ V.T
            qk = Q @ (K.T * sc)
            ct = qk * dp
            b = ct.sum(-1)
            n = torch.maximum(b.abs(), torch.exp(-m)) + EPS
            dn = -(ct * dC).sum(-1) / (n * n)
            db = torch.sign(b) * dn * (b.abs() > torch.exp(-m)).to(dtype)
            c = ct / n[:, None]
            dct = dC / n[:, None] + db[:, None]
            dD = qk * dp * dct
            dq[bi, hi] = (dct * dp) @ (K * sc)
            dk[bi, hi] = (dct * dp).T @ (Q * sc)
            dv[bi, hi] = c.T @ dH
            di[bi, hi] = dD.sum(-2)
            cs = torch.cumsum(dD.sum(-2) - dD.sum(-1), -1)
            g = torch.roll(cs, 1, -1)
            if zero_first_df:
                g[0] = 0.0
            df[bi, hi] = torch.sigmoid(-f[bi, hi]) * g
    return dq, dk, dv, df, di


def stabilizer_scan(f, i, dtype=torch.float64):
    """The scan form's gate stabiliser.  Returns (m, f_stab, i_stab), each [B, NH, S].

    mlstm_scan.py:48-69: m_t = max(logsigmoid(f_t) + m_{t-1}, i_t) with the associative
    scan's first element being the element itself (m_0 = i_0); the rolled m is 0 at t=0;
    i' = exp(i - m), f' = exp(logsigmoid(f) - m + m_shifted).
    """
    f, i = _up(f, dtype), _up(i, dtype)
    lf = torch.nn.functional.logsigmoid(f)
    m = torch.empty_like(f)
    S = f.shape[-1]
    m[..., 0] = i[..., 0]
    for t in range(1, S):
        m[..., t] = torch.maximum(lf[..., t] + m[..., t - 1], i[..., t])
    msh = torch.roll(m, 1, -1)
    msh[..., 0] = 0.0
    return m, torch.exp(lf - m + msh), torch.exp(i - m)


def mlstm_recurrent(q, k, v, f, i, o=None, dtype=torch.float64):
    """Step-by-step recurrence with the silu(o) output gate.  Returns h [B, NH, S, D].

    mlstm_scan.py:343-372.  State starts as m=0, C=0, n=0; per step
    m_t = max(logsigmoid(f_t) + m_{t-1}, i_t), i' = exp(i_t - m_t),
    f' = exp(logsigmoid(f_t) - m_t + m_{t-1}), C_t = f' C_{t-1} + i' v_t (k_t/sqrt(D))^T,
    n_t likewise, h_t = silu(o_t) * (C_t q_t) / (max(|n_t . q_t|, exp(-m_t)) + 1e-6).
    ``o=None`` drops the gate (the matmul form has none).
    """
    q, k, v, f, i = (_up(x, dtype) for x in (q, k, v, f, i))
    B, NH, S, D = q.shape
    lf = torch.nn.functional.logsigmoid(f)
    h = torch.empty_like(q)
    C = torch.zeros((B, NH, D, D), dtype=dtype)
    n = torch.zeros((B, NH, D), dtype=dtype)
    m = torch.zeros((B, NH), dtype=dtype)
    ks = k / math.sqrt(D)
    for t in range(S):
        m_new = torch.maximum(lf[..., t] + m, i[..., t])
        i_st = torch.exp(i[..., t] - m_new)
        f_st = torch.exp(lf[..., t] - m_new + m)
        m = m_new
        C = f_st[..., None, None] * C + i_st[..., None, None] * (v[:, :, t, :, None] * ks[:, :, t, None, :])
        n = f_st[..., None] * n + i_st[..., None] * ks[:, :, t]
        num = torch.einsum("bhvk,bhk->bhv", C, q[:, :, t])
        den = torch.maximum((n * q[:, :, t]).sum(-1).abs(), torch.exp(-m)) + EPS
        h[:, :, t] = num / den[..., None]
    if o is not None:
        h = h * torch.nn.functional.silu(_up(o, dtype))
    return h


def mlstm_scan_dense(q, k, v, f, i, o, dtype=torch.float64):
    """Scan-form result computed through the dense parallel form: silu(o) * h_matmul.

    The two forms are the same function (the stabiliser m_t of mlstm_scan.py:62 is the row
    maximum of mlstm_matmul.py:111, and n_t . q_t is b_t); this is the cheap evaluation of
    the scan oracle for long sequences.  tests/test_oracle_pins.py proves the equality
    against ``mlstm_recurrent``.
    """
    h, _, _ = mlstm_forward_dense(q, k, v, f, i, dtype)
    return h * torch.nn.functional.silu(_up(o, dtype))


def mlstm_gated_backward_dense(dhg, q, k, v, f, i, o, dtype=torch.float64, zero_first_df=False):
    """Backward of ``mlstm_scan_dense`` (the matmul form followed by the gate of mlstm_scan.py:277).
    Returns (dq, dk, dv, df, di, do) in ``dtype``.

    With s = sigmoid(o): d silu(o)/do = s (1 + o (1 - s)); the gate passes dh = dhg * silu(o) to the
    ungated backward (mlstm_matmul.py:336-365) and receives do = dhg * h * silu'(o).  The reference
    has no backward of the gated form; tests/test_oracle_pins.py checks this one against autograd
    through the step-by-step recurrence and against finite differences.
    """
    dhg, o = _up(dhg, dtype), _up(o, dtype)
    h, _, _ = mlstm_forward_dense(q, k, v, f, i, dtype)
    s = torch.sigmoid(o)
    grads = mlstm_backward_dense(dhg * o * s, q, k, v, f, i, dtype, zero_first_df)
    return (*grads, dhg * h * s * (1.0 + o * (1.0 - s)))


def check(*inputs, name="A", atol=1e-2, rtol=1e-2, verbose=True):
    """The reference's comparator (utils.py:4-15): pairs (a0, b0, a1, b1, ...); prints and
    returns True when every pair is allclose."""
    for a, b in zip(inputs[::2], inputs[1::2]):
        if isinstance(b, list):
            b = torch.tensor(b)
        a, b = a.detach().cpu().double(), b.detach().cpu().double()
        close = torch.isclose(a, b, atol=atol, rtol=rtol)
        if not bool(close.all()):
            if verbose:
                print(name)
                print(f"Percentage non-matching: {100 * float((~close).sum()) / a.numel():.10f}")
            return False
    if verbose:
        print(f"{name} -- EQUAL")
    return True


def make_inputs(B, NH, S, D, dtype=torch.float32, seed=0, f_mean=0.0, i_mean=0.0, dh_std=1.0, with_o=False):
    """Seeded synthetic inputs: one CPU generator, draws in the order q, k, v, f, i, dh(, o)
    as float32 normal, affine-transformed, then cast to ``dtype``."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, NH, S, D), generator=g)
    k = torch.randn((B, NH, S, D), generator=g)
    v = torch.randn((B, NH, S, D), generator=g)
    f = torch.randn((B, NH, S), generator=g) + f_mean
    i = torch.randn((B, NH, S), generator=g) + i_mean
    dh = torch.randn((B, NH, S, D), generator=g) * dh_std
    out = [q, k, v, f, i, dh]
    if with_o:
        out.append(torch.randn((B, NH, S, D), generator=g))
    return [x.to(dtype) for x in out]


# ---------------------------------------------------------------------------------------------------------------
# 16-bit weights.  The reference's Triton kernels are fp32 (mlstm_matmul.py:19, :35 "TODO FP 16"); its CUDA kernels
# feed the second product of a tile with the weights rounded to half (cuda-src/mlstm_forward.cu:143-160,
# cutlass-src-ampere/mlstm_forward.cu:308-313), as every tensor-core pipeline does.  The two functions below restate
# that algorithm on the CPU and predict the size of its rounding noise, so that a 16-bit kernel can be held to the
# algorithm it implements, and the distance of that algorithm from the fp32 formulas can be measured rather than
# absorbed into a tolerance.
# ---------------------------------------------------------------------------------------------------------------
def _round_to(x, dtype, terms):
    """x rounded to ``dtype`` as a sum of ``terms`` values of that type (1: plain rounding, 2: hi + lo)."""
    hi = x.to(dtype).to(x.dtype)
    if terms == 1:
        return hi
    return hi + (x - hi).to(dtype).to(x.dtype)


def mlstm_rounded_weights_dense(dh, q, k, v, f, i, dtype, terms=1):
    """Forward and backward (mlstm_matmul.py:104-118, :336-365) with the operands a 16-bit kernel rounds to the
    element type before a tile's second product: C~ (forward, ``P``), dC~ D' (``G``, dQ and dK), C~ / n (``W``, dV),
    and the forward output h where the backward uses it for dn = -(dh . h) / n.  Everything else in float64.
    ``terms=2`` is the split mode (each operand as hi + lo).  Returns (h, dq, dk, dv, df, di), unrounded float64."""
    dh, q, k, v, f, i = (_up(x, torch.float64) for x in (dh, q, k, v, f, i))
    B, NH, S, D = q.shape
    outs = [torch.empty_like(q) for _ in range(4)] + [torch.empty_like(f), torch.empty_like(f)]
    sc = 1.0 / math.sqrt(D)
    rnd = lambda x: _round_to(x, dtype, terms)
    for bi in range(B):
        for hi_ in range(NH):
            Q, K, V, dH = q[bi, hi_], k[bi, hi_], v[bi, hi_], dh[bi, hi_]
            d, m = _decay_matrix(f[bi, hi_], i[bi, hi_])
            dp = torch.exp(d - m[:, None])
            ct = (Q @ K.T) * sc * dp
            b = ct.sum(-1)
            n = torch.maximum(b.abs(), torch.exp(-m)) + EPS
            h = (rnd(ct) @ V) / n[:, None]
            dn = -(dH * rnd(h)).sum(-1) / n
            db = torch.sign(b) * dn * (b.abs() > torch.exp(-m)).to(torch.float64)
            dct = (dH @ V.T) / n[:, None] + db[:, None]
            G = rnd(dct * dp * sc)
            dD = ct * dct
            cs = torch.cumsum(dD.sum(-2) - dD.sum(-1), -1)
            g = torch.roll(cs, 1, -1)
            g[0] = 0.0
            for o_, val in zip(outs, (h, G @ K, G.T @ Q, rnd(ct / n[:, None]).T @ dH, torch.sigmoid(-f[bi, hi_]) * g, dD.sum(-2))):
                o_[bi, hi_] = val
    return tuple(outs)


def rounding_unit_std(dtype):
    """Standard deviation of the relative error of round-to-nearest into ``dtype``, taken at its largest (values just
    above a power of two): ulp / sqrt(12) with ulp = 2^-7 (bfloat16: 8 significant bits) or 2^-10 (float16: 11)."""
    return {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}[dtype] / math.sqrt(12.0)


def mlstm_rounding_noise(dh, q, k, v, f, i, dtype, work_dtype=torch.float64, chunk_len=0):
    """Per-element standard deviation of the error that rounding P, G, W and h to ``dtype`` (see
    mlstm_rounded_weights_dense) leaves in h, dq, dk, dv, df, di, under the usual model of independent rounding errors:
    an output that is sum_j w_j x_j with w rounded has variance u^2 sum_j (w_j x_j)^2, u = rounding_unit_std.  The
    rounding of h enters through db_i = +-(dh_i . h_i) / n_i, which is common to a whole row of dC~ (and of dD, whose
    sums are di and, cumulatively, df).

    ``chunk_len`` = L > 0 models an evaluation in chunks of L positions, where a row meets the keys before its chunk
    through the matrix state of the scan form (mlstm_scan.py:16-26) at the end of the previous chunk, C~ = sum_j w_j k_j
    v_j^T / sqrt(D), and a key meets the queries behind its chunk through the mirror-image state E = sum_i rho_i / n_i
    q_i dh_i^T / sqrt(D), both stored in ``dtype``: every output gains the rounding of the state it is contracted
    with, and the row and column sums of dD of those far pairs, now q_i . dQ_i and k_j . dK_j, gain a per-position
    error that the running sum of df accumulates between the chunk boundaries, where it is pinned to sum <C~, E>
    (a bridge: what a chunk's own sum misses of the next pinned value is spread evenly over the chunk); the pinned
    values carry the rounding of the two states' entries, which averages out over the D^2 products but not to nothing.

    Returns a tuple of tensors shaped like the outputs, in ``work_dtype`` (float32 halves the memory of the S x S
    intermediates of very long sequences)."""
    dh, q, k, v, f, i = (_up(x, work_dtype) for x in (dh, q, k, v, f, i))
    B, NH, S, D = q.shape
    u2 = rounding_unit_std(dtype) ** 2
    outs = [torch.empty_like(q) for _ in range(4)] + [torch.empty_like(f), torch.empty_like(f)]
    sc = 1.0 / math.sqrt(D)
    L = int(chunk_len)
    ncs = (S - 1) // L if L > 0 else 0          # complete chunks with something behind them
    for bi in range(B):
        for hi_ in range(NH):
            Q, K, V, dH = q[bi, hi_], k[bi, hi_], v[bi, hi_], dh[bi, hi_]
            d, m = _decay_matrix(f[bi, hi_], i[bi, hi_])
            dp = torch.exp(d - m[:, None])
            ct = (Q @ K.T) * sc * dp
            b = ct.sum(-1)
            n = torch.maximum(b.abs(), torch.exp(-m)) + EPS
            h = (ct @ V) / n[:, None]
            active = (b.abs() > torch.exp(-m)).to(work_dtype)
            dn = -(dH * h).sum(-1) / n
            db = torch.sign(b) * dn * active
            dct = (dH @ V.T) / n[:, None] + db[:, None]
            G = dct * dp * sc
            W = ct / n[:, None]
            var_h = u2 * ((ct ** 2) @ (V ** 2)) / (n * n)[:, None]
            var_dq = u2 * ((G ** 2) @ (K ** 2))
            var_dk = u2 * ((G ** 2).T @ (Q ** 2))
            var_dv = u2 * ((W ** 2).T @ (dH ** 2))
            var_x = torch.zeros(S, dtype=work_dtype)     # per-position error of (column sum - row sum) of dD, far pairs
            var_anchor = torch.zeros(max(ncs, 1), dtype=work_dtype)   # of the pinned running sums sqrt(D) <C~_c, E_c>
            if ncs > 0:
                pos = torch.arange(S)
                cidx = torch.clamp(pos // L, max=ncs)
                far = (cidx[:, None] > cidx[None, :]).to(work_dtype)          # [row s, key j]: j in an earlier chunk
                T = ((dH / n[:, None]) ** 2) @ (V ** 2).T                     # sum_v (dh_sv v_jv / n_s)^2
                pair = u2 * far * ct ** 2 * T                                 # far pairs seen through rounded chunk sums
                var_x += pair.sum(-1) + pair.sum(-2)
                for c in range(ncs):
                    e = (c + 1) * L - 1
                    rows = slice(e + 1, min(e + 1 + L, S)) if c + 1 < ncs else slice(e + 1, S)   # the rows that read C~_c
                    keys = slice(c * L, e + 1)                                                      # the keys that read E_c
                    Cst = (K * (sc * dp[e])[:, None]).T @ V                                         # [key index, value index]
                    rho = torch.where(pos > e, dp[:, e] / dp[e, e], torch.zeros((), dtype=work_dtype))
                    Est = (Q * (sc * rho / n)[:, None]).T @ dH
                    # both states enter the contraction rounded, every entry on its own: the products' errors add up in
                    # quadrature (they average out over the D^2 entries, but not to nothing)
                    var_anchor[c] = 2.0 * u2 * ((Cst * Est) ** 2).sum() / (sc * sc)
                    dec2 = ((dp[rows, e] / dp[e, e]) / n[rows]) ** 2
                    w2 = dp[e, keys] ** 2
                    var_h[rows] += u2 * ((Q[rows] ** 2) @ (Cst ** 2)) * (dp[rows, e] / dp[e, e] / n[rows])[:, None] ** 2
                    var_dq[rows] += u2 * ((dH[rows] ** 2) @ (Cst ** 2).T) * dec2[:, None]
                    var_dv[keys] += u2 * ((K[keys] ** 2) @ (Est ** 2)) * w2[:, None]
                    var_dk[keys] += u2 * ((V[keys] ** 2) @ (Est ** 2).T) * w2[:, None]
                    var_x[rows] += u2 * dec2 * (((Q[rows] ** 2) @ (Cst ** 2)) * dH[rows] ** 2).sum(-1)
                    var_x[keys] += u2 * w2 * (((K[keys] ** 2) @ (Est ** 2)) * V[keys] ** 2).sum(-1)
            # the h the backward reads carries the noise of the forward's own P as well as its final rounding
            var_db = ((dH ** 2) * (var_h + u2 * h ** 2)).sum(-1) / (n * n) * active   # [S] variance of db_i
            var_dq = var_dq + var_db[:, None] * ((dp * sc) @ K) ** 2
            var_dk = var_dk + ((dp * sc) ** 2).T @ (var_db[:, None] * Q ** 2)
            var_di = (ct ** 2).T @ var_db + var_x                               # dD_ij moves by ct_ij * (error of db_i)
            # df_t = sigmoid(-f_t) sum_{s<t} (col_s - row_s): row i of dD contributes c_i(t) = sum_{s<t} ct_is - [i<t] b_i
            cum = torch.cumsum(ct, -1)
            cum = torch.cat([torch.zeros((S, 1), dtype=cum.dtype), cum[:, :-1]], -1)      # [i, t] = sum_{s<t} ct_is
            lower = torch.tril(torch.ones((S, S), dtype=cum.dtype), -1).T                   # [i, t] = 1 if i < t
            coef = cum - lower * b[:, None]
            var_run = (coef ** 2).T @ var_db
            if ncs > 0:   # running sum of the per-position errors inside each chunk, bridged where the chunk's end is pinned
                for c in range(ncs + 1):
                    lo, hi = c * L, min((c + 1) * L, S) if c < ncs else S
                    vx = var_x[lo:hi]
                    P = torch.cumsum(vx, 0) - vx                                # sum over positions before tau
                    va0 = var_anchor[c - 1] if c > 0 else torch.zeros((), dtype=work_dtype)   # the pinned value the chunk starts from
                    if c < ncs:
                        tau = torch.arange(hi - lo, dtype=work_dtype) / float(L)
                        var_run[lo:hi] += (1 - tau) ** 2 * (P + va0) + tau ** 2 * (vx.sum() - P + var_anchor[c])
                    else:
                        var_run[lo:hi] += P + va0
            var_df = torch.sigmoid(-f[bi, hi_]) ** 2 * var_run
            for o_, val in zip(outs, (var_h, var_dq, var_dk, var_dv, var_df, var_di)):
                o_[bi, hi_] = val.clamp_min(0).sqrt()
    return tuple(outs)
