"""The shapes the library claims beyond what the dense CPU oracle covers head by head: the long-context configuration at
its full batch, single sequences up to 65 600 positions (beyond 65 536 the column kernel leaves its chunked mode while
the row kernel stays in it), and repeatability of the whole backward at the headline shape."""
import pytest
import torch

from _mlstm_pkg import submodule
from oracle import mlstm_oracle as O
from tests.helpers import REL_RMS, assert_close, assert_matches_oracle, literal_violations

pytestmark = pytest.mark.gpu

mm = submodule("mlstm_matmul")
GRADS = ["dq", "dk", "dv", "df", "di"]


def test_long_context_config_at_full_batch():
    """cfg 5: B2 H32 S16384 D128 bf16, f ~ N(3,1), i ~ N(-1,1), dh ~ N(0, 0.1): 64 heads (workgroups dealt out by XCD),
    in chunks of 512.  One head against the fp64 oracle, the rest through properties that do not depend on the size."""
    B, NH, S, D = 2, 32, 16384, 128
    dtype = torch.bfloat16
    q, k, v, f, i, dh = O.make_inputs(B, NH, S, D, dtype, seed=7, f_mean=3.0, i_mean=-1.0, dh_std=0.1)
    dev = [x.cuda() for x in (q, k, v, f, i, dh)]
    h, m, b, saved = mm.mlstm_forward_save_hip(*dev[:5])
    grads = mm.mlstm_backward_saved_hip(dev[5], *dev[:5], h, m, b, saved)
    torch.cuda.synchronize()
    for name, t in zip(["h", "m", "b"] + GRADS, [h, m, b, *grads]):
        assert bool(torch.isfinite(t.float()).all()), name
    assert float(grads[3][..., 0].abs().max()) == 0.0
    # heads are independent, whatever the order their workgroups are dealt out in: a head on its own gives the same bits
    for (bi, hi) in [(0, 0), (1, 17), (1, 31)]:
        one = [x[bi:bi + 1, hi:hi + 1].contiguous() for x in dev]
        h1, m1, b1, s1 = mm.mlstm_forward_save_hip(*one[:5])
        g1 = mm.mlstm_backward_saved_hip(one[5], *one[:5], h1, m1, b1, s1)
        assert torch.equal(h1[0, 0], h[bi, hi]) and torch.equal(m1[0, 0], m[bi, hi]) and torch.equal(b1[0, 0], b[bi, hi])
        for name, a_, w_ in zip(GRADS, g1, grads):
            assert torch.equal(a_[0, 0], w_[bi, hi]), (name, bi, hi)
    # dq, dk, dv are linear in dh for a fixed forward, and scaling by 2 is exact in every rounding on the way
    g2 = mm.mlstm_backward_saved_hip(dev[5] * 2, *dev[:5], h, m, b, saved)
    for name, a_, w_ in zip(GRADS[:3], grads, g2):
        assert torch.equal((a_.float() * 2).to(dtype), w_), name
    bi, hi = 1, 17
    sl = lambda x: x[bi:bi + 1, hi:hi + 1]
    assert_matches_oracle(dtype, *(sl(x) for x in (q, k, v, f, i, dh)), h=sl(h), m=sl(m), grads=[sl(g_) for g_ in grads], chunk_len=512,
                          tag=f"[{bi},{hi}] ")


@pytest.mark.parametrize("S", [32768, 65536 + 64])
def test_single_sequences_beyond_the_dense_oracle(S):
    """One head, D = 128, bf16.  The S x S oracle is out of reach (34 GB per matrix at 65 600), the step-by-step recurrence
    (mlstm_scan.py:343-372, O(S D^2)) is not: the split mode's forward is held to the literal tolerance against it, and
    the default kernels (row side in chunks of 512; column side in chunks at 32 768, over every query tile at 65 600) to
    the split mode's results through the fraction of elements outside the literal bound and the rms error."""
    D, dtype = 128, torch.bfloat16
    q, k, v, f, i, dh = O.make_inputs(1, 1, S, D, dtype, seed=S % 1000, f_mean=3.0)
    dev = [x.cuda() for x in (q, k, v, f, i, dh)]
    out = {}
    for precise in (False, True):
        h, m, b, saved = mm.mlstm_forward_save_hip(*dev[:5], precise=precise)
        grads = mm.mlstm_backward_saved_hip(dev[5], *dev[:5], h, m, b, saved, precise=precise)
        torch.cuda.synchronize()
        out[precise] = [h, *grads]
        if precise:
            assert torch.equal(m, out["m"])
        out["m"] = m
    href = O.mlstm_recurrent(q, k, v, f, i)
    assert_close(out[True][0], href, dtype, "h (split mode) vs recurrence")
    assert float(out[False][4][..., 0].abs().max()) == 0.0 and float(out[True][4][..., 0].abs().max()) == 0.0
    for name, fast, prec in zip(["h"] + GRADS, out[False], out[True]):
        frac, rel = literal_violations(fast, prec.float())
        assert frac <= 0.12 and rel <= REL_RMS[dtype], (name, frac, rel)


def test_backward_at_the_headline_shape_is_repeatable():
    """B4 H8 S4096 D256 bf16: two runs of forward + backward on the same buffers give the same bits (no kernel adds
    across workgroups in launch order; the asynchronous tile copies are waited for before their data is read)."""
    B, NH, S, D = 4, 8, 4096, 256
    dtype = torch.bfloat16
    g = torch.Generator(device="cuda").manual_seed(9)
    mk = lambda *s: torch.randn(s, generator=g, device="cuda", dtype=torch.float32)
    q, k, v, dh = (mk(B, NH, S, D).to(dtype) for _ in range(4))
    f, i = (mk(B, NH, S) + 3.0).to(dtype), mk(B, NH, S).to(dtype)
    runs = []
    for _ in range(3):
        h, m, b, saved = mm.mlstm_forward_save_hip(q, k, v, f, i)
        grads = mm.mlstm_backward_saved_hip(dh, q, k, v, f, i, h, m, b, saved)
        torch.cuda.synchronize()
        runs.append([h, m, b, *[x.clone() for x in grads]])
    for other in runs[1:]:
        for name, a_, w_ in zip(["h", "m", "b"] + GRADS, runs[0], other):
            assert torch.equal(a_, w_), name
