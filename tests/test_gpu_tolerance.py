"""How far the 16-bit kernels are from the fp64 oracle at the statement's literal tolerance (rtol 2e-2, atol 2e-3), measured
per tensor, and what closes the gap.

Three evaluations of the same seeded inputs are compared with the oracle:
  fast     the default kernels (weights of a tile's second product rounded to the element type);
  emulated the same algorithm on the CPU in float64 with just those roundings (oracle.mlstm_rounded_weights_dense);
  precise  the kernels' split mode (MLSTM_PRECISE: weights as hi + lo).
The fast kernels must violate the literal bound exactly as often as the emulation does -- the gap is the algorithm's,
not the kernels' -- and agree with the emulation itself at the literal bound; the split mode must meet the literal
bound on every element.  Run with -s to see the measured fractions.
"""
import pytest
import torch

from _mlstm_pkg import submodule
from oracle import mlstm_oracle as O
from tests.helpers import GRAD_NAMES, assert_close, assert_matches_oracle, literal_violations

pytestmark = pytest.mark.gpu

mm = submodule("mlstm_matmul")
ffi = submodule("_ffi")
NAMES = ["h"] + GRAD_NAMES
# ceilings on the fraction of elements of a tensor outside the literal bound, fast kernels (measured: bf16 h, dv 1 %,
# dq, dk 3-4 %, df, di 4-8 %; fp16 below 1 %)
CEILING = {torch.bfloat16: 0.12, torch.float16: 0.02}


def run_gpu(q, k, v, f, i, dh, precise, chunk_len=0):
    """``chunk_len``: 0 = the library's default for the shape, > 0 forces that chunk length (a multiple of 128)."""
    dev = [x.cuda() for x in (q, k, v, f, i, dh)]
    ffi.set_chunk_length(chunk_len)
    try:
        h, m, b, saved = mm.mlstm_forward_save_hip(*dev[:5], precise=precise)
        grads = mm.mlstm_backward_saved_hip(dev[5], *dev[:5], h, m, b, saved, precise=precise)
    finally:
        ffi.set_chunk_length(0)
    torch.cuda.synchronize()
    return [h, *grads]


def oracle_all(q, k, v, f, i, dh):
    return [O.mlstm_forward_dense(q, k, v, f, i)[0], *O.mlstm_backward_dense(dh, q, k, v, f, i, zero_first_df=True)]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_thirty_seeds_fast_emulated_precise(dtype):
    g = torch.Generator().manual_seed(20240)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    frac = {kind: {n: 0.0 for n in NAMES} for kind in ("fast", "emulated", "precise", "fast_vs_emulated")}
    nseeds = 30
    for seed in range(nseeds):
        S, D, f_mean = r(65, 900), [64, 128, 256][r(0, 2)], [0.0, 3.0][r(0, 1)]
        q, k, v, f, i, dh = O.make_inputs(1, 1, S, D, dtype, seed=seed, f_mean=f_mean)
        ref = oracle_all(q, k, v, f, i, dh)
        emu = O.mlstm_rounded_weights_dense(dh, q, k, v, f, i, dtype)
        fast = run_gpu(q, k, v, f, i, dh, False)
        prec = run_gpu(q, k, v, f, i, dh, True)
        # split mode in chunks of 128 positions (D = 128 and 256; the kernels of D = 64 know no chunks)
        chunked = run_gpu(q, k, v, f, i, dh, True, chunk_len=128)
        for n, r_, c_ in zip(NAMES, ref, chunked):
            cv = literal_violations(c_, r_)[0]
            assert cv == 0.0, f"split mode in chunks: {n} seed {seed} S={S} D={D}: {cv:.2e} of the elements outside the literal bound"
        for n, r_, e_, a_, p_ in zip(NAMES, ref, emu, fast, prec):
            frac["fast"][n] += literal_violations(a_, r_)[0] / nseeds
            frac["emulated"][n] += literal_violations(e_.to(dtype), r_)[0] / nseeds
            frac["fast_vs_emulated"][n] += literal_violations(a_, e_)[0] / nseeds
            pv = literal_violations(p_, r_)[0]
            frac["precise"][n] += pv / nseeds
            assert pv == 0.0, f"split mode: {n} seed {seed} S={S} D={D}: {pv:.2e} of the elements outside the literal bound"
            assert_close(p_, r_, dtype, f"precise {n} (seed {seed})")
    for kind, row in frac.items():
        print(f"{str(dtype)[6:]:9s} {kind:17s} " + "  ".join(f"{n} {row[n]:.2e}" for n in NAMES))
    for n in NAMES:
        a, e = frac["fast"][n], frac["emulated"][n]
        assert a <= CEILING[dtype], (n, a)
        assert abs(a - e) <= 0.25 * e + 1e-3, f"{n}: the kernels violate the literal bound on {a:.2e} of the elements, the emulation on {e:.2e}"
        # against the emulation the kernels' only freedom is which way a weight on a rounding boundary falls
        assert frac["fast_vs_emulated"][n] <= 2e-3, (n, frac["fast_vs_emulated"][n])


def test_headline_shape_two_heads():
    """B4 H8 S4096 D256 bf16 (runs in chunks of 512): the whole batch through the fast kernels, two heads of it against the
    oracle; the same two heads in split mode (in chunks of 512 as well, with two-term states) at the literal bound."""
    dtype = torch.bfloat16
    B, NH, S, D = 4, 8, 4096, 256
    q, k, v, f, i, dh = O.make_inputs(B, NH, S, D, dtype, seed=0, f_mean=3.0)
    fast = run_gpu(q, k, v, f, i, dh, False)
    for (bi, hi) in [(0, 0), (3, 7)]:
        one = [x[bi:bi + 1, hi:hi + 1].contiguous() for x in (q, k, v, f, i, dh)]
        ref = oracle_all(*one)
        prec = run_gpu(*one, True)
        row = {}
        for n, r_, a_, p_ in zip(NAMES, ref, fast, prec):
            row[n] = literal_violations(a_[bi:bi + 1, hi:hi + 1], r_)
            assert row[n][0] <= CEILING[dtype], (n, row[n])
            assert_close(p_, r_, dtype, f"precise {n} [{bi},{hi}]")
        print(f"cfg4 head ({bi},{hi}) fast: " + "  ".join(f"{n} {row[n][0]:.2e} (rms {row[n][1]:.1e})" for n in NAMES))
        assert_matches_oracle(dtype, *one, h=fast[0][bi:bi + 1, hi:hi + 1], grads=[g_[bi:bi + 1, hi:hi + 1] for g_ in fast[1:]], chunk_len=512,
                              tag=f"fast [{bi},{hi}] ")


def test_long_context_shape_one_head():
    """cfg 5 per head: S = 16384, D = 128, bf16, f ~ N(3,1), i ~ N(-1,1), dh ~ N(0, 0.1) (chunks of 512 in both modes;
    split mode with two-term states).  The oracle's S x S matrices are 2 GiB each in float64."""
    dtype = torch.bfloat16
    S, D = 16384, 128
    q, k, v, f, i, dh = O.make_inputs(1, 1, S, D, dtype, seed=5, f_mean=3.0, i_mean=-1.0, dh_std=0.1)
    fast = run_gpu(q, k, v, f, i, dh, False)
    prec = run_gpu(q, k, v, f, i, dh, True)
    ref = oracle_all(q, k, v, f, i, dh)
    row = {}
    for n, r_, a_, p_ in zip(NAMES, ref, fast, prec):
        row[n] = literal_violations(a_, r_)
        assert row[n][0] <= CEILING[dtype], (n, row[n])
        assert_close(p_, r_, dtype, f"precise {n}")
    print("cfg5 one head fast: " + "  ".join(f"{n} {row[n][0]:.2e} (rms {row[n][1]:.1e})" for n in NAMES))
    del ref
    assert_matches_oracle(dtype, q, k, v, f, i, dh, h=fast[0], grads=fast[1:], chunk_len=512, tag="fast ")
