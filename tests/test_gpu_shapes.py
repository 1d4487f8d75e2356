"""Batch / head counts that select the different workgroup orders of the tile kernels, and seeded random shapes."""
import pytest
import torch

from _mlstm_pkg import submodule
from oracle import mlstm_oracle as O
from tests.helpers import assert_matches_oracle

pytestmark = pytest.mark.gpu

mm = submodule("mlstm_matmul")


def check(B, NH, S, D, dtype, seed, heads=None):
    q, k, v, f, i, dh = O.make_inputs(B, NH, S, D, dtype, seed=seed, f_mean=2.0)
    dev = [x.cuda() for x in (q, k, v, f, i, dh)]
    h, m, b = mm.mlstm_forward_hip(*dev[:5])
    grads = mm.mlstm_backward_hip(dev[5], *dev[:5], h, m, b)
    torch.cuda.synchronize()
    # the oracle is dense: compare a few heads, spread over the batch, rather than all of them
    pairs = heads if heads is not None else [(bi, hi) for bi in range(B) for hi in range(NH)]
    for bi, hi in pairs:
        sl = lambda x: x[bi:bi + 1, hi:hi + 1]
        assert_matches_oracle(dtype, *(sl(x) for x in (q, k, v, f, i, dh)), h=sl(h), m=sl(m), b=sl(b), grads=[sl(g_) for g_ in grads],
                              tag=f"[{bi},{hi}] ")


@pytest.mark.parametrize("B,NH", [(1, 8), (3, 8), (2, 8), (5, 8), (1, 7), (3, 3)])
@pytest.mark.parametrize("D,dtype", [(256, torch.bfloat16), (128, torch.float16)])
def test_head_counts_that_change_the_workgroup_order(B, NH, D, dtype):
    # B*NH = 8, 24, 16, 40 (multiples of 8: one, three, two, five heads per XCD, i.e. odd and even numbers of head pairs),
    # 7 and 9 (the plain order); S = 448 gives 3.5 row tiles of 128 and 7 key tiles
    BH = B * NH
    heads = [(0, 0), (B - 1, NH - 1), (B // 2, NH // 2), ((B - 1) // 2, (NH + 1) // 2 % NH)]
    check(B, NH, 448, D, dtype, seed=1000 + BH + D, heads=sorted(set(heads)))


@pytest.mark.parametrize("case", range(18))
def test_seeded_random_shapes(case):
    g = torch.Generator().manual_seed(4242 + case)
    r = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    D = [64, 128, 256][r(0, 2)]
    dtype = [torch.float32, torch.float16, torch.bfloat16][case % 3]
    if D == 256 and dtype == torch.float32:
        dtype = torch.bfloat16
    B, NH, S = r(1, 3), r(1, 4), r(1, 700)
    check(B, NH, S, D, dtype, seed=77 + case, heads=[(0, 0), (B - 1, NH - 1)])


@pytest.mark.parametrize("D", [16, 32])
@pytest.mark.parametrize("dtype,S", [(torch.float32, 200), (torch.float32, 1100), (torch.bfloat16, 333), (torch.float16, 1100)])
def test_head_dimensions_below_the_smallest_tile(D, dtype, S):
    # D = 16 and 32 (the reference's kernels take any power of two from 16 on): the wrappers pad q, k, v with zero columns
    # to the kernels' smallest head dimension and scale q for the 1 / sqrt(D) of the scores; outputs come back at D
    B, NH = 2, 2
    q, k, v, f, i, dh = O.make_inputs(B, NH, S, D, dtype, seed=D + S, f_mean=2.0)
    dev = [x.cuda() for x in (q, k, v, f, i, dh)]
    h, m, b, saved = mm.mlstm_forward_save_hip(*dev[:5])
    assert tuple(h.shape) == (B, NH, S, D) and h.dtype == dtype
    grads = mm.mlstm_backward_saved_hip(dev[5], *dev[:5], h, m, b, saved)
    again = mm.mlstm_backward_hip(dev[5], *dev[:5])               # recomputes the forward
    for g_, a_ in zip(grads, again):
        assert g_.shape == a_.shape and torch.equal(g_, a_)
    assert tuple(grads[0].shape) == (B, NH, S, D) and tuple(grads[3].shape) == (B, NH, S)
    sl = lambda x: x[1:2, 0:1]
    assert_matches_oracle(dtype, *(sl(x) for x in (q, k, v, f, i, dh)), h=sl(h), m=sl(m), b=sl(b), grads=[sl(g_) for g_ in grads])
    # through autograd, like the reference's Triton_mLSTM.apply
    ins = [x.clone().requires_grad_(True) for x in dev[:5]]
    mm.Triton_mLSTM.apply(*ins).backward(dev[5])
    for x, g_ in zip(ins, grads):
        assert torch.equal(x.grad, g_)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_sixteen_bit_head_dimension_512_runs_widened(dtype):
    # beyond the 16-bit tile kernels' head dimensions the wrappers run the fp32 path on widened inputs: results are the
    # fp32 results of the 16-bit inputs, rounded once to the callers' types
    B, NH, S, D = 1, 2, 200, 512
    q, k, v, f, i, dh = O.make_inputs(B, NH, S, D, dtype, seed=512, f_mean=2.0)
    dev = [x.cuda() for x in (q, k, v, f, i, dh)]
    ins = [x.clone().requires_grad_(True) for x in dev[:5]]
    h = mm.Triton_mLSTM.apply(*ins)
    h.backward(dev[5])
    assert h.dtype == dtype and ins[0].grad.dtype == dtype and ins[3].grad.dtype == dtype
    hr, _, _ = O.mlstm_forward_dense(q, k, v, f, i, dtype=torch.float64)
    ref = O.mlstm_backward_dense(dh, q, k, v, f, i, dtype=torch.float64, zero_first_df=True)
    eps = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11     # one rounding to the type: half an ulp, and the fp32 path's 1e-4
    for name, got, want in zip(["h", "dq", "dk", "dv", "df", "di"], [h, *(x.grad for x in ins)], [hr, *ref]):
        got, want = got.detach().cpu().double(), want.double()
        assert torch.all((got - want).abs() <= eps * want.abs() + 2e-4 * float(want.abs().max())), name


@pytest.mark.parametrize("case", range(24))
def test_seeded_random_long_shapes_and_kernel_switches(case):
    # lengths on both sides of the chunking threshold, every type, forced chunk lengths, split mode, each column kernel and
    # both state-kernel forms, three forget-gate regimes: forward + backward (with the forward's saved states, and
    # recomputing them: the same bits) against the oracle under the rule of the arithmetic in use
    import random
    from _mlstm_pkg import submodule
    ffi = submodule("_ffi")
    rng = random.Random(9000 + case)
    dtype = [torch.float32, torch.float16, torch.bfloat16][case % 3]
    D = rng.choice([64, 128] if dtype == torch.float32 else [64, 128, 256])
    B, NH = rng.randint(1, 2), rng.randint(1, 3)
    S = rng.choice([rng.randint(900, 1400), rng.randint(1024, 2600)])
    L = rng.choice([0, 0, 128, 256, 384, -1])
    precise = dtype != torch.float32 and rng.random() < 0.3
    colk, statek = rng.choice([0, 0, 1, 2, 3]), rng.choice([0, 2])
    fmean = rng.choice([0.0, 2.0, 4.0])
    q, k, v, f, i, dh = O.make_inputs(B, NH, S, D, dtype, seed=9000 + case, f_mean=fmean)
    dev = [x.cuda() for x in (dh, q, k, v, f, i)]
    try:
        ffi.set_chunk_length(L)
        ffi.set_column_kernel(colk)
        ffi.set_state_kernel(statek)
        h, m, b, saved = mm.mlstm_forward_save_hip(*dev[1:], precise=precise)
        grads = mm.mlstm_backward_saved_hip(*dev, h, m, b, saved, precise=precise)
        again = mm.mlstm_backward_hip(*dev, precise=precise)
        torch.cuda.synchronize()
        assert ffi.lib().mlstm_kernel_error() == 0
        Lc = int(ffi.lib().mlstm_chunk_length_for(S, D, ffi.dtype_code(dtype)))
    finally:
        ffi.set_chunk_length(0)
        ffi.set_column_kernel(0)
        ffi.set_state_kernel(0)
    for name, x, y in zip(["dq", "dk", "dv", "df", "di"], grads, again):
        assert torch.equal(x, y), name
    sl = lambda x: x[B - 1:B, NH - 1:NH]
    assert_matches_oracle(dtype, *(sl(x) for x in (q, k, v, f, i, dh)), h=sl(h), m=sl(m), b=sl(b), grads=[sl(g_) for g_ in grads],
                          chunk_len=Lc, precise=precise)
