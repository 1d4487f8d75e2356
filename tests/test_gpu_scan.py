"""Parity of the HIP scan form against the CPU oracle (step-by-step recurrence and the dense form)."""
import pytest
import torch

from oracle import mlstm_oracle as O
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu


def run_scan(q, k, v, f, i, o, **kw):
    from mlstm_scan import mlstm_scan
    return mlstm_scan(*(x.cuda() for x in (q, k, v, f, i, o)), **kw)


@pytest.mark.parametrize("S,D", [(1, 64), (16, 64), (64, 64), (100, 128), (192, 128), (130, 256), (256, 512)])
def test_scan_small_vs_recurrence(S, D):
    q, k, v, f, i, _, o = O.make_inputs(1, 2, S, D, torch.float32, seed=S + D, with_o=True)
    h = run_scan(q, k, v, f, i, o)
    ref = O.mlstm_recurrent(q, k, v, f, i, o)          # the reference oracle's own formulation (mlstm_scan.py:343-372)
    assert h.dtype == torch.float32 and h.shape == q.shape
    assert_close(h, ref, torch.float32, "h")


@pytest.mark.parametrize("f_mean,i_mean", [(-3.0, 0.0), (0.0, 2.0), (8.0, -1.0)])
def test_scan_gate_regimes(f_mean, i_mean):
    # strong forgetting (the carried state is rescaled in every chunk), mixed, and almost none (never rescaled)
    q, k, v, f, i, _, o = O.make_inputs(1, 2, 640, 128, torch.float32, seed=11, f_mean=f_mean, i_mean=i_mean, with_o=True)
    h = run_scan(q, k, v, f, i, o)
    assert_close(h, O.mlstm_scan_dense(q, k, v, f, i, o), torch.float32, "h")


def test_scan_many_heads_one_key_range():
    # enough heads to fill the chip without splitting the key range of a value tile
    q, k, v, f, i, _, o = O.make_inputs(4, 4, 200, 512, torch.float32, seed=12, with_o=True)
    h = run_scan(q, k, v, f, i, o)
    assert_close(h, O.mlstm_scan_dense(q, k, v, f, i, o), torch.float32, "h")


def test_scan_tuning_arguments_do_not_change_the_result():
    q, k, v, f, i, _, o = O.make_inputs(1, 2, 128, 64, torch.float32, seed=3, with_o=True)
    h1 = run_scan(q, k, v, f, i, o)
    h2 = run_scan(q, k, v, f, i, o, reduce_block_size=8, value_block_size=16, num_warps=4)
    assert torch.equal(h1, h2)


def test_scan_equals_gated_matmul_form():
    # silu(o) * matmul-form h, both on the GPU
    from mlstm_matmul import mlstm_matmul
    q, k, v, f, i, _, o = O.make_inputs(2, 2, 320, 128, torch.float32, seed=9, with_o=True)
    h = run_scan(q, k, v, f, i, o)
    hm = mlstm_matmul(*(x.cuda() for x in (q, k, v, f, i)))
    assert_close(h, (hm * torch.nn.functional.silu(o.cuda())), torch.float32, "h")


def test_config3_scan_full():
    # B1 H4 S2048 D1024 fp32, reduce_block_size = value_block_size = 4 (the reference's self-check, mlstm_scan.py:375-394)
    q, k, v, f, i, _, o = O.make_inputs(1, 4, 2048, 1024, torch.float32, seed=0, with_o=True)
    h = run_scan(q, k, v, f, i, o, reduce_block_size=4, value_block_size=4)
    ref = O.mlstm_scan_dense(q, k, v, f, i, o)
    assert_close(h, ref, torch.float32, "h")


def test_scan_against_committed_golden_vector():
    import os
    import numpy as np
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "scan_B1_H1_S80_D64_seed2.npz"), allow_pickle=False)
    g = {k_: torch.from_numpy(z[k_]) for k_ in z.files}
    h = run_scan(g["q"], g["k"], g["v"], g["f"], g["i"], g["o"])
    assert_close(h, g["h"], torch.float32, "h")


@pytest.mark.parametrize("S,D", [(8192, 64), (3000, 64), (4096, 128), (2048, 256)])
def test_scan_one_long_sequence_in_segments(S, D):
    # one head: the state walk runs in segments side by side (states at the segment ends from a pass of their own);
    # checked against the step-by-step recurrence, and against the same head inside a batch that fills the chip and
    # therefore walks its chunks in one piece
    q, k, v, f, i, _, o = O.make_inputs(1, 1, S, D, torch.float32, seed=S + D, with_o=True)
    h = run_scan(q, k, v, f, i, o)
    assert_close(h, O.mlstm_recurrent(q, k, v, f, i, o), torch.float32, "h")
    reps = 256 // (D // 32)
    hb = run_scan(*(x.expand(reps, *x.shape[1:]).contiguous() for x in (q, k, v, f, i, o)))
    assert torch.equal(hb[0], hb[reps - 1])
    assert_close(h[0], hb[0].cpu(), torch.float32, "h against the unsegmented walk")


def test_scan_strong_forgetting_across_segments():
    q, k, v, f, i, _, o = O.make_inputs(1, 2, 4096, 64, torch.float32, seed=77, f_mean=-3.0, with_o=True)
    assert_close(run_scan(q, k, v, f, i, o), O.mlstm_recurrent(q, k, v, f, i, o), torch.float32, "h")
