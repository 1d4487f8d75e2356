"""The bounded wait of the eight-wave row kernel: in a normal run no wait expires; with every wait forced to count as
expired (a host-side switch: the kernel skips the wait, reports, and still runs to its end) the error word is set, is
reported once, and is clear again afterwards."""
import pytest
import torch

from _mlstm_pkg import submodule
from oracle import mlstm_oracle as O

pytestmark = pytest.mark.gpu

ffi = submodule("_ffi")
mm = submodule("mlstm_matmul")


def test_expired_wait_is_reported_and_the_kernel_still_ends():
    L = ffi.lib()
    q, k, v, f, i, dh = [x.cuda() for x in O.make_inputs(1, 2, 640, 128, torch.bfloat16, seed=3, f_mean=2.0)]
    h0, m0, b0 = mm.mlstm_forward_hip(q, k, v, f, i)
    assert L.mlstm_kernel_error() == 0
    try:
        assert L.mlstm_set_spin_limit(-1) == 0
        h1, _, _ = mm.mlstm_forward_hip(q, k, v, f, i)        # results undefined; what matters is that the launch drains
        torch.cuda.synchronize()
        assert L.mlstm_kernel_error() == -4
        with pytest.raises(ValueError):
            ffi.check_rc(-4, "mlstm_kernel_error")
        assert L.mlstm_kernel_error() == 0                     # reported once, then clear
    finally:
        L.mlstm_set_spin_limit(0)
    h2, m2, b2 = mm.mlstm_forward_hip(q, k, v, f, i)
    assert torch.equal(h2, h0) and torch.equal(m2, m0) and torch.equal(b2, b0)
    grads = mm.mlstm_backward_hip(dh, q, k, v, f, i, h2, m2, b2)
    torch.cuda.synchronize()
    assert all(bool(torch.isfinite(g.float()).all()) for g in grads)
    assert L.mlstm_kernel_error() == 0
