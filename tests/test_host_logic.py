"""Host-side logic of the ctypes layer that needs no GPU: layouts of gradient tensors, overlap detection."""
import torch

from _mlstm_pkg import submodule

ffi = submodule("_ffi")


def test_expanded_views_are_recognised_as_overlapping():
    B, NH, S, D = 2, 4, 8, 64
    f = torch.zeros(B, 1, S)
    assert ffi.overlaps(f.expand(B, NH, S))                       # gates shared over the heads: stride 0
    q = torch.zeros(1, NH, S, D)
    assert ffi.overlaps(q.expand(B, NH, S, D))
    assert ffi.overlaps(torch.zeros(S + 3).as_strided((2, 3), (2, 1)))   # rows of 3 that start 2 apart
    proj = torch.zeros(B, S, NH, D)
    assert not ffi.overlaps(proj.transpose(1, 2))                 # [B,S,NH,D] activations seen as [B,NH,S,D]
    fused = torch.zeros(B, S, 3, NH, D)
    assert not ffi.overlaps(fused[:, :, 1].transpose(1, 2))       # one slice of a fused q/k/v projection
    assert not ffi.overlaps(torch.zeros(B, NH, S, D))
    assert not ffi.overlaps(torch.zeros(1, 1, S).expand(1, 1, S))  # size-1 dimensions never overlap


def test_overlapping_inputs_are_replaced_by_dense_copies_together():
    B, NH, S = 2, 4, 8
    f = torch.arange(B * S, dtype=torch.float32).reshape(B, 1, S).expand(B, NH, S)
    i = torch.zeros(B, NH, S)
    f2, i2 = ffi.dense_unless_disjoint(f, i)
    assert f2.is_contiguous() and i2.is_contiguous() and torch.equal(f2, f)
    a, b = torch.zeros(B, NH, S), torch.zeros(B, NH, S)
    a2, b2 = ffi.dense_unless_disjoint(a, b)
    assert a2 is a and b2 is b                                     # disjoint tensors pass through untouched


def test_gradient_buffers_of_a_strided_view_keep_its_strides_and_do_not_alias():
    B, NH, S, D = 2, 3, 5, 8
    proj = torch.zeros(B, S, NH, D)
    q = proj.transpose(1, 2)
    dq, dk = ffi.strided_like(q, 2)
    assert dq.stride() == q.stride() and dk.stride() == q.stride() and dq.data_ptr() != dk.data_ptr()
    assert not ffi.overlaps(dq)
    fused = torch.zeros(B, S, 3, NH, D)[:, :, 0].transpose(1, 2)
    g = ffi.strided_like(fused)[0]
    assert g.stride() == fused.stride() and not ffi.overlaps(g)
    g.fill_(1.0)
    assert float(g.sum()) == B * NH * S * D


def test_tile_copy_index_arithmetic_stays_inside_the_tiles():
    """tests/harness/tile_bounds (the kernels' own offset functions, compiled for the host): every block of every tile shape
    is fetched exactly once, lands where the LDS readers expect it, and no fetch ends beyond the tile's last row -- for the
    last tile of the last head that is the end of the caller's tensor; the early touch of the dQ pass stays inside its half row."""
    import os
    import subprocess
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "harness")
    exe = os.path.join(here, "tile_bounds")
    if not os.path.exists(exe):
        subprocess.check_call(["make", "-C", here, "tile_bounds"])
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0 and "tile_bounds: ok" in out.stdout, out.stdout + out.stderr
