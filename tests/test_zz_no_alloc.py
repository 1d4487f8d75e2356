"""The entry point that allocates nothing (mlstm_forward_noalloc_ex: the workspace is a static device array inside the
library) against mlstm_forward_ex, through the C ABI: two calls in a row, the second on a smaller input, bit for bit;
and the size limit."""
import pytest
import torch

from _mlstm_pkg import submodule
from oracle import mlstm_oracle as O

pytestmark = pytest.mark.gpu

ffi = submodule("_ffi")


def forward_both(B, NH, S, D, dtype, seed):
    q, k, v, f, i, _ = [x.cuda() for x in O.make_inputs(B, NH, S, D, dtype, seed=seed, f_mean=2.0)]
    L = ffi.lib()
    dt, gdt = ffi.dtype_code(q.dtype), ffi.dtype_code(f.dtype)
    outs = []
    for which in ("noalloc", "ex"):
        h = torch.zeros_like(q)
        m = torch.zeros((B, NH, S), device="cuda", dtype=torch.float32)
        b = torch.zeros_like(m)
        if which == "noalloc":
            rc = L.mlstm_forward_noalloc_ex(ffi.ptr(q), ffi.ptr(k), ffi.ptr(v), ffi.ptr(f), ffi.ptr(i), ffi.ptr(h), ffi.ptr(m), ffi.ptr(b),
                                            B, NH, S, D, dt, gdt, ffi.stream_ptr())
        else:
            ws, n = ffi.workspace(ffi.OP_FORWARD, B, NH, S, D, dt, q.device)
            rc = L.mlstm_forward_ex(ffi.ptr(q), ffi.ptr(k), ffi.ptr(v), ffi.ptr(f), ffi.ptr(i), ffi.ptr(h), ffi.ptr(m), ffi.ptr(b),
                                    B, NH, S, D, dt, gdt, ffi.ptr(ws), n, ffi.stream_ptr())
        ffi.check_rc(rc, which)
        torch.cuda.synchronize()
        outs.append((h, m, b))
    return outs


def test_noalloc_forward_matches_forward_ex_on_two_calls_in_a_row():
    # first call: a sequence that runs in chunks (states at the chunk ends live in the scratch too); second call: a
    # smaller input of another type and head size, which carves the same array differently
    for (B, NH, S, D, dtype, seed) in [(1, 2, 1536, 128, torch.bfloat16, 11), (2, 1, 300, 256, torch.float16, 12), (1, 1, 77, 64, torch.float32, 13)]:
        assert ffi.lib().mlstm_workspace_bytes(ffi.OP_FORWARD, B, NH, S, D, ffi.dtype_code(dtype)) <= ffi.NOALLOC_MAX_WORKSPACE
        (h0, m0, b0), (h1, m1, b1) = forward_both(B, NH, S, D, dtype, seed)
        assert bool(torch.isfinite(h0.float()).all()) and float(h0.float().abs().max()) > 0
        assert torch.equal(h0, h1) and torch.equal(m0, m1) and torch.equal(b0, b1), (S, D, dtype)


def test_noalloc_forward_leaves_device_memory_as_it_found_it():
    """After one warm-up call per shape (which loads the kernels and looks up the scratch array), further calls must not
    change the device's free memory: nothing is allocated or freed, stream-ordered or otherwise."""
    B, NH, S, D = 1, 2, 1536, 128
    q, k, v, f, i, _ = [x.cuda() for x in O.make_inputs(B, NH, S, D, torch.bfloat16, seed=5, f_mean=2.0)]
    h = torch.empty_like(q)
    m = torch.empty((B, NH, S), device="cuda", dtype=torch.float32)
    b = torch.empty_like(m)
    L = ffi.lib()
    assert L.mlstm_init() == 0
    args = (ffi.ptr(q), ffi.ptr(k), ffi.ptr(v), ffi.ptr(f), ffi.ptr(i), ffi.ptr(h), ffi.ptr(m), ffi.ptr(b), B, NH, S, D, ffi.BF16, ffi.BF16,
            ffi.stream_ptr())
    ffi.check_rc(L.mlstm_forward_noalloc_ex(*args), "warm-up")
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        ffi.check_rc(L.mlstm_forward_noalloc_ex(*args), "mlstm_forward_noalloc_ex")
        free_during, _ = torch.cuda.mem_get_info()
        assert free_during == free0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0


def test_noalloc_forward_rejects_shapes_beyond_its_scratch():
    B, NH, S, D = 4, 8, 4096, 256
    L = ffi.lib()
    assert L.mlstm_workspace_bytes(ffi.OP_FORWARD, B, NH, S, D, ffi.BF16) > ffi.NOALLOC_MAX_WORKSPACE
    q = torch.zeros((B, NH, S, D), device="cuda", dtype=torch.bfloat16)
    f = torch.zeros((B, NH, S), device="cuda", dtype=torch.bfloat16)
    h = torch.empty_like(q)
    rc = L.mlstm_forward_noalloc_ex(ffi.ptr(q), ffi.ptr(q), ffi.ptr(q), ffi.ptr(f), ffi.ptr(f), ffi.ptr(h), None, None,
                                    B, NH, S, D, ffi.BF16, ffi.BF16, ffi.stream_ptr())
    assert rc == -3
    with pytest.raises(ValueError):
        ffi.check_rc(rc, "mlstm_forward_noalloc_ex")
