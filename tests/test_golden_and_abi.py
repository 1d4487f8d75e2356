"""CPU-side checks: the oracle reproduces the committed golden vectors, the C-ABI library loads and exports every
symbol declared in include/mlstm_hip.h, and argument errors are rejected before any GPU work."""
import ctypes
import glob
import os
import re

import numpy as np
import pytest
import torch

from _mlstm_pkg import submodule
from oracle import mlstm_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = os.path.join(ROOT, "tests", "golden")


def load(name):
    z = np.load(os.path.join(GOLD, name), allow_pickle=False)
    return {k: torch.from_numpy(z[k]) for k in z.files}


@pytest.mark.parametrize("name", sorted(os.path.basename(p) for p in glob.glob(os.path.join(GOLD, "matmul_*.npz"))))
def test_oracle_reproduces_matmul_goldens(name):
    g = load(name)
    h, m, b = O.mlstm_forward_dense(g["q"], g["k"], g["v"], g["f"], g["i"])
    grads = O.mlstm_backward_dense(g["dh"], g["q"], g["k"], g["v"], g["f"], g["i"], zero_first_df=True)
    for key, val in [("h", h), ("m", m), ("b", b)] + list(zip(["dq", "dk", "dv", "df", "di"], grads)):
        assert torch.allclose(val.float(), g[key], rtol=1e-6, atol=1e-7), key
    # second, independent evaluation: the recurrence
    hr = O.mlstm_recurrent(g["q"], g["k"], g["v"], g["f"], g["i"], None)
    assert torch.allclose(hr.float(), g["h"], rtol=1e-5, atol=1e-6)


def test_oracle_reproduces_scan_golden():
    g = load("scan_B1_H1_S80_D64_seed2.npz")
    h = O.mlstm_scan_dense(g["q"], g["k"], g["v"], g["f"], g["i"], g["o"])
    assert torch.allclose(h.float(), g["h"], rtol=1e-5, atol=1e-6)


def test_library_exports_every_declared_symbol():
    ffi = submodule("_ffi")
    header = open(os.path.join(ROOT, "include", "mlstm_hip.h")).read()
    declared = set(re.findall(r"^(?:int|size_t|const char\*)\s+((?:mlstm|slstm)_\w+)\s*\(", header, flags=re.M))
    assert declared == set(ffi.exported_symbols()), declared ^ set(ffi.exported_symbols())
    L = ffi.lib()
    for sym in declared:
        assert getattr(L, sym) is not None
    assert L.mlstm_version().decode().startswith("mlstm_hip")


def test_workspace_sizes_and_argument_errors_need_no_gpu():
    ffi = submodule("_ffi")
    L = ffi.lib()
    fwd = L.mlstm_workspace_bytes(ffi.OP_FORWARD, 4, 8, 4096, 256, ffi.BF16)
    bwd = L.mlstm_workspace_bytes(ffi.OP_BACKWARD, 4, 8, 4096, 256, ffi.BF16)
    scan = L.mlstm_workspace_bytes(ffi.OP_SCAN_FORWARD, 1, 4, 2048, 1024, ffi.F32)
    assert 0 < fwd < bwd and scan > 0
    assert L.mlstm_workspace_bytes(ffi.OP_FORWARD_GATED, 4, 8, 4096, 256, ffi.BF16) == fwd
    assert L.mlstm_workspace_bytes(ffi.OP_BACKWARD_GATED, 4, 8, 4096, 256, ffi.BF16) > bwd + 2 * 4 * 8 * 4096 * 256 * 2
    # the scan form's backward walks q, k, v in place from the end and keeps two [BH,S,D] buffers of its own (plus the partial
    # numerators of a second key range at D = 1024): three tensors' worth at the reference's scan shape, not eight
    tensor = 1 * 4 * 2048 * 1024 * 4
    scan_bwd = L.mlstm_workspace_bytes(ffi.OP_SCAN_BACKWARD, 1, 4, 2048, 1024, ffi.F32)
    assert 3 * tensor < scan_bwd < 3 * tensor + 8 * 2**20
    assert L.mlstm_workspace_bytes(ffi.OP_FORWARD, 0, 8, 4096, 256, ffi.BF16) == 0
    assert L.mlstm_workspace_bytes(7, 1, 1, 64, 64, ffi.F32) == 0
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)  # never dereferenced: the shape check comes first
    assert L.mlstm_forward_ex(null, null, null, null, null, null, null, null, 1, 1, 64, 64, ffi.F32, ffi.F32, null, 0, null) == -1
    assert L.mlstm_forward_ex(one, one, one, one, one, one, null, null, 1, 1, 64, 48, ffi.F32, ffi.F32, null, 0, null) == -2
    assert L.mlstm_forward_ex(one, one, one, one, one, one, null, null, 1, 1, 64, 512, ffi.BF16, ffi.F32, null, 0, null) == -2
    assert L.mlstm_forward_ex(one, one, one, one, one, one, null, null, 1, 1, 64, 2048, ffi.F32, ffi.F32, null, 0, null) == -2
    assert L.mlstm_forward_ex(one, one, one, one, one, one, null, null, 1, 1, 64, 64, 9, ffi.F32, null, 0, null) == -1
    assert L.mlstm_forward_ex(one, one, one, one, one, one, null, null, 1, 1, 64, 64, ffi.F32, ffi.F32, one, 8, null) == -3
    assert L.mlstm_backward_ex(*([one] * 6), null, null, null, *([one] * 5), 1, 1, 64, 96, ffi.F16, ffi.F16, null, 0, null) == -2
    assert L.mlstm_forward_gated_ex(*([one] * 5), null, one, one, null, null, 1, 1, 64, 64, ffi.F32, ffi.F32, null, 0, null) == -1
    assert L.mlstm_forward_gated_ex(*([one] * 8), null, null, 1, 1, 64, 512, ffi.F16, ffi.F16, null, 0, null) == -2
    assert L.mlstm_backward_gated_ex(*([one] * 7), null, null, null, *([one] * 5), null, 1, 1, 64, 64, ffi.F16, ffi.F16, null, 0, null) == -1
    assert L.mlstm_backward_gated_ex(*([one] * 7), null, null, null, *([one] * 6), 1, 1, 64, 64, ffi.F16, ffi.F16, one, 8, null) == -3
    assert L.mlstm_scan_forward_ex(*([one] * 7), 1, 1, 64, 64, ffi.BF16, null, 0, null) == -2
    assert L.mlstm_scan_forward_ex(*([one] * 7), 1, 1, 64, 96, ffi.F32, null, 0, null) == -2


def test_python_wrappers_reject_bad_inputs_on_cpu():
    mm = submodule("mlstm_matmul")
    q = torch.zeros(1, 1, 8, 64)
    f = torch.zeros(1, 1, 8)
    with pytest.raises(ValueError):
        mm.mlstm_forward_hip(q, q, q, f, f)                      # CPU tensors: no silent fallback
    with pytest.raises(ValueError):
        mm.mlstm_forward_hip(q[0], q[0], q[0], f[0], f[0])       # wrong rank
