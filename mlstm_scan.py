"""Drop-in module: ``from mlstm_scan import mlstm_scan`` as in the reference's README (README.md:100-123)."""
from _mlstm_pkg import submodule as _sub

_m = _sub("mlstm_scan")
mlstm_scan = _m.mlstm_scan
# the backward of the scan form (the reference's kernel path has none) and the autograd function that carries it
Scan_mLSTM = _m.Scan_mLSTM
mlstm_scan_forward_hip = _m.mlstm_scan_forward_hip
mlstm_scan_forward_save_hip = _m.mlstm_scan_forward_save_hip
mlstm_scan_backward_hip = _m.mlstm_scan_backward_hip
