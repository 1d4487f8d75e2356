"""sLSTM cell (the reference's open item, README.md:9): ``from slstm import slstm``."""
from _mlstm_pkg import submodule as _sub

_m = _sub("slstm")
slstm = _m.slstm
HIP_sLSTM = _m.HIP_sLSTM
slstm_forward_hip = _m.slstm_forward_hip
slstm_backward_hip = _m.slstm_backward_hip
