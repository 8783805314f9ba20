"""MI355X (gfx950) implementation of Zoph_RNN's stacked-LSTM forward path.

csrc/   hand-written HIP kernels and the C-ABI (include/zoph_rnn.h) -> libzoph_rnn_hip.so
host/   C++ classes with the reference's layer-object names, forwarding to the C-ABI
capi.py ctypes plumbing used by the tests and the benchmark
synth.py deterministic synthetic inputs for the benchmark configurations
"""
