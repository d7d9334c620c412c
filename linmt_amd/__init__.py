"""linmt_amd: MI355X (gfx950) HIP kernels and C++ layer classes for LiNMT's per-timestep
LSTM / attention / softmax / beam path.  The product is the C ABI in include/linmt_hip.h
(liblinmt_hip.so) and the C++ host layer on top of it; this package only binds them for Python
tests and the benchmark."""
from . import lib  # noqa: F401
