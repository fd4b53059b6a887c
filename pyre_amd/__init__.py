"""pyre_amd: MI355X-native Qwen-Next (qwen4exp) decode token loop behind pyre's layer API.

The compute lives in the hipcc-built C-ABI library pyre_amd/csrc/libpyre_hip.so (declared in
include/pyre_hip.h); this package is the thin ctypes host mirror used by the tests and bench.py.
"""
