"""The C ABI called from C++ with hipMalloc'ed buffers and a stream of the caller's own (no Python tensors, no torch): add +
RMSNorm + q8_1, the MMQ quantizer, the Q8 KV writer with a refused block, camx_init and the tape's append with its position in a
device word, the decode token's fused norm + rotary + append against the three launches it replaces, an argument refusal; each compared bit for bit with the
oracle inside tests/native/cpp_caller.cpp. Built by __graft_entry__.build() (tests/native/build.py)."""
import ctypes
import os

import pytest

pytestmark = pytest.mark.gpu

SO = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'native', 'libcpp_caller.so')


def test_cpp_caller_matches_the_oracle():
    if not os.path.isfile(SO):
        pytest.fail(f'{SO} is not built: run python -c "import __graft_entry__ as g; g.build()"')
    lib = ctypes.CDLL(SO)
    msg = ctypes.create_string_buffer(256)
    rc = lib.cpp_caller_run(msg, ctypes.c_int(256))
    assert rc == 0, msg.value.decode()
