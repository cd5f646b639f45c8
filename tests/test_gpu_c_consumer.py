"""The C ABI from plain C: tests/c_abi/ring_c_consumer.c (C99, built by the host C compiler against
include/ringattr.h; no Python, torch or C++ on its side) allocates device buffers through the HIP runtime, queries the
workspace sizes, calls ringattr_fwd / ringattr_bwd and checks history, dL/d r_init and dL/dWo against a closed form.
It is built as a shared object so that it can run inside this process."""
import ctypes
import os

import pytest

pytestmark = pytest.mark.gpu

LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_abi", "libring_c_consumer.so")


@pytest.mark.parametrize("N,B,T", [(64, 16, 6), (256, 32, 6), (200, 21, 5), (640, 16, 4)],
                         ids=["streaming", "resident", "resident_masked", "step_per_launch"])
def test_plain_c_caller(N, B, T, gpu_device):
    from rnn_train_ring_attractor_amd import _lib
    print(f"[case] plain-C caller N={N} B={B} T={T}", flush=True)
    _lib.load()                                   # (also resolves the consumer's dependency on libringattr.so)
    if not os.path.exists(LIB):
        pytest.fail(f"{LIB} is missing: run `python -m rnn_train_ring_attractor_amd.build` first")
    consumer = ctypes.CDLL(LIB)
    consumer.test_c_consumer.restype = ctypes.c_int
    consumer.test_c_consumer.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]
    msg = ctypes.create_string_buffer(512)
    rc = consumer.test_c_consumer(N, B, T, msg, len(msg))
    print(f"[measured] {msg.value.decode()}", flush=True)
    assert rc == 0, msg.value.decode()
