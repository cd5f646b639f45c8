"""ringattr_fwd_noalloc (the entry point that allocates nothing: its packed-weight scratch is a fixed array inside
the library) against ringattr_fwd with a caller workspace, through the C ABI.  Both run the same kernels on the
same inputs, so the state history and the saved record must agree bit for bit; two calls in a row, the second
with a smaller input, show that nothing of an earlier call's scratch contents leaks into a later result."""
import numpy as np
import pytest
import torch

from oracle import ring_oracle as O
from tests.ring_cases import make_problem

pytestmark = pytest.mark.gpu


def _run_pair(lib, dev, seed, B, T, k, N, act):
    p = make_problem(seed, B, T, k, N, action="dense" if k != 2 else "lr")
    t = lambda x: torch.tensor(np.ascontiguousarray(x), device=dev)
    A, Wa, Wo, r0 = t(p["A"]), t(p["Wa"]), t(p["Wo"]), t(p["r0"])
    J0, J1, alpha = -0.1, 0.3, 0.15
    stream = torch.cuda.current_stream(dev).cuda_stream
    nsaved = lib.ringattr_saved_bytes(N, k, T, B)
    outs = []
    for entry in ("workspace", "noalloc"):
        hist = torch.full((T, B, N), float("nan"), device=dev)
        saved = torch.zeros(nsaved, dtype=torch.uint8, device=dev)
        if entry == "workspace":
            nws = lib.ringattr_fwd_workspace_bytes(N, k, T, B)
            ws = torch.empty(nws, dtype=torch.uint8, device=dev)
            rc = lib.ringattr_fwd(A.data_ptr(), Wa.data_ptr(), J0, J1, Wo.data_ptr(), r0.data_ptr(), hist.data_ptr(), alpha,
                                  N, k, T, B, act, saved.data_ptr(), ws.data_ptr(), nws, stream)
        else:
            rc = lib.ringattr_fwd_noalloc(A.data_ptr(), Wa.data_ptr(), J0, J1, Wo.data_ptr(), r0.data_ptr(),
                                          hist.data_ptr(), alpha, N, k, T, B, act, saved.data_ptr(), stream)
        assert rc == 0, lib.ringattr_last_error()
        torch.cuda.synchronize()
        outs.append((hist, saved))
    (h_ws, s_ws), (h_na, s_na) = outs
    # What the entry point is for: a warmed call takes nothing from the device allocator and returns nothing to it.
    # hipMemGetInfo (torch.cuda.mem_get_info) reports the device's free bytes; a hipMalloc inside the call, freed
    # or not, would show while the call's work is still queued or after it.
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    rc = lib.ringattr_fwd_noalloc(A.data_ptr(), Wa.data_ptr(), J0, J1, Wo.data_ptr(), r0.data_ptr(), h_na.data_ptr(),
                                  alpha, N, k, T, B, act, s_na.data_ptr(), stream)
    free_queued = torch.cuda.mem_get_info(dev)[0]
    assert rc == 0, lib.ringattr_last_error()
    torch.cuda.synchronize()
    assert free_queued == free_before and torch.cuda.mem_get_info(dev)[0] == free_before
    assert torch.isfinite(h_na).all()
    assert torch.equal(h_na, h_ws)                 # bit-exact: same kernels, same packed weights
    assert torch.equal(s_na, s_ws)
    names = {0: "relu", 1: "gelu", 2: "tanh", 3: "silu"}
    ref, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], alpha, names[act])
    assert O.max_rel_err(h_na.cpu().numpy(), ref) <= 1e-2     # and against the fp64 oracle (trajectory tolerance)


def test_noalloc_forward_matches_workspace_forward_twice(gpu_device):
    from rnn_train_ring_attractor_amd import _lib
    lib = _lib.load()
    with torch.cuda.device(gpu_device):
        print("[case] noalloc fwd N=256 B=48 T=20 k=2 gelu", flush=True)
        _run_pair(lib, gpu_device, 21, 48, 20, 2, 256, 1)
        print("[case] noalloc fwd N=100 B=19 T=7 k=3 silu (smaller, after the first)", flush=True)
        _run_pair(lib, gpu_device, 22, 19, 7, 3, 100, 3)
        # beyond the built-in scratch: N = 512 with a_dim = 8 packs 9 * 512 * 512 * 2 bytes = 4.5 MiB
        z = torch.zeros(16, device=gpu_device)
        rc = lib.ringattr_fwd_noalloc(z.data_ptr(), z.data_ptr(), 0.0, 1.0, z.data_ptr(), z.data_ptr(), z.data_ptr(), 0.15,
                                      512, 8, 4, 16, 0, None, None)
        assert rc == 2 and "built-in scratch" in _lib.last_error()
