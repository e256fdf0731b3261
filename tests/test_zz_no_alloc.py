"""fc_Q4A through the entry point that allocates nothing (llmops_fc_Q4A_noalloc: the workspace is a fixed
array inside the library) against llmops_fc_Q4A with a caller-provided workspace: same kernels, so the
outputs must be bit-equal; and against the CPU oracle at the 1e-3 gate of fp32 FC outputs.  Each case is two
calls in a row on the same device, the second with a smaller input, so that what the first call left in
the shared array is what the second one starts from."""
import ctypes

import numpy as np
import pytest
import torch

import llmops
from llmops import _lib
from conftest import max_rel_err

pytestmark = pytest.mark.gpu


def _case(orc, rng, M, N, K, G):
    dev = torch.device("cuda:0")
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    x = rng.standard_normal((1, M, K)).astype(np.float32)
    wq = llmops.offline_FC_quant_Q4A(torch.from_numpy(w).to(dev), G)
    tx = torch.from_numpy(x).to(dev)
    want = llmops.fc_Q4A(tx, wq, N)
    out = torch.full((1, M, N), float("nan"), dtype=torch.float32, device=dev)
    lib = _lib.load()
    Ng, Kg, _ = wq.shape

    def call():
        rc = lib.llmops_fc_Q4A_noalloc(ctypes.c_void_p(tx.data_ptr()), M, K, ctypes.c_void_p(wq.data_ptr()), Ng, Kg, G, N,
                                       ctypes.c_void_p(out.data_ptr()),
                                       ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
        assert rc == 0, lib.llmops_last_error()
        torch.cuda.synchronize()

    call()  # the first call on a device may load code objects and looks the array's address up
    out.fill_(float("nan"))
    torch.cuda.synchronize()
    # torch's statistics only see torch's allocator; the driver's free-memory figure also sees a hipMalloc made
    # inside the library
    before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    free_before = torch.cuda.mem_get_info(dev)[0]
    call()
    assert torch.cuda.memory_stats(dev)["allocation.all.allocated"] == before
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    assert torch.equal(out, want), (M, N, K, G)
    # the oracle on a few rows (FC rows are independent)
    rows = sorted({0, M // 2, M - 1})
    ref = orc.fc(np.ascontiguousarray(x[:, rows]), orc.quant_w(w, G), N)
    assert max_rel_err(out.cpu().numpy()[:, rows], ref) <= 1e-3


@pytest.mark.parametrize("first,second", [
    ((1, 4096, 4096, 128), (1, 1024, 512, 128)),      # streaming kernel, then a smaller tensor
    ((1, 4096, 11008, 128), (1, 4096, 4096, 32)),     # two k-splits meeting in the exchange slots, then group 32
    ((16, 4096, 4096, 128), (5, 2048, 1024, 128)),    # quantization launch + weight-streaming MFMA kernel (k-halves)
    ((128, 4096, 11008, 128), (40, 4096, 4096, 128)),  # tiled MFMA kernel with split-K, then fewer rows
    ((128, 4096, 11008, 128), (1, 4096, 11008, 128)),  # many rows, then one row over the same array
])
def test_noalloc_matches_workspace_entry_point_twice_in_a_row(orc, first, second):
    rng = np.random.default_rng(11)
    _case(orc, rng, *first)
    _case(orc, rng, *second)


def test_noalloc_refuses_sizes_beyond_its_array():
    lib = _lib.load()
    dev = torch.device("cuda:0")
    t = torch.zeros(4096, dtype=torch.float32, device=dev)
    # 4096 rows x 11008: activation codes alone exceed the array
    rc = lib.llmops_fc_Q4A_noalloc(ctypes.c_void_p(t.data_ptr()), 4096, 11008, ctypes.c_void_p(t.data_ptr()), 128, 86, 128,
                                   4096, ctypes.c_void_p(t.data_ptr()), ctypes.c_void_p(0))
    assert rc == 2 and b"scratch" in lib.llmops_last_error()
    # a refused call enqueues nothing: bad arguments are reported before the zero fill of the array's head is launched
    rc = lib.llmops_fc_Q4A_noalloc(ctypes.c_void_p(0), 1, 4096, ctypes.c_void_p(t.data_ptr()), 128, 32, 128, 4096,
                                   ctypes.c_void_p(t.data_ptr()), ctypes.c_void_p(0))
    assert rc == 1 and b"x != nullptr" in lib.llmops_last_error()
