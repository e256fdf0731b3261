"""No-GPU checks of the C-ABI library: it loads, exports every symbol the header declares, and
rejects bad arguments before touching the device."""
import ctypes
import os
import re

import pytest

from conftest import ROOT

HEADERS = [os.path.join(ROOT, "include", n) for n in ("llmops_hip.h", "llmops_hip_test.h")]
LIB = os.path.join(ROOT, "llama.cl_amd", "llmops", "libllmops_hip.so")


def declared_symbols():
    src = "".join(open(h).read() for h in HEADERS)
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(llmops_[A-Za-z0-9_]+)\s*\(", src)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        pytest.fail(f"{LIB} not built: run `python llama.cl_amd/build.py`")
    return ctypes.CDLL(LIB)


def test_header_declares_the_path():
    names = declared_symbols()
    for must in ("llmops_offline_FC_quant_Q4A", "llmops_offline_FC_dequant_Q4A", "llmops_FC_dynamic_quantize_x",
                 "llmops_fc_Q4A", "llmops_fc_Q4A_partials", "llmops_attention_rope", "llmops_rope_embed", "llmops_softmax"):
        assert must in names


def test_library_exports_every_declared_symbol(lib):
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing


def test_python_binding_covers_every_declared_symbol():
    from llmops import _lib
    assert sorted(_lib.SIGNATURES) == declared_symbols()
    _lib.load()


def test_block_bytes(lib):
    lib.llmops_q4a_block_bytes.restype = ctypes.c_int64
    assert lib.llmops_q4a_block_bytes(32) == 640      # ops/op_fc.hpp:22-24 with G=32
    assert lib.llmops_q4a_block_bytes(128) == 2176
    assert lib.llmops_q4a_block_bytes(64) == 0


def test_argument_validation_without_device(lib):
    """Validation mirrors the reference's ASSERTs and runs before any HIP call, so it works with no GPU."""
    lib.llmops_last_error.restype = ctypes.c_char_p
    i64, vp = ctypes.c_int64, ctypes.c_void_p
    rc = lib.llmops_offline_FC_quant_Q4A(vp(16), i64(32), i64(64), i64(64), 64, vp(16), vp(0))
    assert rc == 1 and b"valid_group" in lib.llmops_last_error()
    rc = lib.llmops_fc_Q4A(vp(256), i64(1), i64(300), vp(256), i64(1), i64(1), 128, i64(32), vp(256), vp(256),
                           ctypes.c_size_t(1 << 20), vp(0))      # 300 activations cannot belong to one k-group of 128
    assert rc == 1 and b"K <= Kg * group_k" in lib.llmops_last_error()
    lib.llmops_fc_Q4A_workspace_bytes.restype = ctypes.c_size_t
    need = lib.llmops_fc_Q4A_workspace_bytes(i64(1), i64(4096), i64(128), i64(32), 128)
    assert need > 65536
    rc = lib.llmops_fc_Q4A(vp(256), i64(1), i64(4096), vp(256), i64(128), i64(32), 128, i64(4096), vp(256), vp(256),
                           ctypes.c_size_t(1024), vp(0))
    assert rc == 2 and b"workspace" in lib.llmops_last_error()
    rc = lib.llmops_attention_rope(vp(256), vp(256), vp(256), i64(1), i64(1), i64(32), i64(64), vp(256), i64(32), vp(256), 0,
                                   i64(2), i64(16), vp(256), 0, 0, vp(256), ctypes.c_size_t(1 << 30), vp(0))
    assert rc == 1 and b"S == 128" in lib.llmops_last_error()
    # the one-token kernels run on a (chunk, head) grid.  With the position by value more than 65535 heads in all take
    # the general kernels (GPU test); with the position in device memory they are refused before any launch
    rc = lib.llmops_attention_rope_decode(vp(256), vp(256), vp(256), i64(2200), i64(32), i64(128), vp(256), i64(64), vp(256), 0,
                                          i64(2), i64(16), vp(256), vp(256), 0, vp(256), ctypes.c_size_t(1 << 40), vp(0))
    assert rc == 1 and b"65535 heads" in lib.llmops_last_error()
    rc = lib.llmops_fc_workspace_reset(vp(0), ctypes.c_size_t(1 << 20), vp(0))
    assert rc == 1 and b"workspace != nullptr" in lib.llmops_last_error()
    # the entry point that allocates nothing validates its arguments before it enqueues anything (no device here:
    # a launch would fail with a HIP error, not with this message)
    rc = lib.llmops_fc_Q4A_noalloc(vp(0), i64(1), i64(4096), vp(256), i64(128), i64(32), 128, i64(4096), vp(256), vp(0))
    assert rc == 1 and b"x != nullptr" in lib.llmops_last_error()


def test_test_hooks_are_refused_unless_the_process_asks_for_them():
    """The planner knobs, dump builds and calibration kernels of include/llmops_hip_test.h live in the product
    library; a process that was not started with LLMOPS_TEST_HOOKS=1 cannot use them."""
    import subprocess
    import sys
    code = (
        "import ctypes, sys\n"
        f"lib = ctypes.CDLL({LIB!r})\n"
        "lib.llmops_last_error.restype = ctypes.c_char_p\n"
        "vp, i64 = ctypes.c_void_p, ctypes.c_int64\n"
        "rc = lib.llmops_test_calib_read(vp(256), i64(1024), 4, vp(256), vp(0))\n"
        "msg = lib.llmops_last_error()\n"
        "lib.llmops_test_fc_set_tuning(64, 8)\n"
        "print(rc, msg.decode())\n"
    )
    env = {k: v for k, v in os.environ.items() if k != "LLMOPS_TEST_HOOKS"}
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert out.stdout.startswith("1 ") and "LLMOPS_TEST_HOOKS=1" in out.stdout
    assert "test hooks are switched off" in out.stderr


def test_gemm_planner_choices(lib):
    """The prefill GEMM's planner is host arithmetic: what it chooses for the shapes its rules were measured
    on (row-tile factor 1, 2, 4 = 32, 64, 128 rows per workgroup, 8 = the 256-row kernel; split-K factor),
    and that every plan covers K exactly once."""
    i64, ci = ctypes.c_int64, ctypes.c_int

    def plan(rows, N, K, G=128):
        rt, S = ci(0), ci(0)
        assert lib.llmops_test_gemm_plan(i64(rows), i64((N + 31) // 32), i64((K + G - 1) // G), G, ctypes.byref(rt),
                                         ctypes.byref(S)) == 0
        return rt.value, S.value

    # many rows: the 256-row kernel, no split where the tiles fill the machine
    assert plan(2048, 11008, 4096) == (8, 1)
    assert plan(2048, 4096, 11008) == (8, 1)
    assert plan(2048, 4096, 512)[0] != 8          # fewer than 8 k-groups: its min-term prologue reads 8 at a time
    # few rows: 32-row tiles and as many splits as still leave runs of 4 k-groups (not 11 runs of 3)
    assert plan(32, 11008, 4096) == (1, 8)
    assert plan(64, 11008, 4096) == (1, 5)
    assert plan(128, 11008, 4096) == (2, 4)
    assert plan(128, 4096, 11008) == (1, 8)
    for rows in (17, 24, 40, 100, 255, 256, 300, 512, 1000, 4096):
        for N, K in ((4096, 4096), (11008, 4096), (4096, 11008), (352, 640), (22016, 4096), (64, 128)):
            rt, S = plan(rows, N, K)
            Kg = (K + 127) // 128
            assert rt in (1, 2, 4, 8) and 1 <= S <= Kg
            per = (Kg + S - 1) // S
            assert (Kg + per - 1) // per == S     # S splits of `per` k-groups, the last possibly short, none empty
    assert lib.llmops_test_gemm_plan(i64(0), i64(1), i64(1), 128, None, None) != 0


def test_python_ops_refuse_host_tensors():
    """The product path has no CPU fallback: host tensors raise instead of being computed elsewhere."""
    import torch
    import llmops
    with pytest.raises(RuntimeError, match="HIP device"):
        llmops.offline_FC_quant_Q4A(torch.zeros(32, 128))
    with pytest.raises(RuntimeError, match="HIP device"):
        llmops.fc_Q4A(torch.zeros(1, 1, 128), torch.zeros(1, 1, 2176, dtype=torch.int8), 32)


def test_kvcache_slot_manager():
    """KVCache.prepare mirrors chatllama/main.py:60-125: ring buffer, protected system slots, early stop."""
    import torch
    from llmops.opset import KVCache
    cfg = {"layer_num": 1, "head_num": 1, "head_size": 128}
    kv = KVCache(cfg, 1, 8, False, device="cpu")
    assert kv.prepare(3, -1, -1) and kv.slots.tolist() == [0, 1, 2] and kv.position_id == 0      # system prompt
    assert kv.prepare(2, 1, 0) and kv.slots.tolist() == [3, 4] and kv.position_id == 3
    assert kv.prepare(3, 2, 0) and kv.slots.tolist() == [5, 6, 7] and kv.cur_kv_len == 8
    # wraps around, skipping the protected system slots 0..2; sentence 1 may be overwritten
    assert kv.prepare(2, 3, 0) and kv.slots.tolist() == [3, 4] and kv.position_id == 8
    # sentence 2 holds the instruction: asked to fail rather than overwrite it
    assert not kv.prepare(1, 4, 2)
    assert kv.cur_kv_len == 8 and kv.slots.dtype == torch.int32


def test_tensor_attributes_the_reference_callers_use():
    """``weight.numel() * weight.item_size`` (chatllama/main.py:171-173) must work on what the ops return."""
    import torch
    import llmops  # noqa: F401  (adds the reference's spelling of the element size)
    t = torch.zeros(3, 5, dtype=torch.int8)
    assert t.item_size == 1 and torch.zeros(2, dtype=torch.float32).item_size == 4
    assert t.numel() * t.item_size == 15 and tuple(t.shape) == (3, 5) and t.clone().numpy().shape == (3, 5)
