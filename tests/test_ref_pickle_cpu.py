"""The reader of reference-format model files (llmops.ref_pickle): structure, arrays, and that nothing
the file names is executed.  No GPU and no compute library involved."""
import importlib.util
import os
import pickle
import sys

import numpy as np
import pytest

import ref_model_file

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("ref_pickle_under_test", os.path.join(ROOT, "llama.cl_amd", "llmops", "ref_pickle.py"))
ref_pickle = importlib.util.module_from_spec(spec)
spec.loader.exec_module(ref_pickle)


def _tiny(rng, G=128):
    blk = {32: 640, 128: 2176}[G]
    H, F, V, L = 256, 512, 320, 2

    def packed(N, K):
        return rng.integers(-128, 128, (N // 32, K // G, blk)).astype(np.int8)

    layers = []
    for _ in range(L):
        layers.append({
            "input_layernorm": (rng.standard_normal(H).astype(np.float32), 1e-5),
            "post_attention_layernorm": (rng.standard_normal(H).astype(np.float32), 1e-5),
            "self_attn.q_proj": (packed(H, H), H), "self_attn.k_proj": (packed(H, H), H),
            "self_attn.v_proj": (packed(H, H), H), "self_attn.o_proj": (packed(H, H), H),
            "mlp.gate_proj": (packed(F, H), F), "mlp.up_proj": (packed(F, H), F), "mlp.down_proj": (packed(H, F), H),
        })
    configs = {"layer_num": L, "head_num": 2, "head_size": 128, "hidden_size": H, "max_position_embeddings": 2048,
               "rotary_dims": 128, "rms_norm_eps": 1e-5}
    embed = (rng.integers(-127, 128, (V, H)).astype(np.int8), rng.random(V).astype(np.float32))
    norm = (rng.standard_normal(H).astype(np.float32), 1e-5)
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, 128, 2, dtype=np.float32) / 128))).astype(np.float32)
    return dict(configs=configs, embed=embed, layers=layers, norm=norm, lm_head=(packed(V, H), V), inv_freq=inv_freq)


@pytest.mark.parametrize("G", [32, 128])
def test_reads_structure_and_arrays_without_executing(tmp_path, G):
    rng = np.random.default_rng(G)
    m = _tiny(rng, G)
    path, marker = tmp_path / "saved_model.pkl", tmp_path / "executed"
    ref_model_file.write(path, marker_path=str(marker), **m)
    # the file really is dangerous for a plain loader ...
    with open(path, "rb") as f:
        raw = f.read()
    assert b"system" in raw and b"llmops" in raw and b"llmop_fc_q4a" in raw
    # ... and the reader neither runs it nor imports what it names
    before = set(sys.modules)
    state = ref_pickle.load(path)
    assert not marker.exists()
    assert not any(k.startswith("transformers") for k in set(sys.modules) - before)
    assert isinstance(state["tokenizer"], ref_pickle.Opaque) and state["tokenizer"].pad_token == "[PAD]"
    assert isinstance(state["tokenizer"].trap, ref_pickle.Opaque)
    t = ref_pickle.model_tensors(state)
    assert t["configs"] == m["configs"]
    assert np.array_equal(t["embed"]["weight"], m["embed"][0]) and np.array_equal(t["embed"]["scales"], m["embed"][1])
    assert np.array_equal(t["inv_freq"], m["inv_freq"])
    assert np.array_equal(t["lm_head"]["weight"], m["lm_head"][0]) and t["lm_head"]["N"] == m["lm_head"][1]
    assert len(t["layers"]) == len(m["layers"])
    for got, want in zip(t["layers"], m["layers"]):
        for name, v in want.items():
            assert np.array_equal(got[name]["weight"], v[0])
            assert (got[name]["eps"] if "layernorm" in name else got[name]["N"]) == v[1]
            if "layernorm" not in name:
                assert got[name]["weight"].dtype == np.int8 and got[name]["bias"] is None


def test_rejects_what_is_not_a_packed_tensor(tmp_path):
    rng = np.random.default_rng(1)
    m = _tiny(rng)
    m["layers"][0]["mlp.down_proj"] = (rng.standard_normal((4, 4, 100)).astype(np.float32), 4)
    path = tmp_path / "m.pkl"
    ref_model_file.write(path, **m)
    with pytest.raises(ValueError):
        ref_pickle.model_tensors(ref_pickle.load(path))


def test_plain_pickle_would_have_run_the_marker(tmp_path):
    """Control: the marker in the test file is live -- a plain loader that can resolve the names runs it.
    (Only the marker object itself is unpickled here, from a stream this test wrote.)"""
    marker = tmp_path / "executed"
    blob = pickle.dumps(ref_model_file._Marker(str(marker)))
    assert not marker.exists()
    pickle.loads(blob)
    assert marker.exists()
