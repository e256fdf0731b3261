"""The decode step at the width it is benchmarked at (hidden 4096, FFN 11008, 32 heads of 128, vocab 55296,
kv-len 2048, Q4_1 group 128; op order of chatllama/main.py:331-380): every launch of the fused plan checked
against the oracle on the GPU's own input to that launch, the fused plan against the reference's op sequence,
one captured graph against the eager step over successive positions, and a 32-layer run with property checks."""
import numpy as np
import pytest
import torch

from conftest import max_rel_err

pytestmark = pytest.mark.gpu

KV = 2048


def h(t):
    return t.detach().cpu().numpy()


def _model(layers, seed, plan="fused", device_rng=False, embed_rows=512):
    from llmops.decode import LLAMA_7B, LlamaDecoder
    cfg = dict(LLAMA_7B)
    cfg["layer_num"] = layers
    model = LlamaDecoder(cfg, group_k=128, seed=seed, plan=plan, embed_rows=embed_rows, device_rng=device_rng)
    # norm weights that are not all ones, so that a norm weight applied to the wrong element shows
    g = torch.Generator(device="cpu").manual_seed(seed + 100)
    for ops in model.layers:
        for name in ("input_layernorm", "post_attention_layernorm"):
            ops[name].weight.copy_((1.0 + 0.25 * torch.randn(cfg["hidden_size"], generator=g)).to(model.device))
    model.norm.weight.copy_((1.0 + 0.25 * torch.randn(cfg["hidden_size"], generator=g)).to(model.device))
    return model, cfg


def _cache(cfg, dtype=torch.float32, seed=0):
    from llmops.opset import KVCache
    kv = KVCache(cfg, 1, KV, dtype=dtype)
    g = torch.Generator(device="cuda").manual_seed(seed)
    kv.cache.copy_(torch.randn(kv.cache.shape, generator=g, device="cuda"))
    return kv


def _strip_sumsq(y):
    y = np.asarray(y, np.float64).reshape(-1, 32)
    return (y * y).sum(1)


def test_full_width_fused_plan_every_launch_vs_oracle(orc):
    """Two layers and the lm_head at full width, position 2047 of a 2048-row cache: each launch of the fused plan
    (q|k|v with the rmsnorm prologue and handed-over sums of squares; attention leaving chunk records; the o projection
    merging them, adding the residual and leaving sums of squares; gate|up with the rmsnorm prologue; the down
    projection taking silu(gate)*up on its way in; the lm_head with the final norm) against the oracle's ops applied
    to the GPU's own input of that launch."""
    import llmops
    model, cfg = _model(2, seed=11)
    H, F, V, eps = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"], cfg["rms_norm_eps"]
    kv = _cache(cfg, seed=1)
    inv = h(model.inv_freq)
    pos = KV - 1
    slots = torch.tensor([pos], dtype=torch.int32, device="cuda")
    ids = torch.tensor([[7]], dtype=torch.int64, device="cuda")
    hidden = model.embed_tokens(ids)
    assert np.array_equal(h(hidden), orc.embedding_q8c(h(ids), h(model.embed_tokens.weight), h(model.embed_tokens.scales)))
    sumsq = None
    worst = {}

    def close(name, got, want, tol):
        e = max_rel_err(h(got), want)
        worst[name] = max(worst.get(name, 0.0), e)
        assert e <= tol, (name, e)

    for i, ops in enumerate(model.layers):
        n1, n2 = ops["input_layernorm"], ops["post_attention_layernorm"]
        assert llmops.attention_records_supported(kv.cache) and model.stacked_gate_up
        # q|k|v: MODE rmsnorm (+ handed-over sums from the second layer on), 384 strips
        qkv = llmops.fc_Q4A_decode(hidden, ops["qkv_proj"].weight, 3 * H, norm=(n1.weight, n1.eps), sumsq_in=sumsq)
        x_n = orc.rmsnorm(h(hidden), h(n1.weight), eps)
        close("qkv", qkv, orc.fc(x_n, h(ops["qkv_proj"].weight), 3 * H), 1e-3)
        q, k, v = qkv[..., :H], qkv[..., H:2 * H], qkv[..., 2 * H:]
        q0, k0, v0 = h(q).copy(), h(k).copy(), h(v).copy()
        cache0 = h(kv.cache[2 * i:2 * i + 2])
        recs = llmops.attention_rope2_records(q, k, v, model.inv_freq, kv.cache, slots, pos, i)
        want_q, want_k, want_c = orc.attention(q0, k0, v0, inv, cache0, h(slots), pos, 0)
        close("k rotated", k, want_k, 1e-5)
        close("cache", kv.cache[2 * i:2 * i + 2], want_c, 1e-5)
        # o projection on the records: merge + residual + sums of squares, 128 strips
        attn, ss = llmops.fc_Q4A_decode(None, ops["o_proj"].weight, H, residual=hidden, want_sumsq=True, attn_records=recs)
        want_attn = orc.iadd(orc.fc(want_q, h(ops["o_proj"].weight), H), h(hidden))
        close("o(records)+residual", attn, want_attn, 1e-3)
        close("o sumsq", ss.reshape(-1), _strip_sumsq(h(attn)), 1e-5)
        # gate|up: rmsnorm from the handed-over sums, 688 strips
        gu = llmops.fc_Q4A_decode(attn, ops["gate_up_proj"].weight, 2 * F, norm=(n2.weight, n2.eps), sumsq_in=ss)
        x_n = orc.rmsnorm(h(attn), h(n2.weight), eps)
        close("gate|up", gu, orc.fc(x_n, h(ops["gate_up_proj"].weight), 2 * F), 1e-3)
        # down: silu(gate)*up on the way in, residual, sums of squares, two k-splits
        hidden_next, sumsq = llmops.fc_Q4A_decode(gu, ops["down_proj"].weight, H, residual=attn, want_sumsq=True, glu_in=True)
        gate, up = h(gu)[..., :F].copy(), h(gu)[..., F:].copy()
        act = orc.imul(up, orc.silu(gate))
        close("down+residual", hidden_next, orc.iadd(orc.fc(act, h(ops["down_proj"].weight), H), h(attn)), 1e-3)
        close("down sumsq", sumsq.reshape(-1), _strip_sumsq(h(hidden_next)), 1e-5)
        hidden = hidden_next
    # lm_head: final norm from the handed-over sums, 1728 strips
    logits = llmops.fc_Q4A_decode(hidden, model.lm_head.weight, V, norm=(model.norm.weight, model.norm.eps), sumsq_in=sumsq)
    x_n = orc.rmsnorm(h(hidden), h(model.norm.weight), eps)
    close("lm_head", logits, orc.fc(x_n, h(model.lm_head.weight), V), 1e-3)
    print("observed max rel err per launch:", {k_: float(f"{e:.2e}") for k_, e in worst.items()})
    # the contract is 1e-3 per op; observed on the MI355X: every launch within 1.1e-6 of the oracle
    assert max(worst.values()) <= 1e-5, worst


def test_full_width_fused_plan_vs_reference_plan_and_oracle(orc):
    """Same weights (same seed, same draw order) through the reference's op sequence (18 launches per layer) and
    through the fused plan (5 launches): logits of a 2-layer full-width step at position 2047, and both against the
    whole step evaluated by the oracle."""
    from test_decode_gpu import oracle_forward
    pos = KV - 1
    ids_h = np.array([[3]], np.int64)
    out = {}
    cfg = None
    for plan in ("reference", "fused"):
        model, cfg = _model(2, seed=12, plan=plan)
        kv = _cache(cfg, seed=2)
        if plan == "reference":
            want, cache_h = oracle_forward(orc, model, ids_h, h(kv.cache), np.array([pos], np.int32), pos, cfg=cfg)
        slots = torch.tensor([pos], dtype=torch.int32, device="cuda")
        logits = model.forward(torch.from_numpy(ids_h).cuda(), kv.cache, slots, pos)
        out[plan] = (h(logits), h(kv.cache))
        del model, kv
        torch.cuda.empty_cache()
    assert out["fused"][0].shape == (1, 1, cfg["vocab_size"])
    assert np.isfinite(out["fused"][0]).all()
    e_ref, e_fused = max_rel_err(out["reference"][0], want), max_rel_err(out["fused"][0], want)
    e_plans = max_rel_err(out["fused"][0], out["reference"][0])
    rms = lambda a, b: float(np.sqrt(np.mean((a.astype(np.float64) - b) ** 2)) / np.sqrt(np.mean(np.asarray(b, np.float64) ** 2)))
    r_ref, r_fused, r_plans = rms(out["reference"][0], want), rms(out["fused"][0], want), rms(out["fused"][0], out["reference"][0])
    print("logits max: reference plan vs oracle", e_ref, "fused plan vs oracle", e_fused, "fused vs reference plan", e_plans)
    print("logits rms: reference plan vs oracle", r_ref, "fused plan vs oracle", r_fused, "fused vs reference plan", r_plans)
    # End to end, any two evaluations drift apart up to the noise floor of the 8-bit activation quantization itself.
    # A 1e-6 difference flips a code now and then (step = amax/127); one flipped code moves an FC output by ~3e-4 of
    # its spread, which flips ~3 % of the next FC's codes, and after three or four FCs the two runs round to
    # independent codes: ~1 % of an output's spread per FC from then on.  Even the reference's own op sequence on
    # the GPU against the oracle shows it (observed over these 9 FCs: rms 2.4-4.9 % of the logits' rms, max 5 % of the
    # largest logit), so this test only bounds the drift; the per-launch test above carries the 1e-3 contract
    # (observed 1e-6).
    assert max(e_ref, e_fused, e_plans) <= 1.5e-1
    assert max(r_ref, r_fused, r_plans) <= 1e-1
    for plan in ("reference", "fused"):
        got = out[plan][1]
        assert np.abs(got[:2] - cache_h[:2]).max() <= 1e-4        # first layer: the new row's k, v are one FC deep
        assert np.abs(got[2:] - cache_h[2:]).max() <= 1.5e-1 * np.abs(cache_h[2:, ..., KV - 1, :]).max()   # second: drift as above
        assert np.array_equal(got[..., :KV - 1, :], cache_h[..., :KV - 1, :])                                # other rows untouched


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.float16])
def test_full_width_graph_equals_eager_over_positions(cache_dtype):
    """One captured graph of the 2-layer full-width step replayed at positions 2045, 2046, 2047 (and once more
    after the ring buffer wrapped, position 2048 into slot 0): bit-identical logits and cache to the eager step
    that reads the same device-side position."""
    model, cfg = _model(2, seed=13)
    kv = _cache(cfg, dtype=cache_dtype, seed=3)
    base = kv.cache.clone()
    dg = model.capture_decode(kv.cache, 0, 0)
    kv.cache.copy_(base)
    pos_t = torch.zeros(1, dtype=torch.int32, device="cuda")
    eager_cache = base.clone()
    for tok, slot, pos in ((5, 2045, 2045), (9, 2046, 2046), (2, 2047, 2047), (4, 0, 2048)):
        ids = torch.tensor([[tok]], dtype=torch.int64, device="cuda")
        slots = torch.tensor([slot], dtype=torch.int32, device="cuda")
        pos_t.fill_(pos)
        want = model.forward(ids, eager_cache, slots, pos_t).clone()
        logits = dg.step(tok, slot, pos)
        torch.cuda.synchronize()
        assert torch.isfinite(logits).all()
        assert torch.equal(logits, want), (tok, slot, pos)
        assert torch.equal(kv.cache, eager_cache), (tok, slot, pos)
        by_value = model.forward(ids, eager_cache.clone(), slots, pos)
        assert max_rel_err(h(logits), h(by_value)) <= 1e-4


def test_config5_all_32_layers_properties():
    """BASELINE config 5 as the benchmark times it: 32 layers, lm_head 55296, kv-len 2048, batch 1.  No oracle at
    this depth (drift); checked: logits finite and not constant, the captured graph replayed three times gives the
    eager step's logits and cache bit for bit, and only the new token's cache row changed in every layer."""
    model, cfg = _model(32, seed=5, device_rng=True)
    kv = _cache(cfg, seed=4)
    base = kv.cache.clone()
    pos = KV - 1
    ids = torch.tensor([[11]], dtype=torch.int64, device="cuda")
    slots = torch.tensor([pos], dtype=torch.int32, device="cuda")
    pos_t = torch.tensor([pos], dtype=torch.int32, device="cuda")
    want = model.forward(ids, kv.cache, slots, pos_t).clone()
    want_cache = kv.cache.clone()
    assert torch.isfinite(want).all() and float(want.std()) > 0
    changed = (want_cache != base).any(dim=-1)                       # [2L, B, H, maxlen]
    assert bool(changed[..., pos].all()) and not bool(changed[..., :pos].any())
    kv.cache.copy_(base)
    dg = model.capture_decode(kv.cache, 0, 0)
    for rep in range(3):
        kv.cache.copy_(base)
        logits = dg.step(11, pos, pos)
        torch.cuda.synchronize()
        assert torch.equal(logits, want), rep
        assert torch.equal(kv.cache, want_cache), rep
