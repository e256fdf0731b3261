"""GPU parity of rope / KV-cache update / attention and of the small neighbour ops.
fp32 outputs: max|err|/max|ref| <= 1e-3 against the reference-made golden vectors and the oracle."""
import numpy as np
import pytest
import torch

from conftest import load_golden, max_rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def ops():
    import llmops
    return llmops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy()


def run_attention(ops, g, cache_dtype=torch.float32, fn="attention_rope2"):
    q, k, v = dev(g["q"]), dev(g["k"]), dev(g["v"])
    cache = dev(g["cache"]).to(cache_dtype)
    getattr(ops, fn)(q, k, v, dev(g["inv_freq"]), cache, dev(g["slots"]), int(g["position_id"]), int(g["layer_id"]))
    return host(q), host(k), host(cache.float())


@pytest.mark.parametrize("name", ["attn_decode", "attn_decode_wrap", "attn_chunk", "attn_prefill"])
@pytest.mark.parametrize("fn", ["attention_rope2", "attention_rope"])
def test_attention_golden_fp32(ops, name, fn):
    g = load_golden(name + ".npz")
    out, k_rot, cache = run_attention(ops, g, fn=fn)
    assert max_rel_err(out, g["out"]) <= TOL
    assert max_rel_err(out, g["out"]) <= 1e-5
    assert np.abs(k_rot - g["k_rot"]).max() <= 1e-5          # k is left rotated in place
    assert np.abs(cache - g["cache_after"]).max() <= 1e-5
    layer = int(g["layer_id"])
    other = np.ones(cache.shape[0], bool)
    other[2 * layer:2 * layer + 2] = False
    assert np.array_equal(cache[other], g["cache"][other])   # other layers' planes untouched
    B, qL, HS = g["q"].shape
    H, S = cache.shape[2], cache.shape[4]
    for l, s in enumerate(g["slots"]):                        # rows written == rotated k / raw v, bit for bit
        assert np.array_equal(cache[2 * layer, :, :, s].reshape(B, HS), k_rot[:, l])
        assert np.array_equal(cache[2 * layer + 1, :, :, s].reshape(B, HS), g["v"][:, l])
    rows = np.ones(cache.shape[3], bool)
    rows[g["slots"]] = False
    assert np.array_equal(cache[2 * layer:2 * layer + 2][:, :, :, rows], g["cache"][2 * layer:2 * layer + 2][:, :, :, rows])


@pytest.mark.parametrize("name", ["attn_decode", "attn_chunk"])
def test_attention_fp16_cache(ops, orc, name):
    """fp16 KV cache is an extension: target = fp32 math on the fp16-rounded cache (new rows included)."""
    g = load_golden(name + ".npz")
    out, k_rot, cache = run_attention(ops, g, cache_dtype=torch.float16)
    g16 = dict(g)
    g16["cache"] = g["cache"].astype(np.float16).astype(np.float32)
    # the oracle writes fp32 k,v rows into the cache; round them as the fp16 cache does before attending
    _, k_ref, cache_ref = orc.attention(g["q"], g["k"], g["v"], g["inv_freq"], g16["cache"], g["slots"],
                                        int(g["position_id"]), int(g["layer_id"]))
    cache_ref = cache_ref.astype(np.float16).astype(np.float32)
    assert np.abs(cache - cache_ref).max() <= 2e-3           # one fp16 ulp at |x| < 4 on the rotated rows
    # attend over the rounded cache: re-run the oracle with the new rows already in place and k,v equal to them
    B, qL, HS = g["q"].shape
    layer = int(g["layer_id"])
    kr = np.stack([cache_ref[2 * layer, :, :, s].reshape(B, HS) for s in g["slots"]], 1)
    vr = np.stack([cache_ref[2 * layer + 1, :, :, s].reshape(B, HS) for s in g["slots"]], 1)
    # feed the already rotated q and zero frequencies so the oracle leaves q,k as given
    zero_f = np.zeros_like(g["inv_freq"])
    q_in = _rotated_q(orc, g)
    want = orc.attention(q_in, kr, vr, zero_f, cache_ref, g["slots"], int(g["position_id"]), layer)[0]
    assert max_rel_err(out, want) <= TOL


def _rotated_q(orc, g):
    B, qL, HS = g["q"].shape
    H = g["cache"].shape[2]
    S = HS // H
    q4 = g["q"].reshape(B, qL, H, S).transpose(0, 2, 1, 3).copy()
    return orc.rope(q4, g["inv_freq"], int(g["position_id"])).transpose(0, 2, 1, 3).reshape(B, qL, HS).copy()


@pytest.mark.parametrize("kv", [256, 2048])
@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.float16])
def test_attention_config4_vs_oracle(ops, orc, kv, cache_dtype):
    """BASELINE config 4: 32 heads x 128, rope base 10000 over 128 dims, one query token, kv-len 256 / 2048."""
    rng = np.random.default_rng(kv)
    B, H, S, layers = 1, 32, 128, 2
    q, k, v = (rng.standard_normal((B, 1, H * S)).astype(np.float32) for _ in range(3))
    cache = rng.standard_normal((2 * layers, B, H, kv, S)).astype(np.float32)
    if cache_dtype == torch.float16:
        cache = cache.astype(np.float16).astype(np.float32)
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, S, 2, dtype=np.float32) / np.float32(S)))).astype(np.float32)
    slots = np.array([kv - 1], np.int32)
    g = dict(q=q, k=k, v=v, cache=cache, inv_freq=inv_freq, slots=slots, position_id=kv - 1, layer_id=1)
    out, k_rot, cache_after = run_attention(ops, g, cache_dtype=cache_dtype)
    want, k_ref, cache_ref = orc.attention(q, k, v, inv_freq, cache, slots, kv - 1, 1)
    tol = TOL if cache_dtype == torch.float32 else 3e-3   # fp16 rounding of the one new K/V row (extension, no reference)
    assert max_rel_err(out, want) <= tol
    if cache_dtype == torch.float32:
        assert max_rel_err(out, want) <= 1e-5
        assert np.abs(k_rot - k_ref).max() <= 1e-4        # position 2047: fp32 sin/cos argument reduction differs slightly
        assert np.abs(cache_after - cache_ref).max() <= 1e-4


def test_attention_kvlen_sweep(ops, orc):
    """Odd and tiny kv lengths (the reference's own sweep uses 30+1, 31+1, 1022..1026) and every chunking."""
    rng = np.random.default_rng(3)
    B, H, S, maxlen = 1, 4, 128, 1100
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, 64, 2, dtype=np.float32) / np.float32(64)))).astype(np.float32)
    cache = rng.standard_normal((2, B, H, maxlen, S)).astype(np.float32)
    for past in (0, 1, 15, 16, 30, 31, 63, 64, 65, 511, 1022, 1023, 1025):
        q, k, v = (rng.standard_normal((B, 1, H * S)).astype(np.float32) for _ in range(3))
        slots = np.array([past], np.int32)
        g = dict(q=q, k=k, v=v, cache=cache, inv_freq=inv_freq, slots=slots, position_id=past, layer_id=0)
        out, _, _ = run_attention(ops, g)
        want = orc.attention(q, k, v, inv_freq, cache, slots, past, 0)[0]
        assert max_rel_err(out, want) <= 1e-5, past


def test_attention_prefill_chunks_vs_oracle(ops, orc):
    rng = np.random.default_rng(4)
    B, H, S, maxlen = 2, 3, 128, 96
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, S, 2, dtype=np.float32) / np.float32(S)))).astype(np.float32)
    cache = rng.standard_normal((4, B, H, maxlen, S)).astype(np.float32)
    for past, qL in ((0, 33), (40, 7), (90, 20)):   # the last one wraps the ring buffer
        q, k, v = (rng.standard_normal((B, qL, H * S)).astype(np.float32) for _ in range(3))
        slots = ((past + np.arange(qL)) % maxlen).astype(np.int32)
        g = dict(q=q, k=k, v=v, cache=cache, inv_freq=inv_freq, slots=slots, position_id=past, layer_id=1)
        out, k_rot, cache_after = run_attention(ops, g)
        want, k_ref, cache_ref = orc.attention(q, k, v, inv_freq, cache, slots, past, 1)
        assert max_rel_err(out, want) <= 1e-5, (past, qL)
        assert np.abs(cache_after - cache_ref).max() <= 1e-5


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.float16])
def test_attention_prefill_tiled_vs_oracle(ops, orc, cache_dtype):
    """Chunks of 32 and more query tokens take the tiled MFMA kernel: several query tiles and waves,
    tiles that are skipped by the in-chunk mask, a chunk that follows earlier context, a chunk that
    wraps the ring buffer, and kv lengths that are not multiples of the 32-row tile."""
    rng = np.random.default_rng(9)
    B, H, S, maxlen = 2, 3, 128, 300
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, S, 2, dtype=np.float32) / np.float32(S)))).astype(np.float32)
    cache = rng.standard_normal((2, B, H, maxlen, S)).astype(np.float32)
    if cache_dtype == torch.float16:
        cache = cache.astype(np.float16).astype(np.float32)
    for past, qL in ((0, 32), (0, 200), (37, 131), (250, 90), (0, 300)):   # (250, 90) wraps the ring buffer
        q, k, v = (rng.standard_normal((B, qL, H * S)).astype(np.float32) for _ in range(3))
        slots = ((past + np.arange(qL)) % maxlen).astype(np.int32)
        g = dict(q=q, k=k, v=v, cache=cache, inv_freq=inv_freq, slots=slots, position_id=past, layer_id=0)
        out, k_rot, cache_after = run_attention(ops, g, cache_dtype=cache_dtype)
        if cache_dtype == torch.float16:   # target: fp32 math on the fp16-rounded cache, new rows included
            kr = orc.rope(k.reshape(B, qL, H, S).transpose(0, 2, 1, 3).copy(), inv_freq, past)
            c16 = cache.copy()
            for l, sl in enumerate(slots):
                c16[0, :, :, sl] = kr[:, :, l].astype(np.float16).astype(np.float32)
                c16[1, :, :, sl] = v[:, l].reshape(B, H, S).astype(np.float16).astype(np.float32)
            want = _attend_cache(orc, q, inv_freq, c16, slots, past, maxlen)
            assert max_rel_err(out, want) <= TOL, (past, qL)
        else:
            want, k_ref, cache_ref = orc.attention(q, k, v, inv_freq, cache, slots, past, 0)
            assert max_rel_err(out, want) <= 1e-4, (past, qL)
            assert np.abs(cache_after - cache_ref).max() <= 1e-5


@pytest.mark.parametrize("order", ["reversed", "shuffled"])
def test_attention_prefill_tiled_with_slots_in_any_order(ops, orc, order):
    """The tiled prompt kernel finds what a query may see from the slot -> token map alone: the chunk's rows are
    written to slots in reversed / shuffled order among rows of earlier context (so the tile with the chunk's last
    tokens comes first, tiles mix visible and masked rows, and the last row a query tile may see is not where a
    prompt written front to back would have it)."""
    rng = np.random.default_rng(21 + len(order))
    B, H, S, maxlen, past, qL = 1, 2, 128, 400, 100, 260
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, S, 2, dtype=np.float32) / np.float32(S)))).astype(np.float32)
    cache = rng.standard_normal((2, B, H, maxlen, S)).astype(np.float32)
    free = np.arange(past, past + qL)
    slots = (free[::-1] if order == "reversed" else rng.permutation(free)).astype(np.int32)
    q, k, v = (rng.standard_normal((B, qL, H * S)).astype(np.float32) for _ in range(3))
    g = dict(q=q, k=k, v=v, cache=cache, inv_freq=inv_freq, slots=slots, position_id=past, layer_id=0)
    out, k_rot, cache_after = run_attention(ops, g)
    want, k_ref, cache_ref = orc.attention(q, k, v, inv_freq, cache, slots, past, 0)
    assert max_rel_err(out, want) <= 1e-5
    assert np.abs(cache_after - cache_ref).max() <= 1e-5


def _attend_cache(orc, q, inv_freq, cache, slots, past, maxlen):
    """fp64 attention of the rotated queries over a finished cache with the reference's in-chunk mask."""
    B, qL, HS = q.shape
    H, S = cache.shape[2], cache.shape[4]
    qr = orc.rope(q.reshape(B, qL, H, S).transpose(0, 2, 1, 3).copy(), inv_freq, past).astype(np.float64)
    kv_len = min(past + qL, maxlen)
    K, V = cache[0, :, :, :kv_len].astype(np.float64), cache[1, :, :, :kv_len].astype(np.float64)
    w = np.einsum("bhqs,bhks->bhqk", qr, K) / np.sqrt(S)
    for pq in range(qL):
        for later in range(pq + 1, qL):
            if slots[later] < kv_len:
                w[:, :, pq, slots[later]] = -np.inf
    w = np.exp(w - w.max(-1, keepdims=True))
    w /= w.sum(-1, keepdims=True)
    o = np.einsum("bhqk,bhks->bhqs", w, V)
    return o.transpose(0, 2, 1, 3).reshape(B, qL, HS)


def test_rope_and_softmax_golden(ops):
    g = load_golden("misc.npz")
    x = dev(g["rope_x"])
    ops.rope_embed(x, dev(g["rope_inv_freq"]), 16)
    assert np.abs(host(x) - g["rope_out"]).max() <= 1e-5     # ops/test_ops.py:211
    assert np.array_equal(host(x)[..., 64:], g["rope_x"][..., 64:])
    s = dev(g["sm_in"])
    ops.softmax(s)
    assert np.allclose(host(s), g["sm"], rtol=1e-5, atol=1e-8)
    lit = dev(g["lit"][None])
    ops.softmax(lit)
    assert np.allclose(host(lit)[0], g["sm_lit"], rtol=1e-5, atol=1e-8) and host(lit)[0, -1] == 0.0
    big = torch.rand(7, 12, 3, 69, device="cuda") - 0.5      # ops/test_ops.py:170
    want = torch.softmax(big, -1)
    ops.softmax(big)
    assert torch.allclose(big, want, rtol=1e-5, atol=1e-8)


def test_neighbours_golden(ops):
    g = load_golden("misc.npz")
    x = dev(g["x"])
    ops.rmsnorm(x, dev(g["wn"]), 1e-5)
    assert np.allclose(host(x), g["rms"], rtol=1e-5, atol=1e-6)
    x = dev(g["x"])
    ops.itrans(x, "silu")
    assert np.allclose(host(x), g["silu"], rtol=1e-3, atol=1e-6)   # the reference itself is ~3e-4 off (rcpps)
    assert np.allclose(host(x), g["x"] / (1 + np.exp(-g["x"].astype(np.float64))), rtol=1e-6, atol=1e-7)
    a = dev(g["x"])
    ops.iadd(a, dev(g["x"][:, ::-1].copy()))
    assert np.array_equal(host(a), g["iadd"])
    a = dev(g["x"])
    ops.imul(a, dev(g["wn"]))
    assert np.array_equal(host(a), g["imul_row"])
    q, s = ops.embedding_q8c_quant_w(dev(g["emb"]))
    assert np.array_equal(host(q), g["eq"]) and np.array_equal(host(s).view(np.uint32), g["es"].view(np.uint32))
    out = ops.empty(2, 3, 64)
    ops.embedding_q8c(out, dev(g["ids"]), q, s)
    assert np.array_equal(host(out), g["emb_out"])
    out = ops.empty(2, 3, 64)
    ops.embedding(out, dev(g["ids"]), dev(g["emb"]))
    assert np.array_equal(host(out), g["emb"][g["ids"]])
    with pytest.raises(RuntimeError):
        ops.itrans(x, "gelu")


@pytest.mark.parametrize("V,E,n", [(50, 30, 7), (9, 4096, 1), (300, 5000, 3), (20, 1026, 4)])
def test_embedding_q8c_vs_oracle(ops, orc, V, E, n):
    """embedding_q8c lookup, bit-equal to the oracle: row lengths that take the four-codes-per-thread kernel
    (a multiple of 4, one or several workgroups per row) and ones that take the byte-wise one."""
    rng = np.random.default_rng(V + E)
    w = rng.standard_normal((V, E)).astype(np.float32)
    ids = rng.integers(0, V, size=(1, n)).astype(np.int64)
    q, s = orc.embedding_q8c_quant_w(w)
    want = orc.embedding_q8c(ids, q, s)
    out = ops.empty(1, n, E)
    ops.embedding_q8c(out, dev(ids), dev(q), dev(s))
    assert np.array_equal(host(out), want)


def test_fused_neighbours_vs_oracle(ops, orc):
    """Extensions used by the decode step: rmsnorm_out == clone+rmsnorm, silu_mul == silu then imul,
    fc_Q4A(residual=) == fc_Q4A then iadd."""
    rng = np.random.default_rng(9)
    for rows, hidden in ((1, 4096), (5, 4096), (2, 11008), (3, 1000)):
        x = rng.standard_normal((1, rows, hidden)).astype(np.float32)
        w = rng.standard_normal(hidden).astype(np.float32)
        dx = dev(x)
        out = ops.rmsnorm_out(dx, dev(w), 1e-5)
        assert np.array_equal(host(dx), x)
        assert np.allclose(host(out), orc.rmsnorm(x, w, 1e-5), rtol=1e-5, atol=1e-6)
        ops.rmsnorm(dx, dev(w), 1e-5)
        assert np.array_equal(host(dx), host(out))
    gu = rng.standard_normal((1, 3, 2 * 11008)).astype(np.float32)
    want = orc.imul(gu[..., 11008:].copy(), orc.silu(gu[..., :11008].copy()))
    assert np.allclose(host(ops.silu_mul(dev(gu))), want, rtol=1e-6, atol=1e-7)
    for rows, N, K in ((1, 4096, 4096), (1, 4096, 11008), (3, 96, 1024), (20, 96, 1024)):
        w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
        x = rng.standard_normal((1, rows, K)).astype(np.float32)
        res = rng.standard_normal((1, rows, N)).astype(np.float32)
        wq = orc.quant_w(w, 128)
        got = host(ops.fc_Q4A(dev(x), dev(wq), N, residual=dev(res)))
        want = orc.iadd(orc.fc(x, wq, N), res)
        assert max_rel_err(got, want) <= 1e-5


# ---- mm_qk / mm_qk42 / mm_qk81 / mm_qk24: the reference's benchmark names for the scaled q.k product ---------
@pytest.mark.parametrize("B,H,qL,kv,S", [(1, 2, 1, 7, 16), (2, 3, 5, 33, 128), (1, 4, 37, 130, 64), (1, 32, 8, 2048, 128),
                                          (1, 2, 129, 257, 128)])
def test_mm_qk_against_oracle(ops, orc, B, H, qL, kv, S):
    rng = np.random.default_rng(qL * 7 + kv)
    q = rng.random((B, qL, H * S), dtype=np.float32)              # ops/perf_ops.py:165-166
    kc = rng.random((B, H, kv, S), dtype=np.float32)
    want = orc.mm_qk(q, kc)
    for name in ("mm_qk", "mm_qk81", "mm_qk24"):
        got = host(getattr(ops, name)(dev(q), dev(kc)))
        assert got.shape == (B, H, qL, kv)
        assert max_rel_err(got, want) <= 1e-5, name
    # mm_qk42: [B,H,qL,S] query, caller's output, cache plane longer than the rows asked for
    q_bhqs = np.ascontiguousarray(q.reshape(B, qL, H, S).transpose(0, 2, 1, 3))
    part = max(1, kv - 3)
    out = torch.full((B, H, qL, part), float("nan"), device="cuda")
    assert ops.mm_qk42(dev(q_bhqs), dev(kc), out) is None
    assert max_rel_err(host(out), orc.mm_qk(q_bhqs, kc, kvLen=part, q_is_bhqs=True)) <= 1e-5
    assert np.isfinite(host(out)).all()                           # every element of the caller's buffer was written


def test_mm_qk_rejects_what_the_reference_asserts(ops):
    q = torch.zeros(1, 4, 2 * 12, device="cuda")
    with pytest.raises(RuntimeError):                              # S % 8 (ops/op_attn.hpp:205)
        ops.mm_qk(q, torch.zeros(1, 2, 5, 12, device="cuda"))
    with pytest.raises(RuntimeError):                              # kcache.size(-4) == B (ops/op_attn.hpp:154)
        ops.mm_qk(torch.zeros(1, 4, 32, device="cuda"), torch.zeros(2, 2, 5, 16, device="cuda"))
    with pytest.raises(RuntimeError):
        ops.mm_qk(torch.zeros(1, 4, 32), torch.zeros(1, 2, 5, 16))  # host tensors: there is no CPU path


def _prefill_case(ops, orc, rng, past, qL, maxlen, half, heads, H=32, S=128):
    """attention over H heads on the device; the oracle on the sampled `heads` (heads are independent)"""
    B = 1
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, 2 * half, 2, dtype=np.float32) / np.float32(2 * half)))).astype(np.float32)
    cache = rng.standard_normal((2, B, H, maxlen, S)).astype(np.float32)
    q, k, v = (rng.standard_normal((B, qL, H * S)).astype(np.float32) for _ in range(3))
    slots = ((past + np.arange(qL)) % maxlen).astype(np.int32)
    g = dict(q=q, k=k, v=v, cache=cache, inv_freq=inv_freq, slots=slots, position_id=past, layer_id=0)
    out, k_rot, cache_after = run_attention(ops, g)
    pick = lambda t: np.ascontiguousarray(t.reshape(B, qL, H, S)[:, :, heads].reshape(B, qL, len(heads) * S))
    want, k_ref, cache_ref = orc.attention(pick(q), pick(k), pick(v), inv_freq, np.ascontiguousarray(cache[:, :, heads]),
                                           slots, past, 0)
    assert max_rel_err(pick(out), want) <= 1e-4, (past, qL, half)
    assert np.abs(pick(k_rot) - k_ref).max() <= 1e-5
    assert np.abs(cache_after[:, :, heads] - cache_ref).max() <= 1e-5
    assert np.isfinite(out).all()


@pytest.mark.parametrize("scale_q,scale_kv", [(1.0, 1.0), (4.0, 0.25), (1e-3, 1e-3), (0.05, 300.0)])
def test_attention_prefill_two_halves_arithmetic_over_a_wide_range(ops, orc, scale_q, scale_kv):
    """The prompt kernel carries fp32 operands as two fp16 halves (22 bits) and multiplies them on the fp16
    matrix cores.  Inputs whose magnitudes are far from 1 -- sharp softmaxes (large q*k), values whose low halves
    fall into the fp16 denormals (1e-3), cache rows in the hundreds, a few outliers 50 times the rest -- stay
    within the contract of 1e-3 of the largest output; what is observed is asserted: 1e-5, as for inputs of
    order 1, except where logits of magnitude ~100 meet cache values up to 6e4 (the last case: the 2^-22 of every
    product then shows in the exponent of the softmax, observed 3e-5)."""
    rng = np.random.default_rng(11)
    B, H, S, qL, past, maxlen, half = 1, 4, 128, 200, 90, 512, 64
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, 2 * half, 2, dtype=np.float32) / np.float32(2 * half)))).astype(np.float32)
    cache = (rng.standard_normal((2, B, H, maxlen, S)) * scale_kv).astype(np.float32)
    q = (rng.standard_normal((B, qL, H * S)) * scale_q).astype(np.float32)
    k = (rng.standard_normal((B, qL, H * S)) * scale_kv).astype(np.float32)
    v = (rng.standard_normal((B, qL, H * S)) * scale_kv).astype(np.float32)
    for t in (q, k, v):
        t[0, ::17, ::29] *= 50.0  # outliers
    cache[:, 0, :, ::13, ::31] *= 50.0
    slots = ((past + np.arange(qL)) % maxlen).astype(np.int32)
    g = dict(q=q, k=k, v=v, cache=cache, inv_freq=inv_freq, slots=slots, position_id=past, layer_id=0)
    out, k_rot, cache_after = run_attention(ops, g)
    want, k_ref, cache_ref = orc.attention(q, k, v, inv_freq, cache, slots, past, 0)
    assert np.isfinite(out).all()
    err = max_rel_err(out, want)
    assert err <= 1e-3
    assert err <= (1e-4 if scale_kv > 100 else 1e-5), err


@pytest.mark.parametrize("past,qL,half", [(0, 1022, 32), (0, 1023, 32), (0, 1024, 32), (0, 1025, 32), (0, 1026, 32),
                                          (0, 1024, 64), (0, 2048, 32), (0, 2048, 64), (0, 128, 64), (0, 512, 64)])
def test_attention_prefill_at_the_reference_sweep_sizes(ops, orc, past, qL, half):
    """The accuracy sweep of the reference's perf script (ops/perf_ops.py:83-100,284-292: 32 heads, head size 128,
    rotary_dims 64, first chunk of 1022..1026 tokens) and the chunk lengths the benchmark publishes (128, 512,
    2048 tokens, full rotary), against the oracle on sampled heads."""
    rng = np.random.default_rng(qL + half)
    _prefill_case(ops, orc, rng, past, qL, 2048, half, heads=[0, 13, 31])


def test_attention_prefill_long_chunk_wrapping_the_ring(ops, orc):
    """a 1024-token chunk whose slots wrap around a cache of 2048 rows that is already full"""
    rng = np.random.default_rng(77)
    _prefill_case(ops, orc, rng, 1500, 1024, 2048, 32, heads=[5, 30])


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.float16])
def test_decode_attention_every_chunking_and_device_position(ops, orc, cache_dtype):
    """Decode attention (one query token) with every chunk size forced in turn and with the position read from
    device memory (the launch is then sized for the whole cache
    and chunks beyond the current length leave at once): all against the oracle, at kv lengths around the
    chunk and tile edges.  The new row's slot lies inside, at the end of, and beyond the attended rows."""
    from llmops import _lib
    lib = _lib.load()
    rng = np.random.default_rng(12)
    B, H, S, maxlen = 1, 5, 128, 1100
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, 64, 2, dtype=np.float32) / np.float32(64)))).astype(np.float32)
    cache0 = rng.standard_normal((2, B, H, maxlen, S)).astype(np.float32)
    if cache_dtype == torch.float16:
        cache0 = cache0.astype(np.float16).astype(np.float32)
    plans = [0] + list((4, 8, 16) if cache_dtype == torch.float32 else (8, 16, 32))
    tol = 1e-5 if cache_dtype == torch.float32 else 3e-3   # fp16: rounding of the one new row (extension, no reference)
    try:
        for kv in (1, 2, 17, 64, 65, 255, 256, 257, 511, 512, 513, 1025, 1100):
            q, k, v = (rng.standard_normal((B, 1, H * S)).astype(np.float32) for _ in range(3))
            pos = kv - 1
            slot = pos if kv % 2 else (pos * 7) % kv          # odd lengths: the last row; even: somewhere inside
            slots = np.array([slot], np.int32)
            want, k_ref, cache_ref = orc.attention(q, k, v, inv_freq, cache0, slots, pos, 0)
            if cache_dtype == torch.float16:
                c16 = cache_ref.astype(np.float16).astype(np.float32)
                want = _attend_cache(orc, q, inv_freq, c16, slots, pos, maxlen)
            for pw in plans:
                lib.llmops_test_attn_set_decode_plan(pw)
                for dev_pos in (False, True):
                    tq, tk, tc = dev(q), dev(k), dev(cache0).to(cache_dtype)
                    p = torch.tensor([pos], dtype=torch.int32, device="cuda") if dev_pos else pos
                    ops.attention_rope2(tq, tk, dev(v), dev(inv_freq), tc, dev(slots), p, 0)
                    assert max_rel_err(host(tq), want) <= tol, (kv, pw, dev_pos)
                    if cache_dtype == torch.float32:
                        assert np.abs(host(tk) - k_ref).max() <= 1e-5
                        assert np.abs(host(tc) - cache_ref).max() <= 1e-5
    finally:
        lib.llmops_test_attn_set_decode_plan(0)


@pytest.mark.parametrize("cache_dtype,maxlen", [(torch.float32, 2048), (torch.float32, 700), (torch.float16, 2048), (torch.float16, 4096)])
def test_attention_records_merged_by_the_o_projection(ops, orc, cache_dtype, maxlen):
    """Decode attention that hands its split-KV chunk records to the o projection (the merge runs on the FC's input
    side): attention_rope2_records + fc_Q4A_decode(attn_records=...) against attention_rope2 + fc_Q4A_decode on
    the same inputs.  Three layers of checks, because two evaluations of the attention output that differ in the
    last bit may quantize an activation on a rounding boundary to neighbouring codes:
    (1) the records, merged on the host in fp64, equal the unfused attention output to 1e-5;
    (2) what the FC kernel itself merged and quantized (its dump build): scales equal to rounding, codes equal but
        for a handful of +-1 boundary cases, and its int32 sums exactly the integer product of ITS codes;
    (3) the outputs agree to 1e-2 and, at selected lengths, with the oracle's attention + FC to the same bar."""
    import ctypes
    from llmops import _lib
    lib = _lib.load()
    rng = np.random.default_rng(31)
    B, H, S, G = 1, 32, 128, 128
    N = K = H * S
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, S, 2, dtype=np.float32) / np.float32(S)))).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    wq = ops.offline_FC_quant_Q4A(dev(w), G)
    pw = host(wq)
    Ng, Kg, _ = pw.shape
    cache0 = rng.standard_normal((2, B, H, maxlen, S)).astype(np.float32)
    if cache_dtype == torch.float16:
        cache0 = cache0.astype(np.float16).astype(np.float32)
    res = rng.standard_normal((1, 1, N)).astype(np.float32)
    kvs = [k_ for k_ in (1, 100, 256, 257, 512, 700, 1024, 2047, 2048, 3000, 4096) if k_ <= maxlen]
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    for kv in kvs:
        q, k, v = (rng.standard_normal((B, 1, H * S)).astype(np.float32) for _ in range(3))
        pos, slots = kv - 1, np.array([kv - 1], np.int32)
        tq, tk, tc = dev(q), dev(k), dev(cache0).to(cache_dtype)
        ops.attention_rope2(tq, tk, dev(v), dev(inv_freq), tc, dev(slots), pos, 0)       # unfused
        att = host(tq)
        want_y, want_ss = ops.fc_Q4A_decode(tq, wq, N, residual=dev(res), want_sumsq=True)
        for dev_pos in (False, True):
            fq, fk, fc = dev(q), dev(k), dev(cache0).to(cache_dtype)
            p = torch.tensor([pos], dtype=torch.int32, device="cuda") if dev_pos else pos
            recs = ops.attention_rope2_records(fq, fk, dev(v), dev(inv_freq), fc, dev(slots), p, 0)
            assert torch.equal(fk, tk) and torch.equal(fc, tc)              # k rotated, cache updated alike
            assert np.array_equal(host(fq), q)                              # q is left as it came in
            # (1) the records themselves (every one of recs.chunks was written; empty ones have sum 0)
            st, ou = host(recs.stats)[:, :recs.chunks].astype(np.float64), host(recs.outs)[:, :recs.chunks].astype(np.float64)
            m, sm = st[..., 0], st[..., 1]
            wgt = np.where(sm > 0, np.exp(m - np.where(sm > 0, m, -np.inf).max(1, keepdims=True)), 0.0)
            merged = ((wgt[..., None] * ou).sum(1) / (wgt * sm).sum(1, keepdims=True)).reshape(1, K)
            assert max_rel_err(merged, att.reshape(1, K)) <= (1e-5 if cache_dtype == torch.float32 else 3e-3), (kv, dev_pos)
            # (2) the FC kernel's own merge + quantization + integer core
            y = torch.empty((1, N), dtype=torch.float32, device="cuda")
            xq = torch.empty((1, K), dtype=torch.int8, device="cuda")
            xd, gs = torch.empty((1, Kg), dtype=torch.float32, device="cuda"), torch.empty((1, Kg), dtype=torch.float32, device="cuda")
            acc = torch.empty((1, Ng * 32, Kg), dtype=torch.int32, device="cuda")
            ws = ops._workspace(y.device, lib.llmops_fc_Q4A_workspace_bytes(1, K, Ng, Kg, G))
            _lib.check(lib.llmops_test_fc_decode_attn_dump(P(recs.stats), P(recs.outs), recs.chunks, H, P(wq), Ng, Kg, N, P(y), P(xq),
                                                           P(xd), P(gs), P(acc), P(ws), ws.numel(),
                                                           ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
            oq, od, og = orc.quant_x(merged.astype(np.float32), G)
            assert np.abs(host(xd) / od - 1.0).max() <= 1e-6
            diff = host(xq).astype(np.int32) - oq.astype(np.int32)
            assert np.abs(diff).max() <= 1 and np.count_nonzero(diff) <= 8, (kv, np.count_nonzero(diff))
            assert np.array_equal(host(acc), orc.fc_partials(host(xq), pw))
            # ... and its fold: y = sum over k-groups of (d*dx)*acc + m*gsum (ops/op_fc.hpp:381-412) evaluated in
            # fp64 on the kernel's OWN scales, group sums and int32 sums
            blocks = np.ascontiguousarray(pw).view(np.uint8)
            wd = blocks[:, :, G // 8 * 128:G // 8 * 128 + 64].copy().view(np.float16).astype(np.float64)      # [Ng, Kg, 32]
            wm = blocks[:, :, G // 8 * 128 + 64:].copy().view(np.float16).astype(np.float64)
            wd, wm = wd.transpose(0, 2, 1).reshape(Ng * 32, Kg), wm.transpose(0, 2, 1).reshape(Ng * 32, Kg)
            dx, sums = host(xd).astype(np.float64)[0], host(gs).astype(np.float64)[0]
            folded = (wd * dx[None, :] * host(acc)[0].astype(np.float64) + wm * sums[None, :]).sum(1)
            assert max_rel_err(host(y)[0], folded[:N]) <= 1e-5, (kv, dev_pos)
            # (3) outputs
            yf, ss = ops.fc_Q4A_decode(None, wq, N, residual=dev(res), want_sumsq=True, attn_records=recs)
            assert np.array_equal(host(yf)[0], host(y) + res[0])            # production build == dump build (+ residual)
            assert max_rel_err(host(yf), host(want_y)) <= 1e-2, (kv, dev_pos)
            assert max_rel_err(host(ss), host(want_ss)) <= 2e-2
        if cache_dtype == torch.float32 and kv in (257, 2048):              # and the oracle's two ops
            oatt, _, _ = orc.attention(q, k, v, inv_freq, cache0, slots, pos, 0)
            assert max_rel_err(host(yf), orc.fc(oatt, pw, N) + res) <= 1e-2


def test_decode_attention_with_more_than_65535_heads_in_all(ops, orc):
    """One query token for 2050 sequences of 32 heads: B*H exceeds what the decode kernels' (chunk, head) grid can
    index, so the call is served by the general kernels (the reference has no such limit, ops/op_attn.hpp:976)."""
    rng = np.random.default_rng(77)
    B, H, S, maxlen, kv = 2050, 32, 128, 8, 6
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, S, 2, dtype=np.float32) / np.float32(S)))).astype(np.float32)
    q, k, v = (rng.standard_normal((B, 1, H * S)).astype(np.float32) for _ in range(3))
    cache = rng.standard_normal((2, B, H, maxlen, S)).astype(np.float32)
    slots = np.array([kv - 1], np.int32)
    tq, tk, tc = dev(q), dev(k), dev(cache)
    ops.attention_rope2(tq, tk, dev(v), dev(inv_freq), tc, dev(slots), kv - 1, 0)
    sel = [0, 1, 1023, 2047, 2048, 2049]                       # the oracle on a few sequences (they are independent)
    want, k_ref, cache_ref = orc.attention(q[sel], k[sel], v[sel], inv_freq, np.ascontiguousarray(cache[:, sel]), slots, kv - 1, 0)
    assert max_rel_err(host(tq)[sel], want) <= 1e-5
    assert np.abs(host(tk)[sel] - k_ref).max() <= 1e-5
    assert np.abs(host(tc)[:, sel] - cache_ref).max() <= 1e-5
    assert torch.isfinite(tq).all()
