"""CPU checks that pin the oracle (oracle/llmops_oracle.c) before anything is compared with it:
committed golden vectors made by the reference's own kernels, the reference build itself where
oracle/_ref exists, closed forms, brute force and textbook formulas."""
import math

import numpy as np
import pytest

import oracle
from conftest import load_golden, max_rel_err


def _ref(G, fresh=False):
    if not oracle.Reference.available(G):
        pytest.skip("oracle/_ref not built on this machine")
    return oracle.Reference(G, fresh=fresh)


# ---- fp16 conversion ----------------------------------------------------------------------------
def test_fp16_to_fp32_all_halves(orc):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = orc.fp16_bits_to_fp32(h)
    fin = ~np.isnan(want)
    assert np.array_equal(got[fin].view(np.uint32), want[fin].view(np.uint32))
    assert np.isnan(got[~fin]).all()


def test_fp32_to_fp16_rne(orc):
    rng = np.random.default_rng(0)
    f16 = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    f16 = f16[np.isfinite(f16)]
    mids = ((f16[:-1].astype(np.float64) + np.sort(f16)[1:].astype(np.float64)) / 2).astype(np.float32)
    vals = np.concatenate([rng.standard_normal(5000).astype(np.float32) * s for s in (1e-8, 1e-6, 1e-4, 1e-2, 1, 100, 7e4)]
                          + [f16[::7], np.nextafter(f16[::7], np.float32(np.inf)), np.nextafter(f16[::7], np.float32(-np.inf)),
                             np.sort(f16)[:-1][::5] / 2 + np.sort(f16)[1:][::5] / 2, mids[::11],
                             np.array([65504, 65519.99, 65520, 1e30, 2.0 ** -25, 2.0 ** -24, 1.5 * 2.0 ** -25, 0.0, -0.0], np.float32)])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.fp32_to_fp16_bits(vals), want)


# ---- weight packing -----------------------------------------------------------------------------
@pytest.mark.parametrize("G", [32, 128])
def test_pack_matches_golden(orc, G):
    g = load_golden(f"fc_g{G}.npz")
    assert np.array_equal(orc.quant_w(g["w"], G), g["wq"])
    assert np.array_equal(orc.dequant_w(g["wq"]).view(np.uint32), g["dq"].view(np.uint32))


@pytest.mark.parametrize("G", [32, 128])
def test_pack_layout_bruteforce(orc, G):
    """byte = (k>>3)*128 + n*4 + (k&3), high nibble iff (k>>2)&1; d,m as fp16 after the nibbles."""
    N, K = 32, G
    codes = np.random.default_rng(1).integers(0, 16, (N, K))
    codes[:, 0] = 0
    codes[:, 1] = 15
    w = (codes / 128.0 - 0.0625).astype(np.float32)  # d = 1/128, m = -1/16 exactly
    blk = orc.quant_w(w, G)[0, 0].view(np.uint8)
    for n in range(N):
        for k in range(K):
            b = int(blk[(k >> 3) * 128 + n * 4 + (k & 3)])
            q = (b >> 4) if ((k >> 2) & 1) else (b & 15)
            assert q == codes[n, k], (n, k)
    d = blk[(G // 8) * 128:(G // 8) * 128 + 64].view(np.float16)
    m = blk[(G // 8) * 128 + 64:].view(np.float16)
    assert np.all(d == np.float16(1 / 128)) and np.all(m == np.float16(-1 / 16))
    assert np.array_equal(orc.unpack_codes(orc.quant_w(w, G)), codes.astype(np.uint8))


@pytest.mark.parametrize("G", [32, 128])
def test_pack_special_groups(orc, G):
    w = np.zeros((32, G), np.float32)
    w[0, :] = 0.37                       # constant group: d = 0 -> id = 0 -> all codes 0, dequant = m
    w[1, :] = np.arange(G) % 16          # d = 1 exactly
    w[2, 0:4] = [0.0, 15.0, 2.5, 3.5]    # d = 1: half-away ties 2.5 -> 3, 3.5 -> 4 (RNE would give 2, 4)
    w[3, 0:3] = [-1.0, 14.0, -0.5]       # m = -1: (w-m)*id = 0.5 -> 1
    wq = orc.quant_w(w, G)
    codes = orc.unpack_codes(wq)
    dq = orc.dequant_w(wq)
    assert np.all(codes[0] == 0) and np.allclose(dq[0], np.float32(np.float16(0.37)))
    assert np.array_equal(codes[1], (np.arange(G) % 16).astype(np.uint8))
    assert list(codes[2, :4]) == [0, 15, 3, 4]
    assert list(codes[3, :3]) == [0, 15, 1]


@pytest.mark.parametrize("G", [32, 128])
def test_pack_invariants_random(orc, G):
    rng = np.random.default_rng(2)
    w = (rng.standard_normal((96, 4 * G)) * 0.02).astype(np.float32)
    wq = orc.quant_w(w, G)
    codes = orc.unpack_codes(wq).reshape(96, 4, G)
    assert codes.min(axis=2).max() == 0 and codes.max(axis=2).min() == 15  # group min -> 0, max -> 15
    wg = w.reshape(96, 4, G)
    d = (wg.max(2) - wg.min(2)) / 15
    err = np.abs(orc.dequant_w(wq).reshape(96, 4, G) - wg)
    # half a step + fp16 rounding of d (15 steps) and m
    assert np.all(err <= d[..., None] * (0.5 + 15 * 2.0 ** -11) + np.abs(wg.min(2))[..., None] * 2.0 ** -11 + 1e-9)


@pytest.mark.parametrize("G", [32, 128])
def test_pack_vs_reference_build(orc, G):
    R = _ref(G)
    rng = np.random.default_rng(3)
    for N, K, scale in ((256, 1024, 0.02), (64, 2048, 1.0), (32, 4 * G, 1e-6)):
        w = (rng.standard_normal((N, K)) * scale).astype(np.float32)
        assert np.array_equal(orc.quant_w(w, G), R.quant_w(w))


# ---- activation quantization --------------------------------------------------------------------
@pytest.mark.parametrize("G", [32, 128])
def test_quant_x_matches_golden(orc, G):
    g = load_golden(f"fc_g{G}.npz")
    xq, xd, gs = orc.quant_x(g["x"], G)
    assert np.array_equal(xq, g["xq"])
    assert np.array_equal(xd.view(np.uint32), g["xd"].view(np.uint32))
    assert np.array_equal(gs.view(np.uint32), g["gsum"].view(np.uint32))


@pytest.mark.parametrize("G", [32, 128])
def test_quant_x_rne_ties_and_edges(orc, G):
    x = np.zeros((3, G), np.float32)
    x[0, :8] = [127, 2.5, 3.5, -2.5, -3.5, 0.5, 1.5, -0.5]  # amax 127 -> d = 1, id = 1
    x[2, 5] = -4.0
    xq, xd, gs = orc.quant_x(x, G)
    assert list(xq[0, :8]) == [127, 2, 4, -2, -4, 0, 2, 0]  # half to even, not half away
    assert xd[0, 0] == 1.0 and xd[1, 0] == 0.0 and np.all(xq[1] == 0) and gs[1, 0] == 0.0
    assert xq[2, 5] == -127 and np.count_nonzero(xq[2]) == 1 and gs[2, 0] == -4.0


@pytest.mark.parametrize("G", [32, 128])
def test_quant_x_closed_form_and_gsum(orc, G):
    x, _ = oracle.closed_form_fc_inputs(4, 32, 8 * G, seed=5)
    xq, xd, gs = orc.quant_x(x, G)
    assert np.all(xd == np.float32(1 / 128))
    assert np.array_equal(xq.astype(np.float32), x * 128)
    rng = np.random.default_rng(6)
    xr = rng.standard_normal((3, 4 * G)).astype(np.float32)
    _, _, gsr = orc.quant_x(xr, G)
    for r in range(3):
        for kb in range(4):
            seg = xr[r, kb * G:(kb + 1) * G]
            s = np.float32(0)
            for v in seg:
                s = np.float32(s + v)
            assert gsr[r, kb] == s
            assert abs(float(gsr[r, kb]) - math.fsum(seg.tolist())) <= G * 2.0 ** -24 * np.abs(seg).sum()


@pytest.mark.parametrize("G", [32, 128])
def test_quant_x_vs_reference_build(orc, G):
    R = _ref(G)
    rng = np.random.default_rng(7)
    for scale in (1.0, 1e-3, 300.0):
        x = (rng.standard_normal((7, 16 * G)) * scale).astype(np.float32)
        a, b = orc.quant_x(x, G), R.quant_x(x)
        assert np.array_equal(a[0], b[0])
        assert np.array_equal(a[1].view(np.uint32), b[1].view(np.uint32))
        assert np.array_equal(a[2].view(np.uint32), b[2].view(np.uint32))


# ---- int32 partial sums and fp32 output ---------------------------------------------------------
@pytest.mark.parametrize("G", [32, 128])
def test_partials_bruteforce(orc, G):
    rng = np.random.default_rng(8)
    N, K, rows = 64, 4 * G, 3
    wq = orc.quant_w((rng.standard_normal((N, K)) * 0.02).astype(np.float32), G)
    xq = rng.integers(-127, 128, (rows, K)).astype(np.int8)
    codes = orc.unpack_codes(wq).astype(np.int64).reshape(N, K // G, G)
    want = np.einsum("rgk,ngk->rng", xq.astype(np.int64).reshape(rows, K // G, G), codes)
    assert np.array_equal(orc.fc_partials(xq, wq), want)
    # extreme codes: |acc| = G*15*127 must survive
    w = np.tile(np.array([0.0, 15.0], np.float32), (32, G // 2))
    w[:, :] = 15.0
    w[:, 0] = 0.0
    wq2 = orc.quant_w(w, G)
    x2 = np.full((1, G), -127, np.int8)
    assert orc.fc_partials(x2, wq2).min() == -(G - 1) * 15 * 127


@pytest.mark.parametrize("G", [32, 128])
def test_fc_matches_golden(orc, G):
    g = load_golden(f"fc_g{G}.npz")
    y = orc.fc(g["x"], g["wq"], g["y"].shape[-1])
    assert np.array_equal(y.view(np.uint32), g["y"].view(np.uint32))


@pytest.mark.parametrize("G", [32, 128])
def test_fc_closed_form_exact(orc, G):
    """ops/test_ops.py:106-149: exactly representable data -> fc == x @ W.T exactly."""
    x, w = oracle.closed_form_fc_inputs(5, 128, 1024, seed=9)
    wq = orc.quant_w(w, G)
    assert np.array_equal(orc.dequant_w(wq), w)
    want = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32)
    assert np.array_equal(orc.fc(x, wq, 128), want)


@pytest.mark.parametrize("G", [32, 128])
def test_fc_formula_fp64(orc, G):
    """General data: y == sum_kb (d16*dx)*acc + m16*gsum evaluated in fp64, within 1e-5."""
    rng = np.random.default_rng(10)
    N, K, rows = 96, 8 * G, 4
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    x = rng.standard_normal((rows, K)).astype(np.float32)
    wq = orc.quant_w(w, G)
    xq, xd, gs = orc.quant_x(x, G)
    acc = orc.fc_partials(xq, wq).astype(np.float64)  # [rows, N, Kg]
    blk = wq.view(np.uint8).reshape(N // 32, K // G, -1)
    d16 = blk[:, :, (G // 8) * 128:(G // 8) * 128 + 64].copy().view(np.float16).astype(np.float64)  # [Ng,Kg,32]
    m16 = blk[:, :, (G // 8) * 128 + 64:].copy().view(np.float16).astype(np.float64)
    d16 = d16.transpose(0, 2, 1).reshape(N, K // G)
    m16 = m16.transpose(0, 2, 1).reshape(N, K // G)
    want = np.einsum("rnk,nk,rk->rn", acc, d16, xd.astype(np.float64)) + np.einsum("nk,rk->rn", m16, gs.astype(np.float64))
    assert max_rel_err(orc.fc(x, wq, N), want) < 1e-5
    # and the quantized product tracks the fp32 product to quantization accuracy
    assert max_rel_err(orc.fc(x, wq, N), x.astype(np.float64) @ w.astype(np.float64).T) < 0.3


@pytest.mark.parametrize("G", [32, 128])
def test_fc_vs_reference_build(orc, G):
    R = _ref(G)
    rng = np.random.default_rng(11)
    w = (rng.standard_normal((128, 2048)) * 0.02).astype(np.float32)
    x = rng.standard_normal((2, 3, 2048)).astype(np.float32)
    wq = R.quant_w(w)
    a = orc.fc(x, wq, 128)
    b = R.fc(x, wq, 128)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


# ---- rope / attention / softmax / neighbours ----------------------------------------------------
def _rope_fp64(x, inv_freq, pos):
    x = x.astype(np.float64).copy()
    half = inv_freq.shape[0]
    for l in range(x.shape[2]):
        th = inv_freq.astype(np.float32) * np.float32(pos + l)
        c, s = np.cos(th.astype(np.float64)), np.sin(th.astype(np.float64))
        x0, x1 = x[:, :, l, :half].copy(), x[:, :, l, half:2 * half].copy()
        x[:, :, l, :half] = c * x0 - s * x1
        x[:, :, l, half:2 * half] = s * x0 + c * x1
    return x


def test_rope_golden_and_textbook(orc):
    g = load_golden("misc.npz")
    got = orc.rope(g["rope_x"], g["rope_inv_freq"], 16)
    assert np.abs(got - g["rope_out"]).max() < 1e-5            # ops/test_ops.py:211 uses atol 1e-5
    assert np.abs(got - _rope_fp64(g["rope_x"], g["rope_inv_freq"], 16)).max() < 1e-5
    assert np.array_equal(got[..., 64:], g["rope_x"][..., 64:])  # partial rotary: dims >= 2*half untouched


def _attention_fp64(q, k, v, inv_freq, cache, slots, pos, layer):
    B, qL, HS = q.shape
    _, _, H, maxlen, S = cache.shape
    q4 = _rope_fp64(q.reshape(B, qL, H, S).transpose(0, 2, 1, 3), inv_freq, pos)
    k4 = _rope_fp64(k.reshape(B, qL, H, S).transpose(0, 2, 1, 3), inv_freq, pos)
    v4 = v.reshape(B, qL, H, S).transpose(0, 2, 1, 3).astype(np.float64)
    cache = cache.astype(np.float64).copy()
    for l in range(qL):
        cache[2 * layer, :, :, slots[l]] = k4[:, :, l]
        cache[2 * layer + 1, :, :, slots[l]] = v4[:, :, l]
    kv = min(pos + qL, maxlen)
    K, V = cache[2 * layer, :, :, :kv], cache[2 * layer + 1, :, :, :kv]
    w = np.einsum("bhqs,bhks->bhqk", q4, K) / math.sqrt(S)
    for l in range(qL):
        for l2 in range(l + 1, qL):
            w[:, :, l, slots[l2]] = -np.inf
    w = np.exp(w - w.max(-1, keepdims=True))
    w /= w.sum(-1, keepdims=True)
    out = np.einsum("bhqk,bhks->bhqs", w, V).transpose(0, 2, 1, 3).reshape(B, qL, HS)
    return out, k4.transpose(0, 2, 1, 3).reshape(B, qL, HS), cache


@pytest.mark.parametrize("name", ["attn_decode", "attn_decode_wrap", "attn_chunk", "attn_prefill"])
def test_attention_golden_and_textbook(orc, name):
    g = load_golden(name + ".npz")
    pos, layer = int(g["position_id"]), int(g["layer_id"])
    out, k_rot, cache_after = orc.attention(g["q"], g["k"], g["v"], g["inv_freq"], g["cache"], g["slots"], pos, layer)
    assert max_rel_err(out, g["out"]) < 1e-5
    assert max_rel_err(out, g["out_v1"]) < 1e-5          # attention_rope (v1) has the same contract
    assert np.abs(k_rot - g["k_rot"]).max() < 1e-5
    assert np.abs(cache_after - g["cache_after"]).max() < 1e-5
    t_out, t_k, t_cache = _attention_fp64(g["q"], g["k"], g["v"], g["inv_freq"], g["cache"], g["slots"], pos, layer)
    assert max_rel_err(out, t_out) < 1e-5
    assert np.abs(k_rot - t_k).max() < 1e-5
    assert np.abs(cache_after - t_cache).max() < 1e-5
    untouched = np.ones(g["cache"].shape[0], bool)
    untouched[2 * layer:2 * layer + 2] = False
    assert np.array_equal(cache_after[untouched], g["cache"][untouched])


def test_softmax_literals_and_golden(orc):
    g = load_golden("misc.npz")
    assert np.allclose(orc.softmax(g["sm_in"]), g["sm"], rtol=1e-5, atol=1e-8)
    lit = orc.softmax(g["lit"][None])[0]                    # ops/test_ops.py:171, last entry is -FLT_MAX
    assert np.allclose(lit, g["sm_lit"], rtol=1e-5, atol=1e-8) and lit[-1] == 0.0
    e = np.exp(g["lit"][:-1].astype(np.float64) - g["lit"][:-1].max())
    assert np.allclose(lit[:-1], e / e.sum(), rtol=1e-6)
    two = orc.softmax(np.array([[0.66046, 0.61789]], np.float32))[0]  # ops/test_ops.py:172
    assert np.allclose(two, [1 / (1 + math.exp(0.61789 - 0.66046)), 1 / (1 + math.exp(0.66046 - 0.61789))], rtol=1e-6)


def test_neighbours_golden(orc):
    g = load_golden("misc.npz")
    x, wn = g["x"], g["wn"]
    assert np.allclose(orc.rmsnorm(x, wn, 1e-5), g["rms"], rtol=1e-5, atol=1e-6)
    ref = wn * (x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-5))
    assert np.allclose(orc.rmsnorm(x, wn, 1e-5), ref, rtol=1e-5, atol=1e-6)
    # the reference's silu uses the 12-bit rcpps approximation (ops/utils.hpp:373-378): ~3e-4 relative
    assert np.allclose(orc.silu(x), g["silu"], rtol=1e-3, atol=1e-6)
    assert np.allclose(orc.silu(x), x / (1 + np.exp(-x.astype(np.float64))), rtol=1e-6, atol=1e-7)
    assert np.array_equal(orc.iadd(x, x[:, ::-1].copy()), g["iadd"])
    assert np.array_equal(orc.imul(x, wn), g["imul_row"])
    eq, es = orc.embedding_q8c_quant_w(g["emb"])
    assert np.array_equal(eq, g["eq"]) and np.array_equal(es.view(np.uint32), g["es"].view(np.uint32))
    assert np.array_equal(orc.embedding_q8c(g["ids"], eq, es), g["emb_out"])


def test_attention_vs_reference_build(orc):
    R = _ref(128, fresh=True)
    g = load_golden("attn_chunk.npz")
    pos, layer = int(g["position_id"]), int(g["layer_id"])
    a = orc.attention(g["q"], g["k"], g["v"], g["inv_freq"], g["cache"], g["slots"], pos, layer)
    b = R.attention(g["q"], g["k"], g["v"], g["inv_freq"], g["cache"], g["slots"], pos, layer)
    for u, v in zip(a, b):
        assert max_rel_err(u, v) < 1e-5


# ---- mm_qk (the four benchmark variants of the scaled q.k product, ops/op_attn.hpp:149-515) -----------
def _qk_fp64(q_bhqs, kc, kvLen):
    return np.einsum("bhqs,bhks->bhqk", q_bhqs.astype(np.float64), kc[:, :, :kvLen].astype(np.float64)) / math.sqrt(kc.shape[-1])


@pytest.mark.parametrize("B,H,qL,kv,S", [(1, 2, 1, 7, 16), (2, 3, 5, 33, 128), (1, 1, 37, 130, 64)])
def test_mm_qk_oracle_against_fp64_einsum(orc, B, H, qL, kv, S):
    rng = np.random.default_rng(B * 1000 + qL)
    q = rng.random((B, qL, H * S), dtype=np.float32)          # ops/perf_ops.py:165-166 draws both from U[0,1)
    kc = rng.standard_normal((B, H, kv, S)).astype(np.float32)
    q_bhqs = np.ascontiguousarray(q.reshape(B, qL, H, S).transpose(0, 2, 1, 3))
    ref = _qk_fp64(q_bhqs, kc, kv)
    assert np.allclose(orc.mm_qk(q, kc), ref, rtol=1e-5, atol=1e-5)
    # the [B,H,qL,S] form with a cache plane longer than the rows asked for (mm_qk42)
    part = max(1, kv - 3)
    got = orc.mm_qk(q_bhqs, kc, kvLen=part, q_is_bhqs=True)
    assert got.shape == (B, H, qL, part)
    assert np.allclose(got, _qk_fp64(q_bhqs, kc, part), rtol=1e-5, atol=1e-5)
    # a transposed operand or a dropped scale would show here: one-hot rows pick single cache entries
    e = np.zeros((B, qL, H * S), np.float32)
    e[:, :, ::S] = 1.0                                          # s = 0 of every head
    assert np.allclose(orc.mm_qk(e, kc), np.broadcast_to((kc[:, :, None, :, 0] / math.sqrt(S)), (B, H, qL, kv)), rtol=1e-6)


@pytest.mark.parametrize("variant", [0, 1, 2, 3])
def test_mm_qk_oracle_against_reference_build(orc, variant):
    ref = _ref(32)
    # crosses the 64-blocks of the AVX variants; those have no tail loops (mm_qk42 steps 4 queries x 2 cache rows,
    # ops/op_attn.hpp:216-218, and writes past the end otherwise), so the sizes are multiples of 8
    B, H, qL, kv, S = 2, 4, 72, 200, 128
    rng = np.random.default_rng(variant)
    kc = rng.standard_normal((B, H, kv, S)).astype(np.float32)
    q = rng.standard_normal((B, qL, H * S)).astype(np.float32)
    q_bhqs = np.ascontiguousarray(q.reshape(B, qL, H, S).transpose(0, 2, 1, 3))
    if variant == 1:
        got = ref.mm_qk(q_bhqs, kc, kvLen=kv - 8, q_is_bhqs=True, variant=1)
        mine = orc.mm_qk(q_bhqs, kc, kvLen=kv - 8, q_is_bhqs=True)
    else:
        got = ref.mm_qk(q, kc, variant=variant)
        mine = orc.mm_qk(q, kc)
    assert got.shape == mine.shape
    assert np.abs(got - mine).max() <= 1e-5 * np.abs(mine).max()


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("K", [5, 100, 333, 1001, 4100])
def test_quant_x_short_last_group_vs_reference_build(orc, G, K):
    """A K that is not a whole number of groups, nor of eights: the reference zero-pads the last group's codes
    (ops/op_fc.hpp:259-261) and its last K % 8 values round half away from zero (ops/utils.hpp:217-219).  The
    restatement against the reference build, bit for bit, ties included."""
    R = _ref(G)
    rng = np.random.default_rng(K + G)
    x = rng.standard_normal((3, K)).astype(np.float32)
    last = (K - 1) // G * G                      # first element of the short group
    x[0, last:] = 0
    x[0, last] = 127.0                            # amax 127 -> d = 1: the products are the values themselves
    ties = np.array([2.5, 3.5, -2.5, -0.5, 0.5, 1.5, -3.5], np.float32)
    n = min(len(ties), K - last - 1)
    x[0, K - n:] = ties[:n]                       # the tail values: where the two roundings differ
    oq, od, og = orc.quant_x(x, G)
    rq, rd, rg = R.quant_x(x)
    assert np.array_equal(oq, rq)
    assert np.array_equal(od.view(np.uint32), rd.view(np.uint32))
    assert np.array_equal(og.view(np.uint32), rg.view(np.uint32))
    assert np.all(oq[:, K:] == 0)


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("rows,N,K", [(1, 64, 100), (3, 96, 1001), (17, 32, 4100)])
def test_fc_short_last_group_vs_reference_build(orc, G, rows, N, K):
    """fc_Q4A with a K that is not a whole number of k-groups: the reference pads the activation codes of the last
    group with zeros, so whatever codes the weights hold beyond K do not matter.  (The weights are packed by the
    restatement, which clips the min/max scan to K; the reference's own packing reads past the row there,
    ops/op_fc.hpp:184.)  Output of the restatement against the reference build's fc_Q4A, bit for bit."""
    R = _ref(G)
    rng = np.random.default_rng(rows + N + K + G)
    wq = orc.quant_w((rng.standard_normal((N, K)) * 0.02).astype(np.float32), G)
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    assert np.array_equal(orc.fc(x, wq, N).view(np.uint32), R.fc(x, wq, N).view(np.uint32))
