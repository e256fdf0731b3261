"""GPU parity of the Q4_1 FC path against the oracle and the committed golden vectors, through
the `llmops` module (ctypes -> C ABI -> HIP kernels).  Bit-exact: packed bytes, Q8 codes, scales,
group sums, int32 partial sums.  fp32 outputs: max|err|/max|ref| <= 1e-3 (the stated contract;
observed errors are ~1e-6)."""
import numpy as np
import pytest
import torch

import oracle
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


# ---- packing ------------------------------------------------------------------------------------
@pytest.mark.parametrize("G", [32, 128])
def test_pack_golden(ops, G):
    g = load_golden(f"fc_g{G}.npz")
    wq = ops.offline_FC_quant_Q4A(dev(g["w"]), G)
    assert np.array_equal(host(wq), g["wq"])
    assert np.array_equal(host(ops.offline_FC_dequant_Q4A(wq)).view(np.uint32), g["dq"].view(np.uint32))


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("N,K", [(4096, 4096), (352, 11008), (100, 1024)])
def test_pack_random_vs_oracle(ops, orc, G, N, K):
    rng = np.random.default_rng(N + K + G)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    w[1, :G] = 0.5                      # constant group
    w[2, :4] = [0.0, 15.0, 2.5, 3.5]    # half-away ties when it spans the group range
    w[3, :G] = np.where(rng.random(G) < 0.5, 0.0, -0.0)  # zero group with mixed signs: sign of m follows first element
    wq = host(ops.offline_FC_quant_Q4A(dev(w), G))
    want = orc.quant_w(w, G)
    assert wq.shape == want.shape
    assert np.array_equal(wq, want)    # includes zero nibbles / zero d,m of padded rows when N % 32 != 0
    assert np.array_equal(host(ops.offline_FC_dequant_Q4A(dev(want))).view(np.uint32), orc.dequant_w(want).view(np.uint32))


def test_pack_row_stride(ops, orc):
    w = (np.random.default_rng(5).standard_normal((64, 640)) * 0.02).astype(np.float32)
    view = dev(w)[:, :512]             # row stride 640, inner contiguous
    assert np.array_equal(host(ops.offline_FC_quant_Q4A(view, 128)), orc.quant_w(w[:, :512], 128))


# ---- activation quantization --------------------------------------------------------------------
@pytest.mark.parametrize("G", [32, 128])
def test_quant_x_golden(ops, G):
    g = load_golden(f"fc_g{G}.npz")
    xq, xd, gs = ops.FC_dynamic_quantize_x(dev(g["x"]), G)
    assert np.array_equal(host(xq), g["xq"])
    assert np.array_equal(host(xd).view(np.uint32), g["xd"].view(np.uint32))
    assert np.array_equal(host(gs).view(np.uint32), g["gsum"].view(np.uint32))


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("rows,K", [(1, 4096), (17, 11008), (2048, 4096)])
def test_quant_x_random_vs_oracle(ops, orc, G, rows, K):
    rng = np.random.default_rng(rows + K)
    x = rng.standard_normal((rows, K)).astype(np.float32)
    x[0, :8] = [127, 2.5, 3.5, -2.5, -3.5, 0.5, 1.5, -0.5]
    x[0, 8:G] = 0
    if rows > 1:
        x[1, G:2 * G] = 0
    xq, xd, gs = ops.FC_dynamic_quantize_x(dev(x), G)
    wq, wd, wg = orc.quant_x(x, G)
    assert np.array_equal(host(xq), wq)
    assert np.array_equal(host(xd).view(np.uint32), wd.view(np.uint32))
    assert np.array_equal(host(gs).view(np.uint32), wg.view(np.uint32))
    assert list(host(xq)[0, :8]) == [127, 2, 4, -2, -4, 0, 2, 0]


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("rows,K", [(1, 4096), (17, 11008), (2048, 4096), (3, 128)])
def test_quant_x_rows_variant_vs_oracle(ops, orc, G, rows, K):
    """The quantizer of the prefill FC: codes and scales bit-exact, group sum within fp32 rounding."""
    rng = np.random.default_rng(rows + K + 1)
    x = rng.standard_normal((rows, K)).astype(np.float32)
    x[0, :8] = [127, 2.5, 3.5, -2.5, -3.5, 0.5, 1.5, -0.5]
    x[0, 8:G] = 0
    x[-1, -G:] = 0
    xq, xd, gs = ops.FC_dynamic_quantize_x(dev(x), G, rows_variant=True)
    wq, wd, wg = orc.quant_x(x, G)
    assert np.array_equal(host(xq), wq)
    assert np.array_equal(host(xd).view(np.uint32), wd.view(np.uint32))
    assert np.abs(host(gs) - wg).max() <= 1e-5 * max(1.0, np.abs(x).max() * G)
    assert list(host(xq)[0, :8]) == [127, 2, 4, -2, -4, 0, 2, 0]


# ---- int32 partial sums -------------------------------------------------------------------------
INNER_LOOPS = [(32, 0), (32, 1), (128, 0), (128, 1), (128, 2)]  # (group, use_mfma); 2 = 256-row kernel, group 128 only


@pytest.mark.parametrize("G,mfma", INNER_LOOPS)
@pytest.mark.parametrize("rows,N,K", [(1, 4096, 4096), (3, 352, 2048), (17, 96, 1024), (40, 32, 384), (300, 160, 640)])
def test_partials_bit_exact(ops, orc, G, mfma, rows, N, K):
    rng = np.random.default_rng(rows * 7 + G)
    wq = orc.quant_w((rng.standard_normal((N, K)) * 0.02).astype(np.float32), G)
    xq = rng.integers(-127, 128, (rows, K)).astype(np.int8)
    xq[0, :G] = -127
    got = host(ops.fc_Q4A_partials(dev(xq), dev(wq), use_mfma=mfma))
    assert np.array_equal(got, orc.fc_partials(xq, wq))


@pytest.mark.parametrize("G,mfma", INNER_LOOPS)
def test_partials_extreme_codes(ops, orc, G, mfma):
    w = np.full((32, 2 * G), 15.0, np.float32)
    w[:, 0::G] = 0.0
    wq = orc.quant_w(w, G)
    xq = np.full((2, 2 * G), -127, np.int8)
    xq[1] = 127
    got = host(ops.fc_Q4A_partials(dev(xq), dev(wq), use_mfma=mfma))
    assert got.min() == -(G - 1) * 15 * 127 and got.max() == (G - 1) * 15 * 127
    assert np.array_equal(got, orc.fc_partials(xq, wq))


# ---- fp32 output --------------------------------------------------------------------------------
@pytest.mark.parametrize("G", [32, 128])
def test_fc_golden(ops, G):
    g = load_golden(f"fc_g{G}.npz")
    y = host(ops.fc_Q4A(dev(g["x"][None]), dev(g["wq"]), g["y"].shape[-1]))[0]
    assert max_rel_err(y, g["y"]) <= TOL
    for r in range(y.shape[0]):          # row by row too: rows differ in magnitude by 1e20
        assert max_rel_err(y[r], g["y"][r]) <= TOL


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("B,M", [(1, 1), (1, 2), (1, 4), (1, 7), (2, 17), (1, 64), (1, 130)])
def test_fc_closed_form_exact(ops, G, B, M):
    """ops/test_ops.py:106-149 (B=2, M=17, N=K=4096 there): every value exactly representable, so
    the result must EQUAL x @ W.T whatever the accumulation order."""
    N = K = 4096 if M <= 17 else 1024
    x, w = oracle.closed_form_fc_inputs(B * M, N, K, seed=M)
    wq = ops.offline_FC_quant_Q4A(dev(w), G)
    assert np.array_equal(host(ops.offline_FC_dequant_Q4A(wq)), w)
    y = host(ops.fc_Q4A(dev(x.reshape(B, M, K)), wq, N))
    want = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32).reshape(B, M, N)
    assert np.array_equal(y, want)


CONFIG_SHAPES = [  # (G, N, K) of BASELINE configs 1 and 2
    (32, 4096, 4096), (128, 4096, 4096), (128, 11008, 4096), (128, 4096, 11008),
]


@pytest.mark.parametrize("G,N,K", CONFIG_SHAPES)
@pytest.mark.parametrize("M", [1, 3, 8, 16, 48])
def test_fc_baseline_shapes_vs_oracle(ops, orc, G, N, K, M):
    rng = np.random.default_rng(G + N + K + M)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    x = rng.standard_normal((1, M, K)).astype(np.float32)
    wq = orc.quant_w(w, G)
    want = orc.fc(x, wq, N)
    dwq, dx = dev(wq), dev(x)
    y1 = host(ops.fc_Q4A(dx, dwq, N))
    assert max_rel_err(y1, want) <= TOL
    assert max_rel_err(y1, want) <= 1e-5   # what the kernels actually achieve
    y2 = host(ops.fc_Q4A(dx, dwq, N))      # split-K partial sums are combined in a fixed order
    assert np.array_equal(y1.view(np.uint32), y2.view(np.uint32))


def test_fc_odd_N_and_fused_strips(ops, orc):
    """N not a multiple of 32 (stores are clipped) and row-wise concatenation of packed tensors
    (q/k/v fused into one launch) give the concatenated outputs."""
    rng = np.random.default_rng(77)
    K = 1024
    x = rng.standard_normal((1, 2, K)).astype(np.float32)
    w = (rng.standard_normal((100, K)) * 0.02).astype(np.float32)
    wq = orc.quant_w(w, 128)
    assert max_rel_err(host(ops.fc_Q4A(dev(x), dev(wq), 100)), orc.fc(x, wq, 100)) <= 1e-5
    ws = [(rng.standard_normal((n, K)) * 0.02).astype(np.float32) for n in (64, 96, 32)]
    packed = [orc.quant_w(a, 128) for a in ws]
    fused = np.concatenate(packed, axis=0)
    y = host(ops.fc_Q4A(dev(x), dev(fused), 192))
    want = np.concatenate([orc.fc(x, p, a.shape[0]) for p, a in zip(packed, ws)], axis=-1)
    assert max_rel_err(y, want) <= 1e-5


def test_fc_size_independent_properties(ops):
    """Full-size (lm_head-like) checks that need no CPU reference: a scaled one-hot activation
    reads back one dequantized weight column, and the op is homogeneous in powers of two."""
    G, N, K = 128, 55296, 4096
    gen = torch.Generator(device="cpu").manual_seed(5)
    w = (torch.randn(N, K, generator=gen) * 0.02).cuda()
    wq = ops.offline_FC_quant_Q4A(w, G)
    dq = ops.offline_FC_dequant_Q4A(wq)
    for k in (0, 1234, K - 1):
        x = torch.zeros(1, 1, K, device="cuda")
        x[0, 0, k] = 127.0                      # dx = 1, code 127, gsum = 127
        y = ops.fc_Q4A(x, wq, N)[0, 0]
        assert torch.allclose(y, 127.0 * dq[:, k], rtol=1e-6, atol=1e-6)
    x = torch.randn(1, 1, K, generator=gen).cuda()
    y1 = ops.fc_Q4A(x, wq, N)
    y2 = ops.fc_Q4A(x * 4.0, wq, N)            # scaling by 2^k is exact through every step
    assert torch.equal(y1 * 4.0, y2)
    assert (y1 - torch.nn.functional.linear(x, dq[:N])).abs().max() / y1.abs().max() < 2e-2  # Q8 activation error only


def test_fc_argument_errors(ops):
    x = torch.zeros(1, 1, 256, device="cuda")
    wq = torch.zeros(1, 2, 2176, dtype=torch.int8, device="cuda")
    with pytest.raises(RuntimeError):
        ops.fc_Q4A(x[0], wq, 32)                                   # rank 2 input (ops/op_fc.hpp:287)
    with pytest.raises(RuntimeError):
        ops.fc_Q4A(x, wq.to(torch.float32), 32)                    # wrong dtype (ops/op_fc.hpp:288)
    with pytest.raises(RuntimeError):
        ops.fc_Q4A(torch.zeros(1, 1, 128, device="cuda"), wq, 32)  # K != Kg*G
    with pytest.raises(RuntimeError):
        ops.fc_Q4A(x, torch.zeros(1, 2, 1000, dtype=torch.int8, device="cuda"), 32)  # not a block size
    with pytest.raises(RuntimeError):
        ops.offline_FC_quant_Q4A(torch.zeros(4, 4, 4, device="cuda"))               # rank 3 weight (ops/op_fc.hpp:152)


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("rows", [1, 2, 3, 8, 20])
def test_fc_decode_folded_ops_vs_oracle(ops, orc, G, rows):
    """fc_Q4A_decode: rmsnorm prologue, residual epilogue and the interleaved gate/up epilogue, each
    against the oracle's separate ops.  A folded rmsnorm may differ from the separate one by an ulp,
    which can flip an int8 code on a rounding boundary, hence 1e-4 instead of 1e-5 there."""
    rng = np.random.default_rng(rows + G)
    K, F = 1024, 352
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    nw = (1.0 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    wg = (rng.standard_normal((F, K)) * 0.02).astype(np.float32)
    wu = (rng.standard_normal((F, K)) * 0.02).astype(np.float32)
    res = rng.standard_normal((1, rows, F)).astype(np.float32)
    pg, pu = orc.quant_w(wg, G), orc.quant_w(wu, G)
    xn = orc.rmsnorm(x, nw, 1e-5)
    # norm only, norm + residual
    got = host(ops.fc_Q4A_decode(dev(x), dev(pg), F, norm=(dev(nw), 1e-5)))
    assert max_rel_err(got, orc.fc(xn, pg, F)) <= 1e-4
    got = host(ops.fc_Q4A_decode(dev(x), dev(pg), F, norm=(dev(nw), 1e-5), residual=dev(res)))
    assert max_rel_err(got, orc.iadd(orc.fc(xn, pg, F), res)) <= 1e-4
    # gate/up epilogue with and without the norm
    il = ops.interleave_gate_up(dev(pg), dev(pu))
    assert np.array_equal(host(il)[0::2], pg) and np.array_equal(host(il)[1::2], pu)
    want = orc.imul(orc.fc(x, pu, F), orc.silu(orc.fc(x, pg, F)))
    assert max_rel_err(host(ops.fc_Q4A_decode(dev(x), il, F, glu=True)), want) <= 1e-5
    want = orc.imul(orc.fc(xn, pu, F), orc.silu(orc.fc(xn, pg, F)))
    assert max_rel_err(host(ops.fc_Q4A_decode(dev(x), il, F, norm=(dev(nw), 1e-5), glu=True)), want) <= 1e-4


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("rows", [1, 3, 8, 20])
@pytest.mark.parametrize("N,K", [(1000, 1024), (4096, 11008)])
def test_fc_decode_sumsq_handover(ops, orc, G, rows, N, K):
    """The per-strip sums of squares an FC leaves behind (also through the split-K hand-off: K = 11008),
    and the rmsnorm of the next FC fed with them instead of reading its input row."""
    rng = np.random.default_rng(rows + G + N)
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    res = rng.standard_normal((1, rows, N)).astype(np.float32)
    pw = dev(orc.quant_w(w, G))
    y, ss = ops.fc_Q4A_decode(dev(x), pw, N, residual=dev(res), want_sumsq=True)
    yh = host(y).astype(np.float64).reshape(rows, N)
    strips = -(-N // 32)
    pad = np.zeros((rows, strips * 32))
    pad[:, :N] = yh
    want = (pad.reshape(rows, strips, 32) ** 2).sum(-1)
    assert host(ss).shape == (rows, strips)
    assert np.abs(host(ss) - want).max() <= 1e-5 * want.max()
    # consumer: rmsnorm(y) @ W2 with and without the handed-over sums must agree to rounding
    if N % G == 0:
        F = 352
        w2 = (rng.standard_normal((F, N)) * 0.02).astype(np.float32)
        nw = (1.0 + 0.1 * rng.standard_normal(N)).astype(np.float32)
        p2 = dev(orc.quant_w(w2, G))
        a = host(ops.fc_Q4A_decode(y, p2, F, norm=(dev(nw), 1e-5)))
        b = host(ops.fc_Q4A_decode(y, p2, F, norm=(dev(nw), 1e-5), sumsq_in=ss))
        assert max_rel_err(b, a) <= 1e-4
        # against the oracle the contract of fc_Q4A applies: the rmsnorm here and there differ by an ulp,
        # which flips an int8 code now and then (K = 4096 values per output)
        assert max_rel_err(b, orc.fc(orc.rmsnorm(host(y), nw, 1e-5), host(p2), F)) <= 1e-3


@pytest.mark.parametrize("rows", [1, 3])
def test_fc_decode_sumsq_handover_many_parts(ops, orc, rows):
    """A producer with more than 256 strips (N = 16384: 512 partial sums): the consumer does not take the
    handed-over sums (it reads at most 256) but computes the statistic from the row -- same result as
    without them, and against the oracle."""
    rng = np.random.default_rng(rows)
    K1, N1, F = 256, 16384, 96
    x = rng.standard_normal((1, rows, K1)).astype(np.float32)
    p1 = dev(orc.quant_w((rng.standard_normal((N1, K1)) * 0.05).astype(np.float32), 128))
    y, ss = ops.fc_Q4A_decode(dev(x), p1, N1, want_sumsq=True)
    assert ss.shape == (rows, 512)
    nw = (1.0 + 0.1 * rng.standard_normal(N1)).astype(np.float32)
    p2 = dev(orc.quant_w((rng.standard_normal((F, N1)) * 0.02).astype(np.float32), 128))
    a = ops.fc_Q4A_decode(y, p2, F, norm=(dev(nw), 1e-5))
    b = ops.fc_Q4A_decode(y, p2, F, norm=(dev(nw), 1e-5), sumsq_in=ss)
    assert torch.equal(a, b)
    assert max_rel_err(host(b), orc.fc(orc.rmsnorm(host(y), nw, 1e-5), host(p2), F)) <= 1e-3


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("rows", [1, 2, 4, 8, 20])
@pytest.mark.parametrize("N,K", [(1000, 1024), (4096, 11008)])
def test_fc_decode_gate_up_input(ops, orc, G, rows, N, K):
    """fc_Q4A_decode(glu_in=True): the input row is [gate | up] (2K floats) and the FC runs on
    silu(gate)*up; against the oracle's silu, imul and fc, with and without the residual and the
    sums of squares (K = 11008 also takes the split-K hand-off), and bit-equal to silu_mul + FC."""
    rng = np.random.default_rng(rows + G + N)
    gu = rng.standard_normal((1, rows, 2 * K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    res = rng.standard_normal((1, rows, N)).astype(np.float32)
    pw = orc.quant_w(w, G)
    act = orc.imul(gu[..., K:].copy(), orc.silu(gu[..., :K].copy()))
    want = orc.fc(act, pw, N)
    got = ops.fc_Q4A_decode(dev(gu), dev(pw), N, glu_in=True)
    assert max_rel_err(host(got), want) <= 1e-4  # expf here and exp there: an int8 code may flip
    two_step = ops.fc_Q4A_decode(ops.silu_mul(dev(gu)), dev(pw), N)
    assert torch.equal(got, two_step)
    got, ss = ops.fc_Q4A_decode(dev(gu), dev(pw), N, residual=dev(res), want_sumsq=True, glu_in=True)
    assert max_rel_err(host(got), want + res) <= 1e-4
    strips = -(-N // 32)
    pad = np.zeros((rows, strips * 32))
    pad[:, :N] = host(got).astype(np.float64).reshape(rows, N)
    ref_ss = (pad.reshape(rows, strips, 32) ** 2).sum(-1)
    assert np.abs(host(ss) - ref_ss).max() <= 1e-5 * ref_ss.max()
    with pytest.raises(RuntimeError):  # no rmsnorm in front of a gate|up row
        ops.fc_Q4A_decode(dev(gu), dev(pw), N, norm=(torch.ones(K, device="cuda"), 1e-5), glu_in=True)


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("rows", [9, 16, 40, 600])
@pytest.mark.parametrize("N,K", [(352, 1024), (2048, 4096), (1000, 8192), (96, 11008)])
def test_fc_decode_many_rows_producer_inside_the_quantization(ops, orc, G, rows, N, K):
    """fc_Q4A_decode with more than 8 rows: the rmsnorm, or silu(gate)*up, runs inside the quantization launch.
    The codes are those of the separate ops, so the results are bit-equal to rmsnorm_out / silu_mul followed by
    fc_Q4A (whose parity with the oracle the other tests hold), with the residual and the sums of squares; and
    against the oracle directly."""
    rng = np.random.default_rng(rows + G + N + K)
    pw = dev(orc.quant_w((rng.standard_normal((N, K)) * 0.02).astype(np.float32), G))
    res = dev(rng.standard_normal((1, rows, N)).astype(np.float32))
    strips = -(-N // 32)

    def sums(y):
        pad = np.zeros((rows, strips * 32))
        pad[:, :N] = host(y).astype(np.float64).reshape(rows, N)
        return (pad.reshape(rows, strips, 32) ** 2).sum(-1)

    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    x[0, 1, :G] = 0.0                # a k-group of zeros: scale 0, codes 0
    x[0, 2, G:2 * G] *= 1e-30        # tiny values
    nw = (1.0 + 0.1 * rng.standard_normal(K)).astype(np.float32)
    if K <= 8192:  # (the oracle's rmsnorm over 600 rows of 11008 adds nothing)
        two_step = ops.fc_Q4A(ops.rmsnorm_out(dev(x), dev(nw), 1e-5), pw, N)
        got = ops.fc_Q4A_decode(dev(x), pw, N, norm=(dev(nw), 1e-5))
        assert torch.equal(got, two_step)
        if rows <= 40:
            # the oracle's product on the normalized rows as this library computes them (its rmsnorm and the
            # oracle's differ by an ulp here and there, which can flip an int8 code: one code is 1e-3 of an
            # output at K = 1024)
            xn = host(ops.rmsnorm_out(dev(x), dev(nw), 1e-5))
            assert max_rel_err(xn, orc.rmsnorm(x, nw, 1e-5)) <= 1e-5
            assert max_rel_err(host(got), orc.fc(xn, host(pw), N)) <= 1e-5
        got, ss = ops.fc_Q4A_decode(dev(x), pw, N, norm=(dev(nw), 1e-5), residual=res, want_sumsq=True)
        assert torch.equal(got, ops.fc_Q4A(ops.rmsnorm_out(dev(x), dev(nw), 1e-5), pw, N, residual=res))
        want_ss = sums(got)
        assert host(ss).shape == (rows, strips) and np.abs(host(ss) - want_ss).max() <= 1e-5 * want_ss.max()
    gu = rng.standard_normal((1, rows, 2 * K)).astype(np.float32)
    gu[0, 0, :G] = -100.0            # silu underflows to -0.0 * up
    two_step = ops.fc_Q4A(ops.silu_mul(dev(gu)), pw, N, residual=res)
    got, ss = ops.fc_Q4A_decode(dev(gu), pw, N, residual=res, want_sumsq=True, glu_in=True)
    assert torch.equal(got, two_step)
    want_ss = sums(got)
    assert np.abs(host(ss) - want_ss).max() <= 1e-5 * want_ss.max()
    if rows <= 40:
        act = host(ops.silu_mul(dev(gu)))
        assert max_rel_err(act, orc.imul(gu[..., K:].copy(), orc.silu(gu[..., :K].copy()))) <= 1e-5
        assert max_rel_err(host(got), orc.fc(act, host(pw), N) + host(res)) <= 1e-5


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("rows", [9, 40, 600])
def test_fc_decode_many_rows_result_in_dense_parts(ops, orc, G, rows):
    """out_parts: the columns of a fused q|k|v projection come out as three dense tensors, bit-equal to the slices
    of the one-tensor result (same quantized rows, same product kernels on a third of the strips each)."""
    rng = np.random.default_rng(rows + G)
    K, N = 1024, 3 * 352
    pw = dev(orc.quant_w((rng.standard_normal((N, K)) * 0.02).astype(np.float32), G))
    x = dev(rng.standard_normal((1, rows, K)).astype(np.float32))
    nw = dev((1.0 + 0.1 * rng.standard_normal(K)).astype(np.float32))
    whole = ops.fc_Q4A_decode(x, pw, N, norm=(nw, 1e-5))
    parts = ops.fc_Q4A_decode(x, pw, N, norm=(nw, 1e-5), out_parts=3)
    assert parts.shape == (3, 1, rows, 352) and parts.is_contiguous()
    for i in range(3):
        # (a third of the strips may be cut into tiles and k-splits differently from the whole: fp32 summation order)
        assert max_rel_err(host(parts[i]), host(whole[..., 352 * i:352 * (i + 1)])) <= 1e-5
    plain = ops.fc_Q4A_decode(x, pw, N, out_parts=3)
    assert max_rel_err(host(plain[1]), host(ops.fc_Q4A(x, pw, N)[..., 352:704])) <= 1e-5
    with pytest.raises(RuntimeError):
        ops.fc_Q4A_decode(x, pw, N, out_parts=4)  # 33 strips do not divide by 4


def test_fc_decode_many_rows_refuses_what_it_cannot_fold(ops, orc):
    """At the C ABI: interleaved gate/up strips on the output side (glu 1) need the 8-row kernel, and the
    silu(gate)*up producer needs group 128; both are refused before anything is enqueued (the Python op composes
    those cases from the separate ops instead)."""
    from llmops import _lib
    lib = _lib.load()
    rng = np.random.default_rng(3)
    K, F, rows = 256, 64, 12
    x = dev(rng.standard_normal((rows, 2 * K)).astype(np.float32))
    y = torch.full((rows, 2 * F), 7.0, device="cuda")
    for G, glu in ((128, 1), (32, 2)):
        pw = dev(orc.quant_w((rng.standard_normal((2 * F, K)) * 0.02).astype(np.float32), G))
        Ng, Kg, _ = pw.shape
        nbytes = lib.llmops_fc_Q4A_workspace_bytes(rows, K, Ng, Kg, G)
        ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        rc = lib.llmops_fc_Q4A_decode(x.data_ptr(), rows, K, pw.data_ptr(), Ng, Kg, G, F if glu == 1 else 2 * F, None, 0.0,
                                      None, glu, None, 0, None, y.data_ptr(), ws.data_ptr(), nbytes,
                                      torch.cuda.current_stream().cuda_stream)
        assert rc != 0
        torch.cuda.synchronize()
        assert bool((y == 7.0).all())
    # the Python op takes both
    pg = dev(orc.quant_w((rng.standard_normal((F, K)) * 0.02).astype(np.float32), 128))
    il = ops.interleave_gate_up(pg, pg)
    assert ops.fc_Q4A_decode(x[:, :K].reshape(1, rows, K).contiguous(), il, F, glu=True).shape == (1, rows, F)
    p32 = dev(orc.quant_w((rng.standard_normal((F, K)) * 0.02).astype(np.float32), 32))
    assert ops.fc_Q4A_decode(x.reshape(1, rows, 2 * K), p32, F, glu_in=True).shape == (1, rows, F)


@pytest.mark.parametrize("rows", [1, 2, 4, 5, 8])
@pytest.mark.parametrize("N,K", [(4096, 11008), (4090, 11008), (3000, 5632)])
def test_fc_two_k_splits_both_handoffs(ops, orc, rows, N, K):
    """Shapes the planner cuts into two k-splits per strip (fewer strips than compute units, long K): the
    splits meet through one 64-bit exchange per output (default) or through the arrival ticket.  Both
    against the oracle, bit-equal to each other, bit-equal over repeated launches (the slots are left
    empty), with and without the residual; ragged N (the padding columns never touch a slot)."""
    from llmops import _lib
    lib = _lib.load()
    rng = np.random.default_rng(rows + N)
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    res = rng.standard_normal((1, rows, N)).astype(np.float32)
    pw = dev(orc.quant_w(w, 128))
    want = orc.fc(x, host(pw), N)
    got = {}
    try:
        for knob in (-2, -3, -2):
            lib.llmops_test_fc_set_tuning(knob, -1)
            a = ops.fc_Q4A(dev(x), pw, N)
            b = ops.fc_Q4A(dev(x), pw, N)
            c = ops.fc_Q4A_decode(dev(x), pw, N, residual=dev(res))
            assert torch.equal(a, b)
            assert max_rel_err(host(a), want) <= 1e-5
            assert max_rel_err(host(c), want + res) <= 1e-5
            if got:
                assert torch.equal(a, got["a"]) and torch.equal(c, got["c"])
            got = {"a": a, "c": c}
    finally:
        lib.llmops_test_fc_set_tuning(-2, -1)


@pytest.mark.parametrize("rows", [3, 5, 8, 9, 13, 16, 17, 24, 32])
@pytest.mark.parametrize("N,K", [(4096, 11008), (4090, 4096), (2070, 2048), (3000, 2176)])
def test_fc_rows_kernel_two_k_halves(ops, orc, rows, N, K):
    """The weight-streaming MFMA kernel on tensors with fewer than 256 strips: two workgroups per strip with
    half of K each, meeting through one 64-bit exchange per output, against one workgroup per strip: both
    against the oracle, bit-equal over repeated launches, with and without the residual; ragged N, odd
    k-group counts (17 = 8 + 9)."""
    from llmops import _lib
    lib = _lib.load()
    rng = np.random.default_rng(rows + N)
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    res = rng.standard_normal((1, rows, N)).astype(np.float32)
    pw = dev(orc.quant_w(w, 128))
    want = orc.fc(x, host(pw), N)
    try:
        for on in (1, 0, 1):
            lib.llmops_test_fc_rows_set_split(on)
            a = ops.fc_Q4A(dev(x), pw, N)
            b = ops.fc_Q4A(dev(x), pw, N)
            c = ops.fc_Q4A(dev(x), pw, N, residual=dev(res))
            assert torch.equal(a, b)
            assert max_rel_err(host(a), want) <= 1e-5
            assert max_rel_err(host(c), want + res) <= 1e-5
    finally:
        lib.llmops_test_fc_rows_set_split(1)


@pytest.mark.parametrize("rows", [2, 3, 4, 6, 8])
@pytest.mark.parametrize("N,K", [(4096, 1024), (9000, 512), (8224, 4480)])
def test_fc_few_rows_either_kernel(ops, orc, rows, N, K):
    """2..8 rows at group 128 can run the streaming kernel that quantizes on the fly or the weight-streaming
    MFMA kernel behind a quantization launch (the row count at which the second takes over is a tuning
    knob): both against the oracle, with and without the residual, for a tensor on either side of 256
    strips and one whose 35 k-groups per workgroup take the MFMA kernel's 16-wave form."""
    from llmops import _lib
    lib = _lib.load()
    rng = np.random.default_rng(rows * 7 + N)
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    res = rng.standard_normal((1, rows, N)).astype(np.float32)
    pw = dev(orc.quant_w(w, 128))
    want = orc.fc(x, host(pw), N)
    try:
        for first in (9, 2, 0):  # streaming kernel for all of 2..8 rows; MFMA kernel from 2 rows; defaults
            lib.llmops_test_fc_set_row_routing(first, first)
            a = ops.fc_Q4A(dev(x), pw, N)
            c = ops.fc_Q4A(dev(x), pw, N, residual=dev(res))
            assert max_rel_err(host(a), want) <= 1e-5
            assert max_rel_err(host(c), want + res) <= 1e-5
    finally:
        lib.llmops_test_fc_set_row_routing(0, 0)


@pytest.mark.parametrize("rows", [17, 48, 100, 128, 129, 200, 256])
@pytest.mark.parametrize("N,K", [(2070, 1024), (4096, 640), (2048, 2816)])
def test_fc_prefill_mid_rows_vs_oracle(ops, orc, rows, N, K):
    """17..256 rows at group 128 as the planner runs them (tiling and split-K factor chosen per shape):
    ragged rows, N not a multiple of 32, k-group counts 8, 5 and 22 (splits of unequal length): output
    and residual epilogue against the oracle, the closed-form construction exactly."""
    rng = np.random.default_rng(rows + N)
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    res = rng.standard_normal((1, rows, N)).astype(np.float32)
    pw = orc.quant_w(w, 128)
    want = orc.fc(x, pw, N)
    assert max_rel_err(host(ops.fc_Q4A(dev(x), dev(pw), N)), want) <= 1e-5
    assert max_rel_err(host(ops.fc_Q4A(dev(x), dev(pw), N, residual=dev(res))), want + res) <= 1e-5
    xe, we = oracle.closed_form_fc_inputs(rows, N, K, seed=rows)
    ye = host(ops.fc_Q4A(dev(xe.reshape(1, rows, K)), ops.offline_FC_quant_Q4A(dev(we), 128), N))
    assert np.array_equal(ye, (xe.astype(np.float64) @ we.astype(np.float64).T).astype(np.float32).reshape(1, rows, N))


@pytest.mark.parametrize("tiling", [1, 2, 4, 8])
@pytest.mark.parametrize("rows,N,K", [(70, 2070, 1024), (300, 2070, 1024), (515, 352, 4096), (1024, 4096, 512)])
def test_fc_prefill_every_tiling_vs_oracle(ops, orc, tiling, rows, N, K):
    """The group-128 MFMA kernels with each row tiling forced in turn (32, 64, 128 rows per workgroup, and
    the 256-row kernel whose two wave groups alternate phases), on shapes with ragged row and column
    edges, with and without split-K: output against the oracle, the residual epilogue, and the
    closed-form construction exactly."""
    from llmops import _lib
    lib = _lib.load()
    rng = np.random.default_rng(rows + N + tiling)
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    res = rng.standard_normal((1, rows, N)).astype(np.float32)
    pw = orc.quant_w(w, 128)
    want = orc.fc(x, pw, N)
    xe, we = oracle.closed_form_fc_inputs(rows, N, K, seed=rows)
    lib.llmops_test_gemm_set_tuning(tiling)
    try:
        got = host(ops.fc_Q4A(dev(x), dev(pw), N))
        got_res = host(ops.fc_Q4A(dev(x), dev(pw), N, residual=dev(res)))
        ye = host(ops.fc_Q4A(dev(xe.reshape(1, rows, K)), ops.offline_FC_quant_Q4A(dev(we), 128), N))
    finally:
        lib.llmops_test_gemm_set_tuning(0)
    assert max_rel_err(got, want) <= 1e-5
    assert max_rel_err(got_res, want + res) <= 1e-5
    assert np.array_equal(ye, (xe.astype(np.float64) @ we.astype(np.float64).T).astype(np.float32).reshape(1, rows, N))


@pytest.mark.parametrize("split", [0, 3])
@pytest.mark.parametrize("K", [1024, 5120, 11008])
def test_fc_prefill_min_term_at_any_activation_scale(ops, orc, K, split):
    """The 256-row kernel forms the min term sum_kg m * gsum once per tile from fp16 halves of the group
    sums, 32 k-groups per MFMA, and falls back to fp32 MFMAs for a round in which some row's sums are too
    small or too large for that.  Rows of ordinary, tiny, huge and zero activations side by side; 8
    k-groups (a quarter of one MFMA's 32), 40 (a short second batch of 32) and 86 (a short third), with
    and without split-K (splits that start off a multiple of 8): every ROW to 1e-5 of its own largest
    output, which is what the fallback exists for."""
    from llmops import _lib
    lib = _lib.load()
    rows, N = 300, 1056
    rng = np.random.default_rng(K + split)
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    x[0, 100:200] *= 1e-4      # group sums far below 1/8
    x[0, 200:290] *= 3000.0    # group sums beyond fp16
    x[0, 290:] = 0.0
    x[0, 5, 128:256] = 0.0     # a zero k-group inside an ordinary row
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    pw = orc.quant_w(w, 128)
    want = orc.fc(x, pw, N)
    lib.llmops_test_gemm_set_tuning(8)
    lib.llmops_test_gemm_set_split(split)
    try:
        got = host(ops.fc_Q4A(dev(x), dev(pw), N))
    finally:
        lib.llmops_test_gemm_set_tuning(0)
        lib.llmops_test_gemm_set_split(0)
    scale = np.abs(want[0]).max(axis=1)
    err = np.abs(got[0] - want[0]).max(axis=1)
    assert np.all(err[290:] == 0.0)
    assert np.all(err[:290] <= 1e-5 * scale[:290]), (err[:290] / scale[:290]).max()


@pytest.mark.parametrize("rows", [9, 12, 16])
@pytest.mark.parametrize("N,K", [(2070, 1024), (4096, 4096)])
def test_fc_rows_9_to_16_streaming_mfma(ops, orc, rows, N, K):
    """9..16 rows at group 128 with at least 64 strips take the weight-streaming MFMA kernel
    (one strip per workgroup): output and residual epilogue against the oracle, N not a multiple of 32."""
    rng = np.random.default_rng(rows + N)
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    res = rng.standard_normal((1, rows, N)).astype(np.float32)
    pw = orc.quant_w(w, 128)
    want = orc.fc(x, pw, N)
    assert max_rel_err(host(ops.fc_Q4A(dev(x), dev(pw), N)), want) <= 1e-5
    assert max_rel_err(host(ops.fc_Q4A(dev(x), dev(pw), N, residual=dev(res))), want + res) <= 1e-5


# ---- ops enqueued on different streams run at the same time and must not share scratch ------------------
def test_fc_on_concurrent_streams_matches_serial(ops):
    G = 128
    rng = np.random.default_rng(11)
    # 4096x11008 is the shape whose k-splits meet through the workspace; 8 rows goes through the prefill pieces
    cases = []
    for N, K, M in [(4096, 11008, 1), (4096, 4096, 1), (4096, 11008, 8), (1024, 11008, 16)]:
        w = dev((rng.standard_normal((N, K)) * 0.02).astype(np.float32))
        cases.append((ops.offline_FC_quant_Q4A(w, G), dev(rng.standard_normal((1, M, K)).astype(np.float32)), N))
    serial = [ops.fc_Q4A(x, wq, N) for wq, x, N in cases]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(3)]
    got = [[] for _ in streams]
    for rep in range(20):
        for si, s in enumerate(streams):
            with torch.cuda.stream(s):
                wq, x, N = cases[(rep + si) % len(cases)]
                got[si].append(((rep + si) % len(cases), ops.fc_Q4A(x, wq, N)))
    torch.cuda.synchronize()
    for per_stream in got:
        for ci, y in per_stream:
            assert torch.equal(y, serial[ci]), ci


# ---- split-K of the prefill GEMM: partial sums added by the product kernel itself or by a second launch ------
@pytest.mark.parametrize("M,N,K", [(128, 11008, 4096), (128, 4096, 11008), (96, 4090, 4096), (40, 1000, 11008), (256, 4096, 11008),
                                   (512, 4096, 11008), (33, 352, 2048), (300, 4090, 11008), (700, 1000, 4096)])
def test_gemm_split_k_reduced_in_kernel_equals_second_launch(ops, M, N, K):
    from llmops import _lib
    lib = _lib.load()
    rng = np.random.default_rng(M + N)
    wq = ops.offline_FC_quant_Q4A(dev((rng.standard_normal((N, K)) * 0.02).astype(np.float32)), 128)
    x = dev(rng.standard_normal((1, M, K)).astype(np.float32))
    res = dev(rng.standard_normal((1, M, N)).astype(np.float32))
    try:
        lib.llmops_test_gemm_set_reduce(0)
        want, want_res = ops.fc_Q4A(x, wq, N), ops.fc_Q4A(x, wq, N, residual=res)
        for mode in (1, 100):                                     # default rule; every split count (several load batches)
            lib.llmops_test_gemm_set_reduce(mode)
            # The planner prices the two ways of adding differently, so the tile size and split count, and with
            # them the order of the fp32 additions, may differ from the second-launch run: equal to rounding.
            # Within a mode the result must not depend on which split arrives last: bit-identical repeats.
            first, first_res = ops.fc_Q4A(x, wq, N), ops.fc_Q4A(x, wq, N, residual=res)
            assert max_rel_err(host(first), host(want)) <= 1e-5
            assert max_rel_err(host(first_res), host(want_res)) <= 1e-5
            for _ in range(3):                                    # the arrival counters are left at zero for the next call
                assert torch.equal(ops.fc_Q4A(x, wq, N), first)
                assert torch.equal(ops.fc_Q4A(x, wq, N, residual=res), first_res)
    finally:
        lib.llmops_test_gemm_set_reduce(1)
    # and the decode kernels, which share the counters, still find them at zero
    y1 = ops.fc_Q4A(x[:, :1].contiguous(), wq, N)
    assert torch.equal(y1, ops.fc_Q4A(x[:, :1].contiguous(), wq, N))
    assert max_rel_err(host(y1)[0, 0], host(want)[0, 0]) <= TOL


# ---- K that is not a whole number of k-groups (nor of eights) ---------------------------------------------------
@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("rows,K", [(1, 5), (3, 100), (2, 333), (17, 1001), (5, 4100)])
def test_quant_x_short_last_group(ops, orc, G, rows, K):
    """codes (zero padded; the last K % 8 values rounded half away from zero like the reference's scalar tail),
    scales and left-to-right sums bit for bit"""
    rng = np.random.default_rng(K + G + rows)
    x = rng.standard_normal((rows, K)).astype(np.float32)
    last = (K - 1) // G * G
    x[0, last:] = 0
    x[0, last] = 127.0
    ties = np.array([2.5, 3.5, -2.5, -0.5, 0.5, 1.5, -3.5], np.float32)
    n = min(len(ties), K - last - 1)
    x[0, K - n:] = ties[:n]
    xq, xd, gs = ops.FC_dynamic_quantize_x(dev(x), G)
    wq, wd, wg = orc.quant_x(x, G)
    assert np.array_equal(host(xq), wq)
    assert np.array_equal(host(xd).view(np.uint32), wd.view(np.uint32))
    assert np.array_equal(host(gs).view(np.uint32), wg.view(np.uint32))


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("rows,N,K", [(1, 4096, 4100), (2, 100, 1001), (8, 352, 333), (17, 96, 1001), (300, 160, 700),
                                      (300, 160, 1100), (300, 160, 5000)])
def test_fc_short_last_group(ops, orc, G, rows, N, K):
    """fc_Q4A with K not a multiple of the group size, on the kernels of few and of many rows, with and without
    the residual epilogue, against the oracle (whose tail handling is pinned by the reference build)."""
    rng = np.random.default_rng(rows + N + K + G)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    pw = orc.quant_w(w, G)
    assert np.array_equal(host(ops.offline_FC_quant_Q4A(dev(w), G)), pw)
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    res = rng.standard_normal((1, rows, N)).astype(np.float32)
    want = orc.fc(x, pw, N)
    assert max_rel_err(host(ops.fc_Q4A(dev(x), dev(pw), N)), want) <= 1e-5
    assert max_rel_err(host(ops.fc_Q4A(dev(x), dev(pw), N, residual=dev(res))), want + res) <= 1e-5


@pytest.mark.parametrize("rows,N,K", [(300, 160, 1100), (300, 160, 5000), (513, 352, 4100)])
def test_fc_256_row_kernel_short_last_group(ops, orc, rows, N, K):
    """The 256-row kernel (forced) on a K that is not a whole number of k-groups: its min-term prologue reads a
    row's group sums eight at a time from rows of 9, 40 and 33 floats (4-byte aligned only), the last k-group
    is zero padded by the quantization."""
    from llmops import _lib
    lib = _lib.load()
    rng = np.random.default_rng(rows + N + K)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    pw = orc.quant_w(w, 128)
    x = rng.standard_normal((1, rows, K)).astype(np.float32)
    res = rng.standard_normal((1, rows, N)).astype(np.float32)
    want = orc.fc(x, pw, N)
    lib.llmops_test_gemm_set_tuning(8)
    try:
        got = host(ops.fc_Q4A(dev(x), dev(pw), N))
        got_res = host(ops.fc_Q4A(dev(x), dev(pw), N, residual=dev(res)))
    finally:
        lib.llmops_test_gemm_set_tuning(0)
    assert max_rel_err(got, want) <= 1e-5
    assert max_rel_err(got_res, want + res) <= 1e-5


@pytest.mark.parametrize("rows,N,K", [(1, 4096, 4096), (2, 4096, 11008), (1, 1000, 2048), (5, 352, 512), (40, 4096, 4096)])
def test_fc_residual_in_place(ops, rows, N, K):
    """y = fc_Q4A(x) + y, the add in place the reference's iadd does (ops/op_misc.hpp:55-79): residual and y one
    buffer, on the one-launch kernels of few rows (with and without k-splits) and on the MFMA kernel: bit-equal to
    the call with a separate residual.  With a short last k-group and few rows the add is a second launch: refused."""
    rng = np.random.default_rng(rows * 7 + N + K)
    G = 128
    wq = ops.offline_FC_quant_Q4A(dev((rng.standard_normal((N, K)) * 0.02).astype(np.float32)), G)
    x = dev(rng.standard_normal((1, rows, K)).astype(np.float32))
    res = dev(rng.standard_normal((1, rows, N)).astype(np.float32))
    want = ops.fc_Q4A(x, wq, N, residual=res)
    lib = ops._lib.load()
    Ng, Kg, _ = wq.shape

    def in_place(xx, kk):
        y = res.clone()
        ws = ops._workspace(xx.device, lib.llmops_fc_Q4A_workspace_bytes(rows, kk, Ng, Kg, G))
        rc = lib.llmops_fc_Q4A_residual(ops._ptr(xx), rows, kk, ops._ptr(wq), Ng, Kg, G, N, ops._ptr(y), ops._ptr(y),
                                        ops._ptr(ws), ws.numel(), ops._stream(xx))
        return rc, y

    for _ in range(3):
        rc, y = in_place(x, K)
        assert rc == 0 and torch.equal(y, want)
    if rows <= 8:
        rc, y = in_place(x[:, :, :K - 3].contiguous(), K - 3)
        assert rc == 1 and b"residual must not be y" in lib.llmops_last_error()        # LLMOPS_EINVAL
        assert torch.equal(y, res)                                                     # nothing was launched
