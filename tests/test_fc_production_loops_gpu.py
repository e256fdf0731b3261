"""Bit-level parity of the loops that actually serve requests, and the prefill GEMM at its headline sizes.

* The decode kernel of fc_Q4A (rows <= 8) quantizes its activations itself and has its own dot4 loop: its
  dump build (llmops_test_fc_decode_dump) stores the Q8 codes, scales and int32 sums it formed, compared
  here bit for bit with the oracle's FC_dynamic_quantize_x / integer core (ops/op_fc.hpp:221-272,337-363;
  quant_row_q8_0 ops/utils.hpp:200-220).  The raw group sum is a tree sum in that kernel (it feeds only the
  fp32 output, ops/op_fc.hpp:408) and is compared to rounding.
* The weight-streaming int8 MFMA kernel of 3..32 rows: its int32 sums (fc_Q4A_partials, use_mfma=3).
* Config 3 (group 128, M in {16,128,512,2048}, 4096->11008 and 11008->4096): the GPU output against the oracle
  on a sample of rows (FC rows are independent), and the 256-row kernel's int32 sums at 2048 rows.

Compared domain of the quantizer: finite activations whose group maximum is a normal fp32 number well inside the
range (|x| in about [1e-30, 1e30]).  NaN, infinities and groups so small that 1/d overflows go through x86's
"integer indefinite" conversion in the reference (ops/utils.hpp:206-214) and are not part of the contract."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import load_golden, max_rel_err

pytestmark = pytest.mark.gpu

TIE = [127, 2.5, 3.5, -2.5, -3.5, 0.5, 1.5, -0.5]      # RNE: 127 2 4 -2 -4 0 2 0 (half-away would give 3 4 -3 -4 1 2 -1)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def decode_dump(x, wq, N, G):
    """x fp32 [rows,K] (numpy), wq packed (numpy) -> y, xq, xd, gsum, acc of the production decode kernel"""
    import llmops
    from llmops import _lib
    lib = _lib.load()
    rows, K = x.shape
    Ng, Kg, _ = wq.shape
    tx, tw = dev(x), dev(wq)
    y = torch.full((rows, N), float("nan"), dtype=torch.float32, device="cuda")
    xq = torch.full((rows, Kg * G), 99, dtype=torch.int8, device="cuda")
    xd = torch.full((rows, Kg), float("nan"), dtype=torch.float32, device="cuda")
    gs = torch.full((rows, Kg), float("nan"), dtype=torch.float32, device="cuda")
    acc = torch.full((rows, Ng * 32, Kg), -(2 ** 31), dtype=torch.int32, device="cuda")
    ws = llmops._workspace(tx.device, lib.llmops_fc_Q4A_workspace_bytes(rows, K, Ng, Kg, G))
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    _lib.check(lib.llmops_test_fc_decode_dump(p(tx), rows, K, p(tw), Ng, Kg, G, N, p(y), p(xq), p(xd), p(gs), p(acc), p(ws),
                                              ws.numel(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    return [t.cpu().numpy() for t in (y, xq, xd, gs, acc)]


def check_dump(orc, x, wq, N, G):
    import llmops
    y, xq, xd, gs, acc = decode_dump(x, wq, N, G)
    oq, od, og = orc.quant_x(x, G)
    assert np.array_equal(xq, oq), "Q8 codes of the decode kernel differ from FC_dynamic_quantize_x"
    assert np.array_equal(xd.view(np.uint32), od.view(np.uint32)), "activation scales differ"
    assert np.abs(gs - og).max() <= 1e-5 * max(1.0, float(np.abs(x).max()) * G)
    assert np.array_equal(acc, orc.fc_partials(oq, wq)), "int32 sums of the decode kernel differ"
    # the dump build computes the same outputs as the kernel llmops.fc_Q4A launches, and both meet the oracle
    prod = llmops.fc_Q4A(dev(x[None]), dev(wq), N)[0].cpu().numpy()
    assert np.array_equal(y.view(np.uint32), prod.view(np.uint32))
    assert max_rel_err(y, orc.fc(x[None], wq, N)[0]) <= 1e-3
    return xq


@pytest.mark.parametrize("G", [32, 128])
def test_decode_kernel_on_golden_rows(orc, G):
    """the committed vectors written by the reference build (their rows hold tie cases and a zero group)"""
    g = load_golden(f"fc_g{G}.npz")
    x = g["x"].reshape(-1, g["x"].shape[-1])
    N = g["y"].shape[-1]
    for r0 in range(0, x.shape[0], 8):
        xs = x[r0:r0 + 8]
        y, xq, xd, gs, acc = decode_dump(xs, g["wq"], N, G)
        assert np.array_equal(xq, g["xq"].reshape(x.shape[0], -1)[r0:r0 + 8])
        assert np.array_equal(xd.view(np.uint32), g["xd"].reshape(x.shape[0], -1)[r0:r0 + 8].view(np.uint32))
        assert np.array_equal(acc, orc.fc_partials(xq, g["wq"]))
        assert max_rel_err(y, g["y"].reshape(x.shape[0], -1)[r0:r0 + 8]) <= 1e-3


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("rows", [1, 2, 3, 4, 8])
def test_decode_kernel_ties_zero_groups_and_scales(orc, G, rows):
    rng = np.random.default_rng(100 * G + rows)
    N, K = 352, 2048
    wq = orc.quant_w((rng.standard_normal((N, K)) * 0.02).astype(np.float32), G)
    x = rng.standard_normal((rows, K)).astype(np.float32)
    x[0, :8] = TIE
    x[0, 8:G] = 0                                  # amax = 127 -> d = 1: the products are the values themselves
    x[-1, G:2 * G] = 0                             # zero group: d = 0 -> id = 0 -> codes 0
    x[-1, 2 * G:3 * G] *= np.float32(1e-30)        # tiny but normal scale
    x[0, 3 * G:4 * G] *= np.float32(1e30)          # huge scale
    x[0, 4 * G] = -np.abs(x[0, 4 * G:5 * G]).max() * 2   # the group maximum is negative -> code -127
    x[-1, 5 * G:6 * G] = np.float32(0.3)           # constant group: every code 127
    x[-1, -G:] = -0.0                              # negative zeros
    xq = check_dump(orc, x, wq, N, G)
    assert list(xq[0, :8]) == [127, 2, 4, -2, -4, 0, 2, 0]
    assert xq[0, 4 * G] == -127 and (xq[-1, 5 * G:6 * G] == 127).all() and (xq[-1, G:2 * G] == 0).all()


@pytest.mark.parametrize("G,N,K", [(32, 4096, 4096),                       # config 1
                                   (128, 4096, 4096), (128, 11008, 4096), (128, 4096, 11008),   # config 2
                                   (32, 4096, 11008), (128, 2070, 1024), (32, 100, 320)])
def test_decode_kernel_config_shapes(orc, G, N, K):
    """one row at the BASELINE shapes (the k-splits of the 11008-long rows included) and ragged sizes"""
    rng = np.random.default_rng(N + K + G)
    wq = orc.quant_w((rng.standard_normal((N, K)) * 0.02).astype(np.float32), G)
    x = rng.standard_normal((1, K)).astype(np.float32)
    x[0, :8] = TIE
    x[0, 8:G] = 0
    check_dump(orc, x, wq, N, G)


@pytest.mark.parametrize("G,N,kgs", [(128, 64, [1, 2, 3, 5, 15, 16, 17, 31, 33, 43, 86, 87, 129]),     # many k-splits
                                     (128, 4096, [33, 43, 47, 80, 86, 87]),                            # two k-splits
                                     (128, 8192, [33, 43, 86, 87]),                                    # none
                                     (32, 64, [1, 3, 4, 5, 8, 9, 63, 65, 127, 344]), (32, 4096, [129, 131, 344])])
def test_decode_kernel_pass_distribution(orc, G, N, kgs):
    """The waves of a workgroup are dealt whole passes of 256 k-values (two blocks at group 128, eight at group
    32), the first few one more than the rest, and the last pass of a split may be partly empty: block counts on
    either side of every boundary of that split, with one, two and many k-splits, one and two rows."""
    rng = np.random.default_rng(G + N)
    for Kg in kgs:
        K = Kg * G
        wq = orc.quant_w((rng.standard_normal((N, K)) * 0.02).astype(np.float32), G)
        # (3..8 rows run 8-wave workgroups; with 64 strips or more and group 128 fc_Q4A sends them to the MFMA kernel,
        # whose output check_dump could not compare bit for bit)
        for rows in ((1, 2, 3, 5, 8) if (N < 2048 or G == 32) else (1, 2)):
            x = rng.standard_normal((rows, K)).astype(np.float32)
            x[0, :8] = TIE
            x[0, 8:G] = 0
            check_dump(orc, x, wq, N, G)


@pytest.mark.parametrize("rows", [3, 9, 16, 17, 32])
@pytest.mark.parametrize("N,K", [(4096, 4096), (4096, 11008), (12288, 4096), (2080, 1024)])
def test_streaming_mfma_kernel_int32_sums(orc, rows, N, K):
    """fc_rows_mfma_kernel (3..32 rows, group 128): every workgroup shape the launcher picks -- two k-halves per
    strip below 256 strips, 16 waves for long runs, two row tiles per wave from 17 rows on"""
    import llmops
    rng = np.random.default_rng(rows + N + K)
    wq = orc.quant_w((rng.standard_normal((N, K)) * 0.02).astype(np.float32), 128)
    xq = rng.integers(-127, 128, (rows, K)).astype(np.int8)
    xq[0, :128] = -127
    got = llmops.fc_Q4A_partials(dev(xq), dev(wq), use_mfma=3).cpu().numpy()
    assert np.array_equal(got, orc.fc_partials(xq, wq))


def sample_rows(M, rng):
    edges = [0, 1, 15, 16, 31, 32, 63, 64, 127, 128, 255, 256, M - 257, M - 256, M - 129, M - 128, M - 33, M - 2, M - 1]
    rows = {r for r in edges if 0 <= r < M}
    rows.update(int(r) for r in rng.integers(0, M, 4))
    return sorted(rows)


@pytest.mark.parametrize("M", [16, 128, 512, 2048])
@pytest.mark.parametrize("N,K", [(11008, 4096), (4096, 11008)])
def test_config3_prefill_gemm_full_size_vs_oracle(orc, M, N, K):
    """Config 3 at its published sizes through llmops.fc_Q4A (whatever kernel and split-K plan the library
    picks): sampled rows -- first and last rows of the first and last row tiles of every tiling -- against the
    oracle; gate 1e-3, observed and asserted <= 1e-5."""
    import llmops
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    x = rng.standard_normal((1, M, K)).astype(np.float32)
    wq = llmops.offline_FC_quant_Q4A(dev(w), 128)
    pw = orc.quant_w(w, 128)
    assert np.array_equal(wq.cpu().numpy(), pw)
    got = llmops.fc_Q4A(dev(x), wq, N).cpu().numpy()
    assert np.isfinite(got).all()
    rows = sample_rows(M, rng)
    want = orc.fc(np.ascontiguousarray(x[:, rows]), pw, N)
    assert max_rel_err(got[:, rows], want) <= 1e-5
    # every row and column, coarsely: x times the dequantized weights in fp64 on the device differs from the FC only
    # by the Q8 rounding of the activations (under 1 % of the output scale); a misplaced tile would be off by 100 %
    y64 = (dev(x)[0].double() @ llmops.offline_FC_dequant_Q4A(wq)[:N].double().T).cpu().numpy()
    assert max_rel_err(got[0], y64) < 0.03


@pytest.mark.parametrize("strips,K", [(4, 4096), (8, 11008)])
def test_config3_256_row_kernel_int32_sums_at_2048_rows(orc, strips, K):
    """fc_gemm_pp_kernel (use_mfma=2) at 2048 rows on a subset of strips: int32 sums of sampled rows bit-equal"""
    import llmops
    rng = np.random.default_rng(strips + K)
    M = 2048
    wq = orc.quant_w((rng.standard_normal((strips * 32, K)) * 0.02).astype(np.float32), 128)
    xq = rng.integers(-127, 128, (M, K)).astype(np.int8)
    xq[0, :128] = -127
    got = llmops.fc_Q4A_partials(dev(xq), dev(wq), use_mfma=2).cpu().numpy()
    rows = sample_rows(M, rng)
    assert np.array_equal(got[rows], orc.fc_partials(np.ascontiguousarray(xq[rows]), wq))


@pytest.mark.parametrize("tiling,splits", [(1, 2), (1, 12), (2, 5), (4, 3), (4, 12)])
@pytest.mark.parametrize("M,N,K", [(128, 11008, 4096), (128, 4096, 11008), (300, 4090, 11008)])
def test_gemm_split_k_in_kernel_reduce_bit_identical_to_second_launch(M, N, K, tiling, splits):
    """With the tiling pinned (row tile factor and split count forced) the partial sums are added in the same
    order by the product kernel's last arrival and by the second launch: identical bits."""
    import llmops
    from llmops import _lib
    lib = _lib.load()
    rng = np.random.default_rng(M + N + tiling)
    wq = llmops.offline_FC_quant_Q4A(dev((rng.standard_normal((N, K)) * 0.02).astype(np.float32)), 128)
    x = dev(rng.standard_normal((1, M, K)).astype(np.float32))
    res = dev(rng.standard_normal((1, M, N)).astype(np.float32))
    try:
        lib.llmops_test_gemm_set_tuning(tiling)
        lib.llmops_test_gemm_set_split(splits)
        lib.llmops_test_gemm_set_reduce(0)
        want, want_res = llmops.fc_Q4A(x, wq, N), llmops.fc_Q4A(x, wq, N, residual=res)
        lib.llmops_test_gemm_set_reduce(1)
        for _ in range(2):
            assert torch.equal(llmops.fc_Q4A(x, wq, N), want)
            assert torch.equal(llmops.fc_Q4A(x, wq, N, residual=res), want_res)
    finally:
        lib.llmops_test_gemm_set_reduce(1)
        lib.llmops_test_gemm_set_split(0)
        lib.llmops_test_gemm_set_tuning(0)


@pytest.mark.parametrize("G", [32, 128])
@pytest.mark.parametrize("scale", [1.0, 1e-6, 1e4, 1e-9, 7e4])
def test_pack_fp16_subnormal_and_overflowing_scales(orc, G, scale):
    """d and m are stored as fp16 (ops/op_fc.hpp:192-193): weights whose group range makes them subnormal halves
    (1e-6), zero halves (1e-9), or infinite halves (1e4 x 15 > 65504 only for m; 7e4 for both) must pack to the
    reference's bytes; the codes use the fp32 d and m and are unaffected."""
    import llmops
    rng = np.random.default_rng(int(G + abs(np.log10(scale)) * 10))
    w = (rng.standard_normal((96, 4 * G)) * scale).astype(np.float32)
    got = llmops.offline_FC_quant_Q4A(dev(w), G).cpu().numpy()
    want = orc.quant_w(w, G)
    assert np.array_equal(got, want)
    dq, ref = llmops.offline_FC_dequant_Q4A(dev(want)).cpu().numpy(), orc.dequant_w(want)
    # (inf * 0 + m: where both sides are NaN the payload bits are not compared)
    assert ((dq.view(np.uint32) == ref.view(np.uint32)) | (np.isnan(dq) & np.isnan(ref))).all()
