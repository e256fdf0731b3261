"""Writes the golden vectors under tests/golden/ from the reference's own kernels.

Runs only where ``oracle/_ref`` has been built from /root/reference (``make -C oracle ref``);
the fixtures it writes are plain arrays (inputs and the reference's outputs) and are committed,
so the tests that read them need neither the reference nor this script.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.abspath(os.path.join(HERE, "..", "..")))
import oracle  # noqa: E402


def fc_case(G, seed):
    R = oracle.Reference(G)
    rng = np.random.default_rng(seed)
    N, K, rows = 64, 512, 6
    w = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
    # special weight groups: constant group (d == 0), a group with exact .5 ties, huge range
    w[3, 0:G] = 0.0123
    w[4, 0:G] = np.float32(0.25) * (rng.integers(0, 31, G) / 2).astype(np.float32)  # codes k/2 -> ties at .5
    w[4, 0] = 0.0
    w[4, 1] = np.float32(0.25 * 15)
    w[5, G:2 * G] *= 1000.0
    x = rng.standard_normal((rows, K)).astype(np.float32)
    # special activation rows: zero group, RNE ties (amax = 127 -> id = 1), tiny values, one-hot
    x[1, 0:G] = 0.0
    x[2, 0:G] = (rng.integers(-250, 250, G) / 2).astype(np.float32)
    x[2, 0] = 127.0
    x[2, 1:6] = [2.5, 3.5, -2.5, -3.5, 0.5]
    x[3] *= 1e-20
    x[4] = 0.0
    x[4, 7] = -3.0
    wq = R.quant_w(w)
    xq, xd, gs = R.quant_x(x)
    y = R.fc(x, wq, N)
    dq = R.dequant_w(wq)
    return dict(w=w, x=x, wq=wq, xq=xq, xd=xd, gsum=gs, y=y, dq=dq)


def attn_case(seed, qL, past, maxlen, half, fp16_round=False):
    R = oracle.Reference(128, fresh=True)
    rng = np.random.default_rng(seed)
    B, H, S, layers = 1, 2, 128, 2
    q = rng.standard_normal((B, qL, H * S)).astype(np.float32)
    k = rng.standard_normal((B, qL, H * S)).astype(np.float32)
    v = rng.standard_normal((B, qL, H * S)).astype(np.float32)
    cache = rng.standard_normal((2 * layers, B, H, maxlen, S)).astype(np.float32)
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, 2 * half, 2, dtype=np.float32) / np.float32(2 * half)))).astype(np.float32)
    slots = ((np.arange(qL) + past) % maxlen).astype(np.int32)
    out, k_rot, cache_after = R.attention(q, k, v, inv_freq, cache, slots, past, 1, version=2)
    out1, _, _ = R.attention(q, k, v, inv_freq, cache, slots, past, 1, version=1)
    return dict(q=q, k=k, v=v, cache=cache, inv_freq=inv_freq, slots=slots, position_id=np.int32(past),
                layer_id=np.int32(1), out=out, out_v1=out1, k_rot=k_rot, cache_after=cache_after)


def misc_case(seed):
    R = oracle.Reference(32, fresh=True)
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((1, 3, 256)).astype(np.float32)
    wn = rng.standard_normal(256).astype(np.float32)
    sm_in = (rng.random((5, 69)).astype(np.float32) - 0.5)
    lit = np.array([0.66046, 0.61789, -0.289624, 0.799137, -0.715343, 0.321021, 1.47277, -3.40282e+38], dtype=np.float32)
    emb = rng.standard_normal((11, 64)).astype(np.float32)
    ids = rng.integers(0, 11, (2, 3)).astype(np.int64)
    eq, es = R.embedding_q8c_quant_w(emb)
    half = 32
    inv_freq = (1.0 / (10000.0 ** (np.arange(0, 2 * half, 2, dtype=np.float32) / np.float32(2 * half)))).astype(np.float32)
    rx = rng.random((2, 3, 5, 128)).astype(np.float32)
    return dict(x=x, wn=wn, rms=R.rmsnorm(x, wn, 1e-5), silu=R.silu(x), sm_in=sm_in, sm=R.softmax(sm_in), lit=lit,
                sm_lit=R.softmax(lit[None])[0], emb=emb, ids=ids, eq=eq, es=es, emb_out=R.embedding_q8c(ids, eq, es),
                rope_x=rx, rope_inv_freq=inv_freq, rope_out=R.rope(rx, inv_freq, 16),
                iadd=R.iadd(x, x[:, ::-1].copy()), imul_row=R.imul(x, wn))


def main():
    for G in (32, 128):
        np.savez_compressed(os.path.join(HERE, f"fc_g{G}.npz"), **fc_case(G, 100 + G))
    np.savez_compressed(os.path.join(HERE, "attn_decode.npz"), **attn_case(7, qL=1, past=37, maxlen=48, half=64))
    np.savez_compressed(os.path.join(HERE, "attn_decode_wrap.npz"), **attn_case(8, qL=1, past=100, maxlen=48, half=32))
    np.savez_compressed(os.path.join(HERE, "attn_chunk.npz"), **attn_case(9, qL=5, past=20, maxlen=48, half=64))
    np.savez_compressed(os.path.join(HERE, "attn_prefill.npz"), **attn_case(10, qL=19, past=0, maxlen=48, half=64))
    np.savez_compressed(os.path.join(HERE, "misc.npz"), **misc_case(11))
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)))


if __name__ == "__main__":
    main()
