"""TEST INFRASTRUCTURE ONLY -- numpy/ctypes front end of the CPU checkers.

Two checkers with one calling convention (numpy arrays in, numpy arrays out):

* :class:`Oracle`    -- this repository's own plain-C restatement (``oracle/llmops_oracle.c``),
                        group size chosen at run time.  Always available once built.
* :class:`Reference` -- the reference's own kernels compiled from ``/root/reference/ops`` by
                        ``oracle/Makefile`` into ``oracle/_ref/`` (group size fixed per library).
                        Available only where those binaries exist.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import this package.  The shipped library never does.
"""
import ctypes
import os
import shutil
import subprocess
import tempfile

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_BUILD = os.path.join(_HERE, "_build")
_REF = os.path.join(_HERE, "_ref")

_i64 = ctypes.c_int64
_int = ctypes.c_int
_f32 = ctypes.c_float


def _p(a):
    return ctypes.c_void_p(a.ctypes.data)


def _isa():
    try:
        with open("/proc/cpuinfo") as f:
            flags = f.read()
    except OSError:
        return "avx2"
    return "vnni" if " avx_vnni" in flags else "avx2"


def build(ref=True, force=False):
    """Compile the checkers (gcc/g++ only).  ``ref`` also builds oracle/_ref when the reference
    sources are present on this machine.  ``force`` recompiles what is already built."""
    flags = ["-B"] if force else []
    subprocess.check_call(["make", "-s"] + flags + ["-C", _HERE, "oracle"])
    if ref and os.path.isdir("/root/reference/ops"):
        subprocess.check_call(["make", "-s"] + flags + ["-C", _HERE, "ref"])


def block_bytes(G):
    return (G // 8) * 128 + 128


def _c32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class Oracle:
    kind = "port"

    def __init__(self, isa=None):
        isa = isa or _isa()
        path = os.path.join(_BUILD, f"liboracle_{isa}.so")
        if not os.path.exists(path):
            build(ref=False)
        self.lib = ctypes.CDLL(path)
        self.lib.orc_fp16_to_fp32.restype = _f32
        self.lib.orc_fp16_to_fp32.argtypes = [ctypes.c_uint16]
        self.lib.orc_fp32_to_fp16.restype = ctypes.c_uint16
        self.lib.orc_fp32_to_fp16.argtypes = [_f32]
        self.lib.orc_block_bytes.restype = _i64
        self.isa = isa

    def max_threads(self):
        return self.lib.orc_max_threads()

    def set_threads(self, n):
        """OpenMP threads of the calls that follow (0 = one per processor)"""
        self.lib.orc_set_threads(int(n))

    def fp32_to_fp16_bits(self, a):
        a = _c32(a).ravel()
        return np.array([self.lib.orc_fp32_to_fp16(float(v)) for v in a], dtype=np.uint16)

    def fp16_bits_to_fp32(self, h):
        return np.array([self.lib.orc_fp16_to_fp32(int(v)) for v in np.asarray(h).ravel()], dtype=np.float32)

    def quant_w(self, w, G):
        w = _c32(w)
        N, K = w.shape
        Ng, Kg = -(-N // 32), -(-K // G)
        out = np.empty((Ng, Kg, block_bytes(G)), dtype=np.int8)
        self.lib.orc_quant_w(_p(w), _i64(N), _i64(K), _int(G), _p(out))
        return out

    def dequant_w(self, wq):
        wq = np.ascontiguousarray(wq, dtype=np.int8)
        Ng, Kg, bb = wq.shape
        G = group_of_block(bb)
        out = np.empty((Ng * 32, Kg * G), dtype=np.float32)
        self.lib.orc_dequant_w(_p(wq), _i64(Ng), _i64(Kg), _int(G), _p(out))
        return out

    def unpack_codes(self, wq):
        wq = np.ascontiguousarray(wq, dtype=np.int8)
        Ng, Kg, bb = wq.shape
        G = group_of_block(bb)
        out = np.empty((Ng * 32, Kg * G), dtype=np.uint8)
        self.lib.orc_unpack_codes(_p(wq), _i64(Ng), _i64(Kg), _int(G), _p(out))
        return out

    def quant_x(self, x, G):
        x = _c32(x)
        lead, K = x.shape[:-1], x.shape[-1]
        rows = int(np.prod(lead)) if lead else 1
        Kg = -(-K // G)
        xq = np.empty(lead + (Kg * G,), dtype=np.int8)
        xd = np.empty(lead + (Kg,), dtype=np.float32)
        gs = np.empty(lead + (Kg,), dtype=np.float32)
        self.lib.orc_quant_x(_p(x), _i64(rows), _i64(K), _int(G), _p(xq), _p(xd), _p(gs))
        return xq, xd, gs

    def fc_partials(self, xq, wq):
        xq = np.ascontiguousarray(xq, dtype=np.int8)
        wq = np.ascontiguousarray(wq, dtype=np.int8)
        Ng, Kg, bb = wq.shape
        G = group_of_block(bb)
        lead = xq.shape[:-1]
        rows = int(np.prod(lead)) if lead else 1
        assert xq.shape[-1] == Kg * G
        acc = np.empty(lead + (Ng * 32, Kg), dtype=np.int32)
        self.lib.orc_fc_partials(_p(xq), _i64(rows), _p(wq), _i64(Ng), _i64(Kg), _int(G), _p(acc))
        return acc

    def fc(self, x, wq, N):
        x = _c32(x)
        wq = np.ascontiguousarray(wq, dtype=np.int8)
        Ng, Kg, bb = wq.shape
        G = group_of_block(bb)
        lead, K = x.shape[:-1], x.shape[-1]
        rows = int(np.prod(lead)) if lead else 1
        y = np.empty(lead + (N,), dtype=np.float32)
        self.lib.orc_fc(_p(x), _i64(rows), _i64(K), _p(wq), _i64(Ng), _i64(Kg), _int(G), _i64(N), _p(y))
        return y

    # --- attention path -------------------------------------------------------------------
    def rope(self, x, inv_freq, position_id):
        x = _c32(x).copy()
        f = _c32(inv_freq)
        B, H, L, S = x.shape
        self.lib.orc_rope(_p(x), _i64(B), _i64(H), _i64(L), _i64(S), _p(f), _i64(f.shape[0]), _int(position_id))
        return x

    def attention(self, q, k, v, inv_freq, kv_cache, slots, position_id, layer_id, version=2):
        """Returns (out, k_rotated, kv_cache_after); inputs are not modified."""
        q, k, v = _c32(q).copy(), _c32(k).copy(), _c32(v).copy()
        cache = _c32(kv_cache).copy()
        f = _c32(inv_freq)
        s = np.ascontiguousarray(slots, dtype=np.int32)
        B, qL, HS = q.shape
        planes, _, H, maxlen, S = cache.shape
        assert HS == H * S
        self.lib.orc_attention(_p(q), _p(k), _p(v), _i64(B), _i64(qL), _i64(H), _i64(S), _p(f), _i64(f.shape[0]),
                               _p(cache), _i64(planes), _i64(maxlen), _p(s), _int(position_id), _int(layer_id))
        return q, k, cache

    def mm_qk(self, q, kcache, kvLen=None, q_is_bhqs=False):
        """attn_w [B,H,qL,kvLen]; q is [B,qL,H*S] (mm_qk, mm_qk81, mm_qk24) or [B,H,qL,S] (mm_qk42)"""
        q = _c32(q)
        kc = _c32(kcache)
        B, H, kmax, S = kc.shape
        kvLen = kmax if kvLen is None else int(kvLen)
        if q_is_bhqs:
            qL = q.shape[2]
            st = (H * qL * S, qL * S, S)
        else:
            qL = q.shape[1]
            st = (qL * H * S, S, H * S)
        out = np.empty((B, H, qL, kvLen), dtype=np.float32)
        self.lib.orc_mm_qk(_p(q), _i64(st[0]), _i64(st[1]), _i64(st[2]), _p(kc), _i64(kmax), _p(out), _i64(B), _i64(H),
                           _i64(qL), _i64(kvLen), _i64(S))
        return out

    def softmax(self, x):
        x = _c32(x).copy()
        K = x.shape[-1]
        self.lib.orc_softmax(_p(x), _i64(x.size // K), _i64(K))
        return x

    def rmsnorm(self, x, w, eps):
        x = _c32(x).copy()
        w = _c32(w)
        Hd = x.shape[-1]
        self.lib.orc_rmsnorm(_p(x), _i64(x.size // Hd), _i64(Hd), _p(w), _f32(eps))
        return x

    def iadd(self, a, b):
        a, b = _c32(a).copy(), _c32(b)
        inner = a.shape[-1]
        self.lib.orc_iadd(_p(a), _p(b), _i64(a.size // inner), _i64(inner), _int(b.ndim == 1))
        return a

    def imul(self, a, b):
        a, b = _c32(a).copy(), _c32(b)
        inner = a.shape[-1]
        self.lib.orc_imul(_p(a), _p(b), _i64(a.size // inner), _i64(inner), _int(b.ndim == 1))
        return a

    def silu(self, a):
        a = _c32(a).copy()
        self.lib.orc_silu(_p(a), _i64(a.size))
        return a

    def embedding_q8c_quant_w(self, w):
        w = _c32(w)
        V, E = w.shape
        q = np.empty((V, E), dtype=np.int8)
        s = np.empty((V,), dtype=np.float32)
        self.lib.orc_embedding_q8c_quant_w(_p(w), _i64(V), _i64(E), _p(q), _p(s))
        return q, s

    def embedding_q8c(self, ids, q, scales):
        ids = np.ascontiguousarray(ids, dtype=np.int64)
        q = np.ascontiguousarray(q, dtype=np.int8)
        scales = _c32(scales)
        E = q.shape[1]
        out = np.empty(ids.shape + (E,), dtype=np.float32)
        self.lib.orc_embedding_q8c(_p(out), _p(ids), _i64(ids.size), _p(q), _p(scales), _i64(E))
        return out


class Reference:
    """The reference's own compiled kernels (oracle/_ref).  ``G`` picks the library.

    ``fresh=True`` loads a private temporary copy of the shared object: the reference keeps a
    process-wide cos/sin table keyed by length only (ops/op_attn.hpp:15-17,45), so a new
    ``inv_freq`` needs fresh statics.
    """

    kind = "reference"

    def __init__(self, G, isa=None, fresh=False):
        isa = isa or _isa()
        path = os.path.join(_REF, f"libref_g{G}_{isa}.so")
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        self._tmp = None
        if fresh:
            fd, tmp = tempfile.mkstemp(suffix=".so", prefix="libref_")
            os.close(fd)
            shutil.copyfile(path, tmp)
            self._tmp = tmp
            path = tmp
        self.lib = ctypes.CDLL(path)
        self.lib.ref_last_error.restype = ctypes.c_char_p
        self.G = self.lib.ref_group_k()
        assert self.G == G and self.lib.ref_block_bytes() == block_bytes(G)
        self.isa = isa

    def __del__(self):
        if getattr(self, "_tmp", None):
            try:
                os.unlink(self._tmp)
            except OSError:
                pass

    @staticmethod
    def available(G=128, isa=None):
        return os.path.exists(os.path.join(_REF, f"libref_g{G}_{isa or _isa()}.so"))

    def max_threads(self):
        return self.lib.ref_max_threads()

    def set_threads(self, n):
        """OpenMP threads of the calls that follow (0 = one per processor)"""
        self.lib.ref_set_threads(int(n))

    def _chk(self, rc):
        if rc != 0:
            raise RuntimeError(self.lib.ref_last_error().decode())

    def quant_w(self, w, G=None):
        assert G in (None, self.G)
        w = _c32(w)
        N, K = w.shape
        Ng, Kg = -(-N // 32), -(-K // self.G)
        out = np.zeros((Ng, Kg, block_bytes(self.G)), dtype=np.int8)
        self._chk(self.lib.ref_offline_FC_quant_Q4A(_p(w), _i64(N), _i64(K), _p(out)))
        return out

    def dequant_w(self, wq):
        wq = np.ascontiguousarray(wq, dtype=np.int8)
        Ng, Kg, bb = wq.shape
        assert bb == block_bytes(self.G)
        out = np.empty((Ng * 32, Kg * self.G), dtype=np.float32)
        self._chk(self.lib.ref_offline_FC_dequant_Q4A(_p(wq), _i64(Ng), _i64(Kg), _p(out)))
        return out

    def quant_x(self, x, G=None):
        assert G in (None, self.G)
        x = _c32(x)
        if x.ndim == 2:
            x3 = x[None]
        else:
            x3 = x
        B, M, K = x3.shape
        Kg = -(-K // self.G)
        xq = np.empty((B, M, Kg * self.G), dtype=np.int8)
        xd = np.empty((B, M, Kg), dtype=np.float32)
        gs = np.empty((B, M, Kg), dtype=np.float32)
        self._chk(self.lib.ref_FC_dynamic_quantize_x(_p(x3), _i64(B), _i64(M), _i64(K), _p(xq), _p(xd), _p(gs)))
        if x.ndim == 2:
            return xq[0], xd[0], gs[0]
        return xq, xd, gs

    def fc(self, x, wq, N):
        x = _c32(x)
        x3 = x[None] if x.ndim == 2 else x
        wq = np.ascontiguousarray(wq, dtype=np.int8)
        Ng, Kg, bb = wq.shape
        assert bb == block_bytes(self.G)
        B, M, K = x3.shape
        # the reference stores 32 floats per strip regardless of N (ops/op_fc.hpp:416-419):
        # give it a padded row and cut afterwards.
        Np = Ng * 32
        if Np == N:
            y = np.empty((B, M, N), dtype=np.float32)
            self._chk(self.lib.ref_fc_Q4A(_p(x3), _i64(B), _i64(M), _i64(K), _p(wq), _i64(Ng), _i64(Kg), _int(N), _p(y)))
        else:
            raise ValueError("Reference.fc needs N % 32 == 0 (the reference overruns its output otherwise)")
        return y[0] if x.ndim == 2 else y

    def _warm_rope_table(self, f):
        """Grow the reference's static cos/sin table past 1 MiB on first use.  Smaller tables come
        from its thread-local buffer pool, whose deleter runs after the pool itself has been
        destroyed at process exit (static vs thread-local destruction order) and corrupts the
        heap; buffers of 1 MiB and more are plain malloc/free (ops/tensor.hpp:164-196)."""
        if getattr(self, "_warmed", False):
            return
        half = f.shape[0]
        pos = -(-(1 << 20) // (8 * half))
        dummy = np.zeros((1, 1, 1, 2 * half), dtype=np.float32)
        self._chk(self.lib.ref_rope_embed(_p(dummy), _i64(1), _i64(1), _i64(1), _i64(2 * half), _p(f), _i64(half), _int(pos)))
        self._warmed = True

    def rope(self, x, inv_freq, position_id):
        x = _c32(x).copy()
        f = _c32(inv_freq)
        self._warm_rope_table(f)
        B, H, L, S = x.shape
        self._chk(self.lib.ref_rope_embed(_p(x), _i64(B), _i64(H), _i64(L), _i64(S), _p(f), _i64(f.shape[0]), _int(position_id)))
        return x

    def attention(self, q, k, v, inv_freq, kv_cache, slots, position_id, layer_id, version=2):
        q, k, v = _c32(q).copy(), _c32(k).copy(), _c32(v).copy()
        cache = _c32(kv_cache).copy()
        f = _c32(inv_freq)
        s = np.ascontiguousarray(slots, dtype=np.int32)
        B, qL, HS = q.shape
        planes, _, H, maxlen, S = cache.shape
        self._warm_rope_table(f)
        self._chk(self.lib.ref_attention_rope(_int(version), _p(q), _p(k), _p(v), _i64(B), _i64(qL), _i64(H), _i64(S),
                                              _p(f), _i64(f.shape[0]), _p(cache), _i64(planes), _i64(maxlen), _p(s),
                                              _int(position_id), _int(layer_id)))
        return q, k, cache

    def mm_qk(self, q, kcache, kvLen=None, q_is_bhqs=False, variant=None):
        """variant: 0 mm_qk, 1 mm_qk42, 2 mm_qk81, 3 mm_qk24 (default: 1 for a [B,H,qL,S] query, else 0)"""
        q = _c32(q).copy()
        kc = _c32(kcache).copy()
        B, H, kmax, S = kc.shape
        kvLen = kmax if kvLen is None else int(kvLen)
        variant = (1 if q_is_bhqs else 0) if variant is None else variant
        assert (variant == 1) == bool(q_is_bhqs) and (variant == 1 or kvLen == kmax)
        qL = q.shape[2] if q_is_bhqs else q.shape[1]
        out = np.zeros((B, H, qL, kvLen), dtype=np.float32)
        self._chk(self.lib.ref_mm_qk(_int(variant), _p(q), _p(kc), _p(out), _i64(B), _i64(H), _i64(qL), _i64(kmax),
                                     _i64(kvLen), _i64(S)))
        return out

    def softmax(self, x):
        x = _c32(x).copy()
        K = x.shape[-1]
        self._chk(self.lib.ref_softmax(_p(x), _i64(x.size // K), _i64(K)))
        return x

    def rmsnorm(self, x, w, eps):
        x = _c32(x).copy()
        w = _c32(w)
        assert x.ndim == 3
        B, L, Hd = x.shape
        self._chk(self.lib.ref_rmsnorm(_p(x), _i64(B), _i64(L), _i64(Hd), _p(w), _f32(eps)))
        return x

    def iadd(self, a, b):
        a, b = _c32(a).copy(), _c32(b)
        inner = a.shape[-1]
        self._chk(self.lib.ref_iadd(_p(a), _p(b), _i64(a.size // inner), _i64(inner), _int(b.ndim == 1)))
        return a

    def imul(self, a, b):
        a, b = _c32(a).copy(), _c32(b)
        inner = a.shape[-1]
        self._chk(self.lib.ref_imul(_p(a), _p(b), _i64(a.size // inner), _i64(inner), _int(b.ndim == 1)))
        return a

    def silu(self, a):
        a = _c32(a).copy()
        inner = a.shape[-1]
        self._chk(self.lib.ref_itrans_silu(_p(a), _i64(a.size // inner), _i64(inner)))
        return a

    def embedding_q8c_quant_w(self, w):
        w = _c32(w)
        V, E = w.shape
        q = np.empty((V, E), dtype=np.int8)
        s = np.empty((V,), dtype=np.float32)
        self._chk(self.lib.ref_embedding_q8c_quant_w(_p(w), _i64(V), _i64(E), _p(q), _p(s)))
        return q, s

    def embedding_q8c(self, ids, q, scales):
        ids = np.ascontiguousarray(ids, dtype=np.int64)
        q = np.ascontiguousarray(q, dtype=np.int8)
        scales = _c32(scales)
        V, E = q.shape
        out = np.empty(ids.shape + (E,), dtype=np.float32)
        self._chk(self.lib.ref_embedding_q8c(_p(out), _p(ids), _i64(ids.size), _p(q), _p(scales), _i64(V), _i64(E)))
        return out


def group_of_block(bb):
    G = (bb - 128) // 16
    if G not in (32, 128) or block_bytes(G) != bb:
        raise ValueError(f"not a Q4_1 block size: {bb}")
    return G


def closed_form_fc_inputs(rows, N, K, seed=0):
    """The exactly-representable construction of ops/test_ops.py:115-123: weights are integers in
    [-8,7]/128 with -8 and 7 forced into every 32-group, inputs integers in [-127,127]/128 with
    +-127 forced, so d_w = 1/128, m = -1/16, d_x = 1/128 and x @ W.T is exact in fp32."""
    rng = np.random.default_rng(seed)
    w = rng.integers(-8, 8, (N, K)).astype(np.float32)
    x = rng.integers(-127, 128, (rows, K)).astype(np.float32)
    w[:, 0::32] = -8
    w[:, 1::32] = 7
    x[:, 0::32] = -127
    x[:, 1::32] = 127
    return x / 128, w / 128
