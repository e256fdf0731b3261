"""``llmops`` for MI355X -- drop-in for the reference's pybind11 module of the same name
(``PYBIND11_MODULE(llmops, m)``, /root/reference/ops/main.cpp:62-179).

Same op names, argument order, shapes, dtypes and in-place behaviour as the reference; the tensor
type at the boundary is a ``torch.Tensor`` on the HIP device instead of the reference's own
``llmops.tensor``.  Every op enqueues hand-written gfx950 kernels from ``libllmops_hip.so`` on the
current torch stream.  There is no CPU or eager fallback: a missing library or a host tensor
raises.

Differences a caller can see:
* The k-group size is a run-time choice (``group_k=32|128`` on ``offline_FC_quant_Q4A``, or
  ``set_default_group_k``) instead of a compile-time constant (ops/op_fc.hpp:109); the other ops
  recover it from the packed tensor's last dimension (640 -> 32, 2176 -> 128).
* ``attention_rope[2]`` also accepts a float16 ``kv_cache`` (fp32 math on fp16-rounded K/V).
* Errors are ``RuntimeError`` with the failed condition, like the reference's ``ASSERT``.
"""
import ctypes

import torch

from . import _lib

__all__ = [
    "offline_FC_quant_Q4A", "offline_FC_dequant_Q4A", "fc_Q4A", "fc_Q4A_noalloc", "fc_Q4A_decode", "interleave_gate_up", "FC_dynamic_quantize_x", "fc_Q4A_partials",
    "attention_rope", "attention_rope2", "attention_rope2_records", "attention_records_supported", "AttentionRecords", "rope_embed", "softmax", "rmsnorm", "iadd", "imul", "itrans", "clone",
    "rmsnorm_out", "silu_mul", "empty", "ones", "embedding", "embedding_q8c_quant_w", "embedding_q8c", "tensor_pool", "set_default_group_k", "reserve_workspace", "reset_workspaces",
    "group_k_of",
]

# Callers of the reference read ``tensor.item_size`` (chatllama/main.py:171-173, ops/perf_ops.py:242; bound at
# ops/main.cpp:95-142).  torch spells it ``itemsize`` / ``element_size()``; the reference's spelling is added as
# a read-only property so that such callers run unchanged on the tensors this module hands out.
if not hasattr(torch.Tensor, "item_size"):
    torch.Tensor.item_size = property(lambda self: self.element_size())

_default_group_k = 32  # the reference's compiled-in default (ops/op_fc.hpp:109)
_workspaces = {}
_captured = set()  # keys of workspaces whose address a stream capture has recorded
_retired = []  # superseded workspaces that a captured graph may still replay into


def set_default_group_k(g):
    global _default_group_k
    _require(g in (32, 128), "group_k in (32, 128)")
    _default_group_k = g


def _require(cond, what):
    if not cond:
        raise RuntimeError(f"assert {what} failed")


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _raw_stream(device):
    """hipStream_t of torch's current stream on `device`, as an int"""
    return torch._C._cuda_getCurrentRawStream(device.index if device.index is not None else torch.cuda.current_device())


def _stream(t):
    return ctypes.c_void_p(_raw_stream(t.device))


def _dev(t, dtype, rank=None, name="tensor"):
    _require(isinstance(t, torch.Tensor), f"{name} is a torch.Tensor")
    _require(t.is_cuda, f"{name} is on the HIP device (llmops has no CPU path)")
    _require(t.dtype == dtype, f"{name}.is<{dtype}>")
    if rank is not None:
        _require(t.dim() == rank, f"{name}.rank == {rank}")
    _require(t.is_contiguous(), f"{name}.is_dense()")


def _workspace(device, nbytes, kind="fc"):
    """Persistent scratch, one per op family, device and stream: ops enqueued on different streams may run
    at the same time and must not share counters or partial sums.  Its first bytes hold arrival counters,
    which must start at zero and which the kernels leave at zero.

    A HIP graph that captured an op replays the raw address of the workspace the op was given, so a workspace
    that a capture has seen is never freed: when a later call needs more, the old tensor is kept (``_retired``)
    and a larger one takes its place for the calls that follow.  A workspace no capture has seen is simply
    replaced, and sizes grow geometrically, so a serving loop whose prefill length creeps upward does not keep
    every intermediate size.  While the stream is capturing nothing may be
    allocated or zero-filled (the fill would be recorded into the graph, and the first replay could find
    counters that were never zeroed): an op that would need a new or larger workspace then raises.  Run the
    op once, at the largest size, on the stream that will capture -- or call ``reserve_workspace`` -- first."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    key = (kind, device.type, index, torch._C._cuda_getCurrentRawStream(index))
    ws = _workspaces.get(key)
    capturing = torch.cuda.is_current_stream_capturing()
    if capturing and ws is not None and ws.numel() >= nbytes:
        _captured.add(key)
    if ws is None or ws.numel() < nbytes:
        if capturing:
            raise RuntimeError(
                f"llmops: the {kind} workspace of this stream would have to be "
                f"{'created' if ws is None else 'enlarged'} ({int(nbytes)} bytes) while the stream is capturing a graph; "
                "run the op once on this stream before the capture, or call llmops.reserve_workspace")
        size = max(int(nbytes), 16 << 20)
        if ws is not None:
            size = max(size, 2 * ws.numel())
            if key in _captured:
                _retired.append(ws)  # a graph captured earlier may still replay its address
                _captured.discard(key)
            else:
                # work enqueued earlier on this stream may still use the old tensor; torch's allocator only hands its
                # memory out again to this same stream, i.e. behind that work
                del ws
        ws = torch.zeros(size, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def reserve_workspace(device=None, fc_bytes=0, attn_bytes=0):
    """Make sure the current stream's FC / attention workspaces on ``device`` hold at least this many bytes
    (``llmops_fc_Q4A_workspace_bytes`` / ``llmops_attention_workspace_bytes`` give the figures), so that a graph
    capture on this stream finds them in place."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    if fc_bytes:
        _workspace(device, fc_bytes, "fc")
    if attn_bytes:
        _workspace(device, attn_bytes, "attn")


def reset_workspaces():
    """Zero the hand-off areas (arrival counters, exchange slots) of every workspace this module holds.  The
    kernels leave them zero after every call that runs to its end; after a launch that did not (a device error in
    the middle of an op) call this once, with no op in flight, before using the module again."""
    torch.cuda.synchronize()
    lib = _lib.load()
    for ws in list(_workspaces.values()) + _retired:
        _lib.check(lib.llmops_fc_workspace_reset(_ptr(ws), ws.numel(), _stream(ws)))
    torch.cuda.synchronize()


def group_k_of(weiq):
    bb = weiq.shape[-1]
    g = (bb - 128) // 16
    _require(g in (32, 128) and (g // 8) * 128 + 128 == bb, "weiq.size(2) == sizeof(q4_block)")
    return g


# ---- Q4_1 fully connected ---------------------------------------------------------------------
def offline_FC_quant_Q4A(wei, group_k=None):
    """fp32 [N,K] -> int8 [ceil(N/32), ceil(K/G), blk(G)] (ops/op_fc.hpp:151-219)."""
    g = _default_group_k if group_k is None else group_k
    _require(g in (32, 128), "group_k in (32, 128)")
    _require(isinstance(wei, torch.Tensor) and wei.is_cuda, "wei is on the HIP device (llmops has no CPU path)")
    _require(wei.dtype == torch.float32 and wei.dim() == 2, "wei.is<float>(2)")
    _require(wei.stride(1) == 1, "wei inner dimension is contiguous")
    N, K = wei.shape
    lib = _lib.load()
    Ng, Kg = -(-N // 32), -(-K // g)
    out = torch.empty((Ng, Kg, lib.llmops_q4a_block_bytes(g)), dtype=torch.int8, device=wei.device)
    _lib.check(lib.llmops_offline_FC_quant_Q4A(_ptr(wei), N, K, wei.stride(0), g, _ptr(out), _stream(wei)))
    return out


def offline_FC_dequant_Q4A(weiq):
    """int8 [Ng,Kg,blk] -> fp32 [Ng*32, Kg*G] (ops/op_fc.hpp:124-149)."""
    _dev(weiq, torch.int8, 3, "weiq")
    g = group_k_of(weiq)
    Ng, Kg, _ = weiq.shape
    out = torch.empty((Ng * 32, Kg * g), dtype=torch.float32, device=weiq.device)
    _lib.check(_lib.load().llmops_offline_FC_dequant_Q4A(_ptr(weiq), Ng, Kg, g, _ptr(out), _stream(weiq)))
    return out


def FC_dynamic_quantize_x(input, group_k, rows_variant=False):
    """fp32 [..,K] -> (xq int8 [..,Kg*G], xd fp32 [..,Kg], gsum fp32 [..,Kg]) (ops/op_fc.hpp:221-272).
    ``rows_variant=True`` runs the kernel the prefill FC uses (same codes and scales, tree-summed gsum)."""
    _dev(input, torch.float32, None, "input")
    _require(group_k in (32, 128), "group_k in (32, 128)")
    K = input.shape[-1]
    lead = tuple(input.shape[:-1])
    rows = input.numel() // K
    Kg = -(-K // group_k)
    xq = torch.empty(lead + (Kg * group_k,), dtype=torch.int8, device=input.device)
    xd = torch.empty(lead + (Kg,), dtype=torch.float32, device=input.device)
    gs = torch.empty(lead + (Kg,), dtype=torch.float32, device=input.device)
    lib = _lib.load()
    fn = lib.llmops_FC_dynamic_quantize_x_rows if rows_variant else lib.llmops_FC_dynamic_quantize_x
    _lib.check(fn(_ptr(input), rows, K, group_k, _ptr(xq), _ptr(xd), _ptr(gs), _stream(input)))
    return xq, xd, gs


def fc_Q4A(input, weiq, N, residual=None):
    """fp32 [B,M,K] x packed [Ng,Kg,blk] -> fp32 [B,M,N] (ops/op_fc.hpp:286-426).
    ``residual`` (extension, fp32 [B,M,N]): returns fc_Q4A(input) + residual in the same launch."""
    _dev(input, torch.float32, 3, "input")
    _dev(weiq, torch.int8, 3, "wei_quantized")
    g = group_k_of(weiq)
    B, M, K = input.shape
    Ng, Kg, _ = weiq.shape
    rows = B * M
    lib = _lib.load()
    need = lib.llmops_fc_Q4A_workspace_bytes(rows, K, Ng, Kg, g)
    ws = _workspace(input.device, need)
    out = torch.empty((B, M, int(N)), dtype=torch.float32, device=input.device)
    if residual is None:
        _lib.check(lib.llmops_fc_Q4A(_ptr(input), rows, K, _ptr(weiq), Ng, Kg, g, int(N), _ptr(out), _ptr(ws), ws.numel(),
                                     _stream(input)))
    else:
        _dev(residual, torch.float32, 3, "residual")
        _require(tuple(residual.shape) == (B, M, int(N)), "residual.is({B, M, N})")
        _lib.check(lib.llmops_fc_Q4A_residual(_ptr(input), rows, K, _ptr(weiq), Ng, Kg, g, int(N), _ptr(residual), _ptr(out),
                                              _ptr(ws), ws.numel(), _stream(input)))
    return out


def fc_Q4A_noalloc(input, weiq, N, out):
    """Extension: fc_Q4A into a caller-provided ``out`` (fp32 [B,M,N]) without allocating anything -- the
    workspace is a fixed array inside the library (``llmops_fc_Q4A_noalloc``).  For callers that cannot
    allocate (graph capture, serving loops); sizes beyond the array raise.  Calls that overlap on one device race."""
    _dev(input, torch.float32, 3, "input")
    _dev(weiq, torch.int8, 3, "wei_quantized")
    _dev(out, torch.float32, 3, "out")
    g = group_k_of(weiq)
    B, M, K = input.shape
    Ng, Kg, _ = weiq.shape
    _require(tuple(out.shape) == (B, M, int(N)), "out.is({B, M, N})")
    _lib.check(_lib.load().llmops_fc_Q4A_noalloc(_ptr(input), B * M, K, _ptr(weiq), Ng, Kg, g, int(N), _ptr(out), _stream(input)))
    return out


def interleave_gate_up(gate_packed, up_packed):
    """Packed gate and up tensors [Ng,Kg,blk] -> one tensor [2*Ng,Kg,blk] with strips alternating
    gate, up, gate, up ... : the layout ``fc_Q4A_decode(..., glu=True)`` consumes."""
    _require(gate_packed.shape == up_packed.shape, "gate.shape() == up.shape()")
    return torch.stack((gate_packed, up_packed), dim=1).reshape(-1, *gate_packed.shape[1:]).contiguous()


def fc_Q4A_decode(input, weiq, N_out, norm=None, residual=None, glu=False, sumsq_in=None, want_sumsq=False,
                  glu_in=False, attn_records=None, out_parts=1):
    """Extension: fc_Q4A with its neighbours of the decode step folded in (one launch for B*M <= 8).

    norm=(weight, eps): input is rmsnorm'ed first;  residual: added to the result;
    glu=True: ``weiq`` holds interleaved gate/up strips (``interleave_gate_up``) and the result is
    silu(gate)*up with N_out = F columns.  glu_in=True: ``input`` is a gate|up row [B, M, 2K] (what an FC
    over the gate and up weights stacked along N leaves behind) and the FC runs on silu(gate)*up.
    attn_records=...: ``input`` is None and the FC's input is the output of decode attention still in chunk records
    (``attention_rope2_records``), merged as it is loaded.
    out_parts=p (more than 8 rows, plain or norm FC): the result comes as p dense tensors [p, B, M, N_out/p] (part i =
    columns i*N_out/p ..), e.g. q, k and v of a fused q|k|v projection, instead of one tensor to be cut up and copied.
    want_sumsq=True returns ``(out, sumsq)`` where ``sumsq``
    [B*M, strips] holds the sum of squares of every 32 outputs; passed as ``sumsq_in`` to the FC that
    rmsnorms ``out`` it saves that FC the pass over the row.  With more than 8 rows the rmsnorm or the
    silu(gate)*up runs inside the quantization launch (same codes as the separate ops give), the residual inside the
    product; shapes that launch does not take, and glu=True, are composed from the separate ops."""
    if attn_records is not None:
        # input = the attention output still in chunk records (attention_rope2_records); merged on the way in
        r = attn_records
        _dev(weiq, torch.int8, 3, "wei_quantized")
        _require(input is None and norm is None and not glu and not glu_in and sumsq_in is None, "attn_records: plain FC")
        _require(r.B == 1 and group_k_of(weiq) == 128 and weiq.shape[1] == r.H, "attn_records: one row, group 128, K = H*128")
        Ng, Kg, _ = weiq.shape
        N_out = int(N_out)
        if residual is not None:
            _dev(residual, torch.float32, 3, "residual")
            _require(tuple(residual.shape) == (1, 1, N_out), "residual.is({B, M, N})")
        lib = _lib.load()
        ws = _workspace(weiq.device, lib.llmops_fc_Q4A_workspace_bytes(1, Kg * 128, Ng, Kg, 128))
        out = torch.empty((1, 1, N_out), dtype=torch.float32, device=weiq.device)
        sumsq = torch.empty((1, Ng), dtype=torch.float32, device=weiq.device) if want_sumsq else None
        _lib.check(lib.llmops_fc_Q4A_decode_attn(_ptr(r.stats), _ptr(r.outs), r.chunks, r.H, _ptr(weiq), Ng, Kg, N_out,
                                                 _ptr(residual) if residual is not None else None,
                                                 _ptr(sumsq) if sumsq is not None else None, _ptr(out), _ptr(ws), ws.numel(),
                                                 _stream(weiq)))
        return (out, sumsq) if want_sumsq else out
    _dev(input, torch.float32, 3, "input")
    _dev(weiq, torch.int8, 3, "wei_quantized")
    g = group_k_of(weiq)
    B, M, K = input.shape
    Ng, Kg, _ = weiq.shape
    rows = B * M
    N_out = int(N_out)
    if glu_in:
        _require(K % 2 == 0 and norm is None and not glu, "glu_in: input.size(2) % 2 == 0, no norm, no glu")
        K //= 2
    if norm is not None:
        _dev(norm[0], torch.float32, 1, "norm weight")
        _require(norm[0].shape[0] == K, "weight.size(0) == K")
    if residual is not None:
        _dev(residual, torch.float32, 3, "residual")
        _require(tuple(residual.shape) == (B, M, N_out), "residual.is({B, M, N})")
    if sumsq_in is not None:
        _dev(sumsq_in, torch.float32, 2, "sumsq_in")
        _require(norm is not None and sumsq_in.shape[0] == rows, "sumsq_in.is({B*M, parts}) with norm")
    _require(not (want_sumsq and glu), "no sumsq with glu")
    fusable = K % g == 0 and input.data_ptr() % 16 == 0 and (norm is None or (K <= 16384 and norm[0].data_ptr() % 16 == 0)) \
        and (not glu_in or g == 128)
    if out_parts != 1 and (rows <= 8 or glu or not fusable):
        whole = fc_Q4A_decode(input, weiq, N_out, norm=norm, glu_in=glu_in, sumsq_in=sumsq_in)
        return torch.stack([c.contiguous() for c in whole.chunk(out_parts, dim=-1)])
    if rows > 8 and (glu or not fusable):
        # gate and up interleaved on the output side (or a shape the fused quantization does not take): separate ops
        x = input if norm is None else rmsnorm_out(input, norm[0], norm[1])
        if glu_in:
            x = silu_mul(input)
        lib = _lib.load()
        if glu:
            _require(N_out % 32 == 0, "F % 32 == 0")
            y = fc_Q4A(x, weiq, 2 * N_out)  # strips alternate gate, up
            act = torch.empty((B, M, N_out), dtype=torch.float32, device=input.device)
            _lib.check(lib.llmops_silu_mul_interleaved(_ptr(y), _ptr(act), rows, N_out, _stream(y)))
            return act
        out = fc_Q4A(x, weiq, N_out, residual=residual)
        if want_sumsq:
            sumsq = torch.empty((rows, Ng), dtype=torch.float32, device=input.device)
            _lib.check(lib.llmops_strip_sumsq(_ptr(out), rows, N_out, _ptr(sumsq), _stream(out)))
            return out, sumsq
        return out
    lib = _lib.load()
    ws = _workspace(input.device, lib.llmops_fc_Q4A_workspace_bytes(rows, K, Ng, Kg, g))
    if out_parts != 1:
        _require(rows > 8 and not glu and residual is None and not want_sumsq and Ng % out_parts == 0 and N_out == Ng * 32,
                 "out_parts: more than 8 rows, whole strips per part, no residual, no sumsq")
        out = torch.empty((out_parts, B, M, N_out // out_parts), dtype=torch.float32, device=input.device)
        _lib.check(lib.llmops_fc_Q4A_decode_parts(_ptr(input), rows, K, _ptr(weiq), Ng, Kg, g, N_out,
                                                  _ptr(norm[0]) if norm is not None else None,
                                                  float(norm[1]) if norm is not None else 0.0, 2 if glu_in else 0, out_parts,
                                                  _ptr(out), _ptr(ws), ws.numel(), _stream(input)))
        return out
    out = torch.empty((B, M, N_out), dtype=torch.float32, device=input.device)
    sumsq = torch.empty((rows, Ng), dtype=torch.float32, device=input.device) if want_sumsq else None
    _lib.check(lib.llmops_fc_Q4A_decode(_ptr(input), rows, K, _ptr(weiq), Ng, Kg, g, N_out,
                                        _ptr(norm[0]) if norm is not None else None, float(norm[1]) if norm is not None else 0.0,
                                        _ptr(residual) if residual is not None else None, 2 if glu_in else int(bool(glu)),
                                        _ptr(sumsq_in) if sumsq_in is not None else None,
                                        sumsq_in.shape[1] if sumsq_in is not None else 0,
                                        _ptr(sumsq) if sumsq is not None else None, _ptr(out), _ptr(ws),
                                        ws.numel(), _stream(input)))
    return (out, sumsq) if want_sumsq else out


def fc_Q4A_partials(xq, weiq, use_mfma=False):
    """The exact int32 core of fc_Q4A: int8 [..,Kg*G] x packed -> int32 [.., Ng*32, Kg]."""
    _dev(xq, torch.int8, None, "xq")
    _dev(weiq, torch.int8, 3, "wei_quantized")
    g = group_k_of(weiq)
    Ng, Kg, _ = weiq.shape
    _require(xq.shape[-1] == Kg * g, "xq.size(-1) == Kgroups * group_k")
    lead = tuple(xq.shape[:-1])
    rows = xq.numel() // (Kg * g)
    acc = torch.empty(lead + (Ng * 32, Kg), dtype=torch.int32, device=xq.device)
    _lib.check(_lib.load().llmops_fc_Q4A_partials(_ptr(xq), rows, _ptr(weiq), Ng, Kg, g, _ptr(acc), int(use_mfma),
                                                  _stream(xq)))
    return acc


# ---- attention --------------------------------------------------------------------------------
def rope_embed(x, inv_freq, position_id):
    """In place on fp32 [B,H,L,S] (ops/op_attn.hpp:44-94)."""
    _dev(x, torch.float32, 4, "x")
    _dev(inv_freq, torch.float32, 1, "inv_freq")
    B, H, L, S = x.shape
    _lib.check(_lib.load().llmops_rope_embed(_ptr(x), B, H, L, S, _ptr(inv_freq), inv_freq.shape[0], int(position_id),
                                            _stream(x)))


def attention_rope2(q, k, v, inv_freq, kv_cache, kvc_slots, position_id, layer_id):
    """q,k,v fp32 [B,qL,H*S]; kv_cache [2*layers,B,H,maxlen,S]; kvc_slots int32 [qL].
    In place: q <- attention output, k <- rotated k, cache rows updated (ops/op_attn.hpp:721-1029).
    Extension: with qL == 1, ``position_id`` may be an int32 tensor [1] on the device; the kernels then read the
    position (and the slot) from memory, so a HIP graph that captured the call serves every following token."""
    _dev(q, torch.float32, 3, "q")
    _dev(k, torch.float32, 3, "k")
    _dev(v, torch.float32, 3, "v")
    _require(isinstance(kv_cache, torch.Tensor) and kv_cache.is_cuda and kv_cache.dim() == 5 and kv_cache.is_contiguous(),
             "kv_cache.is<float>(5)")
    _require(kv_cache.dtype in (torch.float32, torch.float16), "kv_cache.is<float>(5)")
    _dev(kvc_slots, torch.int32, 1, "kvc_slots")
    _dev(inv_freq, torch.float32, 1, "inv_freq")
    B, qL, _ = q.shape
    planes, Bc, H, maxlen, S = kv_cache.shape
    _require(Bc == B, "kv_cache.size(1) == B")
    for t, n in ((q, "q"), (k, "k"), (v, "v")):
        _require(tuple(t.shape) == (B, qL, H * S), f"{n}.is({{B, qL, H * S}})")
    _require(tuple(kvc_slots.shape) == (qL,), "kvc_slots.is({qL})")
    lib = _lib.load()
    need = lib.llmops_attention_workspace_bytes(B, qL, H, S, maxlen)
    ws = _workspace(q.device, need, kind="attn")
    dt = 0 if kv_cache.dtype == torch.float32 else 1
    if isinstance(position_id, torch.Tensor):
        _dev(position_id, torch.int32, 1, "position_id")
        _require(qL == 1 and position_id.numel() == 1, "position_id tensor: one query token, one value")
        _lib.check(lib.llmops_attention_rope_decode(_ptr(q), _ptr(k), _ptr(v), B, H, S, _ptr(inv_freq), inv_freq.shape[0],
                                                    _ptr(kv_cache), dt, planes, maxlen, _ptr(kvc_slots), _ptr(position_id),
                                                    int(layer_id), _ptr(ws), ws.numel(), _stream(q)))
        return
    _lib.check(lib.llmops_attention_rope(_ptr(q), _ptr(k), _ptr(v), B, qL, H, S, _ptr(inv_freq), inv_freq.shape[0],
                                         _ptr(kv_cache), dt, planes, maxlen, _ptr(kvc_slots), int(position_id),
                                         int(layer_id), _ptr(ws), ws.numel(), _stream(q)))


# the reference exports two kernels with one contract (ops/main.cpp:154-155)
attention_rope = attention_rope2


class AttentionRecords:
    """What ``attention_rope2_records`` leaves behind: per head up to 8 split-KV chunk records (max, sum of exp;
    exp-weighted V sum) that ``fc_Q4A_decode(..., attn_records=...)`` merges on its input side."""

    def __init__(self, stats, outs, chunks, B, H):
        self.stats, self.outs, self.chunks, self.B, self.H = stats, outs, chunks, B, H


def attention_records_supported(kv_cache):
    """True if decode attention over this cache can hand its chunk records to the o projection
    (fp32 cache of up to 2048 rows, fp16 of up to 4096)."""
    dt = 0 if kv_cache.dtype == torch.float32 else 1
    return _lib.load().llmops_attention_records_chunks(kv_cache.shape[3], dt) > 0


def attention_rope2_records(q, k, v, inv_freq, kv_cache, kvc_slots, position_id, layer_id, records=None):
    """Extension: ``attention_rope2`` for ONE query token that does not overwrite q with the attention output but
    returns the split-KV chunk records for the FC that consumes the output (``fc_Q4A_decode(attn_records=...)``
    merges them as it loads its input: one launch fewer per decoder layer).  k is rotated in place and the cache
    updated as usual; ``position_id`` is an int or an int32 device tensor [1].  ``records`` reuses an earlier
    result's buffers."""
    _dev(q, torch.float32, 3, "q")
    _dev(k, torch.float32, 3, "k")
    _dev(v, torch.float32, 3, "v")
    _require(isinstance(kv_cache, torch.Tensor) and kv_cache.is_cuda and kv_cache.dim() == 5 and kv_cache.is_contiguous(),
             "kv_cache.is<float>(5)")
    _require(kv_cache.dtype in (torch.float32, torch.float16), "kv_cache.is<float>(5)")
    _dev(kvc_slots, torch.int32, 1, "kvc_slots")
    _dev(inv_freq, torch.float32, 1, "inv_freq")
    B, qL, _ = q.shape
    planes, Bc, H, maxlen, S = kv_cache.shape
    _require(qL == 1 and Bc == B, "one query token; kv_cache.size(1) == B")
    for t, n in ((q, "q"), (k, "k"), (v, "v")):
        _require(tuple(t.shape) == (B, 1, H * S), f"{n}.is({{B, 1, H * S}})")
    lib = _lib.load()
    dt = 0 if kv_cache.dtype == torch.float32 else 1
    chunks = lib.llmops_attention_records_chunks(maxlen, dt)
    _require(chunks > 0, "cache short enough for chunk records (attention_records_supported)")
    if records is None:
        records = AttentionRecords(torch.empty((B * H, chunks, 2), dtype=torch.float32, device=q.device),
                                   torch.empty((B * H, chunks, S), dtype=torch.float32, device=q.device), 0, B, H)
    ws = _workspace(q.device, lib.llmops_attention_workspace_bytes(B, 1, H, S, maxlen), kind="attn")
    on_dev = isinstance(position_id, torch.Tensor)
    if on_dev:
        _dev(position_id, torch.int32, 1, "position_id")
        kv_plan = maxlen
    else:
        kv_plan = min(int(position_id) + 1, maxlen)
    records.chunks = -(-kv_plan // lib.llmops_attention_records_chunk_rows(maxlen, dt))
    _lib.check(lib.llmops_attention_rope_decode_records(_ptr(q), _ptr(k), _ptr(v), B, H, S, _ptr(inv_freq), inv_freq.shape[0],
                                                        _ptr(kv_cache), dt, planes, maxlen, _ptr(kvc_slots),
                                                        0 if on_dev else int(position_id), _ptr(position_id) if on_dev else None,
                                                        int(layer_id), _ptr(records.stats), _ptr(records.outs), _ptr(ws),
                                                        ws.numel(), _stream(q)))
    return records


def softmax(x):
    """In place over the last dimension (ops/op_misc.hpp:183-194)."""
    _dev(x, torch.float32, None, "input")
    K = x.shape[-1]
    _lib.check(_lib.load().llmops_softmax(_ptr(x), x.numel() // K, K, _stream(x)))


def _mm_qk(q, kcache, attn_w, q_is_bhqs):
    _dev(kcache, torch.float32, 4, "kcache")
    _dev(q, torch.float32, 4 if q_is_bhqs else 3, "q")
    B, H, kmax, S = kcache.shape
    _require(q.shape[0] == B, "kcache.size(-4) == B")
    if q_is_bhqs:
        qL = q.shape[2]
        _require(tuple(q.shape) == (B, H, qL, S), "q is [B,H,qL,S]")
        strides = (H * qL * S, qL * S, S)
    else:
        qL = q.shape[1]
        _require(q.shape[2] == H * S, "q is [B,qL,H*S]")
        strides = (qL * H * S, S, H * S)
    if attn_w is None:
        attn_w = torch.empty((B, H, qL, kmax), dtype=torch.float32, device=q.device)
    else:
        _dev(attn_w, torch.float32, 4, "attn_w")
        _require(tuple(attn_w.shape[:3]) == (B, H, qL) and attn_w.shape[3] <= kmax, "attn_w is [B,H,qL,kvLen<=max]")
    _lib.check(_lib.load().llmops_mm_qk(_ptr(q), *strides, _ptr(kcache), kmax, _ptr(attn_w), B, H, qL, attn_w.shape[3], S,
                                        _stream(q)))
    return attn_w


def mm_qk(q, kcache):
    """q [B,qL,H*S], kcache [B,H,kvLen,S] -> (q.k)/sqrt(S) as [B,H,qL,kvLen] (ops/op_attn.hpp:149-193)."""
    return _mm_qk(q, kcache, None, False)


def mm_qk81(q, kcache):
    """Same contract as mm_qk (ops/op_attn.hpp:300-422)."""
    return _mm_qk(q, kcache, None, False)


def mm_qk24(q, kcache):
    """Same contract as mm_qk (ops/op_attn.hpp:424-515)."""
    return _mm_qk(q, kcache, None, False)


def mm_qk42(q, kcache, attn_w):
    """q [B,H,qL,S], kcache [B,H,max-kv-len,S]; fills attn_w [B,H,qL,kvLen] (ops/op_attn.hpp:195-298)."""
    _mm_qk(q, kcache, attn_w, True)


# ---- neighbours -------------------------------------------------------------------------------
def rmsnorm(input, weight, variance_epsilon):
    _dev(input, torch.float32, 3, "input")
    _dev(weight, torch.float32, 1, "weight")
    hidden = weight.shape[0]
    _require(input.shape[-1] == hidden, "input.size(-1) == hidden_states")
    _lib.check(_lib.load().llmops_rmsnorm(_ptr(input), input.numel() // hidden, hidden, _ptr(weight),
                                         float(variance_epsilon), _stream(input)))


def rmsnorm_out(input, weight, variance_epsilon):
    """Extension: clone + rmsnorm in one launch; returns the normalised copy, ``input`` is untouched."""
    _dev(input, torch.float32, 3, "input")
    _dev(weight, torch.float32, 1, "weight")
    hidden = weight.shape[0]
    _require(input.shape[-1] == hidden, "input.size(-1) == hidden_states")
    out = torch.empty_like(input)
    _lib.check(_lib.load().llmops_rmsnorm_out(_ptr(input), _ptr(out), input.numel() // hidden, hidden, _ptr(weight),
                                             float(variance_epsilon), _stream(input)))
    return out


def silu_mul(gate_up):
    """Extension: itrans(gate, "silu") + imul(up, gate) on fp32 [..., 2F] holding gate|up side by side -> [..., F]."""
    _dev(gate_up, torch.float32, None, "gate_up")
    _require(gate_up.shape[-1] % 2 == 0, "gate_up.size(-1) % 2 == 0")
    F = gate_up.shape[-1] // 2
    out = torch.empty(tuple(gate_up.shape[:-1]) + (F,), dtype=torch.float32, device=gate_up.device)
    _lib.check(_lib.load().llmops_silu_mul(_ptr(gate_up), _ptr(out), gate_up.numel() // (2 * F), F, _stream(gate_up)))
    return out


def _ibinary(fn, a, b):
    _dev(a, torch.float32, None, "a")
    _dev(b, torch.float32, None, "b")
    _require(b.dim() == 1 or b.dim() == a.dim(), "b.is<float>(1) || b.is<float>(a.rank())")
    _require(b.shape[-1] == a.shape[-1], "b.size(-1) == a.size(-1)")
    if b.dim() == a.dim() and a.dim() != 1:
        _require(tuple(b.shape) == tuple(a.shape), "b.shape() == a.shape()")
    inner = a.shape[-1]
    _lib.check(fn(_ptr(a), _ptr(b), a.numel() // inner, inner, int(b.dim() == 1), _stream(a)))


def iadd(a, b):
    _ibinary(_lib.load().llmops_iadd, a, b)


def imul(a, b):
    _ibinary(_lib.load().llmops_imul, a, b)


def itrans(a, op):
    _dev(a, torch.float32, None, "a")
    _require(op == "silu", "false")  # the reference ASSERT(false)s on any other op (ops/op_misc.hpp:139)
    _lib.check(_lib.load().llmops_itrans_silu(_ptr(a), a.numel(), _stream(a)))


def clone(t):
    _require(isinstance(t, torch.Tensor) and t.is_cuda and t.is_contiguous(), "d_rank == old.m_rank")
    return t.clone()


def empty(*shape, device="cuda"):
    return torch.empty(shape, dtype=torch.float32, device=device)


def ones(*shape, device="cuda"):
    return torch.ones(shape, dtype=torch.float32, device=device)


def _ids(input):
    _require(isinstance(input, torch.Tensor) and input.is_cuda and input.is_contiguous(), "input is on the HIP device")
    _require(input.dtype in (torch.int32, torch.int64), "input.is<int32_t>() || input.is<int64_t>()")
    return input if input.dtype == torch.int64 else input.to(torch.int64)


def embedding(output, input, weight):
    _dev(weight, torch.float32, 2, "weight")
    _dev(output, torch.float32, None, "output")
    ids = _ids(input)
    V, E = weight.shape
    _require(tuple(output.shape) == tuple(input.shape) + (E,), "infer_shape() == output.shape()")
    _lib.check(_lib.load().llmops_embedding(_ptr(output), _ptr(ids), ids.numel(), _ptr(weight), V, E, _stream(output)))


def embedding_q8c_quant_w(input):
    _dev(input, torch.float32, 2, "input")
    V, E = input.shape
    q = torch.empty((V, E), dtype=torch.int8, device=input.device)
    s = torch.empty((V,), dtype=torch.float32, device=input.device)
    _lib.check(_lib.load().llmops_embedding_q8c_quant_w(_ptr(input), V, E, _ptr(q), _ptr(s), _stream(input)))
    return [q, s]


def embedding_q8c(output, input, weight, scales):
    _dev(weight, torch.int8, 2, "weight")
    _dev(scales, torch.float32, 1, "scales")
    _dev(output, torch.float32, None, "output")
    ids = _ids(input)
    V, E = weight.shape
    _require(tuple(output.shape) == tuple(input.shape) + (E,), "infer_shape() == output.shape()")
    _lib.check(_lib.load().llmops_embedding_q8c(_ptr(output), _ptr(ids), ids.numel(), _ptr(weight), _ptr(scales), V, E,
                                               _stream(output)))


class PoolAllocator:
    """The reference pools small host buffers per thread (ops/tensor.hpp:47-197); device memory here
    comes from torch's caching allocator, so these are the no-ops a caller of
    ``tensor_pool().clear()`` (chatllama/main.py:332-334) expects to exist."""

    def set_policy(self, pol):
        pass

    def summary(self, verbose):
        return "PoolAllocator: device memory is managed by the torch caching allocator"

    def clear(self):
        pass


_pool = PoolAllocator()


def tensor_pool():
    return _pool
