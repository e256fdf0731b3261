"""One Llama-shaped forward step built from ``llmops`` calls in the reference's op order
(``Model.forward``, /root/reference/chatllama/main.py:331-380), on random-initialised weights.

This is the caller of the hot path, kept as thin as the reference's: every arithmetic step is an
``llmops`` op.  Two launch plans are offered:

* ``plan="reference"``: the reference's sequence verbatim -- clone, rmsnorm, q/k/v projections as three
  FCs, attention_rope2, o projection, iadd, clone, rmsnorm, gate, silu, up, imul, down, iadd.
* ``plan="fused"`` (default): the same arithmetic with fewer launches -- q|k|v and gate|up packed
  tensors fused into one FC launch each, rmsnorm folded into the FC that consumes it, silu*up into
  the gate|up epilogue, residual adds into the o and down projections (``llmops.fc_Q4A_decode``).

A decode step (one token, batch 1) has fixed shapes and no host-side decisions, so it can be
captured once as a HIP graph and replayed (``capture_decode``).
"""
import numpy as np
import torch

import llmops
from llmops.opset import KVCache, llmop_embedding_q8c, llmop_fc_q4a, llmop_rmsnorm

LLAMA_7B = dict(layer_num=32, head_num=32, head_size=128, hidden_size=4096, intermediate_size=11008,
                vocab_size=55296, rms_norm_eps=1e-5, rope_base=10000.0)


class LlamaDecoder:
    def __init__(self, configs=None, group_k=128, seed=5, device="cuda", plan="fused", embed_rows=None, device_rng=False):
        """``device_rng``: draw the random weights on the device (much faster for the full-size model; the values
        then differ from the host generator's for the same seed)."""
        cfg = dict(LLAMA_7B)
        cfg.update(configs or {})
        self.configs = cfg
        self.plan = plan
        self.merge_in_o_proj = True  # fused plan, one token: the o projection merges the attention chunks
        self.device = torch.device(device)
        gen = torch.Generator(device=self.device if device_rng else "cpu").manual_seed(seed)
        H, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]

        def randn(*shape):
            return torch.randn(*shape, generator=gen, device=gen.device).to(self.device)

        def fc(N, K, parts=1):
            # parts > 1: several projections sharing one input, packed and concatenated along N
            packed = []
            for _ in range(parts):
                w = randn(N, K) * 0.02
                packed.append(llmops.offline_FC_quant_Q4A(w, group_k))
                del w
            t = torch.cat(packed, dim=0) if parts > 1 else packed[0]
            return llmop_fc_q4a(packed=t, N=N * parts)

        self.layers = []
        for _ in range(cfg["layer_num"]):
            layer = {
                "input_layernorm": llmop_rmsnorm(torch.ones(H, device=self.device), cfg["rms_norm_eps"]),
                "post_attention_layernorm": llmop_rmsnorm(torch.ones(H, device=self.device), cfg["rms_norm_eps"]),
                "o_proj": fc(H, H),
                "down_proj": fc(H, F),
            }
            if plan == "fused":
                layer["qkv_proj"] = fc(H, H, parts=3)
                gate, up = fc(F, H), fc(F, H)
                # gate and up stacked along N: one FC leaves the row [gate | up] and the down projection takes
                # silu(gate)*up on its way in.  That needs F to be whole strips; otherwise the strips are
                # interleaved and silu(gate)*up is the epilogue of the gate|up FC.
                self.stacked_gate_up = F % 32 == 0
                gu = torch.cat((gate.weight, up.weight), dim=0) if self.stacked_gate_up else \
                    llmops.interleave_gate_up(gate.weight, up.weight)
                layer["gate_up_proj"] = llmop_fc_q4a(packed=gu, N=2 * F)
            else:
                layer["q_proj"], layer["k_proj"], layer["v_proj"] = fc(H, H), fc(H, H), fc(H, H)
                layer["gate_proj"], layer["up_proj"] = fc(F, H), fc(F, H)
            self.layers.append(layer)
        self.norm = llmop_rmsnorm(torch.ones(H, device=self.device), cfg["rms_norm_eps"])
        self.lm_head = fc(V, H)
        # the embedding table is only gathered from (one row per token); a small table suffices for timing
        rows = V if embed_rows is None else embed_rows
        self.embed_tokens = llmop_embedding_q8c(randn(rows, H))
        rd = cfg["head_size"]
        inv_freq = 1.0 / (cfg["rope_base"] ** (torch.arange(0, rd, 2).float() / rd))  # chatllama/main.py:294-296
        self.inv_freq = inv_freq.to(self.device)

    @classmethod
    def from_reference(cls, path, device="cuda", plan="fused"):
        """Builds the decoder from a model file written by the reference's ``Model.save``
        (chatllama/main.py:305-308).  The file is read without executing it (``llmops.ref_pickle``); its
        packed Q4_1 tensors have the layout this library uses and go to the device as they are."""
        from llmops import ref_pickle

        t = ref_pickle.model_tensors(ref_pickle.load(path))
        self = cls.__new__(cls)
        self.device = torch.device(device)
        self.plan = plan
        self.merge_in_o_proj = True

        def dev(a):
            return torch.from_numpy(a).to(self.device)

        def fc(*entries):
            for e in entries:
                if e["bias"] is not None:
                    raise ValueError("FC with bias: not part of the Llama family the reference loads")
            packed = [dev(e["weight"]) for e in entries]
            return llmop_fc_q4a(packed=torch.cat(packed, dim=0) if len(packed) > 1 else packed[0],
                                N=sum(e["N"] for e in entries))

        def norm(e):
            return llmop_rmsnorm(dev(e["weight"]), e["eps"])

        ref_cfg = t["configs"]
        first = t["layers"][0]
        H = ref_cfg["hidden_size"]
        F = first["mlp.gate_proj"]["N"]
        self.configs = dict(layer_num=len(t["layers"]), head_num=ref_cfg["head_num"], head_size=ref_cfg["head_size"],
                            hidden_size=H, intermediate_size=F, vocab_size=t["lm_head"]["N"],
                            rms_norm_eps=ref_cfg["rms_norm_eps"], rope_base=10000.0)
        self.layers = []
        self.stacked_gate_up = F % 32 == 0
        for e in t["layers"]:
            layer = {"input_layernorm": norm(e["input_layernorm"]),
                     "post_attention_layernorm": norm(e["post_attention_layernorm"]),
                     "o_proj": fc(e["self_attn.o_proj"]), "down_proj": fc(e["mlp.down_proj"])}
            if plan == "fused":
                # q|k|v stacked along N needs every part to be whole strips (hidden sizes are)
                if H % 32 != 0:
                    raise ValueError("fused plan: hidden_size must be a multiple of 32")
                layer["qkv_proj"] = fc(e["self_attn.q_proj"], e["self_attn.k_proj"], e["self_attn.v_proj"])
                gate, up = dev(e["mlp.gate_proj"]["weight"]), dev(e["mlp.up_proj"]["weight"])
                gu = torch.cat((gate, up), dim=0) if self.stacked_gate_up else llmops.interleave_gate_up(gate, up)
                layer["gate_up_proj"] = llmop_fc_q4a(packed=gu, N=2 * F)
            else:
                layer["q_proj"], layer["k_proj"], layer["v_proj"] = (fc(e["self_attn.q_proj"]), fc(e["self_attn.k_proj"]),
                                                                     fc(e["self_attn.v_proj"]))
                layer["gate_proj"], layer["up_proj"] = fc(e["mlp.gate_proj"]), fc(e["mlp.up_proj"])
            self.layers.append(layer)
        self.norm = norm(t["norm"])
        self.lm_head = fc(t["lm_head"])
        if t["embed"]["scales"] is None:
            raise ValueError("the reference stores the embedding as int8 rows with per-row scales (embedding_q8c)")
        self.embed_tokens = llmop_embedding_q8c(packed=(dev(t["embed"]["weight"]), dev(t["embed"]["scales"])))
        rd = ref_cfg.get("rotary_dims", ref_cfg["head_size"])
        inv_freq = t["inv_freq"] if t["inv_freq"] is not None else \
            (1.0 / (10000.0 ** (torch.arange(0, rd, 2).float() / rd))).numpy()
        self.inv_freq = dev(np.ascontiguousarray(inv_freq, dtype=np.float32))
        return self

    def fc_weight_size(self):
        """bytes of every packed FC tensor a step streams: the layers' projections and the lm_head"""
        n = self.lm_head.weight_size()
        for layer in self.layers:
            n += sum(op.weight_size() for op in layer.values() if isinstance(op, llmop_fc_q4a))
        return n

    def forward(self, input_ids, kv_cache, kv_cache_slots, position_id):
        """input_ids int64 [B, qL]; returns logits fp32 [B, qL, vocab]."""
        llmops.tensor_pool().clear()
        H = self.configs["hidden_size"]
        F = self.configs["intermediate_size"]
        hidden_states = self.embed_tokens(input_ids)
        if self.plan == "fused":
            sumsq = None  # per-strip sums of squares of hidden_states, handed from FC to FC for the rmsnorms
            for i, ops in enumerate(self.layers):
                hidden_states, sumsq = self._layer_fused(i, ops, hidden_states, sumsq, kv_cache, kv_cache_slots, position_id)
            return llmops.fc_Q4A_decode(hidden_states, self.lm_head.weight, self.lm_head.N,
                                        norm=(self.norm.weight, self.norm.eps), sumsq_in=sumsq)
        for i, ops in enumerate(self.layers):
            hidden_states = self._layer_reference(i, ops, hidden_states, kv_cache, kv_cache_slots, position_id)
        self.norm(hidden_states)
        return self.lm_head(hidden_states)

    def _layer_reference(self, i, ops, hidden_states, kv_cache, kv_cache_slots, position_id):
        """chatllama/main.py:344-375 verbatim."""
        input_layernorm = llmops.clone(hidden_states)
        ops["input_layernorm"](input_layernorm)
        q = ops["q_proj"](input_layernorm)
        k = ops["k_proj"](input_layernorm)
        v = ops["v_proj"](input_layernorm)
        llmops.attention_rope2(q, k, v, self.inv_freq, kv_cache, kv_cache_slots, position_id, i)
        attn_output = ops["o_proj"](q)
        llmops.iadd(attn_output, hidden_states)
        post_attention_layernorm = llmops.clone(attn_output)
        ops["post_attention_layernorm"](post_attention_layernorm)
        gate = ops["gate_proj"](post_attention_layernorm)
        llmops.itrans(gate, "silu")
        up = ops["up_proj"](post_attention_layernorm)
        llmops.imul(up, gate)
        hidden_states = ops["down_proj"](up)
        llmops.iadd(hidden_states, attn_output)
        return hidden_states

    def _layer_fused(self, i, ops, hidden_states, sumsq, kv_cache, kv_cache_slots, position_id):
        """Same arithmetic, 6 launches per decode layer instead of 18: rmsnorm inside the q|k|v and
        gate|up FCs (fed with the sums of squares that the FC producing their input leaves behind),
        silu*up on the input side of the down projection, residual adds inside the o and down
        projections, rope + cache update inside the attention kernel."""
        H, F = self.configs["hidden_size"], self.configs["intermediate_size"]
        n1, n2 = ops["input_layernorm"], ops["post_attention_layernorm"]
        rows = hidden_states.shape[0] * hidden_states.shape[1]
        many = rows > 8  # a prompt or a batch: the sums of squares are not handed on (the norms read their rows)
        if many:  # q, k and v as three dense [B,qL,H*S] tensors straight from the product
            q, k, v = llmops.fc_Q4A_decode(hidden_states, ops["qkv_proj"].weight, 3 * H, norm=(n1.weight, n1.eps), out_parts=3)
        else:
            qkv = llmops.fc_Q4A_decode(hidden_states, ops["qkv_proj"].weight, 3 * H, norm=(n1.weight, n1.eps), sumsq_in=sumsq)
            q, k, v = qkv[..., :H], qkv[..., H:2 * H], qkv[..., 2 * H:]
            if not q.is_contiguous():  # more than one token: the op needs dense [B,qL,H*S] tensors
                q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        if rows == 1 and self.merge_in_o_proj and llmops.attention_records_supported(kv_cache) \
                and llmops.group_k_of(ops["o_proj"].weight) == 128 and self.inv_freq.shape[0] % 4 == 0:
            # one token: attention leaves its split-KV chunk records and the o projection merges them on its way in
            recs = llmops.attention_rope2_records(q, k, v, self.inv_freq, kv_cache, kv_cache_slots, position_id, i)
            attn_output, ss = llmops.fc_Q4A_decode(None, ops["o_proj"].weight, H, residual=hidden_states, want_sumsq=True,
                                                   attn_records=recs)
        else:
            llmops.attention_rope2(q, k, v, self.inv_freq, kv_cache, kv_cache_slots, position_id, i)
            if many:
                attn_output, ss = llmops.fc_Q4A_decode(q, ops["o_proj"].weight, H, residual=hidden_states), None
            else:
                attn_output, ss = llmops.fc_Q4A_decode(q, ops["o_proj"].weight, H, residual=hidden_states, want_sumsq=True)
        if self.stacked_gate_up:
            gate_up = llmops.fc_Q4A_decode(attn_output, ops["gate_up_proj"].weight, 2 * F, norm=(n2.weight, n2.eps),
                                           sumsq_in=ss)
            if many:
                return llmops.fc_Q4A_decode(gate_up, ops["down_proj"].weight, H, residual=attn_output, glu_in=True), None
            return llmops.fc_Q4A_decode(gate_up, ops["down_proj"].weight, H, residual=attn_output, want_sumsq=True,
                                        glu_in=True)
        act = llmops.fc_Q4A_decode(attn_output, ops["gate_up_proj"].weight, F, norm=(n2.weight, n2.eps), glu=True,
                                   sumsq_in=ss)
        if many:
            return llmops.fc_Q4A_decode(act, ops["down_proj"].weight, H, residual=attn_output), None
        return llmops.fc_Q4A_decode(act, ops["down_proj"].weight, H, residual=attn_output, want_sumsq=True)

    def capture_decode(self, kv_cache, slot, position_id, stream=None):
        """Capture one decode step (batch 1, one token) as a HIP graph that serves every position: the token id,
        the cache slot and the position live in device memory and are read by the kernels at replay time.
        Returns a DecodeGraph: ``step(token, slot, position_id)`` (or write ``.input_ids``, ``set_position`` and
        ``replay()``), then read ``.logits``."""
        stream = stream or torch.cuda.Stream()
        input_ids = torch.zeros(1, 1, dtype=torch.int64, device=self.device)
        slots = torch.tensor([slot], dtype=torch.int32, device=self.device)
        position = torch.tensor([position_id], dtype=torch.int32, device=self.device)
        with torch.cuda.stream(stream):
            stream.wait_stream(torch.cuda.default_stream(self.device))
            self.forward(input_ids, kv_cache, slots, position)  # warm-up: code objects, workspaces of this stream
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                logits = self.forward(input_ids, kv_cache, slots, position)
        # the workspaces are captured by address too (the module never frees one; the graph object also holds them)
        workspace = [w for key, w in llmops._workspaces.items() if key[1] == self.device.type]
        return DecodeGraph(graph, input_ids, slots, position, kv_cache, logits, stream, workspace)


class DecodeGraph:
    """A captured decode step together with every tensor whose address the graph has recorded.
    The graph replays raw device pointers, so these tensors must live as long as the graph does.
    Token, slot and position are device values the kernels read at replay time: one graph serves a
    whole generation loop."""

    def __init__(self, graph, input_ids, slots, position, kv_cache, logits, stream, workspace):
        self.graph, self.input_ids, self.slots, self.position, self.kv_cache, self.logits, self.stream, self.workspace = \
            graph, input_ids, slots, position, kv_cache, logits, stream, workspace

    def set_position(self, slot, position_id):
        """cache row the next token goes to and its position (kv length = position + 1, up to the cache size)"""
        if not (0 <= int(slot) < self.kv_cache.shape[3]) or int(position_id) < 0:
            raise ValueError("slot outside the cache or negative position")
        with torch.cuda.stream(self.stream):  # (scalar fills: no host buffer that a later call could overwrite too early)
            self.slots.fill_(int(slot))
            self.position.fill_(int(position_id))

    def replay(self):
        with torch.cuda.stream(self.stream):
            self.graph.replay()

    def step(self, token, slot, position_id):
        with torch.cuda.stream(self.stream):
            self.input_ids.fill_(int(token))
        self.set_position(slot, position_id)
        self.replay()
        return self.logits
