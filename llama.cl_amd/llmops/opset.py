"""Python-side wrappers the reference keeps next to its model code (the ``llmop_*`` classes and
``KVCache`` of /root/reference/chatllama/main.py:60-219), re-stated over device tensors.

``to_lt`` / ``to_torch`` are identities here because the tensor type at the boundary already is a
``torch.Tensor`` (the reference converts between torch, numpy and its own tensor class,
chatllama/main.py:136-144).
"""
import torch

import llmops


def to_lt(a):
    return a


def to_torch(a):
    return a


class KVCache:
    """Fixed-size ring-buffer KV cache with slot reuse (chatllama/main.py:60-134).

    ``cache`` is [2*layers, batch, heads, max_kv_len, head_size]; ``prepare`` assigns the cache rows
    ("slots") the next ``query_len`` tokens go to, skipping rows that hold the system prompt
    (mask -1) and refusing (returning False) when it would have to overwrite sentence
    ``fail_on_sid``.
    """

    def __init__(self, configs, batch_size, max_kv_len, verbose=False, device="cuda", dtype=torch.float32):
        self.cache = torch.zeros(configs["layer_num"] * 2, batch_size, configs["head_num"], max_kv_len,
                                 configs["head_size"], dtype=dtype, device=device)
        self.device = device
        self.mask = torch.zeros(max_kv_len, dtype=torch.int32)  # host-side bookkeeping
        self.max_kv_len = max_kv_len
        self.position_id_next = 0
        self.position_id = 0
        self.slots = torch.empty(0, dtype=torch.int32, device=device)
        self.cur_slot = 0
        self.cur_kv_len = 0
        self.verbose = verbose

    def size(self):
        return self.cache.numel() * self.cache.element_size()

    def prepare(self, query_len, sentence_id, fail_on_sid):
        assert query_len > 0
        cur_slot = self.cur_slot
        slots = []
        for _ in range(query_len):
            while self.mask[cur_slot] < 0:  # reserved for the system message
                cur_slot = (cur_slot + 1) % self.max_kv_len
            if self.mask[cur_slot] != 0 and self.mask[cur_slot] == fail_on_sid:
                return False
            slots.append(cur_slot)
            cur_slot = (cur_slot + 1) % self.max_kv_len
        self.cur_slot = cur_slot
        for s in slots:
            self.mask[s] = sentence_id
        self.slots = torch.tensor(slots, dtype=torch.int32, device=self.device)
        self.position_id = self.position_id_next
        self.position_id_next = self.position_id + query_len
        self.cur_kv_len = min(self.cur_kv_len + query_len, self.max_kv_len)
        return True


class llmop_fc_q4a:
    """Holds one packed weight and applies fc_Q4A (+ optional bias) -- chatllama/main.py:158-177."""

    def __init__(self, linear=None, weight=None, bias=None, group_k=None, packed=None, N=None):
        if linear is not None:
            weight, bias = linear.weight, linear.bias
        if packed is not None:
            self.weight, self.N = packed, N
        else:
            self.weight = llmops.offline_FC_quant_Q4A(weight.detach(), group_k)
            self.N = weight.shape[0]
        self.bias = bias.detach() if bias is not None else None

    def __call__(self, input, residual=None):
        out = llmops.fc_Q4A(input, self.weight, self.N, residual=residual)
        if self.bias is not None:
            llmops.iadd(out, self.bias)
        return out

    def weight_size(self):
        size = self.weight.numel() * self.weight.element_size()
        if self.bias is not None:
            size += self.bias.numel() * self.bias.element_size()
        return size

    def __repr__(self):
        return f"llmop_fc_q4a(weight: {list(self.weight.shape)})"


class llmop_rmsnorm:
    """chatllama/main.py:179-191"""

    def __init__(self, weight, variance_epsilon):
        self.weight = weight.detach().clone()
        self.eps = variance_epsilon

    def __call__(self, input):
        llmops.rmsnorm(input, self.weight, self.eps)

    def out_of_place(self, input):
        return llmops.rmsnorm_out(input, self.weight, self.eps)

    def __repr__(self):
        return f"llmop_rmsnorm(weight: {list(self.weight.shape)}, eps: {self.eps})"


class llmop_embedding_q8c:
    """chatllama/main.py:206-219"""

    def __init__(self, weight=None, packed=None):
        # packed = (int8 rows, fp32 per-row scales) as embedding_q8c_quant_w returns them
        self.weight, self.scales = packed if packed is not None else llmops.embedding_q8c_quant_w(weight.detach())

    def __call__(self, input_ids):
        output = llmops.empty(*input_ids.shape, self.weight.shape[1], device=input_ids.device)
        llmops.embedding_q8c(output, input_ids, self.weight, self.scales)
        return output

    def __repr__(self):
        return f"llmop_embedding_q8c(weight: {list(self.weight.shape)})"
