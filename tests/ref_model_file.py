"""Writes a file with the structure of the reference's ``Model.save`` output
(/root/reference/chatllama/main.py:305-308) from numpy arrays, for the loader tests.

The reference pickles ``Model.__dict__``: ``nn.Module`` bookkeeping, the tokenizer object, ``configs``,
``inv_freq`` and ``op_dict`` whose leaves are instances of the script's op wrapper classes
(``__main__.llmop_fc_q4a`` ...) holding ``llmops.tensor`` objects; a ``llmops.tensor`` pickles as an
object with state ``(numpy array,)`` (/root/reference/ops/main.cpp:129-136).  The classes below get
the same module and class names while the file is written, so the byte stream names the same
globals the reference's would.  No reference code is involved.
"""
import collections
import contextlib
import os
import pickle
import sys
import types


def _named(module, name, base=object, **attrs):
    cls = type(name, (base,), dict(attrs))
    cls.__module__ = module
    cls.__qualname__ = name
    return cls


def _tensor_getstate(self):
    return (self.array,)


def _tensor_setstate(self, state):
    self.array = state[0]


class _Marker:
    """Pickles as a call of os.system: a reader that executes the stream would create `path`."""

    def __init__(self, path):
        self.path = path

    def __reduce__(self):
        return (os.system, (f"touch {self.path}",))


@contextlib.contextmanager
def _reference_names():
    tensor = _named("llmops", "tensor", __getstate__=_tensor_getstate, __setstate__=_tensor_setstate)
    ops = {n: _named("__main__", n) for n in ("llmop_fc_q4a", "llmop_rmsnorm", "llmop_embedding_q8c")}
    tok = _named("transformers.models.llama.tokenization_llama_fast", "LlamaTokenizerFast")
    fake_llmops = types.ModuleType("llmops")
    fake_llmops.tensor = tensor
    fake_tok = types.ModuleType(tok.__module__)
    setattr(fake_tok, tok.__name__, tok)
    saved = {k: sys.modules.get(k) for k in ("llmops", tok.__module__)}
    main = sys.modules["__main__"]
    saved_main = {n: getattr(main, n, None) for n in ops}
    sys.modules["llmops"] = fake_llmops
    sys.modules[tok.__module__] = fake_tok
    for n, c in ops.items():
        setattr(main, n, c)
    try:
        yield tensor, ops, tok
    finally:
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v
        for n, v in saved_main.items():
            if v is None:
                delattr(main, n)
            else:
                setattr(main, n, v)


def write(path, configs, embed, layers, norm, lm_head, inv_freq, marker_path=None):
    """embed = (int8 [V,H], fp32 [V]); layers = list of dicts name -> (packed int8, N) for the 7 FCs and
    name -> (weight fp32, eps) for the two norms; norm = (weight, eps); lm_head = (packed, N)."""
    with _reference_names() as (tensor, ops, tok):
        def lt(a):
            t = tensor()
            t.array = a
            return t

        def fc(packed, N):
            o = ops["llmop_fc_q4a"]()
            o.weight, o.bias, o.N = lt(packed), None, N
            return o

        def rms(w, eps):
            o = ops["llmop_rmsnorm"]()
            o.weight, o.eps = lt(w), eps
            return o

        emb = ops["llmop_embedding_q8c"]()
        emb.weight, emb.scales = lt(embed[0]), lt(embed[1])
        tokenizer = tok()
        tokenizer.pad_token = "[PAD]"
        if marker_path is not None:
            tokenizer.trap = _Marker(marker_path)
        op_dict = {
            "model.embed_tokens": emb,
            "layers": [{k: (rms(*v) if "layernorm" in k else fc(*v)) for k, v in layer.items()} for layer in layers],
            "model.norm": rms(*norm),
            "lm_head": fc(*lm_head),
        }
        state = {
            "training": False, "_parameters": collections.OrderedDict(), "_buffers": collections.OrderedDict(),
            "_non_persistent_buffers_set": set(), "_modules": collections.OrderedDict(),
            "tokenizer": tokenizer, "op_dict": op_dict, "configs": dict(configs), "inv_freq": lt(inv_freq),
        }
        with open(path, "wb") as f:
            pickle.dump(state, f)
