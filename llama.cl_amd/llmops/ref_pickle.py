"""Reader for the model file the reference writes with ``Model.save``
(/root/reference/chatllama/main.py:305-308: ``pickle.dump(self.__dict__, f)``), which holds the packed
Q4_1 weights as ``llmops.tensor`` objects (pickled as one numpy array each,
/root/reference/ops/main.cpp:129-136) inside the reference's op wrapper objects
(``llmop_fc_q4a`` & co., chatllama/main.py:158-219), next to things this build has no use for (the
tokenizer object, ``nn.Module`` bookkeeping).

A pickle is a program; this reader does not run it.  Every global the stream names resolves either to
one of a handful of constructors that only build data (numpy array reconstruction, ``OrderedDict``,
``set``) or to an inert stand-in that records what it was given: no class or function named by the
file is imported or called.  ``llmops.tensor`` resolves to a stand-in that keeps the numpy array.

The packed weight layout is the reference's own (``int8 [Ng, Kg, block]``), so the arrays go to the
device as they are -- nothing is re-quantized.
"""
import collections
import io
import pickle

import numpy as np


class Opaque:
    """Inert stand-in for an object of a class this reader does not construct."""
    _ref = ("?", "?")

    def __new__(cls, *args, **kwargs):
        self = object.__new__(cls)
        self._args = args
        return self

    def __init__(self, *args, **kwargs):
        pass

    def __setstate__(self, state):
        # what pickle's BUILD would do for a plain object, minus any class-defined hook
        slots = None
        if isinstance(state, tuple) and len(state) == 2 and (state[0] is None or isinstance(state[0], dict)) \
                and (state[1] is None or isinstance(state[1], dict)):
            state, slots = state
        if isinstance(state, dict):
            self.__dict__.update(state)
        elif state is not None:
            self._state = state
        if slots:
            self.__dict__.update(slots)

    def __call__(self, *args, **kwargs):  # a stand-in used as a callable by REDUCE: still inert
        return Opaque()

    def __repr__(self):
        return f"<{self._ref[0]}.{self._ref[1]} (not constructed)>"


class PackedTensor(Opaque):
    """``llmops.tensor``: its pickled state is ``(numpy array,)`` (ops/main.cpp:129-136)."""
    _ref = ("llmops", "tensor")

    def __setstate__(self, state):
        self.array = state[0] if isinstance(state, tuple) and len(state) == 1 else None
        if not isinstance(self.array, np.ndarray):
            raise pickle.UnpicklingError("llmops.tensor state is not (ndarray,)")


def _reconstructor(cls, base, state):
    """copyreg._reconstructor for stand-ins (protocol < 2 object pickles)."""
    if isinstance(cls, type) and issubclass(cls, Opaque):
        return cls()
    return Opaque()


def _numpy_callables():
    table = {}
    try:
        import numpy._core.multiarray as ma
    except ImportError:  # numpy 1.x
        import numpy.core.multiarray as ma
    for mod in ("numpy.core.multiarray", "numpy._core.multiarray"):  # both spellings occur in files
        table[(mod, "_reconstruct")] = ma._reconstruct
        table[(mod, "scalar")] = ma.scalar
    table[("numpy", "ndarray")] = np.ndarray
    table[("numpy", "dtype")] = np.dtype
    return table


class SafeUnpickler(pickle.Unpickler):
    """Unpickler whose globals are data constructors or inert stand-ins, nothing else."""

    def __init__(self, file):
        super().__init__(file)
        self._standins = {}
        self._safe = {
            ("collections", "OrderedDict"): collections.OrderedDict,
            ("builtins", "set"): set,
            ("builtins", "frozenset"): frozenset,
            ("builtins", "list"): list,
            ("builtins", "dict"): dict,
            ("builtins", "tuple"): tuple,
            ("builtins", "bytearray"): bytearray,
            ("builtins", "complex"): complex,
            ("builtins", "slice"): slice,
            ("builtins", "range"): range,
            ("copyreg", "_reconstructor"): _reconstructor,
            ("copy_reg", "_reconstructor"): _reconstructor,
            ("llmops", "tensor"): PackedTensor,
        }
        self._safe.update(_numpy_callables())

    def find_class(self, module, name):
        key = (module, name)
        if key in self._safe:
            return self._safe[key]
        if key not in self._standins:
            self._standins[key] = type(name.rsplit(".", 1)[-1], (Opaque,), {"_ref": key})
        return self._standins[key]

    def persistent_load(self, pid):  # e.g. torch storages: not needed, not loaded
        return Opaque()


def load(path_or_file):
    """The pickled ``Model.__dict__`` as plain containers, numpy arrays and inert stand-ins."""
    if hasattr(path_or_file, "read"):
        return SafeUnpickler(path_or_file).load()
    with open(path_or_file, "rb") as f:
        return SafeUnpickler(io.BufferedReader(f)).load()


def _array(obj, what):
    if isinstance(obj, PackedTensor):
        return obj.array
    if isinstance(obj, np.ndarray):
        return obj
    raise ValueError(f"{what}: expected an llmops.tensor, found {obj!r}")


def _fc(op, what):
    w = _array(getattr(op, "weight", None), what + ".weight")
    if w.dtype != np.int8 or w.ndim != 3 or w.shape[2] not in (640, 2176):
        raise ValueError(f"{what}.weight is not a packed Q4_1 tensor: {w.dtype} {w.shape}")
    bias = getattr(op, "bias", None)
    return {"weight": w, "N": int(op.N), "bias": None if bias is None else _array(bias, what + ".bias")}


def _norm(op, what):
    return {"weight": _array(getattr(op, "weight", None), what + ".weight").astype(np.float32, copy=False),
            "eps": float(op.eps)}


LAYER_FCS = ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj", "self_attn.o_proj", "mlp.gate_proj",
             "mlp.up_proj", "mlp.down_proj")


def model_tensors(state):
    """Picks the reference's ``op_dict`` (chatllama/main.py:268-287) apart into numpy arrays.

    Returns ``{"configs", "embed": {"weight", "scales"}, "layers": [{name: fc or norm}], "norm", "lm_head",
    "inv_freq"}`` with fc = ``{"weight" int8 [Ng,Kg,block], "N", "bias"}``, norm = ``{"weight", "eps"}``."""
    ops = state["op_dict"]
    emb = ops["model.embed_tokens"]
    out = {
        "configs": dict(state["configs"]),
        "embed": {"weight": _array(emb.weight, "embed_tokens.weight"),
                  "scales": _array(getattr(emb, "scales", None), "embed_tokens.scales") if hasattr(emb, "scales") else None},
        "layers": [],
        "norm": _norm(ops["model.norm"], "model.norm"),
        "lm_head": _fc(ops["lm_head"], "lm_head"),
        "inv_freq": _array(state["inv_freq"], "inv_freq") if "inv_freq" in state else None,
    }
    for i, layer in enumerate(ops["layers"]):
        entry = {name: _fc(layer[name], f"layers[{i}].{name}") for name in LAYER_FCS}
        for name in ("input_layernorm", "post_attention_layernorm"):
            entry[name] = _norm(layer[name], f"layers[{i}].{name}")
        out["layers"].append(entry)
    return out
