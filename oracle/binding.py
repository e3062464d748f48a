"""ctypes binding of the CPU oracle (``liboracle.so``).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and
by the CPU-baseline leg of ``bench.py`` -- never by the product package.
"""
import ctypes
import os
from ctypes import POINTER, byref, c_double, c_float, c_int, c_long, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
MAX_LAYERS = 64
KIND_ATTENTION, KIND_GDN = 0, 1

_PF = POINTER(c_float)


class OrcHParams(ctypes.Structure):
    _fields_ = [
        ("dim", c_int), ("attnHeads", c_int), ("headDim", c_int), ("ffnDim", c_int), ("transformers", c_int),
        ("maxL", c_int), ("vocabSize", c_int), ("ropeDenomBase", c_float), ("qkRmsNorm", c_int),
        ("queryGating", c_int), ("gdnHeads", c_int), ("gdnDk", c_int), ("gdnDv", c_int), ("pleDim", c_int),
        ("layerKinds", c_int * MAX_LAYERS),
    ]


_LAYER_FIELDS = ["rms1", "Wq", "Wk", "Wv", "Wo", "rms2", "W1A", "W1B", "W2", "qRms", "kRms", "Wg", "gdnWa",
                 "gdnBa", "gdnWb", "gdnBb", "pleTable", "pleGate", "pleUp"]


class OrcLayer(ctypes.Structure):
    _fields_ = [(n, _PF) for n in _LAYER_FIELDS]


class OrcWeights(ctypes.Structure):
    _fields_ = [("E", _PF), ("gammaF", _PF), ("layers", OrcLayer * MAX_LAYERS)]


def _lib():
    path = os.path.join(_HERE, "liboracle.so")
    if not os.path.exists(path):
        raise ImportError(f"{path} missing: run `make -C oracle`")
    lib = ctypes.CDLL(path)
    lib.orc_rope_table.argtypes = [c_void_p, c_int, c_int, c_float]
    lib.orc_round_bf16.argtypes = [c_void_p, c_long]
    for sfx, real in (("f32", c_float), ("f64", c_double)):
        g = lambda n: getattr(lib, f"{n}_{sfx}")
        g("orc_rmsnorm").argtypes = [c_void_p, c_void_p, c_int, c_void_p]
        g("orc_head_rmsnorm").argtypes = [c_void_p, c_void_p, c_int, c_int]
        g("orc_rope").argtypes = [c_void_p, c_void_p, c_int, c_int, c_int]
        g("orc_matvec").argtypes = [c_void_p, c_void_p, c_int, c_int, c_void_p]
        g("orc_matmat").argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int]
        g("orc_attend").argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]
        g("orc_gdn_step").argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, real, real, c_int, c_int, c_void_p]
        g("orc_state_new").restype = c_void_p
        g("orc_state_new").argtypes = [POINTER(OrcHParams), POINTER(OrcWeights)]
        g("orc_state_reset").argtypes = [c_void_p]
        g("orc_state_free").argtypes = [c_void_p]
        g("orc_state_pos").argtypes = [c_void_p]
        g("orc_decode_step").argtypes = [c_void_p, c_int, c_void_p]
        g("orc_forward_full").argtypes = [POINTER(OrcHParams), POINTER(OrcWeights), c_void_p, c_int, c_void_p,
                                          c_void_p, c_void_p, c_int]
    return lib


lib = _lib()

# tensor ids of include/mlh.h -> oracle layer field
_TID = {2: "rms1", 3: "Wq", 4: "Wk", 5: "Wv", 6: "Wo", 7: "rms2", 8: "W1A", 9: "W1B", 10: "W2", 11: "qRms",
        12: "kRms", 13: "Wg", 14: "gdnWa", 15: "gdnBa", 16: "gdnWb", 17: "gdnBb", 18: "pleTable", 19: "pleGate",
        20: "pleUp"}


def hparams_from(hp):
    """Copies the shared fields of an mlh_hparams-like object (attribute access) into OrcHParams."""
    o = OrcHParams()
    for f, _ in OrcHParams._fields_:
        if f == "layerKinds":
            for i in range(MAX_LAYERS):
                o.layerKinds[i] = hp.layerKinds[i]
        else:
            setattr(o, f, getattr(hp, f))
    return o


def rope_table(max_l, head_dim, base=10000.0):
    tab = np.empty((max_l, head_dim), dtype=np.float32)
    lib.orc_rope_table(tab.ctypes.data, max_l, head_dim, base)
    return tab


def round_bf16(a):
    a = np.ascontiguousarray(a, dtype=np.float32).copy()
    lib.orc_round_bf16(a.ctypes.data, a.size)
    return a


class Weights:
    """Holds fp32 arrays (keeps them alive) and the OrcWeights struct pointing at them.

    ``tensors``: dict with keys ("E",), ("gammaF",) and (layer, tensor_id) -> ndarray.
    """

    def __init__(self, hp, tensors, bf16=False):
        self.hp = hparams_from(hp)
        self.w = OrcWeights()
        self._keep = []

        def put(arr):
            a = np.ascontiguousarray(arr, dtype=np.float32)
            if bf16 and a.ndim == 2:
                a = round_bf16(a)
            self._keep.append(a)
            return a.ctypes.data_as(_PF)

        self.w.E = put(tensors[("E",)])
        self.w.gammaF = put(tensors[("gammaF",)])
        for (key, arr) in tensors.items():
            if len(key) == 2:
                layer, tid = key
                setattr(self.w.layers[layer], _TID[tid], put(arr))

    @classmethod
    def from_model(cls, model, bf16=False):
        """model: the product's host-side Model (only its tensor() accessor and hparams are used)."""
        hp = model.hparams
        t = {("E",): model.tensor(0, 0), ("gammaF",): model.tensor(0, 1)}
        for layer in range(hp.transformers):
            for tid in _TID:
                a = model.tensor(layer, tid)
                if a is not None:
                    t[(layer, tid)] = a
        w = cls(hp, t, bf16=bf16)
        w._model = model  # the arrays are borrowed views of memory the model owns
        return w


class Decoder:
    """Cached decode with the oracle (float32 or float64 arithmetic)."""

    def __init__(self, weights, dtype="f64"):
        self.sfx = dtype
        self.real = np.float64 if dtype == "f64" else np.float32
        self.weights = weights
        self._st = getattr(lib, f"orc_state_new_{dtype}")(byref(weights.hp), byref(weights.w))
        self.V = weights.hp.vocabSize

    def reset(self):
        getattr(lib, f"orc_state_reset_{self.sfx}")(self._st)

    @property
    def pos(self):
        return getattr(lib, f"orc_state_pos_{self.sfx}")(self._st)

    def step(self, token, want_logits=True):
        logits = np.empty(self.V, dtype=self.real) if want_logits else None
        nxt = getattr(lib, f"orc_decode_step_{self.sfx}")(self._st, int(token),
                                                          logits.ctypes.data if want_logits else None)
        if nxt < 0:
            raise RuntimeError("oracle decode step failed (position or token out of range)")
        return nxt, logits

    def close(self):
        if self._st:
            getattr(lib, f"orc_state_free_{self.sfx}")(self._st)
            self._st = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def forward_full(weights, tokens, dtype="f64", last_only=True, want_probs=False, want_hidden=False):
    """Reference-style full recompute.  Returns dict(logits=..., probs=..., hidden=...)."""
    real = np.float64 if dtype == "f64" else np.float32
    hp = weights.hp
    toks = np.ascontiguousarray(tokens, dtype=np.int32)
    L = toks.size
    ncol = 1 if last_only else L
    logits = np.empty((ncol, hp.vocabSize), dtype=real)
    probs = np.empty((ncol, hp.vocabSize), dtype=real) if want_probs else None
    hidden = np.empty((L, hp.dim), dtype=real) if want_hidden else None
    rc = getattr(lib, f"orc_forward_full_{dtype}")(
        byref(hp), byref(weights.w), toks.ctypes.data, L, logits.ctypes.data,
        probs.ctypes.data if want_probs else None, hidden.ctypes.data if want_hidden else None, int(last_only))
    if rc != 0:
        raise RuntimeError(f"oracle forward failed ({rc})")
    return {"logits": logits, "probs": probs, "hidden": hidden}


# ---------------------------------------------------------------------------------------------------------
# Temperature sampling (test infrastructure like the rest of this package).  The reference has no sampling: its
# loop keeps the top entry of a qsort of the probabilities (inference_orchestrator.cu:120-165).  The rule restated
# here is the one the device documents: p_i = exp((l_i - max l) / T) / Z, pick = smallest i with
# sum_{j <= i} p_j Z > u Z, u a 53-bit uniform from SplitMix64 keyed by (seed, sequence id, position drawn).
# Pinned by: the published first outputs of SplitMix64 seeded with 0, the T -> 0 limit (argmax), the ends of the
# u range, monotonicity in u, and a frequency test against the softmax (tests/test_oracle_sampling.py).
# ---------------------------------------------------------------------------------------------------------
_M64 = (1 << 64) - 1


def splitmix64(x):
    """Output function of SplitMix64 applied to x + golden gamma (Steele, Lea, Flood 2014)."""
    x = (x + 0x9E3779B97F4A7C15) & _M64
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def sample_uniform(seed, seq, pos):
    base = splitmix64(splitmix64(seed & _M64) ^ (((seq + 1) * 0xD1342543DE82EF95) & _M64))
    return (splitmix64((base + pos) & _M64) >> 11) * (1.0 / 9007199254740992.0)


def sample_cdf(logits, temperature):
    """Unnormalised cumulative sums of exp((l - max l) / T) in index order, float64."""
    l = np.asarray(logits, dtype=np.float64)
    return np.cumsum(np.exp((l - l.max()) / float(temperature)))


def sample_token(logits, temperature, u):
    c = sample_cdf(logits, temperature)
    i = int(np.searchsorted(c, u * c[-1], side="right"))  # first index whose cumulative sum exceeds the target
    return min(i, len(c) - 1)
