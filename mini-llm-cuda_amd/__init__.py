"""ctypes bindings of the MI355X inference token loop.

Two shared libraries are loaded from ``lib/`` next to this file:

* ``libmlh.so``      device layer, C ABI of ``include/mlh.h`` (HIP kernels for gfx950)
* ``libminillm.so``  C++ host library, C ABI of ``include/mini_llm_host.h``

There is no CPU fallback: if a library is missing the import fails, and any
forward call without a GPU fails in ``mlh_create``.  The directory name is not
a valid Python identifier; load this package with :func:`importlib.util.spec_from_file_location`
(see ``__graft_entry__.load_package``).
"""
import ctypes
import os
from ctypes import POINTER, byref, c_char_p, c_double, c_float, c_int, c_int32, c_uint64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
MAX_LAYERS = 64

KIND_ATTENTION, KIND_GDN = 0, 1
DTYPE_F32, DTYPE_BF16 = 0, 1

# tensor ids (include/mlh.h)
(T_TOKEN_EMBEDDINGS, T_FINAL_RMS_GAMMA, T_RMS_GAMMA, T_QUERY, T_KEY, T_VALUE, T_OUTPUT_PROJ, T_RMS_GAMMA2,
 T_FFN_1A, T_FFN_1B, T_FFN_2, T_QUERY_RMS_GAMMA, T_KEY_RMS_GAMMA, T_GATED_QUERY, T_GDN_ALPHA_W, T_GDN_ALPHA_B,
 T_GDN_BETA_W, T_GDN_BETA_B, T_PLE_TABLE, T_PLE_GATE, T_PLE_UP, T_COUNT) = range(22)

# kernel ids (include/mlh.h)
K_QKV, K_ATTN, K_OPROJ, K_FFN_GATEUP, K_FFN_DOWN, K_LMHEAD, K_GDN, K_COPY, K_EMBED, K_FINISH = range(10)
K_COUNT = 10


class HParams(ctypes.Structure):
    """mlh_hparams: runtime form of network_meta.h:3-20 plus the extensions."""
    _fields_ = [
        ("dim", c_int32), ("attnHeads", c_int32), ("headDim", c_int32), ("ffnDim", c_int32),
        ("transformers", c_int32), ("maxL", c_int32), ("vocabSize", c_int32), ("ropeDenomBase", c_float),
        ("qkRmsNorm", c_int32), ("queryGating", c_int32), ("gdnHeads", c_int32), ("gdnDk", c_int32),
        ("gdnDv", c_int32), ("pleDim", c_int32), ("weightDtype", c_int32), ("maxSeqs", c_int32),
        ("layerKinds", c_int32 * MAX_LAYERS),
    ]

    def copy(self):
        other = HParams()
        ctypes.memmove(byref(other), byref(self), ctypes.sizeof(HParams))
        return other


class TokenProb(ctypes.Structure):
    _fields_ = [("tokenIdx", c_int), ("prob", c_float)]


def _load(name):
    path = os.path.join(LIB_DIR, name)
    if not os.path.exists(path):
        raise ImportError(f"{path} is missing: build it with __graft_entry__.build() (hipcc, gfx950)")
    return ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)


dev = _load("libmlh.so")
host = _load("libminillm.so")

_P = POINTER
_sigs_dev = {
    "mlh_last_error": (c_char_p, [c_void_p]),
    "mlh_device_count": (c_int, []),
    "mlh_create": (c_int, [_P(HParams), c_int, _P(c_void_p)]),
    "mlh_destroy": (None, [c_void_p]),
    "mlh_upload_tensor": (c_int, [c_void_p, c_int, c_int, c_void_p, c_int, c_int]),
    "mlh_upload_rope_table": (c_int, [c_void_p, c_void_p, c_int]),
    "mlh_finalize": (c_int, [c_void_p]),
    "mlh_reset": (c_int, [c_void_p, c_int]),
    "mlh_seq_len": (c_int, [c_void_p, c_int]),
    "mlh_max_len": (c_int, [c_void_p]),
    "mlh_vocab_size": (c_int, [c_void_p]),
    "mlh_kv_page_size": (c_int, []),
    "mlh_set_page_table": (c_int, [c_void_p, c_void_p, c_int]),
    "mlh_prefill": (c_int, [c_void_p, c_int, c_void_p, c_int]),
    "mlh_prefill_batch": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p]),
    "mlh_set_prefill_mode": (c_int, [c_void_p, c_int]),
    "mlh_forward_full": (c_int, [c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, _P(c_float)]),
    "mlh_decode_step": (c_int, [c_void_p, c_void_p, c_int, c_void_p]),
    "mlh_decode_loop": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "mlh_greedy_token": (c_int, [c_void_p, c_int, _P(c_int32)]),
    "mlh_read_logits": (c_int, [c_void_p, c_int, c_void_p]),
    "mlh_read_probs": (c_int, [c_void_p, c_int, c_void_p]),
    "mlh_set_graph": (c_int, [c_void_p, c_int]),
    "mlh_set_sampling": (c_int, [c_void_p, c_float, ctypes.c_ulonglong]),
    "mlh_set_persistent": (c_int, [c_void_p, c_int]),
    "mlh_get_persistent": (c_int, [c_void_p]),
    "mlh_persistent_fallbacks": (c_int, [c_void_p]),
    "mlh_debug_inject_abort": (c_int, [c_void_p, c_int]),
    "mlh_debug_inject_abort_at_step": (c_int, [c_void_p, c_int]),
    "mlh_debug_set_xcd_tag": (c_int, [c_void_p, ctypes.c_uint]),
    "mlh_xcd_decode_supported": (c_int, [c_void_p]),
    "mlh_synchronize": (c_int, [c_void_p]),
    "mlh_time_kernel": (c_int, [c_void_p, c_int, c_int, c_int, c_int, _P(c_double), _P(c_double)]),
    "mlh_kernel_name": (c_char_p, [c_int]),
    "mlh_time_decode": (c_int, [c_void_p, c_void_p, c_int, c_int, _P(c_double)]),
    "mlh_selftest_gemm": (c_int, [c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, _P(c_double)]),
    "mlh_gemm_device_init": (c_int, [c_int]),
    "mlh_gemm_device": (c_int, [c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "mlh_probe_hops": (c_int, [c_void_p, c_int, _P(c_double)]),
    "mlh_probe_mfma": (c_int, [c_void_p, c_int, c_int, c_int, _P(c_double)]),
    "mlh_probe_lds_loads": (c_int, [c_void_p, c_int, _P(c_double)]),
    "mlh_profile_decode": (c_int, [c_void_p, c_void_p, c_int, c_int, _P(c_double), _P(c_int32)]),
}
_sigs_host = {
    "mll_hparams_reference_defaults": (None, [_P(HParams)]),
    "mll_hparams_config": (c_int, [c_int, _P(HParams)]),
    "mll_set_layer_pattern": (None, [_P(HParams), c_int]),
    "mll_rope_table": (None, [c_void_p, c_int, c_int, c_float]),
    "mll_model_new": (c_void_p, [_P(HParams)]),
    "mll_model_free": (None, [c_void_p]),
    "mll_model_hparams": (_P(HParams), [c_void_p]),
    "mll_model_tensor": (_P(c_float), [c_void_p, c_int, c_int, _P(c_int), _P(c_int)]),
    "mll_model_init_normal": (None, [c_void_p, c_uint64, c_float]),
    "mll_model_init_uniform": (None, [c_void_p, c_uint64, c_float]),
    "mll_random_tokens": (None, [c_uint64, c_int, c_int, c_int, c_void_p]),
    "mll_model_load": (c_void_p, [c_char_p, _P(HParams), c_char_p, c_int]),
    "mll_model_save": (c_int, [c_void_p, c_char_p, c_int]),
    "mll_model_upload": (c_int, [c_void_p, c_void_p]),
    "mll_vocab_load": (c_void_p, [c_char_p, c_int]),
    "mll_vocab_free": (None, [c_void_p]),
    "mll_vocab_size": (c_int, [c_void_p]),
    "mll_vocab_token": (c_char_p, [c_void_p, c_int]),
    "mll_vocab_lookup": (c_int, [c_void_p, c_char_p]),
    "mll_hash_token": (ctypes.c_uint, [c_char_p]),
    "mll_load_story_context": (c_int, [c_char_p, c_int, c_int, c_void_p, c_int, c_void_p]),
    "mll_load_stories": (c_int, [c_char_p, c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "mll_prefill_stories": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int]),
    "mll_story_loss": (c_int, [c_void_p, c_void_p, c_int, _P(c_float), _P(c_int)]),
    "mll_generate": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, _P(c_double)]),
    "mll_top_k": (c_int, [c_void_p, c_int, c_int, _P(TokenProb)]),
}
for _lib, _sigs in ((dev, _sigs_dev), (host, _sigs_host)):
    for _name, (_res, _args) in _sigs.items():
        _fn = getattr(_lib, _name)  # AttributeError here = the library does not export a declared symbol
        _fn.restype = _res
        _fn.argtypes = _args

DEVICE_SYMBOLS = tuple(_sigs_dev)
HOST_SYMBOLS = tuple(_sigs_host)


class MlhError(RuntimeError):
    pass


def config(n, **overrides):
    """Hyper-parameters of benchmark configuration n (1..5), with optional field overrides."""
    hp = HParams()
    if not host.mll_hparams_config(n, byref(hp)):
        raise ValueError(f"unknown configuration {n}")
    for k, v in overrides.items():
        setattr(hp, k, v)
    return hp


def reference_defaults():
    hp = HParams()
    host.mll_hparams_reference_defaults(byref(hp))
    host.mll_set_layer_pattern(byref(hp), 0)
    return hp


def set_layer_pattern(hp, gdn_per_attn):
    host.mll_set_layer_pattern(byref(hp), gdn_per_attn)


def rope_table(max_l, head_dim, base=10000.0):
    tab = np.empty((max_l, head_dim), dtype=np.float32)
    host.mll_rope_table(tab.ctypes.data, max_l, head_dim, base)
    return tab


def random_tokens(seed, stream, vocab, n):
    out = np.empty(n, dtype=np.int32)
    host.mll_random_tokens(seed, stream, vocab, n, out.ctypes.data)
    return out


class Model:
    """Host-side model (fp32 tensors in model.bin order)."""

    def __init__(self, handle):
        if not handle:
            raise MlhError("model handle is NULL")
        self._h = handle

    @classmethod
    def new(cls, hp):
        return cls(host.mll_model_new(byref(hp)))

    @classmethod
    def generate(cls, hp, seed, std=0.02):
        m = cls.new(hp)
        host.mll_model_init_normal(m._h, seed, std)
        return m

    @classmethod
    def load(cls, path, hint=None):
        err = ctypes.create_string_buffer(512)
        h = host.mll_model_load(os.fsencode(path), byref(hint) if hint is not None else None, err, 512)
        if not h:
            raise MlhError(err.value.decode(errors="replace"))
        return cls(h)

    def save(self, path, float64=False):
        if not host.mll_model_save(self._h, os.fsencode(path), int(float64)):
            raise MlhError(f"cannot write {path}")

    @property
    def hparams(self):
        return host.mll_model_hparams(self._h).contents

    def tensor(self, layer, tid):
        """Borrowed NumPy view of a tensor ([rows, cols], 1-D for vectors), or None if absent."""
        r, c = c_int(), c_int()
        p = host.mll_model_tensor(self._h, layer, tid, byref(r), byref(c))
        if not p:
            return None
        arr = np.ctypeslib.as_array(p, shape=(r.value * c.value,))
        return arr.reshape(r.value, c.value) if c.value > 1 else arr

    def init_uniform(self, seed, rng):
        host.mll_model_init_uniform(self._h, seed, rng)

    GAIN_TENSORS = (T_FINAL_RMS_GAMMA, T_RMS_GAMMA, T_RMS_GAMMA2, T_QUERY_RMS_GAMMA, T_KEY_RMS_GAMMA)

    def randomize_gains(self, seed, spread=0.3):
        """Replaces every RMSNorm gain vector (finalRMSNormGamma, rmsGamma, rmsGamma2, queryRMSGamma, keyRMSGamma;
        the generators set them to 1 as an untrained model has them) by 1 + spread * U(-1, 1), every element its
        own draw -- what a trained model.bin carries (load_model.cu:378-390, 411-450).  Deterministic in seed."""
        rng = np.random.default_rng([int(seed), 0x6761696E])
        t = self.tensor(0, T_FINAL_RMS_GAMMA)
        t[:] = 1 + spread * rng.uniform(-1, 1, size=t.shape)
        for layer in range(self.hparams.transformers):
            for tid in self.GAIN_TENSORS[1:]:
                t = self.tensor(layer, tid)
                if t is not None:
                    t[:] = 1 + spread * rng.uniform(-1, 1, size=t.shape)
        return self

    def close(self):
        if self._h:
            host.mll_model_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Device:
    """One device context (mlh_ctx): weights, KV pages, GDN states, stream and decode graph."""

    def __init__(self, hp, device=0):
        h = c_void_p()
        rc = dev.mlh_create(byref(hp), device, byref(h))
        if rc != 0:
            raise MlhError(f"mlh_create failed ({rc}): {dev.mlh_last_error(None).decode()}")
        self._h = h
        self.hp = hp.copy()

    def _check(self, rc):
        if rc != 0:
            raise MlhError(f"device layer error {rc}: {dev.mlh_last_error(self._h).decode()}")

    def upload(self, model):
        if not host.mll_model_upload(model._h, self._h):
            raise MlhError(f"upload failed: {dev.mlh_last_error(self._h).decode()}")

    def upload_tensor(self, layer, tid, arr):
        a = np.ascontiguousarray(arr, dtype=np.float32)
        rows, cols = (a.shape[0], a.shape[1]) if a.ndim == 2 else (a.shape[0], 1)
        self._check(dev.mlh_upload_tensor(self._h, layer, tid, a.ctypes.data, rows, cols))

    def upload_rope(self, tab):
        a = np.ascontiguousarray(tab, dtype=np.float32)
        self._check(dev.mlh_upload_rope_table(self._h, a.ctypes.data, a.size))

    def finalize(self):
        self._check(dev.mlh_finalize(self._h))

    def reset(self, seq=-1):
        self._check(dev.mlh_reset(self._h, seq))

    def seq_len(self, seq):
        return dev.mlh_seq_len(self._h, seq)

    def set_page_table(self, table):
        t = np.ascontiguousarray(table, dtype=np.int32)
        self._check(dev.mlh_set_page_table(self._h, t.ctypes.data, t.size))

    def prefill(self, seq, ids):
        a = np.ascontiguousarray(ids, dtype=np.int32)
        self._check(dev.mlh_prefill(self._h, seq, a.ctypes.data, a.size))

    def prefill_batch(self, seqs, prompts):
        """Appends prompts[i] to sequence seqs[i] for all i in one pass."""
        sq = np.ascontiguousarray(seqs, dtype=np.int32)
        lens = np.array([len(p) for p in prompts], dtype=np.int32)
        ids = np.ascontiguousarray(np.concatenate([np.asarray(p, dtype=np.int32) for p in prompts]), dtype=np.int32)
        self._check(dev.mlh_prefill_batch(self._h, sq.size, sq.ctypes.data, ids.ctypes.data, lens.ctypes.data))

    def forward_full(self, seq, ids, want_probs=True):
        """Teacher-forced forward over ids appended to seq: (logits [n, V], probs [n, V] or None, mean NLL)."""
        a = np.ascontiguousarray(ids, dtype=np.int32)
        lg = np.empty((a.size, self.hp.vocabSize), dtype=np.float32)
        pr = np.empty_like(lg) if want_probs else None
        nll = c_float(0)
        self._check(dev.mlh_forward_full(self._h, seq, a.ctypes.data, a.size, lg.ctypes.data,
                                         pr.ctypes.data if pr is not None else None, byref(nll)))
        return lg, pr, float(nll.value)

    def set_prefill_mode(self, mode):
        self._check(dev.mlh_set_prefill_mode(self._h, int(mode)))

    def decode_step(self, last_ids):
        a = np.ascontiguousarray(last_ids, dtype=np.int32)
        out = np.empty_like(a)
        self._check(dev.mlh_decode_step(self._h, a.ctypes.data, a.size, out.ctypes.data))
        return out

    def decode_loop(self, first_ids, steps):
        a = np.ascontiguousarray(first_ids, dtype=np.int32)
        out = np.empty((steps, a.size), dtype=np.int32)
        self._check(dev.mlh_decode_loop(self._h, a.ctypes.data, a.size, steps, out.ctypes.data))
        return out

    def time_decode(self, first_ids, steps):
        a = np.ascontiguousarray(first_ids, dtype=np.int32)
        ms = c_double()
        self._check(dev.mlh_time_decode(self._h, a.ctypes.data, a.size, steps, byref(ms)))
        return ms.value

    def greedy_token(self, seq=0):
        t = c_int32()
        self._check(dev.mlh_greedy_token(self._h, seq, byref(t)))
        return t.value

    def logits(self, seq=0):
        out = np.empty(self.hp.vocabSize, dtype=np.float32)
        self._check(dev.mlh_read_logits(self._h, seq, out.ctypes.data))
        return out

    def probs(self, seq=0):
        out = np.empty(self.hp.vocabSize, dtype=np.float32)
        self._check(dev.mlh_read_probs(self._h, seq, out.ctypes.data))
        return out

    def set_graph(self, enabled):
        self._check(dev.mlh_set_graph(self._h, int(enabled)))

    def set_sampling(self, temperature, seed=0):
        """temperature 0: greedy (default); > 0: tokens are drawn from softmax(logits / temperature)."""
        self._check(dev.mlh_set_sampling(self._h, float(temperature), int(seed)))

    def set_persistent(self, enabled):
        self._check(dev.mlh_set_persistent(self._h, int(enabled)))

    def get_persistent(self):
        return dev.mlh_get_persistent(self._h)

    def persistent_fallbacks(self):
        return dev.mlh_persistent_fallbacks(self._h)

    def debug_inject_abort(self, launches):
        self._check(dev.mlh_debug_inject_abort(self._h, int(launches)))

    def debug_inject_abort_at_step(self, step):
        self._check(dev.mlh_debug_inject_abort_at_step(self._h, int(step)))

    def debug_set_xcd_tag(self, tags_used):
        self._check(dev.mlh_debug_set_xcd_tag(self._h, int(tags_used)))

    def xcd_decode_supported(self):
        return bool(dev.mlh_xcd_decode_supported(self._h))

    def synchronize(self):
        self._check(dev.mlh_synchronize(self._h))

    def time_kernel(self, kernel, layer=0, nseq=1, iters=50):
        us, nbytes = c_double(), c_double()
        self._check(dev.mlh_time_kernel(self._h, kernel, layer, nseq, iters, byref(us), byref(nbytes)))
        return us.value, nbytes.value

    def probe_hops(self, iters=2000):
        """Microseconds per dependent exchange: (inside one XCD, across XCDs, grid barrier); -1 where a wait expired."""
        us = (c_double * 3)()
        self._check(dev.mlh_probe_hops(self._h, iters, us))
        return tuple(us)

    def probe_mfma(self, form, data, iters=20000):
        """TFLOP/s of a register-only half-precision MFMA loop on every SIMD: form 0 = 32x32x16, 1 = 16x16x32;
        data 0 = all-zero operands, 1 = unit-variance operands."""
        t = c_double()
        self._check(dev.mlh_probe_mfma(self._h, form, data, iters, byref(t)))
        return t.value

    def probe_lds_loads(self, slices=4000):
        """TB/s of the GEMM's direct global -> LDS load pattern alone (L2-resident operands, nothing multiplied)."""
        t = c_double()
        self._check(dev.mlh_probe_lds_loads(self._h, slices, byref(t)))
        return t.value

    def profile_decode(self, first_ids, steps):
        """In-sequence mean microseconds per launch (run time plus the launch gap before it) and
        launches per step, by kernel name, over `steps` plain-launch decode steps."""
        a = np.ascontiguousarray(first_ids, dtype=np.int32)
        us = (c_double * K_COUNT)()
        n = (c_int32 * K_COUNT)()
        self._check(dev.mlh_profile_decode(self._h, a.ctypes.data, a.size, steps, us, n))
        return {dev.mlh_kernel_name(k).decode(): (us[k], n[k]) for k in range(K_COUNT) if n[k] > 0}

    def generate(self, prompt, max_new):
        """Greedy generation on sequence 0 (mll_generate): returns (ids, elapsed ms)."""
        a = np.ascontiguousarray(prompt, dtype=np.int32)
        out = np.empty(max(max_new, 1), dtype=np.int32)
        ms = c_double()
        n = host.mll_generate(self._h, a.ctypes.data, a.size, max_new, out.ctypes.data, byref(ms))
        if n < 0:
            raise MlhError(f"generate failed: {dev.mlh_last_error(self._h).decode()}")
        return out[:n].copy(), ms.value

    def prefill_stories(self, tokens, right_end, first, count):
        t = np.ascontiguousarray(tokens, dtype=np.int32)
        r = np.ascontiguousarray(right_end, dtype=np.int32)
        if host.mll_prefill_stories(self._h, t.ctypes.data, r.ctypes.data, t.shape[1] - 1, first, count) != 0:
            raise MlhError(f"prefill_stories failed: {dev.mlh_last_error(self._h).decode()}")

    def story_loss(self, story, right_end):
        """(total loss, predictions) of one loaded story: the forward half of the reference's processSequence."""
        t = np.ascontiguousarray(story, dtype=np.int32)
        loss, n = c_float(), c_int()
        if host.mll_story_loss(self._h, t.ctypes.data, int(right_end), byref(loss), byref(n)) != 0:
            raise MlhError(f"story_loss failed: {dev.mlh_last_error(self._h).decode()}")
        return float(loss.value), int(n.value)

    def top_k(self, k, seq=0):
        buf = (TokenProb * k)()
        n = host.mll_top_k(self._h, seq, k, buf)
        if n < 0:
            raise MlhError("top_k failed")
        return [(buf[i].tokenIdx, buf[i].prob) for i in range(n)]

    def close(self):
        if self._h:
            dev.mlh_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Vocab:
    def __init__(self, path, expect_size=0):
        self._h = host.mll_vocab_load(os.fsencode(path), expect_size)
        if not self._h:
            raise MlhError(f"cannot load vocabulary {path}")

    def __len__(self):
        return host.mll_vocab_size(self._h)

    def token(self, idx):
        return host.mll_vocab_token(self._h, idx)

    def lookup(self, token):
        return host.mll_vocab_lookup(self._h, token if isinstance(token, bytes) else token.encode())

    def story_context(self, path, story_index, percentage, max_l):
        out = np.zeros(max_l + 1, dtype=np.int32)
        n = host.mll_load_story_context(os.fsencode(path), story_index, percentage, self._h, max_l, out.ctypes.data)
        return out[:n].copy()

    def load_stories(self, path, max_l, max_stories=2000):
        """All stories of a tokenised-stories file: (tokens [n, max_l+1], rightEnd [n]), or None on error."""
        toks = np.zeros((max(max_stories, 1), max_l + 1), dtype=np.int32)
        right = np.zeros(max(max_stories, 1), dtype=np.int32)
        n = host.mll_load_stories(os.fsencode(path), self._h, max_l, max_stories, toks.ctypes.data, right.ctypes.data)
        if n < 0:
            return None
        return toks[:n].copy(), right[:n].copy()

    def close(self):
        if self._h:
            host.mll_vocab_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def selftest_gemm(a, b, r=None, bf16=False, iters=0, f16=False, swiglu=False):
    """C = a . b^T (+ r) through the device GEMM kernel; returns (C, mean microseconds or None).  swiglu: the
    gate/up epilogue instead, C[m, j] = silu(P[m, 2j]) * P[m, 2j+1] in the operand type, shape [M, N/2]."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    m, k = a.shape
    n = b.shape[0]
    if r is not None:
        r = np.ascontiguousarray(r, dtype=np.float32)
    c = np.empty((m, n // 2 if swiglu else n), dtype=np.float32)
    us = c_double()
    code = (2 if f16 else (DTYPE_BF16 if bf16 else DTYPE_F32)) | (0x100 if swiglu else 0)
    rc = dev.mlh_selftest_gemm(code, m, n, k, a.ctypes.data, b.ctypes.data,
                               r.ctypes.data if r is not None else None, c.ctypes.data, iters, byref(us))
    if rc != 0:
        raise MlhError(f"GEMM self-test failed ({rc}): unsupported shape or no device")
    return c, (us.value if iters > 0 else None)


def device_count():
    return dev.mlh_device_count()
