"""Host library: model.bin reader/writer, vocab.json tokenizer, story loader, generator, presets.
CPU only.  The fixtures under tests/golden/ are the reference's own data files."""
import ctypes
import json
import os
import struct

import numpy as np
import pytest

from conftest import GOLDEN, ROOT

VOCAB_PV = os.path.join(GOLDEN, "vocab_pytorch_verification.json")
VOCAB_MODEL = os.path.join(GOLDEN, "vocab_model.json")
SAMPLE = os.path.join(GOLDEN, "sample.json")

BLOCK_KEYS = ["rmsGamma", "queryWeights", "keyWeights", "valueWeights", "outputProjectionWeights", "rmsGamma2",
              "feedForwardWeights1A", "feedForwardWeights1B", "feedForwardWeights2"]  # load_model.cu:411-421


# --------------------------------------------------------------------------- independent NumPy reader
def numpy_read_model_bin(path):
    """Straight from the format description (load_model.cu:320-343): u64 LE header length, JSON
    header, data at the next multiple of 8, tensors back to back in header order."""
    raw = open(path, "rb").read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    meta = json.loads(raw[8:8 + hlen].decode())
    off = 8 + hlen
    off += (8 - off % 8) % 8

    def take(entry):
        nonlocal off
        dt = np.float32 if entry["dtype"] == "float32" else np.float64
        n = int(np.prod(entry["shape"]))
        a = np.frombuffer(raw, dtype=dt, count=n, offset=off).reshape(entry["shape"])
        off += n * a.itemsize
        return a.astype(np.float32)

    out = {"tokenEmbeddings": take(meta["tokenEmbeddings"]), "finalRMSNormGamma": take(meta["finalRMSNormGamma"]),
           "blocks": []}
    for blk in meta["transformerBlocks"]:
        out["blocks"].append({k: take(v) for k, v in blk.items()})
    return meta, out, off, len(raw)


def small_hp(pkg, **kw):
    hp = pkg.config(3, dim=64, attnHeads=1, headDim=64, ffnDim=96, transformers=3, vocabSize=50, gdnHeads=1,
                    pleDim=8, maxL=16, qkRmsNorm=1, queryGating=1, **kw)
    pkg.set_layer_pattern(hp, 1)
    return hp


def test_model_bin_round_trip_and_layout(pkg, tmp_path):
    hp = small_hp(pkg)
    model = pkg.Model.generate(hp, 5)
    for f64 in (False, True):
        path = str(tmp_path / f"m{int(f64)}.bin")
        model.save(path, float64=f64)
        meta, t, end, size = numpy_read_model_bin(path)
        assert end == size  # every byte accounted for, no per-tensor padding
        # 2-D tensors are row-major [out, in]; the embedding is [vocab, dim], one token's vector contiguous
        assert meta["tokenEmbeddings"]["shape"] == [50, 64]
        assert np.array_equal(t["tokenEmbeddings"], model.tensor(0, 0))
        assert meta["transformerBlocks"][0]["feedForwardWeights1A"]["shape"] == [96, 64]
        assert meta["transformerBlocks"][0]["feedForwardWeights2"]["shape"] == [64, 96]
        assert list(hp.layerKinds[:3]) == [1, 0, 1]  # applied first = file block 2 (GDN), then attention, then GDN
        keys1 = list(meta["transformerBlocks"][1].keys())  # block 1 is attention with both flags
        assert keys1[:9] == BLOCK_KEYS
        assert keys1[9:12] == ["queryRMSGamma", "keyRMSGamma", "gatedQueryWeights"]
        assert keys1[12:] == ["perLayerEmbeddings", "pleGateWeights", "pleUpWeights"]
        keys0 = list(meta["transformerBlocks"][0].keys())  # block 0 is GDN
        assert keys0[:9] == BLOCK_KEYS
        assert keys0[9:13] == ["gdnAlphaWeights", "gdnAlphaBias", "gdnBetaWeights", "gdnBetaBias"]
        assert keys0[13:] == ["perLayerEmbeddings", "pleGateWeights", "pleUpWeights"]
        assert np.array_equal(t["blocks"][2]["feedForwardWeights1B"], model.tensor(2, 9))
        back = pkg.Model.load(path)  # hyper-parameters come from the header's networkMeta
        hb = back.hparams
        assert (hb.dim, hb.headDim, hb.ffnDim, hb.vocabSize, hb.pleDim, hb.qkRmsNorm) == (64, 64, 96, 50, 8, 1)
        assert list(hb.layerKinds[:3]) == list(hp.layerKinds[:3])
        for l in range(3):
            for tid in range(2, 21):
                a, b = model.tensor(l, tid), back.tensor(l, tid)
                assert (a is None) == (b is None)
                if a is not None:
                    assert np.array_equal(a, b)


def write_reference_style(path, hp_dims, pad_to=None, dtype="float32", drop_key=None, truncate=0, rng=None,
                          extra_dims=False):
    """A checkpoint as the reference's loaders expect it (no networkMeta), written by hand."""
    V, d, F, NL = hp_dims
    rng = rng or np.random.default_rng(0)
    np_dt = np.float32 if dtype == "float32" else np.float64
    entry = lambda shape: {"shape": list(shape), "dtype": dtype}
    tensors, header = [], {"tokenEmbeddings": entry((V, d)), "finalRMSNormGamma": entry((d,)), "transformerBlocks": []}
    tensors += [rng.normal(size=(V, d)), rng.normal(size=(d,))]
    shapes = {"rmsGamma": (d,), "queryWeights": (d, d), "keyWeights": (d, d), "valueWeights": (d, d),
              "outputProjectionWeights": (d, d), "rmsGamma2": (d,), "feedForwardWeights1A": (F, d),
              "feedForwardWeights1B": (F, d), "feedForwardWeights2": (d, F)}
    for _ in range(NL):
        blk = {}
        for k in BLOCK_KEYS:
            if k == drop_key:
                continue
            blk[k] = entry(shapes[k] + ((1,) if extra_dims and k == "queryWeights" else ()))
            tensors.append(rng.normal(size=shapes[k]))
        header["transformerBlocks"].append(blk)
    hj = json.dumps(header)
    if pad_to is not None:  # pad the header with spaces until (8 + len) % 8 == pad_to
        while (8 + len(hj)) % 8 != pad_to:
            hj += " "
    hb = hj.encode()
    data = b"".join(np.asarray(t, dtype=np_dt).tobytes() for t in tensors)
    blob = struct.pack("<Q", len(hb)) + hb + b"\0" * ((8 - (8 + len(hb)) % 8) % 8) + data
    if truncate:
        blob = blob[:-truncate]
    open(path, "wb").write(blob)
    return [np.asarray(t, dtype=np_dt).astype(np.float32) for t in tensors]


@pytest.mark.parametrize("pad", range(8))
def test_reference_style_file_all_header_alignments(pkg, tmp_path, pad):
    path = str(tmp_path / "ref.bin")
    tensors = write_reference_style(path, (40, 64, 96, 2), pad_to=pad)
    hint = pkg.config(1, dim=64, attnHeads=1, headDim=64, ffnDim=96, transformers=2, vocabSize=40, maxL=8)
    m = pkg.Model.load(path, hint)
    assert np.array_equal(m.tensor(0, 0), tensors[0])
    assert np.array_equal(m.tensor(0, 1), tensors[1])
    assert np.array_equal(m.tensor(0, 3), tensors[3])          # block 0 queryWeights, row-major as stored
    assert np.array_equal(m.tensor(1, 10), tensors[2 + 9 + 8])  # block 1 feedForwardWeights2


def test_float64_file_is_narrowed(pkg, tmp_path):
    path = str(tmp_path / "f64.bin")
    tensors = write_reference_style(path, (40, 64, 96, 1), dtype="float64")
    hint = pkg.config(1, dim=64, attnHeads=1, headDim=64, ffnDim=96, transformers=1, vocabSize=40, maxL=8)
    m = pkg.Model.load(path, hint)
    assert np.array_equal(m.tensor(0, 8), tensors[2 + 6])


def test_missing_key_does_not_advance_offset(pkg, tmp_path):
    """load_model.cu:436-438: a key absent from the header only warns; the next tensor is read from
    the position the missing one would have had."""
    path = str(tmp_path / "miss.bin")
    tensors = write_reference_style(path, (40, 64, 96, 1), drop_key="rmsGamma2")
    hint = pkg.config(1, dim=64, attnHeads=1, headDim=64, ffnDim=96, transformers=1, vocabSize=40, maxL=8)
    m = pkg.Model.load(path, hint)
    assert np.all(m.tensor(0, 7) == 0)                    # never read: stays at its zero initial value
    assert np.array_equal(m.tensor(0, 8), tensors[2 + 5])  # feedForwardWeights1A follows outputProjection directly


def test_loader_failures(pkg, tmp_path):
    hint = pkg.config(1, dim=64, attnHeads=1, headDim=64, ffnDim=96, transformers=1, vocabSize=40, maxL=8)
    with pytest.raises(pkg.MlhError, match="not found"):
        pkg.Model.load(str(tmp_path / "nope.bin"), hint)
    p = str(tmp_path / "trunc.bin")
    write_reference_style(p, (40, 64, 96, 1), truncate=100)
    with pytest.raises(pkg.MlhError, match="past buffer end"):
        pkg.Model.load(p, hint)
    p = str(tmp_path / "hdr.bin")
    open(p, "wb").write(struct.pack("<Q", 10 ** 9) + b"{}")
    with pytest.raises(pkg.MlhError, match="larger than the file"):
        pkg.Model.load(p, hint)
    p = str(tmp_path / "short.bin")
    open(p, "wb").write(b"\1\2\3")
    with pytest.raises(pkg.MlhError):
        pkg.Model.load(p, hint)
    p = str(tmp_path / "badjson.bin")
    open(p, "wb").write(struct.pack("<Q", 5) + b"{nope")
    with pytest.raises(pkg.MlhError, match="JSON"):
        pkg.Model.load(p, hint)
    p = str(tmp_path / "dtype.bin")
    write_reference_style(p, (40, 64, 96, 1), dtype="float32")
    raw = open(p, "rb").read().replace(b'"float32"', b'"int8000"', 1)
    open(p, "wb").write(raw)
    with pytest.raises(pkg.MlhError, match="Unsupported dtype"):
        pkg.Model.load(p, hint)
    p = str(tmp_path / "dims.bin")
    write_reference_style(p, (40, 64, 96, 1), extra_dims=True)
    with pytest.raises(pkg.MlhError, match="dimension"):
        pkg.Model.load(p, hint)
    p = str(tmp_path / "nometa.bin")
    write_reference_style(p, (40, 64, 96, 1))
    with pytest.raises(pkg.MlhError, match="networkMeta"):
        pkg.Model.load(p)  # neither a hint nor a networkMeta object
    # the transposed layout that the reference's writer produces ([dim, vocab] embedding) is refused
    p = str(tmp_path / "transposed.bin")
    write_reference_style(p, (40, 64, 96, 1))
    raw = open(p, "rb").read().replace(b'"shape": [40, 64]', b'"shape": [64, 40]', 1)
    open(p, "wb").write(raw)
    with pytest.raises(pkg.MlhError, match="vocabSize, dim"):
        pkg.Model.load(p, hint)


# --------------------------------------------------------------------------- tokenizer
def py_hash(token_bytes):
    h = 5381
    for c in token_bytes:
        c = c - 256 if c >= 128 else c  # plain char is signed on this platform
        h = (h * 33 + c) & 0xFFFFFFFF
    return h % 20011


def test_vocab_fixtures_and_lookup(pkg):
    v = pkg.Vocab(VOCAB_PV)
    strings = json.load(open(VOCAB_PV))
    assert len(v) == 10097 == len(strings)
    sample = json.load(open(SAMPLE))
    assert len(sample) == 166
    ids = [v.lookup(t) for t in sample]
    assert ids[:16] == [181, 190, 13, 151, 0, 154, 37, 13, 2925, 3448, 155, 2169, 1, 71, 383, 68]
    assert all(i >= 0 for i in ids)
    assert [v.lookup(t) for t in ("\n", "\t", " ", ",")] == [8, 9, 10, 0]
    assert v.lookup("~") == 10096
    for i in (0, 8, 9, 10, 5000, 10096):
        assert v.token(i) == strings[i].encode()
    for i, s in enumerate(strings):  # every entry maps back to its own index
        assert v.lookup(s) == i
    assert v.lookup("definitely-not-a-token") == -1 and v.lookup("") == -1
    assert v.token(-1) is None and v.token(10097) is None
    v2 = pkg.Vocab(VOCAB_MODEL)
    assert len(v2) == 10096 and v2.lookup("{") == -1 and v.lookup("{") == 10079


def test_vocab_size_mismatch_only_warns(pkg):
    v = pkg.Vocab(VOCAB_PV, expect_size=20160)  # the reference's vocabSize: larger than the file
    assert len(v) == 20160 and v.token(10096) == b"~" and v.token(15000) is None and v.lookup("~") == 10096
    v = pkg.Vocab(VOCAB_PV, expect_size=100)    # smaller: entries beyond are dropped
    assert len(v) == 100 and v.lookup("~") == -1 and v.lookup(",") == 0


def test_hash_token_is_djb2_mod_20011(pkg):
    assert pkg.host.mll_hash_token(b"") == 5381 % 20011
    assert pkg.host.mll_hash_token(b"a") == (5381 * 33 + 97) % 20011
    for s in (b"Once", b" upon", b"\n", b"~", b" Ollie's", "café".encode()):
        assert pkg.host.mll_hash_token(s) == py_hash(s)


def test_vocab_errors(pkg, tmp_path):
    with pytest.raises(pkg.MlhError):
        pkg.Vocab(str(tmp_path / "missing.json"))
    p = tmp_path / "obj.json"
    p.write_text('{"a": 1}')
    with pytest.raises(pkg.MlhError):
        pkg.Vocab(str(p))
    p = tmp_path / "bad.json"
    p.write_text('["a", "b"')
    with pytest.raises(pkg.MlhError):
        pkg.Vocab(str(p))
    p = tmp_path / "esc.json"
    p.write_text('["a\\"b", "\\u00e9\\n", 7, "\\ud83d\\ude00", "x\\\\y"]')
    v = pkg.Vocab(str(p))
    assert v.token(0) == b'a"b' and v.token(1) == "é\n".encode() and v.token(2) is None
    assert v.token(3) == "\U0001F600".encode() and v.token(4) == b"x\\y" and v.lookup('a"b') == 0


def test_json_reader_against_reference_cjson(pkg):
    """The host library's JSON reader and the reference's vendored cJSON (compiled as
    oracle/_ref/libcjson_ref.so) must hand out identical token strings for both vocabularies."""
    ref_path = os.path.join(ROOT, "oracle", "_ref", "libcjson_ref.so")
    if not os.path.exists(ref_path):
        pytest.skip("oracle/_ref/libcjson_ref.so not built (reference tree absent)")
    cj = ctypes.CDLL(ref_path)

    class CJ(ctypes.Structure):
        pass
    CJ._fields_ = [("next", ctypes.POINTER(CJ)), ("prev", ctypes.POINTER(CJ)), ("child", ctypes.POINTER(CJ)),
                   ("type", ctypes.c_int), ("valuestring", ctypes.c_char_p), ("valueint", ctypes.c_int),
                   ("valuedouble", ctypes.c_double), ("string", ctypes.c_char_p)]
    cj.cJSON_Parse.restype = ctypes.POINTER(CJ)
    cj.cJSON_Parse.argtypes = [ctypes.c_char_p]
    cj.cJSON_Delete.argtypes = [ctypes.POINTER(CJ)]
    for path in (VOCAB_PV, VOCAB_MODEL):
        root = cj.cJSON_Parse(open(path, "rb").read())
        assert root
        want, node = [], root.contents.child
        while node:
            want.append(node.contents.valuestring)
            node = node.contents.next
        cj.cJSON_Delete(root)
        v = pkg.Vocab(path)
        assert len(v) == len(want)
        assert [v.token(i) for i in range(len(v))] == want


# --------------------------------------------------------------------------- story loader
def test_story_context_rules(pkg, tmp_path):
    v = pkg.Vocab(VOCAB_PV)
    sample = json.load(open(SAMPLE))
    stories = tmp_path / "stories.json"
    stories.write_text(json.dumps([sample, sample[:3], [], ["Once", 5], ["Once", "zzzz-not-in-vocab"]]))
    path = str(stories)
    want = [v.lookup(t) for t in sample]
    assert v.story_context(path, 0, 100, 1280).tolist() == want
    assert v.story_context(path, 0, 50, 1280).tolist() == want[:83]        # 166 * 50 / 100
    assert v.story_context(path, 0, 0, 1280).tolist() == want[:1]          # at least one token
    assert v.story_context(path, 1, 34, 1280).tolist() == want[:1]         # 3 * 34 / 100 = 1
    assert v.story_context(path, 0, 100, 100).tolist() == want[:101]       # capped at maxL + 1
    for bad in (5, -1):
        assert len(v.story_context(path, bad, 100, 1280)) == 0             # index out of range
    assert len(v.story_context(path, 2, 100, 1280)) == 0                   # empty story
    assert len(v.story_context(path, 3, 100, 1280)) == 0                   # non-string token
    assert len(v.story_context(path, 4, 100, 1280)) == 0                   # unknown token
    assert len(v.story_context(str(tmp_path / "none.json"), 0, 100, 1280)) == 0
    notarr = tmp_path / "obj.json"
    notarr.write_text('{"a": []}')
    assert len(v.story_context(str(notarr), 0, 100, 1280)) == 0


def test_load_all_stories_of_a_file(pkg, tmp_path, capfd):
    """The multi-story loader (reference: loadStoriesFromFile, training_orchestrator.cu:103-273): slab of
    maxL+1 ids per loaded story padded with token 89, rightEnd = ids loaded - 2, bad stories skipped with
    the slot reused, file truncated to the story limit."""
    v = pkg.Vocab(VOCAB_PV)
    sample = json.load(open(SAMPLE))
    want = [v.lookup(t) for t in sample]
    stories = tmp_path / "stories.json"
    docs = [sample, "not an array", [], ["Once"], sample[:2], ["Once", 5], ["Once", " upon", "zzzz-not-in-vocab"],
            sample[:41], sample[:40], sample[:100]]
    stories.write_text(json.dumps(docs))
    maxL = 40
    flush = lambda: ctypes.CDLL(None).fflush(None)  # the library prints through C stdio
    toks, right = v.load_stories(str(stories), maxL)
    flush()
    out = capfd.readouterr().out
    assert toks.shape == (5, maxL + 1)
    assert right.tolist() == [39, 0, 39, 38, 39]        # 166 -> 41 loaded; 2; 41; 40; 100 -> 41
    assert toks[0].tolist() == want[:41] and toks[2].tolist() == want[:41] and toks[4].tolist() == want[:41]
    assert toks[1].tolist() == want[:2] + [89] * 39      # padded with the padding token
    assert toks[3].tolist() == want[:40] + [89]
    for msg in ("Processing 10 stories...", "Story at index 1 is not an array, skipping.",
                "Story at index 2 has no tokens, skipping.", "Story at index 3 has fewer than 2 tokens, skipping.",
                "Token at position 1 in story 5 is not a string.",
                "Token 'zzzz-not-in-vocab' not found in vocabulary (story 6, pos 2).",
                "Successfully processed 5 stories (out of 10 in file)."):
        assert msg in out, msg
    # the story limit truncates the FILE (stories looked at), as the reference's MAX_TRAINING_STORIES does
    toks2, right2 = v.load_stories(str(stories), maxL, max_stories=5)
    flush()
    assert right2.tolist() == [39, 0] and "File contains 10 stories, truncating to 5." in capfd.readouterr().out
    # a long maxL loads whole stories; rightEnd follows the story length
    toks3, right3 = v.load_stories(str(stories), 1280)
    assert right3.tolist() == [164, 0, 39, 38, 98] and toks3[0, :166].tolist() == want and np.all(toks3[0, 166:] == 89)
    # errors: missing file, not JSON, not an array -> -1; empty array -> 0 stories
    assert v.load_stories(str(tmp_path / "none.json"), maxL) is None
    bad = tmp_path / "bad.json"
    bad.write_text("[[")
    assert v.load_stories(str(bad), maxL) is None
    bad.write_text('{"a": []}')
    assert v.load_stories(str(bad), maxL) is None
    bad.write_text("[]")
    t0, r0 = v.load_stories(str(bad), maxL)
    assert t0.shape[0] == 0 and r0.shape[0] == 0


# --------------------------------------------------------------------------- generator and presets
M64 = (1 << 64) - 1


def splitmix64(x):
    x = (x + 0x9E3779B97F4A7C15) & M64
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M64
    return z ^ (z >> 31)


def stream_base(seed, key):
    return splitmix64(splitmix64(seed) ^ ((key * 0xD1342543DE82EF95) & M64))


def test_generator_is_counter_based_and_reproducible_in_python(pkg):
    toks = pkg.random_tokens(1, 0, 8192, 64)
    base = stream_base(1, 0x7000)
    assert toks.tolist() == [splitmix64((base + i) & M64) % 8192 for i in range(64)]
    assert not np.array_equal(toks, pkg.random_tokens(1, 1, 8192, 64))
    assert toks.min() >= 0 and toks.max() < 8192
    hp = pkg.config(1)
    model = pkg.Model.generate(hp, 0)
    Wq = model.tensor(2, 3)  # block 2, queryWeights: key (2+1)*64 + 3
    base = stream_base(0, 3 * 64 + 3)
    for p in (0, 1, 1000):
        a, b = splitmix64((base + 2 * p) & M64), splitmix64((base + 2 * p + 1) & M64)
        u1, u2 = ((a >> 11) + 1) / 2.0 ** 53, (b >> 11) / 2.0 ** 53
        r = np.sqrt(-2 * np.log(u1))
        flat = Wq.reshape(-1)
        assert abs(flat[2 * p] - 0.02 * r * np.cos(2 * np.pi * u2)) < 1e-8
        assert abs(flat[2 * p + 1] - 0.02 * r * np.sin(2 * np.pi * u2)) < 1e-8
    E = model.tensor(0, 0)
    assert abs(E.std() - 0.02) < 2e-4 and abs(E.mean()) < 1e-4
    for l in range(4):
        assert np.all(model.tensor(l, 2) == 1) and np.all(model.tensor(l, 7) == 1)  # RMSNorm gains 1
    assert np.all(model.tensor(0, 1) == 1)
    again = pkg.Model.generate(hp, 0)
    assert np.array_equal(again.tensor(3, 10), model.tensor(3, 10))
    other = pkg.Model.generate(hp, 1)
    assert not np.array_equal(other.tensor(3, 10), model.tensor(3, 10))
    # GDN gate biases are N(0, 1); uniform init stays inside its range
    hp3 = pkg.config(3)
    m3 = pkg.Model.generate(hp3, 2)
    biases = np.concatenate([m3.tensor(l, t) for l in range(12) for t in (15, 17) if m3.tensor(l, t) is not None])
    assert biases.size == 9 * 2 * 12 and 0.7 < biases.std() < 1.3
    m3.init_uniform(42, 0.02)
    w = m3.tensor(1, 8)
    assert w.min() >= -0.02 and w.max() < 0.02 and abs(w.std() - 0.02 / np.sqrt(3)) < 2e-4


def test_presets(pkg):
    ref = pkg.reference_defaults()  # network_meta.h:3-20
    assert (ref.dim, ref.attnHeads, ref.headDim, ref.ffnDim, ref.transformers, ref.maxL, ref.vocabSize) == \
        (768, 6, 128, 3072, 16, 1280, 20160)
    assert ref.qkRmsNorm == 1 and ref.queryGating == 1 and ref.ropeDenomBase == 10000.0
    c1, c2, c3, c4, c5 = (pkg.config(i) for i in range(1, 6))
    assert (c1.dim, c1.transformers, c1.attnHeads, c1.headDim, c1.ffnDim, c1.vocabSize, c1.maxL) == (256, 4, 4, 64, 704, 4096, 144)
    assert (c2.dim, c2.transformers, c2.attnHeads, c2.headDim, c2.ffnDim, c2.vocabSize, c2.maxL) == (768, 12, 12, 64, 2048, 8192, 576)
    assert all(k == 0 for k in c2.layerKinds[:12]) and c2.qkRmsNorm == 0 and c2.queryGating == 0
    # 3 GDN : 1 attention in application order; file index 0 (top) is applied last
    assert list(c3.layerKinds[:12]) == [0, 1, 1, 1, 0, 1, 1, 1, 0, 1, 1, 1]
    assert (c3.gdnHeads, c3.gdnDk, c3.gdnDv, c3.pleDim, c3.maxL, c3.maxSeqs) == (12, 64, 64, 64, 1152, 1)
    assert (c4.maxSeqs, c4.maxL) == (64, 2048)
    assert (c5.dim, c5.transformers, c5.attnHeads, c5.headDim, c5.ffnDim, c5.vocabSize, c5.weightDtype, c5.maxSeqs) == \
        (2048, 24, 16, 128, 5632, 32000, pkg.DTYPE_BF16, 8)
    assert sum(1 for k in c5.layerKinds[:24] if k == 0) == 6
    with pytest.raises(ValueError):
        pkg.config(6)
