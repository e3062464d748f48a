"""The reference-shaped main() builds against the replacement headers alone (CPU), and on the GPU it
runs the whole loop -- vocab.json, tokenised story, model.bin, greedy generation to maxL -- with ids equal
to the oracle's."""
import json
import os
import subprocess

import numpy as np
import pytest

from conftest import GOLDEN, ROOT, check_greedy_against_oracle

LIB = os.path.join(ROOT, "mini-llm-cuda_amd", "lib")


def build_main(tmp_path):
    exe = str(tmp_path / "dropin_main")
    subprocess.run(["g++", "-std=c++17", os.path.join(ROOT, "tests", "cpp", "dropin_main.cpp"),
                    "-I" + os.path.join(ROOT, "include"), "-L" + LIB, "-lminillm", "-lmlh",
                    "-Wl,-rpath," + LIB, "-o", exe], check=True)
    return exe


def test_reference_shaped_main_builds_and_reports_missing_gpu(pkg, tmp_path):
    exe = build_main(tmp_path)
    if pkg.device_count() > 0:
        pytest.skip("a GPU is present")
    r = subprocess.run([exe, "1", "v", "s", "0", "50"], capture_output=True, text=True)
    assert r.returncode == 3 and "no HIP device" in r.stdout


@pytest.mark.gpu
def test_reference_shaped_main_generates_like_the_oracle(pkg, orc, tmp_path):
    exe = build_main(tmp_path)
    vocab = os.path.join(GOLDEN, "vocab_pytorch_verification.json")
    sample = json.load(open(os.path.join(GOLDEN, "sample.json")))
    stories = tmp_path / "stories.json"
    stories.write_text(json.dumps([sample[:40], sample]))
    hp = pkg.config(1, vocabSize=10097, maxL=96)
    model = pkg.Model.generate(hp, seed=3)
    path = str(tmp_path / "model.bin")
    model.save(path)
    # config 1 preset has vocab 4096; run the reference defaults' code path with an explicit model instead
    r = subprocess.run([exe, "1", vocab, str(stories), "1", "25", path], capture_output=True, text=True)
    # config 1's compiled-in vocabulary (4096) does not match this file: loadModelFile must refuse it
    assert r.returncode == 4 and "Error" in r.stdout
    hp1 = pkg.config(1)
    model1 = pkg.Model.generate(hp1, seed=3)
    path1 = str(tmp_path / "model1.bin")
    model1.save(path1)
    small = tmp_path / "small_vocab.json"
    small.write_text(json.dumps(json.load(open(vocab))[:4096]))
    story = [t for t in sample if json.load(open(small)).count(t)][:60]
    stories.write_text(json.dumps([story]))
    r = subprocess.run([exe, "1", str(small), str(stories), "0", "50", path1], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "Generation complete. Generated 114 new tokens." in r.stdout  # 144 - 30
    ids = [int(x) for x in r.stdout.strip().splitlines()[-1].split()[1:]]
    v = pkg.Vocab(str(small))
    prompt = [v.lookup(t) for t in story[:30]]
    assert ids[:30] == prompt
    dec = orc.Decoder(orc.Weights.from_model(model1), "f64")
    check_greedy_against_oracle(dec, prompt, ids[30:144], 2e-5, what="drop-in main")


def build_exe(tmp_path, name):
    exe = str(tmp_path / name)
    subprocess.run(["g++", "-std=c++17", os.path.join(ROOT, "tests", "cpp", name + ".cpp"),
                    "-I" + os.path.join(ROOT, "include"), "-L" + LIB, "-lminillm", "-lmlh",
                    "-Wl,-rpath," + LIB, "-o", exe], check=True)
    return exe


def _small_setup(pkg, tmp_path, max_l=None):
    """Config 1 with its 4096-token vocabulary cut from the reference's vocabulary fixture, a story made of
    the sample's tokens that survive the cut, and a written model.bin."""
    vocab = os.path.join(GOLDEN, "vocab_pytorch_verification.json")
    sample = json.load(open(os.path.join(GOLDEN, "sample.json")))
    hp1 = pkg.config(1) if max_l is None else pkg.config(1, maxL=max_l)
    model1 = pkg.Model.generate(hp1, seed=3)
    path1 = str(tmp_path / "model1.bin")
    model1.save(path1)
    words = json.load(open(vocab))[:4096]
    small = tmp_path / "small_vocab.json"
    small.write_text(json.dumps(words))
    keep = set(words)
    story = [t for t in sample if t in keep][:60]
    stories = tmp_path / "stories.json"
    stories.write_text(json.dumps([story]))
    return hp1, model1, path1, str(small), str(stories), story


def _parse_verbose(stdout):
    """[(position, [(rank, idx, prob)...], picked idx)] from the reference's top-10 blocks."""
    import re
    blocks = []
    cur = None
    for line in stdout.splitlines():
        m = re.match(r"--- Top 10 Most Probable Next Tokens \(position (\d+)\) ---", line)
        if m:
            cur = [int(m.group(1)), [], None]
            blocks.append(cur)
            continue
        m = re.match(r"\s*(\d+)\. .*\(idx:\s*(\d+), prob: ([0-9.]+)\)$", line)
        if m and cur is not None:
            cur[1].append((int(m.group(1)), int(m.group(2)), float(m.group(3))))
            continue
        m = re.match(r"Most probable token: .* \(index: (\d+)\)$", line)
        if m and cur is not None:
            cur[2] = int(m.group(1))
    return blocks


@pytest.mark.gpu
def test_verbose_and_interactive_branches(pkg, orc, tmp_path):
    """runInferenceLoop(skipUserInput=true, verboseOutput=true): the reference's top-10 block per token
    (inference_orchestrator.cu:86-146) with probabilities and order equal to the oracle's softmax, the same ids
    as the quiet device-resident branch; and the interactive branch stepping on Enter and stopping on 'q'."""
    exe = build_exe(tmp_path, "dropin_main")
    hp1, model1, path1, small, stories, story = _small_setup(pkg, tmp_path, max_l=48)
    args = [exe, "1", small, stories, "0", "50", path1]
    fast = subprocess.run(args + ["fast", "48"], capture_output=True, text=True)
    verb = subprocess.run(args + ["verbose", "48"], capture_output=True, text=True)
    assert fast.returncode == 0 and verb.returncode == 0, verb.stdout[-2000:]
    ids_fast = [int(x) for x in fast.stdout.strip().splitlines()[-1].split()[1:]]
    ids_verb = [int(x) for x in verb.stdout.strip().splitlines()[-1].split()[1:]]
    assert ids_fast == ids_verb and len(ids_verb) == 48
    assert "Generation complete. Generated 18 new tokens." in verb.stdout
    blocks = _parse_verbose(verb.stdout)
    assert [b[0] for b in blocks] == list(range(30, 48))
    assert verb.stdout.count("[Token added. Total context:") == 18
    v = pkg.Vocab(small)
    dec = orc.Decoder(orc.Weights.from_model(model1), "f64")
    for t in ids_verb[:29]:
        dec.step(t, want_logits=False)
    for (pos, rows, picked) in blocks:
        _, lg = dec.step(ids_verb[pos - 1])
        p = np.exp(lg - lg.max())
        p /= p.sum()
        order = sorted(range(len(p)), key=lambda i: (-p[i], i))[:10]
        assert [r[0] for r in rows] == list(range(1, 11))
        for rank, (_, idx, prob) in enumerate(rows):
            assert abs(prob - p[idx]) <= 1e-6 + 1e-4 * p[idx]            # printed with six decimals
            assert idx == order[rank] or abs(p[idx] - p[order[rank]]) <= 2e-5 * p[order[rank]] + 1e-9
        assert picked == ids_verb[pos] and (picked == order[0] or lg[order[0]] - lg[picked] <= 2e-5)
    # interactive: three tokens accepted with Enter, then 'q'
    inter = subprocess.run(args + ["interactive", "48"], input="\n\n\nq\n", capture_output=True, text=True)
    assert inter.returncode == 0
    assert "Generation stopped by user." in inter.stdout and "Generation complete. Generated 3 new tokens." in inter.stdout
    assert inter.stdout.count("Press Enter to add this token and continue") == 4
    ids_int = [int(x) for x in inter.stdout.strip().splitlines()[-1].split()[1:]]
    assert ids_int[:33] == ids_verb[:33]
    # stdin closed: the loop ends as the reference's does on fgets == NULL
    eof = subprocess.run(args + ["interactive", "48"], input="", capture_output=True, text=True)
    assert eof.returncode == 0 and "Generation complete. Generated 0 new tokens." in eof.stdout


@pytest.mark.gpu
def test_run_inference_calls_and_all_positions(pkg, orc, tmp_path):
    """runInference(L) on a grown, unchanged, edited, shortened and regrown seqTokenIndices (cache reuse or
    rebuild), mlh_read_probs / mll_top_k after each, and runInferenceAllPositions, against the oracle's
    reference-style full recompute of the same token lists."""
    exe = build_exe(tmp_path, "dropin_calls")
    hp1, model1, path1, small, stories, story = _small_setup(pkg, tmp_path)
    out = tmp_path / "out"
    out.mkdir()
    r = subprocess.run([exe, "1", small, stories, path1, str(out)], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-2000:]
    w = orc.Weights.from_model(model1)
    lines = dict((l.split()[0], l.split()[1:]) for l in open(out / "tokens.txt").read().splitlines())
    V = hp1.vocabSize
    lens = {}
    for name in ("first", "grown", "unchanged", "edited", "shorter", "regrown", "after_allpos"):
        toks = np.array([int(x) for x in lines[name]], np.int32)
        lens[name] = len(toks)
        ref = orc.forward_full(w, toks, "f64", want_probs=True)
        lg = np.fromfile(out / f"{name}_logits.f32", dtype=np.float32)
        pr = np.fromfile(out / f"{name}_probs.f32", dtype=np.float32)
        assert lg.shape == (V,) and pr.shape == (V,)
        from conftest import assert_logits_close
        assert_logits_close(lg, ref["logits"][0], 1e-3, name)
        p = ref["probs"][0]
        assert np.max(np.abs(pr - p) / p) < 1e-4 and abs(float(pr.sum()) - 1) < 1e-5      # softmax of the logits
        top = [int(x) for x in lines[name + "_top"]]
        order = sorted(range(V), key=lambda i: (-p[i], i))[:10]
        for rank, idx in enumerate(top):  # descending probability, ties (within fp32 of the softmax) aside
            assert idx == order[rank] or abs(p[idx] - p[order[rank]]) <= 2e-5 * p[order[rank]]
        assert len(set(top)) == 10 and all(pr[top[i]] >= pr[top[i + 1]] for i in range(9))
    assert lens["grown"] == lens["first"] + 2 and lens["shorter"] == lens["first"] - 5
    toks = np.array([int(x) for x in lines["allpos"]], np.int32)
    ref = orc.forward_full(w, toks, "f64", last_only=False, want_probs=True)
    pr = np.fromfile(out / "allpos_probs.f32", dtype=np.float32).reshape(len(toks), V)  # position i at i * vocabSize
    assert np.max(np.abs(pr - ref["probs"]) / ref["probs"]) < 1e-4
    nll = -np.log(np.maximum(ref["probs"][np.arange(len(toks) - 1), toks[1:]], 1e-4))
    assert abs(float(lines["loss"][0]) - nll.mean()) < 1e-5 * nll.mean()


@pytest.mark.gpu
def test_top_k_ties_and_story_feeders(pkg, orc, tmp_path):
    """mll_top_k orders equal probabilities by the lower id; the multi-story loader's slab feeds one batched
    prefill (logits per story against the oracle) and the per-story loss of the reference's processSequence."""
    from conftest import assert_logits_close
    vocab = os.path.join(GOLDEN, "vocab_pytorch_verification.json")
    sample = json.load(open(os.path.join(GOLDEN, "sample.json")))
    words = json.load(open(vocab))[:4096]
    small = tmp_path / "small_vocab.json"
    small.write_text(json.dumps(words))
    keep = set(words)
    story = [t for t in sample if t in keep]
    stories = tmp_path / "stories.json"
    stories.write_text(json.dumps([story[:70], story[5:30], ["Once"], story[10:12], story[:131]]))
    hp = pkg.config(1, maxL=96, maxSeqs=4)
    model = pkg.Model.generate(hp, seed=8)
    E = model.tensor(0, 0)
    E[4000] = E[17]
    E[123] = E[17]  # three identical embedding rows: identical logits and probabilities
    dev = pkg.Device(hp, 0)
    dev.upload(model)
    w = orc.Weights.from_model(model)
    v = pkg.Vocab(str(small))
    toks, right = v.load_stories(str(stories), hp.maxL)
    assert right.tolist() == [68, 23, 0, 95]
    dev.prefill_stories(toks, right, 0, 4)
    for i in range(4):
        L = int(right[i]) + 1
        assert dev.seq_len(i) == L
        ref = orc.forward_full(w, toks[i, :L], "f64", want_probs=True)
        assert_logits_close(dev.logits(i), ref["logits"][0], 1e-3, f"story {i}")
        pr = dev.probs(i)
        assert np.max(np.abs(pr - ref["probs"][0]) / ref["probs"][0]) < 1e-4
        top = dev.top_k(4096, seq=i)   # the whole vocabulary, sorted
        ids = [t[0] for t in top]
        assert sorted(ids) == list(range(4096))
        for a, b in zip(top, top[1:]):
            assert a[1] > b[1] or (a[1] == b[1] and a[0] < b[0])
        at = ids.index(17)
        assert ids[at:at + 3] == [17, 123, 4000] or pr[17] != pr[123] or pr[123] != pr[4000]
        assert pr[17] == pr[123] == pr[4000]
    for i in range(4):
        L = int(right[i]) + 1
        loss, n = dev.story_loss(toks[i], right[i])
        ref = orc.forward_full(w, toks[i, :L], "f64", last_only=False, want_probs=True)["probs"]
        tgt = toks[i, 1:L + 1]
        mask = tgt != 89
        want = -np.log(np.maximum(ref[np.arange(L)[mask], tgt[mask]], 1e-4)).sum()
        assert n == int(mask.sum()) and abs(loss - want) < 1e-4 * want
    dev.close()
