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
