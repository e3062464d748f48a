#!/usr/bin/env python3
"""Writes cfg5_prefill_golden.npz: configuration 5 at its full size (d2048, 24 layers 3 GDN : 1 attention, 16 heads
x 128, ffn 5632, vocab 32000, PLE 64, weights N(0, 0.02) from seed 5 rounded to bf16) and ONE 2048-token prompt
(seed 5, sequence 0) through the float64 CPU oracle's full recompute on the same bf16-rounded weights: the logits
at a handful of positions, kept as float32.  Eleven minutes and about 20 GB on eight cores (three minutes for the 2048-token pass).
Run from the repository root: python tests/golden/make_cfg5_golden.py"""
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

POSITIONS = (0, 63, 64, 127, 128, 999, 1000, 1535, 2047)  # chunk and page edges, odd places, the end


def main():
    m, orc = entry.load_package(), entry.load_oracle()
    hp = m.config(5, maxSeqs=1)
    model = m.Model.generate(hp, seed=5)
    toks = m.random_tokens(5, 0, hp.vocabSize, 2048)
    w = orc.Weights.from_model(model, bf16=True)
    t0 = time.time()
    hid = orc.forward_full(w, toks, "f64", last_only=True, want_hidden=True)
    print(f"oracle pass: {time.time() - t0:.0f} s", flush=True)
    # last-position logits come from the pass itself; the other positions' from one pass per prefix would cost the
    # same again each, so they are taken from prefixes only where that is cheap (the short ones) ...
    out = {2047: hid["logits"][0].astype(np.float32)}
    for p in POSITIONS:
        if p == 2047:
            continue
        t0 = time.time()
        out[p] = orc.forward_full(w, toks[:p + 1], "f64", last_only=True)["logits"][0].astype(np.float32)
        print(f"prefix of {p + 1}: {time.time() - t0:.0f} s", flush=True)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "cfg5_prefill_golden.npz"),
                        tokens=toks.astype(np.int32), positions=np.array(POSITIONS, dtype=np.int32),
                        logits=np.stack([out[p] for p in POSITIONS]),
                        embedding_head=model.tensor(0, 0)[:4, :8].copy())
    print("argmax per position:", [int(np.argmax(out[p])) for p in POSITIONS])


if __name__ == "__main__":
    main()
