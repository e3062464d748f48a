#!/usr/bin/env python3
"""Writes cfg1_golden.npz: configuration 1 (d256, 4 layers, 4 heads x 64, ffn 704, vocab 4096,
fp32 weights N(0, 0.02) from seed 0, gains 1, 16-token uniform-random prompt, 128 greedy steps)
run through the float64 CPU oracle.  Run from the repository root: python tests/golden/make_golden.py"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402


def main():
    m, orc = entry.load_package(), entry.load_oracle()
    hp = m.config(1)
    model = m.Model.generate(hp, seed=0)
    prompt = m.random_tokens(0, 0, hp.vocabSize, 16)
    dec = orc.Decoder(orc.Weights.from_model(model), "f64")
    lg = None
    for t in prompt:
        _, lg = dec.step(int(t))
    ids, top_idx, top_val, full = [], [], [], {}
    keep = (0, 1, 63, 127)
    for step in range(128):
        order = np.argsort(-lg, kind="stable")[:4]
        top_idx.append(order)
        top_val.append(lg[order])
        if step in keep:
            full[step] = lg.astype(np.float32)
        ids.append(int(order[0]))
        if step < 127:
            _, lg = dec.step(ids[-1])
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "cfg1_golden.npz"),
                        prompt=prompt.astype(np.int32), ids=np.array(ids, dtype=np.int32),
                        top_idx=np.array(top_idx, dtype=np.int32), top_val=np.array(top_val, dtype=np.float64),
                        full_steps=np.array(keep, dtype=np.int32),
                        full_logits=np.stack([full[s] for s in keep]),
                        embedding_head=model.tensor(0, 0)[:4, :8].copy())
    print("ids:", ids[:16], "... distinct:", len(set(ids)))


if __name__ == "__main__":
    main()
