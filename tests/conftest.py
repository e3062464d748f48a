import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    """The product package (ctypes bindings over libmlh.so / libminillm.so).  Built libraries are
    loaded as they are; only when none exist is the build run."""
    lib = os.path.join(entry.PKG_DIR, "lib")
    if not (os.path.exists(os.path.join(lib, "libmlh.so")) and os.path.exists(os.path.join(lib, "libminillm.so"))):
        entry.build()
    return entry.load_package()


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (test infrastructure)."""
    if not os.path.exists(os.path.join(ROOT, "oracle", "liboracle.so")):
        import subprocess
        subprocess.run(["make", "liboracle.so"], cwd=os.path.join(ROOT, "oracle"), check=True)
    return entry.load_oracle()


def rel_diff(a, b):
    """The reference's comparison metric |a-b| / max(|a|,|b|) (comparison_logits_grad.js:26-38;
    cuda_pytorch_grad_comparison.js:281-289), elementwise, 0 where both are 0."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    den = np.maximum(np.abs(a), np.abs(b))
    return np.where(den > 0, np.abs(a - b) / np.where(den > 0, den, 1), 0.0)


def assert_logits_close(got, want, rtol, what=""):
    """Logits agree within rtol in the reference's relative metric.  Elements whose magnitude is
    below 1e-2 of the largest logit are compared absolutely against rtol * that floor: a relative
    test on values near zero measures nothing but the cancellation in the dot product (fp32 sums over
    a few hundred terms of O(1) logits carry ~1e-6 of absolute noise)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert np.all(np.isfinite(got)), f"{what}: non-finite logits"
    floor = 1e-2 * np.max(np.abs(want))
    den = np.maximum(np.maximum(np.abs(got), np.abs(want)), floor)
    r = np.abs(got - want) / den
    worst = int(np.argmax(r))
    assert r[worst] <= rtol, (f"{what}: logit {worst} differs: got {got[worst]!r} want {want[worst]!r} "
                              f"rel {r[worst]:.3e} > {rtol}")
    # independent of the floor: the largest absolute error, relative to the largest logit
    amax = float(np.max(np.abs(got - want)) / np.max(np.abs(want)))
    assert amax <= rtol * 0.1, f"{what}: max |diff| / max |logit| = {amax:.3e}"
    return float(r[worst])


def check_greedy_against_oracle(decoder, prompt, gpu_ids, gap_tol, gpu_logits_per_step=None, rtol=None,
                                what=""):
    """Feeds the oracle the prompt and then the GPU's own tokens, so both see the same history.
    At every step the GPU's pick must be the oracle's argmax, or lie within gap_tol of the
    oracle's best logit (a top-2 gap below tolerance).  Returns (#exact, #tolerated)."""
    decoder.reset()
    lg = None
    for t in prompt:
        _, lg = decoder.step(int(t))
    exact = tolerated = 0
    for i, gid in enumerate(gpu_ids):
        best = int(np.argmax(lg))
        if isinstance(gpu_logits_per_step, dict):  # logits recorded at some steps only
            if i in gpu_logits_per_step:
                assert_logits_close(gpu_logits_per_step[i], lg, rtol, f"{what} step {i}")
        elif gpu_logits_per_step is not None:
            assert_logits_close(gpu_logits_per_step[i], lg, rtol, f"{what} step {i}")
        if int(gid) == best:
            exact += 1
        else:
            gap = float(lg[best] - lg[int(gid)])
            assert gap <= gap_tol, (f"{what} step {i}: GPU picked {int(gid)} (logit {lg[int(gid)]:.8f}), oracle "
                                    f"{best} (logit {lg[best]:.8f}), gap {gap:.3e} > {gap_tol}")
            tolerated += 1
        if i + 1 < len(gpu_ids):
            _, lg = decoder.step(int(gid))
    return exact, tolerated
