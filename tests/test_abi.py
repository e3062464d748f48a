"""The C-ABI libraries load without a GPU, export every symbol the headers declare, and refuse
loudly to compute when no device is present.  CPU only (no compute calls)."""
import os
import re
import subprocess

import pytest

from conftest import ROOT

INCLUDE = os.path.join(ROOT, "include")


def declared_functions(header):
    text = open(os.path.join(INCLUDE, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    text = re.sub(r"typedef\s+struct\s*\{.*?\}\s*\w+\s*;", "", text, flags=re.S)
    text = re.sub(r"enum\s*\{.*?\}\s*;", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b([A-Za-z_]\w*)\s*\([^;{]*\)\s*;", text)))


def exported(lib):
    out = subprocess.run(["nm", "-D", "--defined-only", lib], capture_output=True, text=True, check=True).stdout
    return {line.split()[-1] for line in out.splitlines() if line.strip()}


def exported_demangled(lib):
    out = subprocess.run(["nm", "-D", "-C", "--defined-only", lib], capture_output=True, text=True, check=True).stdout
    return out


def test_device_library_exports_every_declared_symbol(pkg):
    names = declared_functions("mlh.h")
    assert len(names) >= 20 and "mlh_decode_loop" in names and "mlh_create" in names
    have = exported(os.path.join(pkg.LIB_DIR, "libmlh.so"))
    missing = [n for n in names if n not in have]
    assert not missing, f"libmlh.so does not export {missing}"
    assert sorted(pkg.DEVICE_SYMBOLS) == names  # the Python binding covers the whole header


def test_host_library_exports_every_declared_symbol(pkg):
    names = declared_functions("mini_llm_host.h")
    assert len(names) >= 15 and "mll_model_load" in names
    have = exported(os.path.join(pkg.LIB_DIR, "libminillm.so"))
    missing = [n for n in names if n not in have]
    assert not missing, f"libminillm.so does not export {missing}"
    assert sorted(pkg.HOST_SYMBOLS) == names


def test_reference_named_surface_is_exported_with_cxx_linkage(pkg):
    """The reference declares these with C++ linkage (load_model.h:3-6, inference.h:3-4,
    inference_orchestrator.h:17-18, memory_allocation.h:5, random_weights.h:4, main.cu:45)."""
    dem = exported_demangled(os.path.join(pkg.LIB_DIR, "libminillm.so"))
    for sig in ("allocateMemory(bool)", "loadVocab(char const*)", "vocabGetToken(int)", "vocabLookup(char const*)",
                "loadModel(char const*)", "initializeRandomWeights(float)", "runInference(int)",
                "runInferenceAllPositions(int, float*, float*)",
                "getPreComputedRopeTheta(float*, int)", "loadStoryContext(char const*, int, int)",
                "runInferenceLoop(char const*, int, int, bool, bool)", "seqTokenIndices"):
        assert sig in dem, f"{sig} not exported"
    for name in declared_functions("mini_llm_reference_api.h"):
        assert name in dem


def test_no_gpu_means_loud_failure_not_a_fallback(pkg):
    if pkg.device_count() > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(pkg.MlhError, match="no HIP device"):
        pkg.Device(pkg.config(1), 0)


def test_create_validates_hyperparameters(pkg):
    if pkg.device_count() == 0:
        bad = pkg.config(1, headDim=32)  # attnHeads * headDim != dim is rejected before any device call
        with pytest.raises(pkg.MlhError, match="attnHeads"):
            pkg.Device(bad, 0)
        with pytest.raises(pkg.MlhError, match="positive"):
            pkg.Device(pkg.config(1, maxSeqs=0), 0)


def test_product_never_links_the_oracle(pkg):
    for lib in ("libmlh.so", "libminillm.so"):
        out = subprocess.run(["ldd", os.path.join(pkg.LIB_DIR, lib)], capture_output=True, text=True).stdout
        assert "oracle" not in out
    for dirpath, _, files in os.walk(os.path.join(ROOT, "mini-llm-cuda_amd")):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"
