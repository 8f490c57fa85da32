"""Reference-named C++ call sites (include/lyradiff_compat.h) on the GPU through the C ABI."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_reference_style_call_sites(dev):
    exe = os.path.join(ROOT, "tests", "cpp", "compat_check")
    assert os.path.exists(exe), "build it with `python -m lyradiff_amd.build` (prebuilt binaries travel to the GPU box)"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count(": 0 mismatches") == 4 and "0 outliers" in r.stdout and "prefix: yes" in r.stdout


def test_cpp_layer_types(dev):
    """Tensor/TensorMap/Allocator/W4A4Gemm/CutlassInt8GemmRunner/profiler (include/lyradiff_layers.h)."""
    exe = os.path.join(ROOT, "tests", "cpp", "layers_check")
    assert os.path.exists(exe), "build it with `python -m lyradiff_amd.build` (prebuilt binaries travel to the GPU box)"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("0 mismatches") == 3 and r.stdout.count(": yes") == 3 and "0 outliers" in r.stdout


def test_cpp_flux_fp8_types(dev):
    """FluxAttnPostFP8Processor / FluxSingleTransformerFP8Mlp / FP8LoraWeight (include/lyradiff_layers.h) and the rope launchers: each fused
    forward equals the reference's launch sequence run step by step, bit for bit."""
    exe = os.path.join(ROOT, "tests", "cpp", "flux_fp8_check")
    assert os.path.exists(exe), "build it with `python -m lyradiff_amd.build` (prebuilt binaries travel to the GPU box)"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count(" 0 mismatches") == 5
