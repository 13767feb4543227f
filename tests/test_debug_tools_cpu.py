"""The debug-build plumbing, without a GPU: FA_PAGED_ATTENTION_LIBRARY names another build of the library
(a build with the in-kernel timeline or a cost probe compiled in), the build module takes an output path and
extra compiler flags, and the timeline reader's percentile helper ignores the slots a wavefront left empty."""
import importlib
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_override_is_read_from_the_environment(tmp_path):
    other = tmp_path / "libfa_other.so"
    code = "from flash_attention_factory_amd import _cabi; print(_cabi.LIBRARY)"
    env = dict(os.environ, FA_PAGED_ATTENTION_LIBRARY=str(other), PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, check=True).stdout.strip()
    assert out == str(other)
    # a library that is not there is an error, never a fallback to the product library
    code = "from flash_attention_factory_amd import _cabi; _cabi.load()"
    res = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True)
    assert res.returncode != 0 and "libfa_other.so" in res.stderr
    env.pop("FA_PAGED_ATTENTION_LIBRARY")
    out = subprocess.run([sys.executable, "-c", "from flash_attention_factory_amd import _cabi; print(_cabi.LIBRARY)"],
                         env=env, capture_output=True, text=True, check=True).stdout.strip()
    assert out == os.path.join(ROOT, "flash_attention_factory_amd", "libfa_paged_attention.so")


def test_build_command_line(monkeypatch, tmp_path):
    from flash_attention_factory_amd import _build
    seen = {}

    def fake_run(cmd, capture_output, text):
        seen["cmd"] = cmd
        return subprocess.CompletedProcess(cmd, 0, "", "")

    monkeypatch.setattr(_build.subprocess, "run", fake_run)
    out = _build.build(extra_flags=["-DFA_TIMELINE"], output=str(tmp_path / "libfa_timeline.so"))
    assert out.endswith("libfa_timeline.so")
    cmd = seen["cmd"]
    assert "-DFA_TIMELINE" in cmd and cmd[-1] == out and cmd[-2] == "-o" and _build.SOURCE in cmd
    assert "--offload-arch=gfx950" in cmd and "-packed-fp32-ops" in cmd
    _build.build()
    assert seen["cmd"][-1] == _build.LIBRARY  # the product library by default


def test_timeline_percentiles_skip_empty_slots():
    dt = importlib.import_module("flash_attention_factory_amd.debug_timeline")
    assert dt._pct([1.0, float("nan"), 3.0], (0, 50, 100)) == [1.0, 2.0, 3.0]
    assert all(np.isnan(v) for v in dt._pct([float("nan")] * 3))
