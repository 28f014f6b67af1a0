"""Command-line flags of `llava` that are decided before any device is touched (reference: llava_context.cpp:163-212)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "llama-vulkan_amd", "bin", "llava")

pytestmark = pytest.mark.skipif(not os.path.exists(EXE), reason="bin/llava is not built")


def run(*args, env=None):
    e = dict(os.environ)
    e.pop("LLAVA_MODEL", None)
    e.update(env or {})
    return subprocess.run([EXE, *args], capture_output=True, timeout=60, env=e)


@pytest.mark.parametrize("flag", ["-c", "--control"])
def test_control_mode_is_refused_like_the_reference(flag):
    r = run(flag)
    assert r.returncode == 1
    assert b"Control disabled for now" in r.stderr


@pytest.mark.parametrize("flag", ["-v", "--verbose"])
def test_verbose_long_and_short_form_are_accepted(flag):
    # accepted, then the missing model path is what ends the run
    r = run(flag)
    assert r.returncode == 1
    assert b"Unknown argument" not in r.stderr
    assert b"model" in r.stderr.lower()


def test_help_prints_usage():
    r = run("--help")
    assert r.returncode == 0
    assert b"usage" in (r.stdout + r.stderr).lower()


def test_unknown_flag_is_an_error():
    r = run("--no-such-flag")
    assert r.returncode == 1
    assert b"Unknown argument" in r.stderr
