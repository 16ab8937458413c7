"""The counter protocol (tile stores -> release-ordered signal -> polling waiter -> reset ->
per-group consumer -> join before the next call) as a multi-threaded CPU model under
ThreadSanitizer: oracle/counter_protocol.cpp.  No GPU is involved; the failure-handling cases
(a count that never arrives) are forced from the host here, never on the device."""
import os
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "oracle", "counter_protocol.cpp")


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    exe = str(tmp_path_factory.mktemp("tsan") / "counter_protocol")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=thread", "-pthread", SRC, "-o", exe]
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0 and "tsan" in (p.stderr or "").lower():
        pytest.skip("ThreadSanitizer runtime not available: " + p.stderr[-200:])
    assert p.returncode == 0, p.stderr
    return exe


def _run(exe, *args):
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1 exitcode=66")
    return subprocess.run([exe, *args], capture_output=True, text=True, env=env, timeout=300)


def test_protocol_is_race_free_and_correct(model):
    p = _run(model, "--calls", "6", "--producers", "6")
    assert p.returncode == 0, p.stdout + p.stderr
    assert "ok: 6 calls" in p.stdout and "data race" not in p.stderr


def test_short_count_trips_the_bounded_wait(model):
    p = _run(model, "--short-count")
    assert p.returncode == 0, p.stdout + p.stderr
    assert "bounded wait expired on group 5 after releasing 5 groups" in p.stdout


def test_sanitizer_sees_the_race_when_the_ordering_is_removed(model):
    p = _run(model, "--relaxed-signal", "--calls", "3")
    assert p.returncode == 66 and "data race" in p.stderr, (p.returncode, p.stdout, p.stderr[-500:])
