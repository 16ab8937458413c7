"""The library's process-wide knobs (fo_tune, fo_set_wait_timeout_ms) under ThreadSanitizer:
threads that set them while other threads read them the way every launch does.  Host code only
(flashoverlap_amd/csrc/fo_knobs.h is plain C++); no GPU is involved."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "knobs_threads.cpp")


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
    if shutil.which("g++") is None:
        pytest.skip("no g++")
    exe = str(tmp_path_factory.mktemp("knobs") / "knobs_threads")
    p = subprocess.run(["g++", "-std=c++17", "-O1", "-g", "-fsanitize=thread", "-pthread", SRC, "-o", exe],
                       capture_output=True, text=True)
    if p.returncode != 0 and "tsan" in (p.stderr or "").lower():
        pytest.skip("ThreadSanitizer runtime not available: " + p.stderr[-200:])
    assert p.returncode == 0, p.stderr
    return exe


def _run(exe, *args):
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1 exitcode=66")
    return subprocess.run([exe, *args], capture_output=True, text=True, env=env, timeout=300)


def test_knobs_are_race_free_and_stay_in_range(harness):
    p = _run(harness)
    assert p.returncode == 0, p.stdout + p.stderr
    assert p.stdout.startswith("ok:") and "data race" not in p.stderr


def test_sanitizer_reports_the_same_traffic_on_plain_ints(harness):
    p = _run(harness, "--plain-int")
    assert p.returncode == 66 and "data race" in p.stderr, (p.returncode, p.stdout, p.stderr[-400:])


def test_library_uses_the_knobs_header_and_keeps_no_plain_globals():
    """The launchers read the knobs through fo_knobs.h; no translation unit keeps an int of its own."""
    import re
    csrc = os.path.join(ROOT, "flashoverlap_amd", "csrc")
    for name in ("fo_gemm.hip", "fo_sync.hip"):
        text = open(os.path.join(csrc, name)).read()
        assert '#include "fo_knobs.h"' in text
        assert not re.search(r"^\s*(static\s+|extern\s+)?int\s+g_(store_mode|release_mode|timeout_ms|copy_streaming_stores)\b",
                             text, flags=re.M), name
