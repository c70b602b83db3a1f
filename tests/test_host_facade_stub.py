"""Host logic of the C++ facade without a GPU: tests/cpp/facade_test.cpp is built against a stand-in for the device library
(every entry point succeeds, memory calls act on host memory, graph handles are tracked, nothing is computed) with
AddressSanitizer and UBSan, and its scenarios are run for what the host side does on its own: the order and lifetime of
allocations, recordings and staged batches, the bookkeeping of deferred and left-out work, the per-sample views.  The
numbers the scenarios compare are meaningless here (they print FAIL for them); what counts is that every scenario runs to
its end with no sanitizer report, no abort of the stand-in (a replay or destroy of a dead recording) and no exception."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SCENARIOS = ["mnist", "resblock", "persample", "loss_map", "embedding", "adam", "pipeline", "frozen_input", "deferred", "real_batches",
             "upstream_nets", "three_products", "errors", "token_model", "accessors"]


@pytest.fixture(scope="module")
def stub_binary(tmp_path_factory):
    work = tmp_path_factory.mktemp("stub")
    stub = str(work / "stub_backend.cpp")
    subprocess.run([sys.executable, os.path.join(ROOT, "tests", "cpp", "make_stub_backend.py"),
                    os.path.join(ROOT, "include", "cnet_hip.h"), stub], check=True)
    exe = str(work / "facade_stub")
    cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fopenmp",
           "-I" + os.path.join(ROOT, "include"), "-I" + ROOT, os.path.join(ROOT, "tests", "cpp", "facade_test.cpp"), stub, "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    return exe


@pytest.mark.parametrize("scenario", SCENARIOS)
def test_facade_scenario_runs_clean_on_the_stand_in(stub_binary, scenario):
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", OMP_NUM_THREADS="4")
    r = subprocess.run([stub_binary, scenario], capture_output=True, text=True, timeout=600, env=env)
    text = r.stdout + r.stderr
    assert r.returncode >= 0, "killed by signal %d\n%s" % (-r.returncode, text[-2000:])
    for bad in ("AddressSanitizer", "runtime error:", "stub:", "terminate called", "what():"):
        assert bad not in text, text[-3000:]
    assert "%s:" % scenario in text and "failure(s)" in text, text[-1500:]   # the scenario reached its summary line
