"""The cache policies of the 128-bit accesses (plain; hint on loads and stores; hinted stores; hinted loads + device-scope
stores) must not change a bit of any result.  A launch picks its policy from its footprint, and the library reads the two
overrides CNET_STREAM_MIN_MB / CNET_STREAM_POLICY once per process, so each policy runs tests/gpu_stream_policy_check.py in
a process of its own on small, 128-bit-aligned shapes (every elementwise, one-gradient, fused and row-normalising entry
point, with and without accumulation, with and without the planes of the conjugate half) and prints a hash of every result;
this process computes the same results under the plain policy, checks a few of them against the CPU oracle, and compares
the hashes.  The same kernels at a size that streams by itself are in tests/test_gpu_streaming.py."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from tests import gpu_stream_policy_check as check
from tests.gpu_util import gpu, rel_c  # noqa: F401

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def plain(gpu):
    if os.environ.get("CNET_STREAM_MIN_MB") or os.environ.get("CNET_STREAM_POLICY"):
        pytest.skip("this process already runs under a policy override")
    return check.results()


def test_plain_policy_results_agree_with_the_oracle(plain, port):
    """Anchors the hashes: the arrays they are taken from are the oracle's results (every entry point has its own parity
    test elsewhere; here a forward pass, a fused pass and a one-gradient pass of the same run)."""
    B, n = check.SHAPES[0]
    tag = "%dx%d" % (B, n)
    xr, xi = check._planes((1, B, n), (B, n), 2, 2.0)
    gp = check._pair((3, B, n), (B, n))
    base = check._pair((7, B, n), (B, n))
    assert rel_c(plain[tag + " gelu_fwd"], port.gelu_fwd(xr, xi)) < 1e-5
    want = port.gelu_bwd(xr, xi, gp)
    got = plain[tag + " gelu_bwd_sym acc=1 mirror=1"]
    assert rel_c([got[0] - base[0], got[1] - base[1]], want[0:2]) < 1e-5
    assert rel_c([got[2] - base[2], got[3] - base[3]], want[2:4]) < 1e-5
    v1 = check._planes((6, B, n), (1, n), 2, 0.7)
    hr, hi = port.hadamard_fwd(xr, xi, v1[0][0], v1[1][0])
    got = plain[tag + " hadamard_gelu_fwd shared=1"]
    assert rel_c(got[0:2], (hr, hi)) < 1e-6 and rel_c(got[2:4], port.gelu_fwd(hr, hi)) < 1e-5


@pytest.mark.parametrize("policy", [1, 2, 3])
def test_every_policy_moves_the_same_bits(plain, policy):
    env = dict(os.environ, CNET_STREAM_MIN_MB="0", CNET_STREAM_POLICY=str(policy))
    r = subprocess.run([sys.executable, os.path.join(HERE, "gpu_stream_policy_check.py")], env=env, capture_output=True, text=True,
                       timeout=240, cwd=os.path.dirname(HERE))
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-3000:]
    line = [l for l in r.stdout.splitlines() if l.startswith("DIGESTS ")]
    assert line, r.stdout[-2000:]
    got = json.loads(line[-1][len("DIGESTS "):])
    want = {k: check.digest(v) for k, v in plain.items()}
    assert set(got) == set(want) and len(want) > 400
    differ = sorted(k for k in want if got[k] != want[k])
    assert not differ, ("policy %d" % policy, len(differ), differ[:12])
