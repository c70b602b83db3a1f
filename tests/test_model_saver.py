"""The .mod model files of upstream CNet (impl/model_saver.h:483-967): the facade's ModelSaver and the Python reader
against files written by upstream's own ModelSaver (tests/golden/*.mod, see tests/golden/make_golden.py).  Host only."""
import os
import subprocess

import numpy as np

from cnet_amd import modfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = os.path.join(ROOT, "tests", "golden")
BIN = os.path.join(ROOT, "tests", "bin", "saver_test")


def test_facade_model_saver_reads_and_rewrites_upstream_files(tmp_path):
    if not os.path.exists(BIN):
        subprocess.run(["make", "-C", os.path.join(ROOT, "cnet_amd", "host"), BIN], check=True, capture_output=True)
    res = subprocess.run([BIN, GOLD, str(tmp_path)], capture_output=True, text=True, timeout=120)
    print(res.stdout)
    assert res.returncode == 0 and "FAIL" not in res.stdout and res.stdout.count("PASS") >= 25, res.stdout + res.stderr


def test_python_reader_and_writer_on_upstream_files():
    gold = np.load(os.path.join(GOLD, "golden.npz"))
    for name, kinds in (("readme", [8, 4, 8, 1, 10, 8, 3, 5]), ("token", [2, 8, 6, 12, 8, 3, 6, 7, 9, 8, 1, 8, 3, 5, 11])):
        blob = open(os.path.join(GOLD, "%s_net.mod" % name), "rb").read()
        assert blob == gold["model_files/%s_mod" % name].tobytes()
        recs = modfile.loads(blob)
        assert [r["type"] for r in recs] == kinds
        assert [r["uid"] for r in recs] == list(gold["model_files/%s_uids" % name])
        assert modfile.dumps(recs) == blob
        for r in recs:
            if r["type"] in (modfile.INPUT, modfile.EMBEDDING):
                assert r["re"].dtype == np.float32 and r["re"].shape == (r["in_len"],) and r["im"].shape == (r["in_len"],)
            if r["type"] == modfile.LINEAR:
                assert r["in1"] + r["in2"] == r["in_len"] and r["in2"] // r["in1"] == r["out_size"]
    # the README net: weights as planted by the recipe (tests/golden/recipes.py: seeds 41..44)
    recs = modfile.loads(open(os.path.join(GOLD, "readme_net.mod"), "rb").read())
    hw = recs[2]
    want = np.random.RandomState(41).randn(100).astype(np.float32) * np.float32(0.3) + 1
    assert np.array_equal(hw["re"], want.astype(np.float32))
    assert recs[6]["prev"] == [recs[4]["uid"], recs[5]["uid"]]


def test_python_reader_refusals():
    blob = open(os.path.join(GOLD, "token_net.mod"), "rb").read()
    for bad in (b"", b"\x00\x00\x00\x01" + blob[4:], blob[:50], blob[:4] + b"\x00\x00\x00\x63" + blob[8:]):
        try:
            modfile.loads(bad)
        except ValueError:
            continue
        raise AssertionError("accepted a broken stream")
