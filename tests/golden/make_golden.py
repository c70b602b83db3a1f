"""Writes tests/golden/golden.npz from the compiled UPSTREAM CPU classes (oracle/_ref/libcnet_ref.so).

Run in a container where the upstream tree is mounted:  make -C oracle && python tests/golden/make_golden.py
The fixture holds data only: seeded inputs and the planes the upstream code produced for them.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import binding  # noqa: E402
from tests.golden import recipes  # noqa: E402


def main():
    ref = binding.load_ref()
    if ref is None:
        raise SystemExit("oracle/_ref/libcnet_ref.so missing: build it with `make -C oracle` first")
    assert ref.backend == "reference"
    blob = {}
    for fn in recipes.SCENARIOS:
        for key, val in fn(ref).items():
            blob["%s/%s" % (fn.__name__, key)] = np.asarray(val)
    # the two model streams also as files, for the readers that take a path
    for name in ("readme", "token"):
        with open(os.path.join(HERE, "%s_net.mod" % name), "wb") as f:
            f.write(blob["model_files/%s_mod" % name].tobytes())
    path = os.path.join(HERE, "golden.npz")
    np.savez_compressed(path, **blob)
    print("wrote %s: %d arrays, %.1f KB" % (path, len(blob), os.path.getsize(path) / 1024))


if __name__ == "__main__":
    main()
