"""Writes ``tests/golden/golden.json``: SHA-256 digests (plus shape and a few raw
words) of the outputs of RepDL's own C++ CPU backend on the cases of
``cases.py``.

The backend is the reference's ``backend/cpu/*.cpp`` compiled as they lie by
``oracle/build.py`` (``build_ref``) -- compiled C++, not the reference's Python
package.  Runs only where ``/root/reference`` exists; the JSON it writes is the
committed fixture.  Usage: ``python tests/golden/make_golden.py``.
"""
from __future__ import annotations

import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(HERE))

import torch  # noqa: E402

import cases  # noqa: E402
import gen  # noqa: E402
from oracle import build, ref  # noqa: E402


def main() -> None:
    if ref.load() is None:
        build.build_ref()
    cpu, cpu_math = ref.load()
    out = {}
    for case in cases.CASES:
        try:
            y = cases.run(case, cpu, cpu_math)
        except Exception as e:  # the reference itself rejects this input
            out[case["name"]] = {"error": type(e).__name__}
            continue
        out[case["name"]] = {
            "sha256": gen.sha256(y),
            "shape": list(y.shape),
            "words": gen.words(y),
        }
        print(case["name"], out[case["name"]]["sha256"][:16], flush=True)
    meta = {
        "_meta": {
            "producer": "RepDL backend/cpu/*.cpp compiled with g++ -O2 -fopenmp (oracle/build.py build_ref)",
            "torch": torch.__version__,
            "cases": len(out),
        }
    }
    meta.update(out)
    with open(os.path.join(HERE, "golden.json"), "w") as f:
        json.dump(meta, f, indent=1, sort_keys=True)


if __name__ == "__main__":
    main()
