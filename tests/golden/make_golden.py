"""Writes tests/golden/wigner_3j.npz from the reference's own ``wigner_3j``.

The sign convention of the real-basis coupling tensors is the one thing about
the oracle that no invariant, special case or third-party library fixes (a
global sign per (l1, l2, l3) survives all of them), so these vectors are taken
from the reference itself.  The reference file is numpy-only and is loaded by
path, in the build container only; the output is plain data.

    python tests/golden/make_golden.py [/root/reference]
"""
import importlib.util
import pathlib
import sys

import numpy as np

LMAX = 4


def main():
    root = pathlib.Path(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
    src = root / "openequivariance" / "implementations" / "e3nn_lite.py"
    spec = importlib.util.spec_from_file_location("_ref_e3nn_lite", src)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    out = {}
    for l1 in range(LMAX + 1):
        for l2 in range(LMAX + 1):
            for l3 in range(abs(l1 - l2), min(LMAX, l1 + l2) + 1):
                out[f"{l1}_{l2}_{l3}"] = mod.wigner_3j(l1, l2, l3).astype(np.float64)
    dest = pathlib.Path(__file__).with_name("wigner_3j.npz")
    np.savez_compressed(dest, **out)
    print(f"wrote {len(out)} tensors to {dest}")


if __name__ == "__main__":
    main()
