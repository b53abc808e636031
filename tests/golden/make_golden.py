"""Writes tests/golden/wigner_3j.npz from the reference's own ``wigner_3j`` and
tests/golden/tpproblem.json from the reference's own ``TPProblem``.

The sign convention of the real-basis coupling tensors is the one thing about
the oracle that no invariant, special case or third-party library fixes (a
global sign per (l1, l2, l3) survives all of them), so these vectors are taken
from the reference itself.  The reference file is numpy-only and is loaded by
path, in the build container only; the output is plain data.

The second fixture pins the normalisation: for literal instruction lists (written out below, no
reference enumeration helper is used) it records what the reference's ``TPProblem`` computes - the
final coefficient of every instruction, its weight shape, ``weight_numel`` and the irreps' sizes -
for the default and the non-default normalisation modes, variances and user path weights.

    python tests/golden/make_golden.py [/root/reference]
"""
import importlib.util
import json
import pathlib
import sys

import numpy as np

LMAX = 7

SH2, SH3 = "1x0e+1x1o+1x2e", "1x0e+1x1o+1x2e+1x3o"


def _parse(irreps):
    out = []
    for tok in irreps.replace(" ", "").split("+"):
        mul, ir = tok.split("x") if "x" in tok else ("1", tok)
        out.append((int(mul), int(ir[:-1]), 1 if ir[-1] == "e" else -1))
    return out


def _channelwise(in1, in2, lmax_out, natural):
    """Instruction list of a channelwise product: every allowed (i1, i2) -> l3 <= lmax_out path gets an
    output slot of its own; slots sorted by (l, parity) then creation order, parity -1 first."""
    a, b = _parse(in1), _parse(in2)
    slots = []
    for i, (m1, l1, p1) in enumerate(a):
        for j, (_, l2, p2) in enumerate(b):
            for l3 in range(abs(l1 - l2), l1 + l2 + 1):
                p3 = p1 * p2
                if l3 <= lmax_out and (not natural or p3 == (-1) ** l3):
                    slots.append((l3, p3, len(slots), i, j, m1))
    slots.sort(key=lambda t: (t[0], t[1], t[2]))
    out = "+".join(f"{m}x{l}{'e' if p == 1 else 'o'}" for l, p, _, _, _, m in slots)
    ins = [(i, j, k, "uvu", True) for k, (_, _, _, i, j, _) in enumerate(slots)]
    return out, ins


def _fully_connected(in1, in2, out):
    a, b, c = _parse(in1), _parse(in2), _parse(out)
    return [(i, j, k, "uvw", True, 1.0) for i, (_, l1, p1) in enumerate(a) for j, (_, l2, p2) in enumerate(b)
            for k, (_, l3, p3) in enumerate(c) if p3 == p1 * p2 and abs(l1 - l2) <= l3 <= l1 + l2]


def problem_cases():
    cases = [dict(name="readme", in1="1x2e", in2="1x3e", out="1x2e", ins=[(0, 0, 0, "uvu", True)], kw={})]
    for name, in1, in2, lmax in (("mace", "128x0e+128x1o+128x2e", SH3, 3), ("nequip", "32x0e+32x1o+32x2e", SH2, 2),
                                 ("large", "256x0e+256x1o+256x2e", SH3, 2)):
        out, ins = _channelwise(in1, in2, lmax, natural=True)
        cases.append(dict(name=name, in1=in1, in2=in2, out=out, ins=ins, kw={}))
    out, ins = _channelwise("128x0e+128x1o+128x2e", SH3, 3, natural=False)
    cases.append(dict(name="mace_all_parities", in1="128x0e+128x1o+128x2e", in2=SH3, out=out, ins=ins, kw={}))
    d = "64x0e+64x1o+64x2e"
    cases.append(dict(name="dense_uvw", in1=d, in2=SH2, out=d, ins=_fully_connected(d, SH2, d), kw=dict(shared_weights=True)))
    # non-default modes on a small mixed problem, with user path weights and variances
    in1, in2, out = "3x0e+2x1o", "2x0e+1x1o", "4x0e+3x1o+2x1e"
    ins = [(0, 0, 0, "uvw", True, 1.0), (1, 1, 0, "uvw", True, 2.5), (0, 1, 1, "uvw", True, 0.5),
           (1, 0, 1, "uvw", True, 1.0), (1, 1, 2, "uvw", True, 3.0)]
    for irn in ("component", "norm", "none"):
        for pn in ("element", "path", "none"):
            cases.append(dict(name=f"modes_{irn}_{pn}", in1=in1, in2=in2, out=out, ins=ins,
                              kw=dict(irrep_normalization=irn, path_normalization=pn)))
    cases.append(dict(name="variances", in1=in1, in2=in2, out=out, ins=ins,
                      kw=dict(in1_var=[1.0, 0.5], in2_var=[2.0, 0.25], out_var=[3.0, 0.125, 1.5])))
    cases.append(dict(name="uvu_mul2", in1="4x0e+4x1o", in2="2x0e+2x1o", out="4x0e+4x1o+4x1o",
                      ins=[(0, 0, 0, "uvu", True), (0, 1, 1, "uvu", True, 2.0), (1, 0, 2, "uvu", True), (1, 1, 0, "uvu", True)], kw={}))
    return cases


IRREPS_CASES = ["1x0e", "0e + 1o + 2e", "32x0e+32x1o+32x2e", "2x1o + 3x0e + 2x1o + 0x2e + 1x1e", "4x0o+4x0e+4x1o",
                "128x0e+128x1o+128x2e+128x3o", "10x1o + 10x1e + 48x0e + 48x0o", "3x2e+0x0e+3x2e", "7x5o"]


def write_irreps_fixture(mod, dest):
    """What the reference's Irreps reports for a few strings: text form, sizes and the derived forms."""
    out = []
    for text in IRREPS_CASES:
        ir = mod.Irreps(text)
        srt = ir.sort()
        out.append(dict(text=text, repr=repr(ir), dim=int(ir.dim), num_irreps=int(ir.num_irreps), ls=[int(l) for l in ir.ls],
                        lmax=int(ir.lmax), length=len(ir), muls=[int(m) for m, _ in ir], parities=[int(i.p) for _, i in ir],
                        slices=[[sl.start, sl.stop] for sl in ir.slices()], simplify=repr(ir.simplify()),
                        remove_zero=repr(ir.remove_zero_multiplicities()), sort=repr(srt.irreps), sort_p=list(srt.p),
                        sort_inv=list(srt.inv), regroup=repr(ir.regroup()), count_1o=int(ir.count("1o")),
                        contains_2e=bool("2e" in ir), times2=repr(ir * 2), plus=repr(ir + mod.Irreps("1x3e"))))
    sh = {str(l): repr(mod.Irreps.spherical_harmonics(l)) for l in range(4)}
    prod = {f"{a}*{b}": [repr(x) for x in mod.Irrep(a) * mod.Irrep(b)] for a, b in (("1o", "1o"), ("2e", "1o"), ("0e", "3o"), ("2o", "2e"))}
    dest.write_text(json.dumps(dict(irreps=out, spherical_harmonics=sh, products=prod), indent=1) + "\n")
    print(f"wrote {len(out)} irreps cases to {dest}")


def write_problem_fixture(mod, dest):
    out = []
    for c in problem_cases():
        tpp = mod.TPProblem(c["in1"], c["in2"], c["out"], [tuple(t) for t in c["ins"]], **c["kw"])
        out.append(dict(name=c["name"], irreps_in1=c["in1"], irreps_in2=c["in2"], irreps_out=c["out"],
                        instructions=[list(t) for t in c["ins"]], kwargs=c["kw"],
                        expect=dict(path_weights=[float(i.path_weight) for i in tpp.instructions],
                                    path_shapes=[list(i.path_shape) for i in tpp.instructions],
                                    weight_numel=int(tpp.weight_numel),
                                    dims=[int(tpp.irreps_in1.dim), int(tpp.irreps_in2.dim), int(tpp.irreps_out.dim)],
                                    shared_weights=bool(tpp.shared_weights), internal_weights=bool(tpp.internal_weights),
                                    text=str(tpp), repr=repr(tpp),
                                    weight_ranges=[[int(a), int(b), list(sh)] for a, b, sh in
                                                   (tpp.weight_range_and_shape_for_instruction(i) for i in range(len(tpp.instructions)))])))
    dest.write_text(json.dumps(out, indent=1) + "\n")
    print(f"wrote {len(out)} problems to {dest}")


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
    write_problem_fixture(mod, pathlib.Path(__file__).with_name("tpproblem.json"))
    write_irreps_fixture(mod, pathlib.Path(__file__).with_name("irreps.json"))


if __name__ == "__main__":
    main()
