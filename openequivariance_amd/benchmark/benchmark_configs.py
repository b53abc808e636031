"""The problem families of the reference's benchmarks, as lists of problems (reference:
openequivariance/benchmark/benchmark_configs.py and test/benchmark.py:37-70).  The irreps are
facts about the published models (e3nn's tetris examples, DiffDock, MACE, NequIP)."""
from ..problem import ChannelwiseTPP as CTPP
from ..problem import FullyConnectedTPProblem as FCTPP
from ..problem import SingleInstruction

# fully connected layers of e3nn's tetris example, layer by layer (sc, lin1, lin2, alpha)
_TETRIS = [
    ("1x0e", "150x0e + 50x1o + 50x2e"), ("1x0e", "1x0e"),
    ("1x0e + 1x1o + 1x2e", "150x0e + 50x1o + 50x2e"), ("1x0e + 1x1o + 1x2e", "1x0e"),
    ("50x0e + 50x1o + 50x2e", "250x0e + 50x1o + 50x1e + 50x2o + 50x2e"), ("50x0e + 50x1o + 50x2e", "50x0e + 50x1o + 50x2e"),
    ("150x0e + 200x1o + 100x1e + 100x2o + 200x2e", "250x0e + 50x1o + 50x1e + 50x2o + 50x2e"),
    ("150x0e + 200x1o + 100x1e + 100x2o + 200x2e", "1x0e"),
    ("50x0e + 50x1o + 50x1e + 50x2o + 50x2e", "50x0o + 250x0e + 50x1o + 50x1e + 50x2o + 50x2e"),
    ("50x0e + 50x1o + 50x1e + 50x2o + 50x2e", "50x0e + 50x1o + 50x1e + 50x2o + 50x2e"),
    ("100x0o + 150x0e + 300x1o + 250x1e + 250x2o + 300x2e", "50x0o + 250x0e + 50x1o + 50x1e + 50x2o + 50x2e"),
    ("100x0o + 150x0e + 300x1o + 250x1e + 250x2o + 300x2e", "1x0e"),
    ("50x0o + 50x0e + 50x1o + 50x1e + 50x2o + 50x2e", "1x0o + 6x0e"),
    ("50x0o + 50x0e + 50x1o + 50x1e + 50x2o + 50x2e", "50x0o + 50x0e + 50x1o + 50x1e + 50x2o + 50x2e"),
    ("150x0o + 150x0e", "1x0o + 6x0e"), ("150x0o + 150x0e", "1x0e"),
]
e3nn_torch_tetris = [FCTPP(a, "1x0e", c) for a, c in _TETRIS]

_SH3 = "1x0e + 1x1o + 1x2e + 1x3o"
e3nn_torch_tetris_polynomial = [
    FCTPP(_SH3, _SH3, "64x0e + 24x1e + 24x1o + 16x2e + 16x2o", label="tetris-poly-1"),
    FCTPP("64x0e + 24x1e + 24x1o + 16x2e + 16x2o", _SH3, "0o + 6x0e", label="tetris-poly-2"),
]

_DD = "10x1o + 10x1e + 48x0e + 48x0o"
diffdock_configs = [
    FCTPP(_DD, "1x0e + 1x1o", _DD, shared_weights=False, label="DiffDock-L=1"),
    FCTPP(_DD, "1x0e + 1x1o + 1x2e", _DD, shared_weights=False, label="DiffDock-L=2"),
]

mace_conv = [
    ("128x0e+128x1o+128x2e", "1x0e+1x1o+1x2e+1x3o", "128x0e+128x1o+128x2e+128x3o", "mace-large"),
    ("128x0e+128x1o", "1x0e+1x1o+1x2e+1x3o", "128x0e+128x1o+128x2e", "mace-medium"),
]


def _both_parities(mul: int, lmax: int) -> str:
    return " + ".join(f"{mul}x{l}{p}" for l in range(lmax + 1) for p in "oe")


def _natural(lmax: int) -> str:
    return " + ".join(f"{l}{'eo'[l % 2]}" for l in range(lmax + 1))


nequip_conv = [(_both_parities(mul, lmax), _natural(lmax), _both_parities(mul, lmax), label) for mul, lmax, label in
               [(32, 2, "nequip-lips"), (64, 1, "nequip-revmd17-aspirin"), (64, 2, "nequip-revmd17-toluene"),
                (64, 3, "nequip-revmd17-benzene"), (32, 1, "nequip-water")]]

mace_problems = [CTPP(*c) for c in mace_conv]
nequip_problems = [CTPP(*c) for c in nequip_conv]

roofline_configs = [
    SingleInstruction(L1, L2, L3, "uvu", f"[{i + 1}]#{L1} x {L2} -> {L3} (uvu)")
    for i, (L1, L2, L3) in enumerate([("128x1e", "1x1e", "128x1e"), ("128x2e", "1x1e", "128x2e"),
                                      ("128x3e", "1x3e", "128x3e"), ("128x5e", "1x5e", "128x3e"),
                                      ("128x5e", "1x3e", "128x5e"), ("128x6e", "1x3e", "128x6e"),
                                      ("128x7e", "1x4e", "128x7e"), ("128x7e", "1x7e", "128x7e")])
]
