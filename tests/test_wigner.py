"""Pins the real-basis Clebsch-Gordan tensors of the oracle and of the product."""
import itertools
import pathlib

import numpy as np
import pytest

from openequivariance_amd.wigner import wigner_3j as w3j_product, su2_clebsch_gordan
from oracle.cg import wigner_3j as w3j_oracle, su2_cg

GOLDEN = np.load(pathlib.Path(__file__).parent / "golden" / "wigner_3j.npz")
TRIPLES = [tuple(map(int, k.split("_"))) for k in GOLDEN.files]


@pytest.mark.parametrize("impl", [w3j_oracle, w3j_product], ids=["oracle", "product"])
def test_matches_reference_golden_vectors(impl):
    """260 tensors (l1, l2, l3 <= 7: everything the problem families of the benchmarks use) written from
    the reference's own wigner_3j: fixes the sign convention."""
    assert len(TRIPLES) == 260 and max(max(t) for t in TRIPLES) == 7
    for (l1, l2, l3) in TRIPLES:
        np.testing.assert_allclose(impl(l1, l2, l3), GOLDEN[f"{l1}_{l2}_{l3}"], atol=1e-13, rtol=0)


def test_su2_coefficients_against_sympy():
    """Independent library: sympy's Clebsch-Gordan coefficients (complex basis)."""
    from sympy.physics.quantum.cg import CG
    for j1, j2, j3 in [(1, 1, 0), (1, 1, 1), (1, 1, 2), (2, 1, 2), (2, 2, 3), (2, 3, 2), (3, 3, 0)]:
        ref = np.zeros((2 * j1 + 1, 2 * j2 + 1, 2 * j3 + 1))
        for m1 in range(-j1, j1 + 1):
            for m2 in range(-j2, j2 + 1):
                if abs(m1 + m2) <= j3:
                    ref[j1 + m1, j2 + m2, j3 + m1 + m2] = float(CG(j1, m1, j2, m2, j3, m1 + m2).doit())
        np.testing.assert_allclose(su2_cg(j1, j2, j3), ref, atol=1e-12)
        np.testing.assert_allclose(su2_clebsch_gordan(j1, j2, j3), ref, atol=1e-12)


@pytest.mark.parametrize("impl", [w3j_oracle, w3j_product], ids=["oracle", "product"])
def test_closed_form_special_cases(impl):
    assert impl(0, 0, 0).item() == pytest.approx(1.0)
    for l in range(4):                                   # C(l,0,l)_{i0k} = delta_ik / sqrt(2l+1)
        np.testing.assert_allclose(impl(l, 0, l)[:, 0, :], np.eye(2 * l + 1) / np.sqrt(2 * l + 1), atol=1e-14)
        np.testing.assert_allclose(impl(l, l, 0)[:, :, 0], np.eye(2 * l + 1) / np.sqrt(2 * l + 1), atol=1e-14)
    eps = np.zeros((3, 3, 3))                            # C(1,1,1) = +-epsilon / sqrt(6)
    for i, j, k in itertools.permutations(range(3)):
        eps[i, j, k] = np.linalg.det(np.eye(3)[[i, j, k]])
    c = impl(1, 1, 1)
    assert np.allclose(c, eps / np.sqrt(6)) or np.allclose(c, -eps / np.sqrt(6))
    assert np.count_nonzero(np.abs(impl(2, 3, 2)) > 1e-12) == 28


@pytest.mark.parametrize("impl", [w3j_oracle, w3j_product], ids=["oracle", "product"])
def test_norm_and_exchange_symmetry(impl):
    for l1, l2, l3 in TRIPLES:
        c = impl(l1, l2, l3)
        assert np.sum(c * c) == pytest.approx(1.0, abs=1e-13)
        swapped = impl(l2, l1, l3).transpose(1, 0, 2)
        assert np.allclose(c, swapped, atol=1e-13) or np.allclose(c, -swapped, atol=1e-13)


def _rotation_generators(l):
    """so(3) generators in the real basis, obtained from the l=1 coupling: for l = 1 they are
    (J_a)_{ik} = epsilon_{aik}; higher l are built by coupling with the CG tensors themselves is
    circular, so use the complex ladder construction and the real<->complex change of basis."""
    from openequivariance_amd.wigner import real_to_complex
    m = np.arange(-l, l + 1)
    jz = np.diag(m).astype(complex)
    jp = np.zeros((2 * l + 1, 2 * l + 1), dtype=complex)
    for a in range(2 * l):
        mm = m[a]
        jp[a + 1, a] = np.sqrt(l * (l + 1) - mm * (mm + 1))
    jm = jp.conj().T
    jx, jy = (jp + jm) / 2, (jp - jm) / 2j
    q = real_to_complex(l)
    out = []
    for j in (jx, jy, jz):
        r = q.conj().T @ (-1j * j) @ q               # real antisymmetric generator
        assert np.abs(r.imag).max() < 1e-12
        out.append(r.real)
    return out


@pytest.mark.parametrize("impl", [w3j_oracle, w3j_product], ids=["oracle", "product"])
def test_rotation_invariance(impl):
    """C is an invariant tensor: sum over the three slots of (generator acting on that slot) = 0."""
    for l1, l2, l3 in [(1, 1, 1), (1, 1, 2), (2, 1, 2), (2, 2, 2), (2, 3, 2), (3, 2, 1), (2, 3, 3)]:
        c = impl(l1, l2, l3)
        g1, g2, g3 = _rotation_generators(l1), _rotation_generators(l2), _rotation_generators(l3)
        for a in range(3):
            viol = (np.einsum("ai,ijk->ajk", g1[a], c) + np.einsum("bj,ijk->ibk", g2[a], c)
                    + np.einsum("ck,ijk->ijc", g3[a], c))
            assert np.abs(viol).max() < 1e-12
