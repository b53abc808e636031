"""CPU oracle for the Clebsch-Gordan tensor product and the fused graph convolution.

THIS PACKAGE IS TEST INFRASTRUCTURE.  It is a self-contained fp64 restatement
of what the reference checks itself against (e3nn's ``o3.TensorProduct``
semantics as cloned in the reference's ``e3nn_lite.py``) and it is imported
only by the tests, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline``
leg of ``bench.py``.  Nothing in ``openequivariance_amd`` imports it, and it
imports nothing from ``openequivariance_amd``: the coupling tensors, the path
normalisation, the instruction enumeration, the weight orders and the
contraction are all restated here so that a mistake on either side shows up as
a parity failure.

How each function is pinned (a function with no such check would be marked
"parity unpinned" here; none is):

=====================  ======================================================
``cg.wigner_3j``       golden vectors written from the reference's own
                       ``e3nn_lite.wigner_3j`` (tests/golden/wigner_3j.npz);
                       sympy's Clebsch-Gordan coefficients; closed-form special
                       cases; ``|C| = 1``; rotation invariance
``spec.Problem``       golden path coefficients from the reference's
                       ``TPProblem`` (tests/golden/tpproblem.json, all normalisation modes); hand values
                       (sqrt 5; sqrt(2l3+1); sqrt(1/192), sqrt(3/256), sqrt(5/256))
``spec.channelwise``   path counts / dims / weight counts of the five benchmark
``spec.fully_conn..``  configurations and the explicit column tables
``tp.forward``         brute-force triple loops on tiny inputs; tri-linearity;
                       O(3) equivariance; the README example's structure
``tp.backward``        central finite differences; torch autograd through an
                       independent einsum; <G,Z> = <X,dX> = <Y,dY> = <W,dW>
``tp.conv_*``          gather + scatter-add of per-edge products, checked
                       against an explicit per-edge loop
``weights.*``          identity for uvu with mul(Y) = 1; round trip; a hand case;
                       the closed-form index formula for 64x64 uvw blocks
=====================  ======================================================
"""
