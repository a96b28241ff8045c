"""CPU oracle for the Clebsch-Gordan layer hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package (``cgnet_amd``) may
import this directory; it is used by ``tests/``, by ``__graft_entry__.smoke()``
and by the ``cpu_baseline`` leg of ``bench.py`` as the checker / the timed CPU
baseline, never as the product path.

The oracle restates, on the CPU in numpy / torch, what the reference's python
path computes (file:line relative to the reference checkout):

* ``cg_coeff``   Clebsch-Gordan coefficients           CGNet/ClebschGordan/ClebschGordan.cpp:360-394
                 (textbook Racah sum), matrix layout    CGNet/ClebschGordan/CGmodule.cpp:70-119
* ``triples``    kept (l1,l2)->l lists, MST, encodings  CGNet/CGutils.py:73-187
* ``cg_layer``   CG product, fragment norm, weight mix  CGNet/CG_layers_python.py:65-133,136-184,248-269
                 Kronecker / complex bmm helpers        CGNet/Complex_math.py:12-74, CGNet/CGutils.py:15-21
                 l=0 skip-connection stack              CGNet/CGNet.py:52-69
* ``bruteforce`` dense definitions used to pin the above on tiny inputs

Pinning status (what each function is checked against, in tests/test_oracle_*.py):

* cg_coeff.cg_exact / cg_matrix / flat_cg_table: sympy fixture (all entries L<=4,
  spot entries at L=6,11,15,20), textbook values, unitarity, exchange symmetry.
* triples.*: closed-form counts (23/489/1124/2486), the reference's recorded
  parameter shapes (1643, 31023), scipy MST fixture.  The MST tie-breaking is
  "parity unpinned" by any test the reference holds (it pins no scipy version);
  it is pinned here to scipy 1.15.3's output.
* cg_layer.cg_product: dense six-index einsum, l2=0 and l=0 closed forms,
  rotation equivariance with Wigner-D matrices.
* cg_layer.fragment_norm_update: numpy.std closed form, scaling law, eps floor.
* cg_layer.weight_mix: complex einsum (library routine).
* gradients: torch.autograd.gradcheck in float64, adjoint identity.

The reference's own tests hold no golden vectors for this path
(CGNet/test.py:81-130 is an unasserted live printout), so at the reference level
the path is "parity unpinned"; the checks above are what fixes the oracle.
"""
