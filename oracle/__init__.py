"""CPU oracle for the e3nn message-passing hot path.

TEST INFRASTRUCTURE ONLY.  This package restates, in numpy (fp64 by default), the
algorithm of the reference e3nn implementation for

* irreps parsing / feature layout           (irreps.py)
* real-basis Wigner 3j / Clebsch-Gordan     (wigner.py)
* TensorProduct normalisation + ``uvu`` / ``uvw`` contraction (tensor_product.py)
* cartesian spherical harmonics             (spherical_harmonics.py)
* edge gather + destination scatter-sum     (message_passing.py)
* the node-wise blocks either side of the message: o3.Linear, nn.Activation, nn.Gate,
  nn.FullyConnectedNet, the v2106 Convolution  (nn.py)
* a multi-threaded torch-CPU einsum restatement used only as the timed CPU
  baseline                                   (torch_cpu.py)

Only tests, the smoke check and the ``cpu_baseline`` leg of the benchmark may
import it; the shipped package never does.

Pin status (what independently fixes each function; see tests/test_oracle_*.py):

* wigner_3j ............ pinned: golden tensors written from the reference for all
                         l <= 4, closed forms (epsilon/sqrt6, identity/sqrt(2l+1)),
                         permutation symmetry, Frobenius norm, sympy CG.
* normalisation ........ pinned: golden instruction tables from the reference for the
                         five benchmark configurations, the 10x0e == 3x0e+7x0e identity,
                         unit output variance.
* uvu / uvw contraction  pinned: golden outputs from the reference on small seeded
                         inputs, brute-force 7-index loops, special cases that reduce
                         to dot / cross / scalar products.
* spherical harmonics .. pinned: golden values from the reference (l <= 8, three
                         normalisations), scipy's complex harmonics, norm / parity /
                         zero-vector identities, the w3j recurrence.
* gather / scatter ..... pinned: integer-valued payloads (bit-exact), golden output.
* Linear / Activation / Gate / FullyConnectedNet / Convolution
                         pinned: golden outputs from the reference (instruction tables,
                         irreps, normalisation constants, outputs), Linear's closed form on scalars.
"""
