"""CPU oracle for the LogicLayer kernel family.  TEST INFRASTRUCTURE, NOT PRODUCT.

Everything in this directory is a CPU restatement of the algorithms the reference
implements in ``difflogic/functional.py``, ``difflogic/difflogic.py``,
``difflogic/compiled_model.py`` and ``difflogic/cuda/difflogic_kernel.cu``.  It exists so
that the hand-written HIP kernels can be checked against something that does not share
their code.  Only the test-suite, the smoke check and the ``cpu_baseline`` leg of the
benchmark may import it; the shipped package ``difflogic_amd`` never does.

Modules
-------
``gates``          the 16-gate truth table in its three forms (table, real-valued, bitwise).
``float_oracle``   fp32/fp64 relaxed forward, GroupSum, and autograd gradients
                   (functional.py:26-70, difflogic.py:94-108, 175-196).
``packed_oracle``  numpy restatement of bit packing, packed gate evaluation and the
                   per-class bit count (difflogic_kernel.cu:437-501, 547-581, 631-664).
``connections``    the two connectivity initialisers and the reverse (CSR) index
                   (difflogic.py:56-69, 154-169; functional.py:76-124).
``cgen``           generator of a C translation unit equivalent to the one the reference
                   emits for CPU inference, plus gcc + ctypes plumbing
                   (compiled_model.py:94-239, 281-319, 342-370).
``c/packed_interp.c``  table-driven C interpreter of a discretised net on 64-sample words
                   (same arithmetic as the generated C, without one line of C per gate).

How each function is pinned (see tests/test_oracle_*.py)
--------------------------------------------------------
* gate table         : op ``i``'s truth-table row is the 4-bit binary expansion of ``i``;
                       the real-valued and bitwise forms are evaluated on {0,1}^2 against it.
* float forward      : equals the multilinear extension of the table (closed form), and
                       equals the boolean gate exactly on {0,1} inputs with one-hot weights.
* gradients          : torch.autograd.gradcheck in fp64 + closed-form partial derivatives.
* packbits           : numpy.packbits(bitorder='little') viewed as little-endian words.
* packed eval        : brute force over 16 ops x 4 input pairs; bit-at-a-time interpreter.
* groupbitsum        : numpy.unpackbits -> reshape -> sum.
* generated C / interp: outputs of the reference's own CompiledLogicNet (gcc) on seeded
                       tiny nets, stored under tests/golden/ (fixtures written by
                       tests/golden/make_golden.py in the build container).
* connections        : index tensors the reference's initialisers return for fixed seeds,
                       stored under tests/golden/.
"""
