"""CPU oracle for the KernelMatmul hot path.  TEST INFRASTRUCTURE ONLY.

Nothing under this directory is part of the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import it, and
only as the checker.  The product (``kernel_matmul_amd``) never imports this package.

Contents
--------
``kernels.py``        float64 closed forms of the kernel functions, their hyper-parameter
                      derivatives, the block-row mask, and the four operators built from
                      them (matmul, parameter gradient, index, dense).
``ranges.py`` +       literal restatement of the reference's range builders
``ranges_oracle.c``   (native/ranges/ranges.cpp) in plain C, loaded through ctypes.
``dense_cpu.py``      the reference's dense build-K-then-matmul check path in fp32 torch on
                      the CPU; this is what ``bench.py`` times as ``cpu_baseline``.
``build_ref.sh``      compiles the reference's own ``native/ranges/ranges.cpp`` (where the
                      reference tree is present) into ``oracle/_ref/`` to validate
                      ``ranges_oracle.c`` against the real thing.

Parity status of each oracle function is listed in the header of the file defining it.
"""
