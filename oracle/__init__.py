"""CPU oracle for the kernel hot path — TEST INFRASTRUCTURE ONLY.

Nothing in ``deplodock_amd`` may import this package.  It is imported by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``, always as the checker and never as the thing measured or shipped.

Two layers:

``oracle.emmy_ops``  numpy restatements of what the reference's frontend ops
                     and streaming carriers compute (each function cites the
                     reference file:line it follows).
``oracle.eager``     the oracle the task prescribes: PyTorch eager on the same
                     ``nn.Module`` and seeded inputs (the workloads themselves —
                     modules and input recipes — live in
                     ``deplodock_amd.workloads`` and are re-exported here).

Every function of ``emmy_ops`` is pinned in ``tests/test_oracle.py`` against
PyTorch eager on the reference's own test recipes, against committed golden
vectors (``tests/golden``), and against what the mathematics fixes (row sums,
shift invariance, brute force on tiny inputs).  No function is left
"parity unpinned".
"""
