"""TEST INFRASTRUCTURE ONLY — CPU oracle for the Select-then-Prune decode path.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import this package;
the shipped package (``twilight_amd``) never does.

* :mod:`oracle.native`  — ctypes binding of ``twl_oracle.c`` (top-p bisection, nucleus set,
  INT4 group quantisation), built by ``oracle/Makefile``.
* :mod:`oracle.pyimpl_port` — torch-CPU / numpy restatement of the ``twilight/pyimpl`` decode
  math (quantiser, Quest selector, estimator GEMV, softmax + top-p, masked attention) plus the
  storage-format helpers (INT4 records, Quest metadata records, paging).

The reference's own implementation cannot be built or imported for this path (CUDA/CUB/FlashInfer
for the top-p kernel; the INT4 GEMV and sparse attention live in an un-vendored submodule), so
there is no ``oracle/_ref``.
"""
