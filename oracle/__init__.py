"""TEST INFRASTRUCTURE — CPU oracle for the batched-prediction hot path.

A CPU restatement of the reference's algorithm, used only as the checker by
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py``.  Nothing under ``habitat_amd/`` imports this package.

  occupancy.c      thread-block occupancy        (cpp/src/cuda/kernel.cpp:29-56,
                                                  cpp/src/cuda/cuda_occupancy.h:1289-1420)
  wave_scaling.c   per-record wave scaling in C  (analysis/wave_scaling/*.py)
  wave_scaling.py  the same, line by line in Python, raising what the reference raises
  mlp.py           the per-op MLPs in numpy fp64 and torch-CPU fp32
                                                 (analysis/mlp/mlp.py:17-131,252-267)
  predictor.py     operation-level arithmetic    (analysis/predictor.py:111-148,
                                                  analysis/run_time.py:50-58, analysis/trace.py:27-36)
  ref_shim.cpp     C face of the reference's own kernel.cpp → oracle/_ref/ (only
                   where the reference tree is mounted)

Parity pins (what each function is checked against before it is trusted) are
listed in each file's header and exercised by tests/test_oracle*.py.
"""
