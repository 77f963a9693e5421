"""TEST INFRASTRUCTURE ONLY.

CPU checkers for the HIP selection kernels.  Importable only from ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``; the product package
``evox_amd`` never imports this package and has no CPU fallback.

  eager_restatement.py  torch-CPU restatement of the reference's eager path (the checker proper)
  brute_force.py        independent numpy definitions that pin the restatement
  nd_oracle.c           plain-C restatement for sizes where the dense formulation cannot allocate
"""
