"""CPU oracle for the Gaussian fmmv / fdmmv hot path.

THIS PACKAGE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the test-suite,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it, and only as the checker.  Nothing under ``falkon_amd/`` imports it.

Contents
--------
``gaussian_ref``  op-for-op restatement (torch CPU ops) of the reference's
                  per-block arithmetic: ``square_norm``, ``_sq_dist``,
                  ``rbf_core`` (falkon/kernels/distance_kernel.py:88-101,140-159).
``mmv_ref``       restatement of the reference's blocked CPU drivers
                  ``mmv_run_thread`` / ``dmmv_run_thread`` and of the block-size
                  solvers that feed them (falkon/mmv_ops/fmmv.py:60-114,309-402,
                  488-544,683-767; falkon/utils/helpers.py:24-31,74-85,149-195).
``brute``         closed-form ``exp(-1/2 sum_k ((x_k-c_k)/s_k)^2)`` in fp64
                  difference form; independent of the expanded-norm route.
``brute_c``       ctypes binding of ``brute.c`` (the same closed form in plain C
                  with long-double accumulation), a second independent witness.
``inputs``        seeded generators: the reference test fixtures
                  (falkon/tests/gen_random.py:17-22, tests/test_kernels.py:32-71)
                  and the five benchmark configurations.

How each function is pinned (see tests/test_oracle.py):
  * ``rbf_core``     vs ``brute`` and ``brute_c`` on the reference's own test
                     shapes and seeds, vs ``torch.cdist`` (the reference's own
                     naive oracle, falkon/tests/naive_kernels.py:23-25), unit
                     diagonal when X==C, sigma->inf limit, per-dimension sigma ==
                     isotropic sigma=1 on pre-divided data.
  * ``fmmv_ref``     == ``K_brute @ v``; one-hot v returns columns of K;
                     blocked == unblocked (a tiny budget forces many blocks).
  * ``fdmmv_ref``    == ``K_brute.T @ (K_brute @ v + w)``; adjoint identity
                     ``u.T (K v) == (K.T u).T v``; ``w=None`` == two mmv calls.
  * block solvers    never exceed the budget / the maximum dims
                     (falkon/tests/test_dim_selectors.py:12-90 properties).
No function of this oracle is "parity unpinned".
"""
