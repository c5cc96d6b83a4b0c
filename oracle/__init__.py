"""CPU oracle for the MI355X VJP/JVP path.  TEST INFRASTRUCTURE, NOT PRODUCT.

What is here
------------
* ``np_namespace`` / ``np_boxes`` / ``np_vjps`` / ``np_jvps`` / ``special``:
  a NumPy value type (ndarray boxes, vspaces and derivative rules) plugged
  into the repository's tracer through its public extension API.  Every rule
  restates, formula by formula and in the same operation order, the rule of
  the reference it cites (autograd/numpy/numpy_vjps.py, numpy_jvps.py,
  numpy_boxes.py, numpy_vspaces.py, numpy_wrapper.py, scipy/special.py), so
  that on the same seeded inputs it reproduces what reference autograd+NumPy
  computes on the host.
* ``misc`` / ``convolution``: container flattening and the optimizers (autograd/misc/flatten.py,
  optimizers.py) and the N-d convolution with its cotangents (autograd/scipy/signal.py), restated
  the same way.
* ``closed_forms``: answers that do not come from any tracer at all (textbook
  derivatives, brute-force sums, dense Hessians) for the five workloads and the
  rule families; they are what pins the restatement where the reference's own
  tests hold no vectors.

Who may use it
--------------
Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py``, and only as the checker / the reported CPU baseline.  Nothing
under ``autograd_amd/`` imports this package; the device path has no CPU
fallback and raises when its HIP library is missing.

How it is pinned
----------------
``tests/test_oracle_*.py`` check it against (1) the known answers the
reference's tests and README hold (tests/test_direct.py:13-24, README.md:27-34,
tests/test_tuple.py:11-24, tests/test_wrappers.py:54-64,147-153,268-283,
tests/test_scalar_ops.py:134-143, tests/test_numpy.py:881-890,1032-1038, ...),
(2) ``closed_forms``, (3) central finite differences (the reference's
``check_grads`` construction) over the shape lists of the reference's
systematic tests, and (4) fixtures under ``tests/golden/`` written by the real
reference in the build container (whole-workload outputs at reduced sizes, a
sweep of every rule and namespace form in reverse mode, forward mode and second
order with their result dtypes, the differential operators, convolutions in
every mode, gradients of seeded random programs), against which the restatement
is bit-identical.  No function here is "parity unpinned".

Python ``float`` is deliberately NOT registered as an oracle value type (the
device namespace owns it); use ``numpy.float64`` scalars or 0-d arrays.
"""
