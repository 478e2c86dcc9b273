"""CPU oracle for the Scatterbrain / block-sparse hot path.

TEST INFRASTRUCTURE ONLY.  This package restates, on the CPU with plain PyTorch /
numpy ops, the algorithms of the reference implementation (HazyResearch/fly) for
the path the HIP kernels accelerate.  It exists so that parity tests, the smoke
check and the benchmark's CPU-baseline leg have something to compare against; the
product package ``fly_amd`` never imports it and has no CPU fallback.

Every function cites the reference file:line it follows (paths relative to the
reference checkout).  The pinning status of each function -- which independent
check (closed form, brute force, invariant) holds it in place -- is recorded in
the docstring of the module that defines it and exercised by ``tests/test_oracle_*``.

Third-party arithmetic that the reference calls but does not vendor:

* ``fast_transformers.local_product`` (idiap/fast-transformers, unpinned master
  clone, reference Dockerfile:108-111): ``local_dot_product`` and
  ``local_weighted_average``.  Restated in ``oracle.local_product`` from the
  reference's call sites and the band masks its tests build.
* ``triton.ops.blocksparse.softmax`` (triton==2.0.0.dev20220711, Dockerfile:123):
  restated in ``oracle.blocksparse.block_softmax`` from the reference's call site
  and its dense-softmax test.
* ``libtriton.superblock`` (same package): restated in ``oracle.blocksparse.sdd_lut``.
* ``deepspeed.ops.sparse_attention.*SparsityConfig`` (deepspeed==0.6.5): NOT
  restated -- parity unpinned for DeepSpeed-generated layouts; the product accepts
  them only as duck-typed objects.
"""
