"""CPU oracle for the SpargeAttn hot path.  TEST INFRASTRUCTURE ONLY.

This package restates, in numpy, the algorithm of the reference path
``spas_sage2_attn_meansim_topk_cuda`` / ``block_sparse_sage2_attn_cuda``
(spas_sage_attn/core.py:105-233 of thu-ml/SpargeAttn).  It is the checker the
HIP kernels are compared against; nothing in the product package may import
it.  Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg
of ``bench.py`` use it.

Arithmetic contract
-------------------
The reference leaves reduction order, tie-breaking and several roundings to
Triton / cuBLAS / ATen.  The oracle fixes them so that "bit-exact" is a
well-defined statement:

* every reduction whose addends are exactly representable (sums of T-typed
  values, of products of two T-typed values, of squares) is accumulated in
  IEEE binary64, which is exact for inputs whose dynamic range inside one
  reduction stays below 2**28;
* a tensor is rounded exactly once, round-to-nearest-even, at each point
  where the reference materialises it in the input dtype T (bf16 or fp16);
* fp32 steps the reference performs in fp32 (norm, quantisation scale,
  divide, +-0.5, truncate) are IEEE binary32 with correctly rounded
  divide / sqrt;
* the compressed softmax uses a fixed sequence of binary64 operations
  (``cexp``) and a fixed summation tree, so that a GPU can reproduce it bit
  for bit;
* the descending sort is stable (ties -> lower block index first).

Pinning status (what checks each function beyond re-typing its formula) is
listed in each module's docstring; functions whose bit pattern only a run of
the real CUDA/Triton reference could pin say "parity unpinned".
"""
