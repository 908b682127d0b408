"""CPU oracle for the quantized-matmul hot path -- TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package (`rmlx_amd/`) may import this module.  It is used by
`tests/`, by `__graft_entry__.smoke()` and by the `cpu_baseline` leg of `bench.py`,
always as the checker and never as the thing measured or shipped.

Two layers:

* `oracle.refpath` -- ctypes bindings of `affine_qmm_ref.c`, a plain-C restatement of the
  reference's scalar CPU path (same loop nests, f32, no FMA contraction).
* `oracle.model`   -- NumPy restatement of the reference's *semantics* in float64
  (dequantize-then-matmul, routing, expert grouping, SwiGLU, weighted combine), the
  tolerance oracle the HIP kernels are compared against.

Parity status per function is recorded in each function's docstring ("pinned by ...").
"""
