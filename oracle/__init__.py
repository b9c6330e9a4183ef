"""CPU oracle for the SageAttention forward path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this directory.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
use it, and only as the checker: never as the thing that is measured or shipped.

Pinning status of each oracle function (what independent evidence fixes it):

* ``quant.quant_per_block_int8`` / ``quant.per_block_int8`` -- restates
  backends/_enflame/ops/sage_attention/quant_per_block.py:20-101 with the zero-tile
  guard of backends/_hygon/ops/sageattention/sageattention_triton.py:35.  The
  reference holds no golden vectors for it; pinned by closed-form invariants
  (arg-max element -> +-127, |x - q*scale| <= scale/2, round-half-away ties, masked
  tail rows), a second, independent big-rational restatement on small tiles
  (tests/test_oracle_quant.py) and golden vectors that the reference's own quantiser
  produced (tests/golden/quant_golden.npz, written by tests/golden/make_quant_golden.py).
* ``quant.k_mean`` -- the reference never computes the K mean (it is only an argument,
  quant_per_block.py:53-54): **parity unpinned**; definition stated in its docstring.
* ``quant.quant_v_fp8`` -- FP8 P.V is not in the reference's own kernels: **parity
  unpinned**; the e4m3fn value set is pinned against the reference's bit decoder
  backends/_enflame/ops/hpc_ops_attention/fp8_utils.py:19-38 (restated in the test) and
  torch's float8_e4m3fn CPU cast.
* ``attention.sage_reference`` -- restates the test oracles
  backends/_hygon/test/sageattention/test_sageattention_hip.py:12-28 and
  backends/_enflame/test/test_sage_attention_native.py:62-81; pinned against
  torch.nn.functional.scaled_dot_product_attention and brute-force loops on tiny
  shapes.  Its causal / varlen extensions are not in the reference: **parity unpinned**
  there, pinned by SDPA ``is_causal=True`` and a per-sequence loop.
* ``fp8_model.fp8_attention_model`` -- the arithmetic of this build's FP8 P.V kernel (e4m3 P
  and V, lazily moved reference maximum, denominator from the rounded probabilities); the
  reference has no FP8 kernel: **parity unpinned** there, pinned by scalar-loop closed forms,
  exact invariants and closeness to ``sage_reference`` (tests/test_oracle_fp8_model.py).
"""
