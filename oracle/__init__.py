"""CPU oracle for the calibration-time quantization hot path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the shipped
product: only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline``
leg of ``bench.py`` may import it, and only as the checker.  The product
(``llmcompressor_amd``) never imports this package and fails loudly when its
HIP library is missing.

The oracle restates, op for op, the eager-torch arithmetic of the reference's
hot path (``modifiers/gptq/gptq_quantize.py``, ``observers/*.py``) and of the
compressed-tensors numerics those files call (``calculate_qparams``,
``generate_gparam``, ``fake_quantize``, the pack routines).  compressed-tensors
(pinned ``==0.18.0`` by the reference's ``setup.py:138-143``) is not vendored in
the reference tree and is not installed, so those functions are restated from
its published algorithm and pinned by the golden vectors the reference's own
tests hold (see ``tests/test_oracle_golden.py``).

Parity status per function (a function not pinned by a reference-held vector,
closed form or invariant says so here):

* pinned: ``calculate_qparams`` (int sym/asym, fp4 tensor_group),
  ``generate_gparam``, ``fake_quantize`` (int4 tensor/channel/group/block,
  nvfp4 tensor_group, activation tensor / dynamic-local), min-max observers
  (memoryless / static / moving average), MSE grid search (eight known-answer
  losses), ``flatten_for_calibration`` shape contract, ``accumulate_hessian``
  (fp64 closed form), ``quantize_weight`` (diagonal-Hessian == RTN, textbook
  un-blocked GPTQ in fp64, block-size independence, grid membership),
  ``moe.experts_forward`` (the reference's routing counts for 4 experts / top-2,
  the dense fp64 closed form).
* pinned by independent definitions importable here (``tests/test_oracle_formats.py``; no reference-held bytes
  exist for these): ``pack_fp4_to_uint8`` nibble order, sign bit and the -0 nibble, and the E8M0 byte with its
  bias (the MXFP4 consumer decode of ``transformers.integrations.mxfp4`` gives back ``fake_quantize`` bit for
  bit; swapped nibbles, a dropped -0 or a bias off by one fail); ``cast_to_fp4`` rounding and the e2m1 codes
  (triton's OCP reference encoder over every bf16 value); the NVFP4 triple nibble / e4m3 scale byte / global
  scale (decode written from the format); fp8 storage (nearest-even over a table of the 256 e4m3fn bytes built
  from the bit fields, every bf16 input); ``pack_to_int32`` (shift-and-mask decode written from the published
  ``pack_factor = 32 // num_bits`` definition, every code in every slot, and the reference-held int4 group
  matrix of ``test_lifecycle.py`` through the packed words); the BLOCK strategy inside the GPTQ column loop
  (diagonal Hessian => the reference-held block [2, 3] matrix of ``test_lifecycle.py``).
* parity unpinned (no reference-held vector exists and nothing importable decides them; each sits behind one
  function): MXFP4 E8M0 scale *generation* for group maxima with mantissa >= 1.75 (``mxfp4_scale_exponent``: the
  bit-pattern rule's rounding bump carries there and gives one more than the OCP floor rule -- brute force over
  every bf16 maximum in ``tests/test_oracle_golden.py`` shows the two rules differ exactly there); the zero-scale
  epsilon substitution (``calculate_qparams``); the per-token dynamic FP8 reduce / scale-dtype path
  (``compute_dynamic_scales_and_zp``; cross-checked against the per-row helper a consumer applies: same reduce
  dimension, scales equal after rounding to bf16, >= 95 % equal bytes, the rest one e4m3 step away); the dtype in
  which ``q * scale`` is formed when x is fp32 and the scale bf16 (``_dequantize``); the checkpoint format name of
  int weights with quantised activations.
* parity unpinned by reference vectors, pinned by mathematics only:
  ``sparsegpt.accumulate_hessian`` / ``sparsegpt.sparsify_weight`` (the
  reference's SparseGPT tests need hub models; see ``tests/test_oracle_sparsegpt.py``:
  closed-form running-average Hessian, diagonal-Hessian == saliency pruning,
  exact zero counts, un-blocked fp64 textbook elimination, the OBS step against
  a constrained least-squares solve); ``observers.imatrix_grid_search`` /
  ``observers.prepare_importance`` (``tests/test_oracle_imatrix.py``: the
  reference's uniform-importance == plain-search property, brute-force fp64
  argmin, patience rule).
"""
