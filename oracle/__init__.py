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
* parity unpinned (no reference-held vector exists; follows the public format
  specs): MXFP4 E8M0 scale generation, ``pack_to_int32`` / ``pack_fp4_to_uint8``
  byte layouts, fp8 storage, per-token dynamic FP8 scales, zero-scale epsilon
  substitution, the BLOCK strategy inside the GPTQ column loop, the checkpoint
  format name of int weights with quantised activations.  Cross-checks that do
  not lift the status (``tests/test_oracle_golden.py``): the MXFP4 exponent rule
  against the OCP Microscaling definition over every bf16 maximum (equal, or one
  more where the rounding bump carries, mantissas >= 1.75); the E8M0 byte against
  ``torch.float8_e8m0fnu``; per-token FP8 against the per-row helper a consumer
  of such checkpoints applies (same reduce dimension, scales equal after rounding
  to bf16, >= 95 % equal bytes, the rest one e4m3 step away).
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
