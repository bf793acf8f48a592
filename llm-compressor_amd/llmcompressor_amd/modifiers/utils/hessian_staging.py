"""Staging of calibration batches for the Hessian kernel, shared by the modifiers that accumulate
``H += 2 X^T X`` in a forward hook (GPTQ: modifiers/gptq/base.py:240-262; SparseGPT:
modifiers/pruning/sparsegpt/base.py:88-117 in the reference).

The ``[K,K]`` accumulator is read and written once per launch, so several hook calls are accumulated by one
launch: either by reference (the hook's input tensors are held and handed to the kernel as a list of buffers)
or through a staging buffer.  A class using the mixin provides ``_hessians``, ``_num_samples``, ``_staged``,
``_held`` (dicts keyed by module), ``_held_bytes`` and the fields ``hessian_batch_tokens``, ``stage_by_reference``
and ``stage_max_bytes`` (bound on the activations held by reference over all modules).
"""
from __future__ import annotations

import torch

from ... import ops
from ...torch_ops import llmc

__all__ = ["HessianStagingMixin"]


class HessianStagingMixin:
    # The hook runs once per Linear per batch, so it is kept cheap: the sample count stays on the host
    # until the flush.
    def _stage(self, module, inp):
        k = inp.shape[-1]
        n = inp.numel() // k
        samples = 1 if inp.ndim == 2 else inp.shape[0]  # accumulate_hessian counts a 2-D input as one sample
        if self.stage_by_reference and inp.is_contiguous():
            x = inp.view(n, k)
            held = self._held.get(module)
            fits = ops.segment_ok(x) and (held is None or not held[0] or (
                held[0][0].shape == x.shape and held[0][0].dtype == x.dtype))
            if fits:
                st = self._staged.get(module)
                if st is not None and st[1] > 0:
                    self._flush(module)
                if held is None:
                    held = self._held[module] = [[], [], 0]  # views, (tensor, version at hook time), samples
                held[0].append(x)
                held[1].append((inp, inp._version))
                held[2] += samples
                self._held_bytes = getattr(self, "_held_bytes", 0) + x.numel() * x.element_size()
                if len(held[0]) * n >= self.hessian_batch_tokens or len(held[0]) >= ops.SEGMENTS_MAX:
                    self._flush(module)
                elif self._held_bytes > getattr(self, "stage_max_bytes", 1 << 62):
                    # many modules holding batches at once (a pipeline that runs the whole model per batch):
                    # accumulate everything pending rather than keep more activations alive
                    for other in [m for m, h in self._held.items() if h[0]]:
                        self._flush(other)
                return
            if held is not None and held[0]:
                self._flush(module)
        st = self._staged.get(module)
        if st is None or st[0].shape[0] < n or st[0].dtype != inp.dtype or st[0].device != inp.device:
            if st is not None:
                self._flush(module)
            cap = max(self.hessian_batch_tokens, n)
            st = [torch.empty((cap, k), dtype=inp.dtype, device=inp.device), 0, 0]
            self._staged[module] = st
        elif st[1] + n > st[0].shape[0]:
            self._flush(module)
        used = st[1]
        st[0].narrow(0, used, n).copy_(inp.reshape(n, k))
        st[1] = used + n
        st[2] += samples
        if st[1] >= self.hessian_batch_tokens:
            self._flush(module)

    def _flush(self, module):
        held = self._held.get(module)
        if held is not None and held[0]:
            for t, version in held[1]:
                if t._version != version:
                    raise RuntimeError(
                        "an activation that was held for Hessian accumulation was modified in place "
                        "after the forward hook saw it; set stage_by_reference=False for this model")
            llmc.hessian_accum_segments_(self._hessians[module], held[0], 2.0, True)
            self._num_samples[module] += held[2]
            self._held_bytes = getattr(self, "_held_bytes", 0) - sum(x.numel() * x.element_size() for x in held[0])
            self._held[module] = [[], [], 0]
        st = self._staged.get(module)
        if st is None or st[1] == 0:
            return
        llmc.hessian_accum_(self._hessians[module], st[0].narrow(0, 0, st[1]), 2.0, True)
        self._num_samples[module] += st[2]
        st[1] = 0
        st[2] = 0
