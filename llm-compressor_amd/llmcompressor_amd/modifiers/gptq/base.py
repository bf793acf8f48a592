"""GPTQModifier (reference: modifiers/gptq/base.py:47-399).

Same fields and lifecycle as the reference.  One MI355X-specific addition: the forward hook
stages calibration batches and accumulates several of them with one Hessian launch
(``hessian_batch_tokens``), which amortises the read-modify-write of the [K,K] accumulator;
the sum over tokens is unchanged up to fp32 summation order.
"""
from __future__ import annotations

import contextlib
import logging

import torch
from pydantic import PrivateAttr

from ... import ops  # noqa: F401
from ...torch_ops import llmc
from ...core import Event, State
from ...observers import ACTIVATION_OBS
from ...quantization import (
    ActivationOrdering,
    QuantizationConfig,
    QuantizationScheme,
    QuantizationStrategy,
    getattr_chain,
    is_module_quantized,
    match_named_modules,
    update_offload_parameter,
)
from ...sentinel import Sentinel
from ...utils.metric_logging import CompressionLogger
from ..modifier import Modifier
from ..quantization.calibration import observe, update_qparams
from ..quantization.quantization import QuantizationMixin
from ..utils.concurrent import SIDE_STREAMS, run_on_streams
from ..utils.hessian_staging import HessianStagingMixin
from .gptq_quantize import (accumulate_hessian, begin_weight_group, finish_weight_group, make_empty_hessian,
                            quantize_weight, quantize_weight_group,
                            width_key)

logger = logging.getLogger("llmcompressor_amd")

__all__ = ["GPTQModifier"]

_GPTQ_Q_PARAMS = ["weight", "weight_scale", "weight_zero_point", "weight_g_idx"]


_WIDE_SET = 16  # problems per lock-step set from which the set runs alone on the calling stream


class GPTQModifier(Modifier, QuantizationMixin, HessianStagingMixin):
    """GPTQ (https://arxiv.org/abs/2210.17323): calibrate a Hessian per targeted Linear with forward
    hooks, then quantise the weight column by column with error feedback.

    :param block_size: number of columns compressed in one pass
    :param dampening_frac: dampening applied to H, as a fraction of the diagonal mean
    :param actorder: column order; defaults to "static" (quantise in descending diag(H) order, no g_idx)
    :param offload_hessians: keep Hessians on the CPU between hook calls
    :param hessian_batch_tokens: stage activations and launch the Hessian kernel once this many tokens
        are pending (0 = one launch per hook call, the reference's behaviour).  The [K,K] accumulator is read
        and written once per launch, so for wide Linears many hook calls per launch are what keeps the kernel
        on the matrix cores instead of on memory

    :param share_identical_inputs: Linears that are fed the very same tensor on every call (q/k/v, gate/up)
        have the same Hessian; accumulate it once and hand each of them a copy when it is compressed.
        Results are bit-identical to one accumulation per module.  A module shares only while the tensor it
        receives is the very object (address, shape, strides, version) its leader has just accumulated, starting
        with its first call; a module that shared and later receives another tensor, or misses a call of its
        leader, raises (its leader has then already taken in a call the module did not see, so the two Hessians
        cannot be separated after the fact) -- pass ``share_identical_inputs=False`` for such a model

    :param stage_by_reference: while staging, keep references to the hook's input tensors instead of copying
        them into a staging buffer, and hand the kernel the list of buffers.  Taken only for contiguous
        bf16/f16 inputs whose token count is a multiple of 64; anything else is copied.  An input that is
        modified in place before its batch is accumulated raises at the flush (tensor version check)
    :param stage_max_bytes: bound on the activations held by reference over all modules; beyond it everything
        pending is accumulated at once (matters when a pipeline runs the whole model per batch)
    :param group_min_modules: when at least this many Linears of one ``compress_module_list`` call have the same
        number of input features (the experts of an MoE layer; q/k/v/o/gate/up of a decoder layer), their
        Cholesky chains run in lock-step in grouped kernels, and so do the column loops of those among them
        that share shape and scheme (0 = never); ``group_max_bytes`` bounds the work buffers of one such job
    :param compress_concurrency: how many modules of one ``compress_module_list`` call are quantised at the
        same time, each on its own HIP stream (1 = one after the other, the reference's behaviour)

    Expert Linears inside a ``LinearExperts2D`` block are handled together: while the block's forward
    runs, their hook calls are only recorded, and when it returns all experts' Hessians of one width
    are updated by a single grouped launch (384 tiny launches per batch become three).
    """

    requires_calibration_data: bool = True

    block_size: int = 128
    dampening_frac: float | None = 0.01
    actorder: ActivationOrdering | Sentinel | None = Sentinel("static")
    offload_hessians: bool = False
    hessian_batch_tokens: int = 65536
    share_identical_inputs: bool = True
    compress_concurrency: int = 4
    group_min_modules: int = 3
    group_max_bytes: int = 8 << 30
    stage_by_reference: bool = True
    stage_max_bytes: int = 16 << 30

    _module_names: dict = PrivateAttr(default_factory=dict)
    _hessians: dict = PrivateAttr(default_factory=dict)
    _num_samples: dict = PrivateAttr(default_factory=dict)
    _staged: dict = PrivateAttr(default_factory=dict)
    _held: dict = PrivateAttr(default_factory=dict)
    _held_bytes: int = PrivateAttr(default=0)
    _group_pending: list | None = PrivateAttr(default=None)
    _leader: dict = PrivateAttr(default_factory=dict)  # follower module -> module whose Hessian it shares
    # per input width: (tensor kept alive, its version, leader) of the last input that was accumulated
    _recent_input: dict = PrivateAttr(default_factory=dict)
    _hook_calls: dict = PrivateAttr(default_factory=dict)  # module -> hook calls so far (leaders and followers)
    _streams: dict = PrivateAttr(default_factory=lambda: SIDE_STREAMS)

    def resolve_quantization_config(self) -> QuantizationConfig:
        config = super().resolve_quantization_config()

        def resolve_actorder(existing):
            if self.actorder == Sentinel("static"):
                return ActivationOrdering.STATIC if existing is None else existing
            if existing is None or self.actorder == existing:
                return self.actorder
            raise ValueError(
                "Cannot resolve activation ordering when both `GPTQModifier.actorder` and "
                f"`QuantizationScheme.actorder` are provided and differ ({self.actorder}, {existing}). "
                "Either unset `GPTQModifier.actorder` or remove `actorder` from config groups.")

        grouped = (QuantizationStrategy.GROUP, QuantizationStrategy.TENSOR_GROUP)
        for scheme in config.config_groups.values():
            assert isinstance(scheme, QuantizationScheme)
            strategy = getattr_chain(scheme, "weights.strategy", None)
            if strategy in (QuantizationStrategy.GROUP, QuantizationStrategy.TENSOR_GROUP,
                            QuantizationStrategy.CHANNEL, QuantizationStrategy.TENSOR, QuantizationStrategy.BLOCK):
                scheme.weights.actorder = resolve_actorder(scheme.weights.actorder)
                if scheme.weights.actorder == ActivationOrdering.GROUP:
                    logger.warning("ActivationOrdering.GROUP is deprecated and will be removed in a future "
                                   "release. Use default actorder='static' instead. ")
                    if strategy not in grouped:
                        logger.warning(f"ActivationOrdering.GROUP is not compatible with strategy={strategy}; "
                                       "falling back to actorder=None for this scheme.")
                        scheme.weights.actorder = None
        return config

    def on_initialize(self, state: State, **kwargs) -> bool:
        if QuantizationMixin.has_config(self):
            QuantizationMixin.initialize_quantization(self, state.model)
        self._module_names = {m: name for name, m in match_named_modules(state.model, self.resolved_targets,
                                                                         self.ignore)}
        return True

    def on_calibration_start(self, state: State, event: Event, **kwargs):
        QuantizationMixin.start_calibration(self, state.model)
        added_hook = False
        for _, module in match_named_modules(state.model, self.resolved_targets, self.ignore):
            if getattr_chain(module, "quantization_scheme.weights", None) is not None:
                if not isinstance(module, torch.nn.Embedding):
                    self.register_hook(module, self.calibrate_module, "forward")
                    added_hook = True
        if not added_hook:
            raise ValueError("GPTQModifier was unable to find any modules to quantize. Please check quantization "
                             "`config_groups` and `targets` in recipe")
        from llmcompressor_amd.modeling.moe import LinearExperts2D

        for module in state.model.modules():
            if isinstance(module, LinearExperts2D):
                self.register_hook(module, self._begin_expert_group, "forward_pre")
                self.register_hook(module, self._end_expert_group, "forward")

    def on_sequential_epoch_end(self, state: State, event: Event, modules: list[torch.nn.Module] = (), **kwargs):
        modules = [m for m in modules if is_module_quantized(m)]
        # The Cholesky chains of wide lock-step sets (the experts of an MoE layer) need the Hessians only: they
        # are enqueued first, and the weights are observed on the host while they run.
        started = self._begin_compress(list(self._num_samples.keys()))
        observe(modules, base_name="weight")
        self.sync_obs_act_stats(modules)
        update_qparams(modules, ACTIVATION_OBS)
        self._finish_compress(started)

    def on_calibration_end(self, state: State, event: Event, **kwargs):
        QuantizationMixin.end_calibration(self, state.model)
        self.remove_hooks()

    def calibrate_module(self, module: torch.nn.Module, args: tuple[torch.Tensor, ...], _output: torch.Tensor):
        """Forward hook: accumulate the Hessian of the module's input.

        The hook runs once per Linear and batch (384 times per forward of an MoE layer), so it reads the modifier's
        private state through the one dictionary pydantic keeps it in instead of one attribute lookup each (those
        go through ``BaseModel.__getattr__``, about a microsecond apiece)."""
        inp = args[0]
        priv = self.__pydantic_private__
        if self.share_identical_inputs:
            calls = priv["_hook_calls"]
            calls[module] = calls.get(module, 0) + 1
            if self._follows_recent_input(module, inp, priv):
                return
        num_samples = priv["_num_samples"]
        pending = priv["_group_pending"]
        grouped = (pending is not None and isinstance(module, torch.nn.Linear) and inp.is_cuda
                   and not self.offload_hessians and inp.dtype in (torch.bfloat16, torch.float16))
        if module not in num_samples:
            device = inp.device if inp.is_cuda else module.weight.device
            init_device = "cpu" if self.offload_hessians else device
            priv["_hessians"][module] = make_empty_hessian(module, device=init_device)
            # an expert's tally stays on the host: hundreds of one-element device additions per forward otherwise
            num_samples[module] = 0.0 if grouped else torch.zeros(tuple(), device=device)
        if grouped:
            pending.append((module, inp))
            return
        if (self.hessian_batch_tokens > 0 and not self.offload_hessians and isinstance(module, torch.nn.Linear)
                and inp.dtype in (torch.bfloat16, torch.float16)):  # fp32 inputs go straight to the fp32 product
            self._stage(module, inp)
            return
        with self._maybe_onload_hessian(module):
            self._hessians[module], self._num_samples[module] = accumulate_hessian(
                inp, module, self._hessians[module], self._num_samples[module])

    # -- shared Hessians (see ``share_identical_inputs``)
    def _follows_recent_input(self, module, inp, priv=None) -> bool:
        """True when `module` received the tensor that the last accumulating hook call of its input width took
        in for another module; then only its sample count advances.  Kept per width, so that modules of another
        width called in between (an expert's down_proj between its own and the next expert's gate_proj, which with
        ``moe_calibrate_all_experts`` all receive the block's input) do not end the run.  The previous inputs are
        kept referenced, so no later tensor can take their address while it is being compared."""
        priv = self.__pydantic_private__ if priv is None else priv
        width = module.in_features if isinstance(module, torch.nn.Linear) else None
        recent = priv["_recent_input"].get(width) if width is not None else None
        # an empty tensor is "the same" only as the very object: the empty row ranges of two neighbouring experts
        # without tokens start at one address and have one shape, and are still two inputs
        same = (recent is not None and recent[2] is not module and inp.data_ptr() == recent[0].data_ptr()
                and inp.shape == recent[0].shape and inp.dtype == recent[0].dtype and inp.stride() == recent[0].stride()
                and inp._version == recent[1] and (inp.numel() > 0 or inp is recent[0]))
        leaders, num_samples = priv["_leader"], priv["_num_samples"]
        leader = leaders.get(module)
        if same and (leader is recent[2] or (leader is None and module not in num_samples)):
            leaders[module] = recent[2]
            n = 1 if inp.ndim == 2 else inp.shape[0]
            num_samples[module] = num_samples.get(module, 0) + n
            return True
        if leader is not None:
            raise RuntimeError("share_identical_inputs: a module that shared its input with another one received a "
                               "different tensor on a later call; pass share_identical_inputs=False for this model")
        if width is not None:
            priv["_recent_input"][width] = (inp, inp._version, module)
        return False

    # -- expert groups (see the class docstring)
    def _begin_expert_group(self, _module, _args):
        if self._group_pending is None:
            self._group_pending = []

    def _end_expert_group(self, _module, _args, _output):
        pending, self._group_pending = self._group_pending, None
        by_width = {}
        for module, inp in pending or ():
            # accumulate_hessian counts a 2-D input as one sample, a batched one by its batch entries
            self._num_samples[module] += 1 if inp.ndim == 2 else inp.shape[0]
            x = inp.reshape(-1, inp.shape[-1])
            by_width.setdefault((x.shape[1], x.dtype), []).append((self._hessians[module], x))
        for group in by_width.values():
            llmc.hessian_accum_grouped_([h for h, _ in group], [x for _, x in group], 2.0, True)

    def compress_modules(self):
        self.compress_module_list(list(self._num_samples.keys()))

    def compress_module_list(self, module_list):
        self._finish_compress(self._begin_compress(module_list))

    def _begin_compress(self, module_list):
        """Flush what is pending, plan the jobs and enqueue the chains of the wide sets.  Returns
        (launched wide sets, remaining jobs) for ``_finish_compress``; no weight observer is read here."""
        followers = {}
        for module in module_list:
            leader = self._leader.pop(module, None)
            if leader is not None:
                if self._hook_calls.get(module) != self._hook_calls.get(leader):
                    raise RuntimeError("share_identical_inputs: a module that shared its input with another one was "
                                       f"called {self._hook_calls.get(module)} times, the module it shared with "
                                       f"{self._hook_calls.get(leader)} times; pass share_identical_inputs=False for "
                                       "this model")
                followers[module] = leader
        self._recent_input = dict()
        for module in module_list:
            self._hook_calls.pop(module, None)
        for leader in followers.values():
            self._flush(leader)
        for module in module_list:  # pending activations go in on the calibration stream
            self._flush(module)
            self._staged.pop(module, None)
            self._held.pop(module, None)
        for module, leader in followers.items():
            # the leader's tensor itself for now, and the tally in the form the leader keeps it (host number for
            # experts, device scalar otherwise), filled on the device: no host transfer or wait per follower
            self._hessians[module] = self._hessians[leader]
            tally = self._num_samples[leader]
            count = float(self._num_samples[module])
            self._num_samples[module] = torch.full_like(tally, count) if isinstance(tally, torch.Tensor) else count
        jobs = self._plan_jobs(list(module_list))
        # A lock-step set leaves its Hessians untouched and factors a tensor it meets twice only once, so members of
        # such sets keep sharing the leader's tensor.  The per-module path factors in place: a follower gets its own
        # copy (made here, before any job starts) unless it and its leader both sit in lock-step sets.
        in_sets = {m for job in jobs if isinstance(job, list) for m in job}
        for module, leader in followers.items():
            if not (module in in_sets and leader in in_sets):
                self._hessians[module] = self._hessians[module].clone()
        # a set of many problems (the experts of an MoE layer) fills the chip by itself: such sets are enqueued one
        # after the other on the calling stream, with one host wait for all of them
        wide = [job for job in jobs if isinstance(job, list) and len(job) >= _WIDE_SET]
        jobs = [job for job in jobs if not (isinstance(job, list) and len(job) >= _WIDE_SET)]
        return [self._begin_set(part) for part in wide], jobs

    def _finish_compress(self, started):
        begun, jobs = started
        if begun:
            self._finish_sets([self._end_set(b) for b in begun])
        if not jobs:
            return
        members = [m for job in jobs for m in (job if isinstance(job, list) else [job])]
        workers = min(int(self.compress_concurrency), len(jobs))
        on_gpu = (all(m.weight.is_cuda and self._hessians[m].is_cuda for m in members)
                  and len({m.weight.device for m in members}) == 1)  # one device per call
        if workers <= 1 or not on_gpu or self.offload_hessians:
            for job in jobs:
                self._compress_job(job)
            return
        # several jobs at once, one host thread and one HIP stream each, most expensive first so that the
        # widest module does not start last (see modifiers/utils/concurrent.py); results are unchanged

        def cost(job):
            return sum(float(m.weight.shape[1]) ** 3 + float(m.weight.shape[0]) * m.weight.shape[1] ** 2
                       for m in (job if isinstance(job, list) else [job]))

        jobs.sort(key=lambda job: -cost(job))
        run_on_streams(jobs, self._compress_job, workers, members[0].weight.device, self._streams)

    def _plan_jobs(self, modules):
        """Split the modules of one call into jobs: a list = Linears of one width that share a lock-step
        Cholesky chain (at least ``group_min_modules`` of them; the work buffers of one job stay within
        ``group_max_bytes``), a module = the per-module path."""
        if self.group_min_modules <= 0 or self.offload_hessians:
            return modules
        sets = {}
        for m in modules:
            key = width_key(m, getattr_chain(m, "quantization_scheme.weights"), self._hessians[m])
            if key is not None:
                sets.setdefault(key, []).append(m)
        planned, taken = [], set()
        for members in sets.values():
            if len(members) < max(2, self.group_min_modules):
                continue
            K = members[0].weight.shape[1]
            # factors + work matrices: about 10 K^2 bytes per problem
            per_call = max(1, min(len(members), int(self.group_max_bytes // (10 * K * K))))
            for i in range(0, len(members), per_call):
                part = members[i:i + per_call]
                planned.append(part if len(part) > 1 else part[0])
            taken.update(members)
        return planned + [m for m in modules if m not in taken]

    def _compress_job(self, job, produced_on=None, consumed_on=None):
        if isinstance(job, list):
            self._compress_set(job, produced_on, consumed_on)
        else:
            self._compress_one(job, produced_on, consumed_on)

    def _compress_set(self, part, produced_on=None, consumed_on=None):
        """Linears of one width in lock-step (``quantize_weight_group``); parameters as on the per-module path."""
        self._finish_sets([self._end_set(self._begin_set(part, produced_on))], consumed_on)

    def _begin_set(self, part, produced_on=None):
        hs = [self._hessians.pop(m) for m in part]
        tallies = [self._num_samples.pop(m) for m in part]
        if all(isinstance(t, torch.Tensor) and t.is_cuda for t in tallies):  # one transfer, not one per module
            tallies = torch.stack([t.reshape(()) for t in tallies]).tolist()
        tallies = [float(t) for t in tallies]
        if produced_on is not None:  # allocated on the calibration stream, last read on this one
            for h in hs:
                h.record_stream(produced_on)
        names = [self._module_names.get(m, m.__class__.__name__) for m in part]
        logger.info(f"Quantizing {len(part)} modules in lock-step ({names[0]} .. {names[-1]})")
        with torch.no_grad():
            ctx = begin_weight_group(part, hs, tallies, self.dampening_frac, self.block_size)
        return part, names, ctx

    def _end_set(self, begun):
        part, names, ctx = begun
        with torch.no_grad():
            results = finish_weight_group(ctx, self.block_size)
        return part, names, results

    def _finish_sets(self, launched, consumed_on=None):
        # one host wait for everything enqueued so far
        failed = torch.cat([torch.stack([r[2] for r in results]) for _, _, results in launched]).tolist()
        at = 0
        for part, names, results in launched:
            for m, name, (loss, q_param_dict, _) in zip(part, names, results):
                if failed[at]:
                    logger.warning(f"Failed to invert hessian of {name} due to numerical instability. Falling "
                                   "back to round-to-nearest for this module.")
                at += 1
                for attr, val in q_param_dict.items():
                    if consumed_on is not None and val.is_cuda:  # allocated on a side stream, read by later forwards
                        val.record_stream(consumed_on)
                    update_offload_parameter(m, attr, val)

    def _compress_one(self, module, produced_on=None, consumed_on=None):
        name = self._module_names.get(module, module.__class__.__name__)
        hessian = self._hessians.pop(module)
        num_samples = self._num_samples.pop(module)
        if produced_on is not None:  # allocated on the calibration stream, last read on this one
            hessian.record_stream(produced_on)
        logger.info(f"Quantizing {name} using {int(num_samples)} samples")
        with torch.no_grad(), CompressionLogger(module) as comp_logger:
            if self.offload_hessians:
                hessian = hessian.to(device=module.weight.device)
            loss, q_param_dict = quantize_weight(
                module=module,
                quant_args=getattr_chain(module, "quantization_scheme.weights"),
                hessian=hessian,
                blocksize=self.block_size,
                percdamp=self.dampening_frac,
                hessian_divisor=float(num_samples),
            )
            comp_logger.set_results(name="GPTQ", loss=loss)
        for attr, val in q_param_dict.items():
            if consumed_on is not None and val.is_cuda:  # allocated on this stream, read by later forwards
                val.record_stream(consumed_on)
            update_offload_parameter(module, attr, val)

    def on_finalize(self, state: State, **kwargs) -> bool:
        if not self.ended_:
            self.on_end(state, None)
        if len(self._num_samples) > 0:
            raise ValueError(f"Failed to compress {len(self._num_samples)} modules")
        self._hessians = dict()
        self._num_samples = dict()
        self._staged = dict()
        self._held = dict()
        self._held_bytes = 0
        self._leader = dict()
        self._hook_calls = dict()
        self._recent_input = dict()
        return True

    @contextlib.contextmanager
    def _maybe_onload_hessian(self, module: torch.nn.Module):
        if self.offload_hessians:
            self._hessians[module] = self._hessians[module].to(device=module.weight.device)
        yield
        if self.offload_hessians:
            if module in self._hessians:
                self._hessians[module] = self._hessians[module].to(device="cpu")


# the Hessian hook reads the module and its input, never the output: an experts block may then call it with the
# rows the Linear would have received without running that Linear by itself
GPTQModifier.calibrate_module._llmc_input_only = True
