"""oneshot(): apply a recipe to a model with optional calibration data (reference: entrypoints/oneshot.py:316-481).

Accepts an instantiated ``torch.nn.Module`` and, as ``dataset``, a ready ``DataLoader`` / list of batches (the
reference passes a DataLoader straight through, datasets/utils.py:143-144) or an in-memory ``datasets.Dataset``
(sampled, truncated and batched as the reference does, ``llmcompressor_amd.datasets``).  Loading models or
datasets by hub name needs network access and is not part of this build.
"""
from __future__ import annotations

import logging
import os
from typing import Optional

import torch

from ..core import active_session
from ..pipelines import CalibrationPipeline

logger = logging.getLogger("llmcompressor_amd")

__all__ = ["Oneshot", "oneshot"]


class _DatasetArgs:
    def __init__(self, **kw):
        self.__dict__.update(kw)


class Oneshot:
    def __init__(self, model, recipe=None, dataset=None, output_dir: Optional[str] = None, pipeline: str = "independent",
                 sequential_targets=None, stage: Optional[str] = None, save_compressed: bool = True,
                 moe_calibrate_all_experts: bool = True, moe_grouped_calibration: bool = False, **kwargs):
        if isinstance(model, str):
            raise ValueError("oneshot: pass an instantiated torch.nn.Module; loading by name is not available offline")
        self.model = model
        self.recipe = recipe
        self.dataset = dataset
        self.output_dir = output_dir
        self.pipeline = pipeline
        self.stage = stage
        self.save_compressed = save_compressed
        self.processor = kwargs.pop("processor", None) or kwargs.pop("tokenizer", None)
        self.dataset_args = _DatasetArgs(sequential_targets=sequential_targets, pipeline=pipeline,
                                         moe_calibrate_all_experts=moe_calibrate_all_experts,
                                         moe_grouped_calibration=moe_grouped_calibration, **kwargs)

    def __call__(self):
        from ..modeling.moe import get_non_linearized_moes, linearize_moe
        from ..transformers.compression.compressed_tensors_utils import modify_save_pretrained

        # reference: entrypoints/utils.py:96 -- from here on ``model.save_pretrained(dir, save_compressed=True,
        # quantization_format=None)`` writes the compressed checkpoint
        modify_save_pretrained(self.model)
        if get_non_linearized_moes(self.model):  # reference: entrypoints/oneshot.py:237-243
            logger.warning("Detected an MoE model whose experts are stored as fused 3-D tensors; replacing them "
                           "by per-expert Linears so that they can be calibrated and quantized.")
            linearize_moe(self.model)
        left = [name for name, m in self.model.named_modules()
                if isinstance(getattr(m, "down_proj", None), torch.nn.Parameter) and m.down_proj.ndim == 3]
        if left:
            logger.warning(f"{len(left)} fused expert modules have a layout or forward signature that is not "
                           f"recognised ({left[0]}, ...); they stay as they are and their weights are not quantized.")
        from ..datasets import get_calibration_dataloader
        from ..pipelines.onload import place_model

        # reference: set_onload_device(model, get_main_device()) at the head of every pipeline -- a model that
        # arrives on the host is computed on the GPU: moved there whole if it fits, else layer by layer
        self.dataset_args.onload_device = place_model(self.model)

        # an in-memory `datasets.Dataset` becomes a DataLoader (num_calibration_samples, max_seq_length,
        # batch_size, shuffle_calibration_samples, data_collator, ...); loaders and lists of batches pass through
        self.apply_recipe_modifiers(get_calibration_dataloader(self.dataset, self.processor,
                                                               **vars(self.dataset_args)))
        if self.output_dir is not None:
            if getattr(getattr(self.model, "save_pretrained", None), "_overridden", False):
                # reference: entrypoints/utils.py:122-124
                self.model.save_pretrained(self.output_dir, save_compressed=self.save_compressed)
            else:  # a plain torch module has no writer of its own
                from ..compressors import save_pretrained_compressed

                save_pretrained_compressed(self.model, self.output_dir, save_compressed=self.save_compressed,
                                           recipe=active_session().lifecycle.recipe)
        return self.model

    def apply_recipe_modifiers(self, calibration_dataloader):
        from ..modeling.moe import moe_calibration_context

        session = active_session()
        session.reset()
        # reference: entrypoints/oneshot.py:247-250 -- the whole calibration runs inside the MoE context when
        # ``moe_calibrate_all_experts`` is set: every expert is then called on every token while hooks observe it.
        # ``moe_grouped_calibration`` (this build's own switch, off by default) lets an experts block whose live
        # hooks only read their inputs take its grouped launches in the observed pass as well.
        with moe_calibration_context(bool(self.dataset_args.moe_calibrate_all_experts),
                                     grouped=bool(self.dataset_args.moe_grouped_calibration)):
            session.initialize(model=self.model, recipe=self.recipe, recipe_stage=self.stage,
                               calib_data=calibration_dataloader)
            mods = session.get_modifiers()
            user = self.pipeline
            pipeline = CalibrationPipeline.from_modifiers(mods, user=user)
            if calibration_dataloader is None and any(m.requires_calibration_data for m in mods):
                raise ValueError("the recipe requires calibration data but no `dataset` was given")
            pipeline(self.model, calibration_dataloader, self.dataset_args)
            session.finalize()


def oneshot(model, recipe=None, dataset=None, output_dir: Optional[str] = None, pipeline: str = "independent",
            sequential_targets=None, stage: Optional[str] = None, save_compressed: bool = True, **kwargs):
    """Quantise ``model`` in place according to ``recipe`` and return it; save when ``output_dir`` is given."""
    return Oneshot(model=model, recipe=recipe, dataset=dataset, output_dir=output_dir, pipeline=pipeline,
                   sequential_targets=sequential_targets, stage=stage, save_compressed=save_compressed, **kwargs)()
