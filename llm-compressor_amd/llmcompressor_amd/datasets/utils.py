"""From the ``dataset=`` argument of ``oneshot`` to the batches the calibration pipelines iterate.

Mirrors what the reference does between its entry point and the first forward (datasets/utils.py:122-431,
args/dataset_arguments.py): a ready ``DataLoader`` (or any plain iterable of batches) passes through; an in-memory
``datasets.Dataset`` / ``DatasetDict`` is tokenised if it has no ``input_ids`` column yet, cut to
``num_calibration_samples`` by a sampler (random order by default, longest-first without shuffling) and batched by a
collator that truncates each batch to its shortest sequence (``"truncation"``, the default) or pads it
(``"padding"``).  Loading a dataset by hub name needs the network and is refused.
"""
from __future__ import annotations

import logging
from typing import Any, Callable, Iterator, Optional

import torch
from torch.utils.data import DataLoader, RandomSampler, Sampler

logger = logging.getLogger("llmcompressor_amd")

__all__ = ["get_calibration_dataloader", "format_calibration_data", "DataCollatorWithTruncation",
           "LengthAwareSampler", "DATASET_DEFAULTS", "get_rank_partition"]

# reference: args/dataset_arguments.py (the fields this path reads, with their defaults)
DATASET_DEFAULTS = dict(num_calibration_samples=512, shuffle_calibration_samples=True, batch_size=1,
                        data_collator="truncation", max_seq_length=None, text_column="text",
                        pad_to_max_length=True, splits=None, preprocessing_func=None, remove_columns=None,
                        dataloader_num_workers=0)
_TOKEN_KEYS = ("input_ids", "labels", "attention_mask", "loss_mask")


class DataCollatorWithTruncation:
    """Cut every sequence of a batch to the batch's shortest one (and to ``max_seq_length``), then stack
    (reference: datasets/utils.py:301-318)."""

    def __init__(self, max_seq_length: Optional[int] = None):
        self.max_seq_length = max_seq_length

    def __call__(self, features, return_tensors: str = "pt"):
        from transformers import default_data_collator

        features = [dict(f) for f in features]
        for key in _TOKEN_KEYS:
            if any(key not in f for f in features):
                continue
            keep = min(len(f[key]) for f in features)
            if self.max_seq_length is not None:
                keep = min(keep, self.max_seq_length)
            for f in features:
                f[key] = f[key][:keep]
        return default_data_collator(features, return_tensors)


class LengthAwareSampler(Sampler):
    """Indices in order of descending ``input_ids`` length, the first ``num_samples`` of them: without
    shuffling, neighbours in a batch have similar lengths and the shortest samples are the ones left out
    (reference: datasets/utils.py:321-393)."""

    def __init__(self, data_source, num_samples: Optional[int] = None, batch_size: int = 1):
        self.data_source = data_source
        self._num_samples = num_samples or len(data_source)
        self.batch_size = batch_size
        columns = getattr(data_source, "column_names", None) or []
        name = next((c for c in ("input_ids", "decoder_input_ids") if c in columns), None)
        if name is None:
            logger.warning(f"Could not find input ids in {columns}")
            self.order = list(range(len(data_source)))
            return
        lengths = torch.tensor([len(sample) for sample in data_source[name]])
        self.order = torch.argsort(lengths, descending=True, stable=True).tolist()

    @property
    def num_samples(self) -> int:
        return self._num_samples

    def __iter__(self) -> Iterator[int]:
        return iter(self.order[: self._num_samples])

    def __len__(self) -> int:
        return min(self._num_samples, len(self.order))


def _make_sampler(dataset, num_samples, shuffle: bool, batch_size: int) -> Sampler:
    if num_samples is not None and num_samples > len(dataset):
        logger.warning(f"Requested {num_samples} samples but the provided dataset only has {len(dataset)} samples.")
        num_samples = len(dataset)
    if shuffle:
        if batch_size > 1:
            logger.warning("Shuffling the dataset can lead to unoptimal batching for sequences of non-uniform "
                           "length; consider calling `oneshot` with `batch_size=1`")
        return RandomSampler(dataset, num_samples=num_samples)
    return LengthAwareSampler(dataset, num_samples=num_samples, batch_size=batch_size)


def _make_collate_fn(data_collator, max_seq_length, processor) -> Callable:
    if callable(data_collator):
        return data_collator
    if data_collator == "truncation":
        return DataCollatorWithTruncation(max_seq_length)
    if data_collator == "padding":
        from transformers import DataCollatorWithPadding

        tokenizer = getattr(processor, "tokenizer", processor)
        if tokenizer is None:
            raise ValueError("`data_collator='padding'` needs the model's tokenizer: pass `processor=` / `tokenizer=`")
        if tokenizer.pad_token is None or tokenizer.pad_token_id < 0:
            tokenizer.pad_token = tokenizer.eos_token
        if max_seq_length is not None:
            logger.warning("Cannot use `data_collator='padding'` with `max_seq_length`. Ignoring truncation "
                           "specified by `max_seq_length`")
        return DataCollatorWithPadding(tokenizer)
    raise ValueError(f"Unknown data collator {data_collator}")


def format_calibration_data(tokenized_dataset, processor=None, **args) -> DataLoader:
    """DataLoader over a tokenised dataset (reference: datasets/utils.py:154-179)."""
    a = {**DATASET_DEFAULTS, **{k: v for k, v in args.items() if k in DATASET_DEFAULTS}}
    workers = a["dataloader_num_workers"]
    extra = {"persistent_workers": True} if workers > 0 else {}
    return DataLoader(
        tokenized_dataset, batch_size=a["batch_size"],
        sampler=_make_sampler(tokenized_dataset, a["num_calibration_samples"], a["shuffle_calibration_samples"],
                              a["batch_size"]),
        collate_fn=_make_collate_fn(a["data_collator"], a["max_seq_length"], processor),
        pin_memory=torch.cuda.is_available() and workers > 0, num_workers=workers, **extra)


def _select_split(dataset, splits):
    """One split of a ``DatasetDict`` (reference: datasets/utils.py:46-119)."""
    if hasattr(dataset, "column_names") and not isinstance(dataset.column_names, dict):
        return dataset
    if isinstance(splits, dict):
        if "calibration" not in splits:
            raise ValueError("Passing `splits` as a dict is only supported when it contains a `'calibration'` key")
        splits = splits["calibration"]
    elif isinstance(splits, (list, tuple)):
        splits = splits[0] if splits else None
    elif splits is not None and not isinstance(splits, str):
        raise ValueError(f"Invalid splits type: {type(splits)}. Expected a split string")
    if splits is not None:
        return dataset[splits]
    if "train" in dataset:
        logger.warning("No split was specified, but a multi-split dataset was given. Falling back to the 'train' "
                       "split for calibration.")
        return dataset["train"]
    raise ValueError("No split specified and 'train' split not found in dataset. Please specify `splits` explicitly.")


def _tokenize(dataset, processor, a):
    """Rows of text to ``input_ids`` / ``attention_mask`` (reference: transformers/data/base.py:131-325):
    optional ``preprocessing_func`` per row, the tokenizer over ``text_column`` with truncation to
    ``max_seq_length`` and -- ``pad_to_max_length`` being on by default -- padding to it."""
    if processor is None:
        raise ValueError("the dataset has no `input_ids` column and no `processor` / `tokenizer` was given to "
                         "tokenize it")
    if a["preprocessing_func"] is not None:
        if not callable(a["preprocessing_func"]):
            raise ValueError("`preprocessing_func` must be a callable here (registry names are not available)")
        dataset = dataset.map(a["preprocessing_func"])
    column = a["text_column"]
    if column not in dataset.column_names:
        raise ValueError(f"text_column {column!r} not found in the dataset's columns {dataset.column_names}")
    tokenizer = getattr(processor, "tokenizer", processor)
    max_len = a["max_seq_length"]
    limit = getattr(tokenizer, "model_max_length", None)
    if max_len is not None and isinstance(limit, int) and max_len > limit:
        logger.warning(f"max_seq_length {max_len} exceeds the tokenizer's model_max_length {limit}; using {limit}")
        max_len = limit
    padding = "max_length" if (a["pad_to_max_length"] and max_len is not None) else False

    def encode(row):
        return dict(processor(row[column], padding=padding, max_length=max_len, truncation=max_len is not None))

    drop = list(dataset.column_names)
    extra = a["remove_columns"]
    if isinstance(extra, str):
        extra = [extra]
    return dataset.map(encode, remove_columns=sorted(set(drop) | set(extra or [])))


def get_calibration_dataloader(dataset, processor=None, **args):
    """What the pipelines iterate, from ``oneshot``'s ``dataset`` argument (reference: datasets/utils.py:122-151).
    ``None`` (data-free recipes), a ``DataLoader`` and any other ready iterable of batches pass through."""
    if dataset is None or isinstance(dataset, DataLoader):
        return dataset
    if isinstance(dataset, str):
        raise ValueError(f"dataset {dataset!r}: loading a dataset by name needs network access; pass a "
                         "`datasets.Dataset`, a `DataLoader` or a list of batches")
    if not hasattr(dataset, "column_names"):
        return dataset  # a list / generator of ready batches
    a = {**DATASET_DEFAULTS, **{k: v for k, v in args.items() if k in DATASET_DEFAULTS}}
    dataset = _select_split(dataset, a["splits"])
    if "input_ids" not in dataset.column_names:
        dataset = _tokenize(dataset, processor, a)
    return format_calibration_data(dataset, processor, **a)


def get_rank_partition(split: str, num_samples: int) -> str:
    """``"train[start:end]"`` for this process's share of ``num_samples`` (reference: datasets/utils.py:398-431);
    with one process that is all of them."""
    import math

    import torch.distributed as dist

    assert "[" not in split, "Split string should not already contain partitioning brackets"
    rank = dist.get_rank() if dist.is_available() and dist.is_initialized() else 0
    world = dist.get_world_size() if dist.is_available() and dist.is_initialized() else 1
    start = math.floor(num_samples * (rank / world))
    end = math.floor(num_samples * ((rank + 1) / world))
    return f"{split}[{start}:{end}]"
