"""Tensor-level entry points: extract pointers, sizes and the current HIP stream
from torch tensors and call the C ABI.  torch is only memory and streams here."""
from __future__ import annotations

import torch

from . import _lib

BF16, F16, F32 = 0, 1, 2
_DT = {torch.bfloat16: BF16, torch.float16: F16, torch.float32: F32}


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _require_gpu(*ts: torch.Tensor) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "llmcompressor_amd kernels run on MI355X device tensors only; got a "
                f"{t.device} tensor (there is no CPU fallback)"
            )


def hessian_accumulate_(H: torch.Tensor, x: torch.Tensor, alpha: float = 2.0, assume_symmetric: bool = True):
    """H[K,K] (fp32, in place) += alpha * x^T x for x = [T,K] bf16/f16."""
    _require_gpu(H, x)
    assert H.dtype == torch.float32 and H.ndim == 2 and H.shape[0] == H.shape[1]
    assert x.ndim == 2 and x.shape[1] == H.shape[0]
    if x.dtype not in (torch.bfloat16, torch.float16):
        x = x.to(torch.bfloat16) if x.dtype == torch.float32 and False else x
        raise TypeError(f"hessian_accumulate_: unsupported activation dtype {x.dtype}")
    if x.stride(1) != 1:
        x = x.contiguous()
    assert H.stride(1) == 1
    with torch.cuda.device(H.device):
        rc = _lib.lib().llmc_hessian_accumulate(
            H.data_ptr(), H.stride(0), x.data_ptr(), x.stride(0), x.shape[0], x.shape[1],
            _DT[x.dtype], float(alpha), 1 if assume_symmetric else 0, _stream(H),
        )
    _lib.check(rc, "llmc_hessian_accumulate")
    return H
