"""Tensor-level entry points: extract pointers, sizes and the current HIP stream
from torch tensors and call the C ABI.  torch is only memory and streams here."""
from __future__ import annotations

import threading
import weakref

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


def hessian_accumulate_(H: torch.Tensor, x: torch.Tensor, alpha: float = 2.0, assume_symmetric: bool = True,
                        use_workspace: bool = True):
    """H[K,K] (fp32, in place) += alpha * x^T x for x = [T,K] bf16/f16 (exact products on the 16-bit matrix
    cores) or fp32 (the fp32 matrix-core GEMM over the full matrix).

    With `use_workspace` a per-stream scratch buffer lets tiles that do not fill the chip be cut along
    the tokens (summed in fixed order, so results stay reproducible); without it every output tile
    is one workgroup."""
    _require_gpu(H, x)
    assert H.dtype == torch.float32 and H.ndim == 2 and H.shape[0] == H.shape[1]
    assert x.ndim == 2 and x.shape[1] == H.shape[0]
    if x.dtype not in (torch.bfloat16, torch.float16, torch.float32):
        raise TypeError(f"hessian_accumulate_: unsupported activation dtype {x.dtype}")
    if x.stride(1) != 1:
        x = x.contiguous()
    assert H.stride(1) == 1
    with torch.cuda.device(H.device):
        ws, nws = None, 0
        if use_workspace and x.dtype != torch.float32:
            nws = int(_lib.lib().llmc_hessian_workspace_bytes(x.shape[0], x.shape[1]))
            ws = _workspace(H.device, nws) if nws else None
        rc = _lib.lib().llmc_hessian_accumulate(
            H.data_ptr(), H.stride(0), x.data_ptr(), x.stride(0), x.shape[0], x.shape[1],
            _DT[x.dtype], float(alpha), 1 if assume_symmetric else 0, _ptr(ws), nws, _stream(H),
        )
    _lib.check(rc, "llmc_hessian_accumulate")
    return H


SEGMENTS_MAX = 64  # buffers per llmc_hessian_accumulate_segments launch


def segment_ok(x: torch.Tensor) -> bool:
    """Can `x` ([T, K] view) be one buffer of hessian_accumulate_segments_ (not the last one)?"""
    return (x.is_cuda and x.ndim == 2 and x.dtype in (torch.bfloat16, torch.float16) and x.stride(1) == 1
            and x.shape[0] > 0 and x.shape[0] % 64 == 0 and x.shape[1] % 8 == 0 and x.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0)


def hessian_accumulate_segments_(H: torch.Tensor, xs, alpha: float = 2.0, assume_symmetric: bool = True):
    """H (fp32 [K,K], in place) += alpha * X^T X where X is the row-wise concatenation of xs, without
    building it: xs[i] = [T_i, K] with one common row stride and dtype, T_i equal and a multiple of 64
    for all but the last (which may hold fewer rows).  Bit-identical to hessian_accumulate_ on torch.cat(xs)."""
    import ctypes

    if not xs:
        return H
    x0 = xs[0]
    _require_gpu(H, x0)
    K = H.shape[0]
    assert H.dtype == torch.float32 and H.shape == (K, K) and H.stride(1) == 1
    seg = x0.shape[0] if len(xs) > 1 else -(-x0.shape[0] // 64) * 64
    for i, x in enumerate(xs):
        last = i == len(xs) - 1
        if not (x.ndim == 2 and x.shape[1] == K and x.dtype == x0.dtype and x.stride(1) == 1
                and x.stride(0) == x0.stride(0) and x.device == H.device and x.data_ptr() % 16 == 0
                and (x.shape[0] == seg or (last and 0 < x.shape[0] <= seg))):
            raise ValueError("hessian_accumulate_segments_: buffers need one width, dtype, row stride and row count "
                             "(the last may be shorter) and 16-byte alignment")
    if x0.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"hessian_accumulate_segments_: unsupported activation dtype {x0.dtype}")
    if seg % 64 or K % 8 or x0.stride(0) % 8:
        raise ValueError("hessian_accumulate_segments_: rows per buffer must be a multiple of 64, K and the row "
                         "stride multiples of 8")
    with torch.cuda.device(H.device):
        for b in range(0, len(xs), SEGMENTS_MAX):
            part = xs[b:b + SEGMENTS_MAX]
            T = seg * (len(part) - 1) + part[-1].shape[0]
            xp = (ctypes.c_void_p * len(part))(*[x.data_ptr() for x in part])
            nws = int(_lib.lib().llmc_hessian_workspace_bytes(T, K))
            ws = _workspace(H.device, nws) if nws else None
            rc = _lib.lib().llmc_hessian_accumulate_segments(
                H.data_ptr(), H.stride(0), xp, len(part), seg, part[-1].shape[0], x0.stride(0), K, _DT[x0.dtype],
                float(alpha), 1 if assume_symmetric else 0, _ptr(ws), nws, _stream(H))
            _lib.check(rc, "llmc_hessian_accumulate_segments")
    return H


def hessian_accumulate_grouped_(Hs, xs, alpha: float = 2.0, assume_symmetric: bool = True):
    """One launch for many independent problems of the same width (the per-expert Hessians of an MoE
    layer): Hs[i] (fp32 [K,K], in place) += alpha * xs[i]^T xs[i] with xs[i] = [T_i, K], T_i >= 0.
    All Hs share a row stride, all xs a row stride and dtype; every xs[i] is 16-byte aligned."""
    import ctypes

    assert len(Hs) == len(xs)
    if not Hs:
        return Hs
    H0 = Hs[0]
    K = H0.shape[0]
    x_ref = next((x for x in xs if x.shape[0] > 0), None)
    if x_ref is None:
        return Hs
    _require_gpu(H0, x_ref)
    if x_ref.dtype not in (torch.bfloat16, torch.float16):
        raise TypeError(f"hessian_accumulate_grouped_: unsupported activation dtype {x_ref.dtype}")
    n = len(Hs)
    hp = (ctypes.c_void_p * n)()
    xp = (ctypes.c_void_p * n)()
    tc = (ctypes.c_int64 * n)()
    keep = []
    for i, (H, x) in enumerate(zip(Hs, xs)):
        assert H.dtype == torch.float32 and H.shape == (K, K) and H.stride(1) == 1 and H.stride(0) == H0.stride(0)
        assert x.ndim == 2 and x.shape[1] == K and H.device == H0.device
        tc[i] = x.shape[0]
        hp[i] = H.data_ptr()
        if x.shape[0] > 0:
            if x.dtype != x_ref.dtype:
                raise TypeError("hessian_accumulate_grouped_: mixed activation dtypes")
            if x.stride(1) != 1 or x.stride(0) != x_ref.stride(0) or x.data_ptr() % 16:
                x = x.contiguous()
                if x.stride(0) != x_ref.stride(0):
                    raise ValueError("hessian_accumulate_grouped_: activation blocks need one common row stride")
                keep.append(x)
            xp[i] = x.data_ptr()
    with torch.cuda.device(H0.device):
        rc = _lib.lib().llmc_hessian_accumulate_grouped(
            hp, H0.stride(0), xp, x_ref.stride(0), tc, n, K, _DT[x_ref.dtype], float(alpha),
            1 if assume_symmetric else 0, _stream(H0))
    _lib.check(rc, "llmc_hessian_accumulate_grouped")
    return Hs


FMT_INT, FMT_FP8, FMT_FP4 = 0, 1, 2
SCALE_PLAIN, SCALE_NVFP4, SCALE_MXFP4 = 0, 1, 2
OUT_FAKEQUANT, OUT_CODES, OUT_PACKED = 0, 1, 2
_TD = {BF16: torch.bfloat16, F16: torch.float16, F32: torch.float32}

class _WorkspaceStore(dict):
    """The scratch buffers of one host thread, keyed by (device, stream)."""

    __slots__ = ("__weakref__",)
    __hash__ = object.__hash__  # kept in a WeakSet: identity, not contents

    def __eq__(self, other):
        return self is other


_ws_local = threading.local()  # a thread's store goes away with the thread, and its buffers with it
_ws_stores = weakref.WeakSet()  # the stores of the threads still alive, for release_workspaces()


def _workspace(device, nbytes: int) -> torch.Tensor:
    """Scratch memory for one C call, cached per (device, stream, host thread).

    Several entry points issue more than one launch over their workspace, and ctypes releases the GIL during
    a call, so two host threads on one stream could interleave their launches: each thread therefore owns its
    buffer (work of one thread on one stream is ordered by the stream).  The buffers of a thread live in
    thread-local storage: a worker thread that ends (a pool that is torn down) gives its buffers back."""
    store = getattr(_ws_local, "store", None)
    if store is None:
        store = _ws_local.store = _WorkspaceStore()
        _ws_stores.add(store)
    key = (device, torch.cuda.current_stream(device).cuda_stream)
    ws = store.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 16), dtype=torch.uint8, device=device)
        store[key] = ws
    return ws


def release_workspaces() -> None:
    """Drop the cached scratch buffers of every thread (the largest GPTQ workspace is R * K * 4 bytes and more).
    Call it between phases when the memory is wanted back; work already enqueued keeps its buffer alive through
    the caching allocator's stream ordering, and the next call allocates afresh."""
    for store in list(_ws_stores):
        store.clear()


def _ptr(t):
    return 0 if t is None else t.data_ptr()


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}; expected bf16/f16/f32") from None


def minmax_groups(w: torch.Tensor, group: int):
    """min/max of each run of `group` consecutive columns of w [R,K] -> two [R, K/group] tensors."""
    _require_gpu(w)
    assert w.ndim == 2 and w.stride(1) == 1
    R, K = w.shape
    mn = torch.empty((R, K // group), dtype=w.dtype, device=w.device)
    mx = torch.empty_like(mn)
    ws = _workspace(w.device, 1 << 16)
    with torch.cuda.device(w.device):
        rc = _lib.lib().llmc_minmax_groups(w.data_ptr(), _dt(w), R, K, w.stride(0), group, mn.data_ptr(),
                                           mx.data_ptr(), ws.data_ptr(), ws.numel(), _stream(w))
    _lib.check(rc, "llmc_minmax_groups")
    return mn, mx


def minmax_blocks(w: torch.Tensor, bh: int, bw: int):
    _require_gpu(w)
    assert w.ndim == 2 and w.stride(1) == 1
    R, K = w.shape
    shape = ((R + bh - 1) // bh, (K + bw - 1) // bw)
    mn = torch.empty(shape, dtype=w.dtype, device=w.device)
    mx = torch.empty_like(mn)
    with torch.cuda.device(w.device):
        rc = _lib.lib().llmc_minmax_blocks(w.data_ptr(), _dt(w), R, K, w.stride(0), bh, bw, mn.data_ptr(),
                                           mx.data_ptr(), _stream(w))
    _lib.check(rc, "llmc_minmax_blocks")
    return mn, mx


def minmax_strided(x: torch.Tensor, n0: int, n1: int, group: int, s0: int, s1: int):
    """x viewed as (n0, n1, group) with element strides (s0, s1, 1): reduce dims (0,-1) -> [n1]."""
    _require_gpu(x)
    mn = torch.empty((n1,), dtype=x.dtype, device=x.device)
    mx = torch.empty_like(mn)
    with torch.cuda.device(x.device):
        rc = _lib.lib().llmc_minmax_strided(x.data_ptr(), _dt(x), n0, n1, group, s0, s1, mn.data_ptr(),
                                            mx.data_ptr(), _stream(x))
    _lib.check(rc, "llmc_minmax_strided")
    return mn, mx


def _gs32(global_scale):
    """The kernels read the global scale as one fp32 value."""
    if global_scale is None:
        return None
    return global_scale.to(torch.float32).contiguous()


def global_scale_from_stats(stats):
    """NVFP4 global scale from the (min, max) arrays of every observer of a fused group -> fp32 [1]."""
    mn0 = stats[0][0]
    _require_gpu(mn0)
    absmax = torch.zeros(1, dtype=torch.float32, device=mn0.device)
    out = torch.empty(1, dtype=torch.float32, device=mn0.device)
    with torch.cuda.device(mn0.device):
        for mn, mx in stats:
            mn, mx = mn.contiguous(), mx.contiguous()
            rc = _lib.lib().llmc_absmax_accumulate(mn.data_ptr(), mx.data_ptr(), mn.numel(), _dt(mn),
                                                   absmax.data_ptr(), _stream(mn0))
            _lib.check(rc, "llmc_absmax_accumulate")
        rc = _lib.lib().llmc_generate_gparam(absmax.data_ptr(), _dt(mn0), out.data_ptr(), _stream(mn0))
    _lib.check(rc, "llmc_generate_gparam")
    return out


def calculate_qparams(mn, mx, fmt: int, bits: int, symmetric: bool, scale_mode: int = SCALE_PLAIN,
                      global_scale=None, want_codes: bool = False):
    """(min,max) -> (scale, zero_point int8, scale_code uint8|None); shapes follow `mn`."""
    global_scale = _gs32(global_scale)
    _require_gpu(mn, mx)
    mn, mx = mn.contiguous(), mx.contiguous()
    sdt = torch.float32 if scale_mode == SCALE_NVFP4 else mn.dtype
    scale = torch.empty(mn.shape, dtype=sdt, device=mn.device)
    zp = torch.zeros(mn.shape, dtype=torch.int8, device=mn.device)
    codes = torch.empty(mn.shape, dtype=torch.uint8, device=mn.device) if want_codes else None
    with torch.cuda.device(mn.device):
        rc = _lib.lib().llmc_calculate_qparams(
            mn.data_ptr(), mx.data_ptr(), mn.numel(), _dt(mn), fmt, bits, 1 if symmetric else 0, scale_mode,
            _ptr(global_scale), scale.data_ptr(), _DT[sdt], 0 if symmetric else zp.data_ptr(), _ptr(codes),
            _stream(mn))
    _lib.check(rc, "llmc_calculate_qparams")
    return scale, zp, codes


def quantize(x, scale, zero_point, fmt: int, bits: int, row_div: int, scale_row_stride: int, col_div: int,
             out_mode: int = OUT_FAKEQUANT, g_idx=None, global_scale=None, out_dtype=None):
    """Element-wise quantise of x [R,K]; see llmc_quantize in include/llmc_amd.h for the scale indexing."""
    global_scale = _gs32(global_scale)
    _require_gpu(x, scale)
    assert x.ndim == 2 and x.stride(1) == 1
    R, K = x.shape
    scale = scale.contiguous()
    if zero_point is not None:
        zero_point = zero_point.contiguous()
        assert zero_point.dtype == torch.int8
    if g_idx is not None:
        g_idx = g_idx.to(torch.int32).contiguous()
    if out_mode == OUT_FAKEQUANT:
        out_dtype = out_dtype or x.dtype
        out = torch.empty((R, K), dtype=out_dtype, device=x.device)
        odt, ldo = _DT[out_dtype], K
    elif out_mode == OUT_CODES:
        tdt = torch.int8 if fmt == FMT_INT else (torch.float8_e4m3fn if fmt == FMT_FP8 else torch.uint8)
        out = torch.empty((R, K), dtype=tdt, device=x.device)
        odt, ldo = 0, K
    else:
        if fmt == FMT_INT:
            pf = 32 // bits
            ldo = (K + pf - 1) // pf
            out = torch.empty((R, ldo), dtype=torch.int32, device=x.device)
        elif fmt == FMT_FP4:
            ldo = (K + 1) // 2
            out = torch.empty((R, ldo), dtype=torch.uint8, device=x.device)
        else:
            ldo = K
            out = torch.empty((R, K), dtype=torch.float8_e4m3fn, device=x.device)
        odt = 0
    with torch.cuda.device(x.device):
        rc = _lib.lib().llmc_quantize(
            x.data_ptr(), _dt(x), R, K, x.stride(0), scale.data_ptr(), _dt(scale), _ptr(zero_point),
            _ptr(g_idx), _ptr(global_scale), fmt, bits, row_div, scale_row_stride, col_div, out_mode,
            out.data_ptr(), odt, ldo, _stream(x))
    _lib.check(rc, "llmc_quantize")
    return out


def dynamic_per_token_quantize(x, fmt: int = FMT_FP8, bits: int = 8, out_mode: int = OUT_FAKEQUANT):
    """x [N,K] bf16/f16 -> (fake-quantised x | code bytes, per-row scale [N,1])."""
    _require_gpu(x)
    assert x.ndim == 2 and x.stride(1) == 1
    N, K = x.shape
    scale = torch.empty((N, 1), dtype=x.dtype, device=x.device)
    if out_mode == OUT_FAKEQUANT:
        out = torch.empty((N, K), dtype=x.dtype, device=x.device)
    else:
        out = torch.empty((N, K), dtype=torch.float8_e4m3fn if fmt == FMT_FP8 else torch.int8, device=x.device)
    with torch.cuda.device(x.device):
        rc = _lib.lib().llmc_dynamic_per_token_quantize(x.data_ptr(), _dt(x), N, K, x.stride(0), fmt, bits,
                                                        out_mode, out.data_ptr(), K, scale.data_ptr(),
                                                        _stream(x))
    _lib.check(rc, "llmc_dynamic_per_token_quantize")
    return out, scale


FACTOR_INVERSE, FACTOR_GROUPS, FACTOR_GROUP_WIDTH = 0, 1, 512


def gptq_factor_form(K: int, blocksize: int = 128) -> int:
    """The form of the factor the library prefers for a quantize_weight call on K columns: FACTOR_GROUPS where
    the column loop can work from the Cholesky factor of H itself and the shorter chain pays for the loop's extra
    launches (K a multiple of 128, from 8192 columns on), else FACTOR_INVERSE."""
    return int(_lib.lib().llmc_gptq_factor_form(int(K), int(blocksize)))


def gptq_hinv_(H: torch.Tensor, perm=None, divisor: float = 1.0, percdamp: float = 0.01, form: int = FACTOR_INVERSE):
    """In place: H -> upper factor U of (H/divisor [permuted] + damping)^-1; with form = FACTOR_GROUPS only inside
    the 512-column diagonal blocks (aligned to the last column), the upper Cholesky factor of the damped H itself
    outside them.

    Returns (U (= H), dead uint8 [K], info int32 [1] on device)."""
    _require_gpu(H)
    assert H.dtype == torch.float32 and H.ndim == 2 and H.shape[0] == H.shape[1] and H.stride(1) == 1
    K = H.shape[0]
    dead = torch.empty(K, dtype=torch.uint8, device=H.device)
    info = torch.zeros(1, dtype=torch.int32, device=H.device)
    if perm is not None:
        perm = perm.to(torch.int32).contiguous()
    nbytes = _lib.lib().llmc_gptq_hinv_workspace_bytes(K)
    ws = _workspace(H.device, nbytes)
    with torch.cuda.device(H.device):
        rc = _lib.lib().llmc_gptq_hinv(H.data_ptr(), H.stride(0), K, _ptr(perm), float(divisor), float(percdamp),
                                       int(form), dead.data_ptr(), ws.data_ptr(), ws.numel(), info.data_ptr(),
                                       _stream(H))
    _lib.check(rc, "llmc_gptq_hinv")
    return H, dead, info


def gptq_hinv_grouped(Hs, perms=None, divisors=None, percdamp: float = 0.01, form: int = FACTOR_INVERSE):
    """gptq_hinv_ for n Hessians of one width in lock-step.  Hs: list of fp32 [K,K] (left untouched); perms:
    int32 [n,K] tensor or None; divisors: list of floats.  Returns (U [n,K,K] fp32, dead [n,K] uint8, info [n])."""
    import ctypes

    n = len(Hs)
    H0 = Hs[0]
    _require_gpu(H0)
    K = H0.shape[0]
    for H in Hs:
        assert H.dtype == torch.float32 and H.shape == (K, K) and H.stride(1) == 1 and H.stride(0) == H0.stride(0)
        assert H.device == H0.device
    U = torch.empty((n, K, K), dtype=torch.float32, device=H0.device)
    dead = torch.empty((n, K), dtype=torch.uint8, device=H0.device)
    info = torch.zeros(n, dtype=torch.int32, device=H0.device)
    hp = (ctypes.c_void_p * n)(*[H.data_ptr() for H in Hs])
    pp = None
    if perms is not None:
        perms = perms.to(torch.int32).contiguous()
        assert perms.shape == (n, K)
        pp = (ctypes.c_void_p * n)(*[perms.data_ptr() + 4 * K * b for b in range(n)])
    dv = (ctypes.c_float * n)(*[float(d) for d in (divisors if divisors is not None else [1.0] * n)])
    nbytes = _lib.lib().llmc_gptq_hinv_grouped_workspace_bytes(n, K)
    ws = _workspace(H0.device, nbytes)
    with torch.cuda.device(H0.device):
        rc = _lib.lib().llmc_gptq_hinv_grouped(hp, H0.stride(0), n, K, pp, dv, float(percdamp), int(form),
                                              dead.data_ptr(), U.data_ptr(), K, ws.data_ptr(), ws.numel(),
                                              info.data_ptr(), _stream(H0))
    _lib.check(rc, "llmc_gptq_hinv_grouped")
    return U, dead, info


def gptq_quantize(weight, U, scale, zero_point, fmt: int, bits: int, row_div: int, scale_row_stride: int,
                  g_idx=None, perm=None, dead=None, global_scale=None, blocksize: int = 128,
                  form: int = FACTOR_INVERSE):
    """The GPTQ column loop on a factor of the given form (see gptq_hinv_).  Returns (quantised-dequantised weight
    in weight.dtype, loss fp32 [1])."""
    global_scale = _gs32(global_scale)
    _require_gpu(weight, U, scale)
    assert weight.ndim == 2 and weight.stride(1) == 1 and U.stride(1) == 1
    R, K = weight.shape
    scale = scale.contiguous()
    if zero_point is not None:
        zero_point = zero_point.contiguous()
        assert zero_point.dtype == torch.int8
    if g_idx is not None:
        g_idx = g_idx.to(torch.int32).contiguous()
    if perm is not None:
        perm = perm.to(torch.int32).contiguous()
    out = torch.empty((R, K), dtype=weight.dtype, device=weight.device)
    loss = torch.empty(1, dtype=torch.float32, device=weight.device)
    nbytes = _lib.lib().llmc_gptq_quantize_workspace_bytes(R, K, int(form))
    ws = _workspace(weight.device, nbytes)
    with torch.cuda.device(weight.device):
        rc = _lib.lib().llmc_gptq_quantize(
            weight.data_ptr(), _dt(weight), R, K, weight.stride(0), U.data_ptr(), U.stride(0), _ptr(perm),
            _ptr(dead), scale.data_ptr(), _dt(scale), _ptr(zero_point), _ptr(global_scale), _ptr(g_idx), row_div,
            scale_row_stride, fmt, bits, blocksize, int(form), out.data_ptr(), K, loss.data_ptr(), ws.data_ptr(),
            ws.numel(), _stream(weight))
    _lib.check(rc, "llmc_gptq_quantize")
    return out, loss


def gptq_quantize_grouped(weights, U, scales, zero_points, fmt: int, bits: int, row_div: int, scale_row_stride: int,
                          g_idxs=None, perms=None, dead=None, global_scales=None, blocksize: int = 128,
                          form: int = FACTOR_INVERSE):
    """gptq_quantize for n weights of one shape in lock-step.  weights / scales / zero_points / g_idxs /
    global_scales: lists of n tensors (the last three may be None); U [n,K,K] fp32; perms [n,K] int32 or None;
    dead [n,K] uint8 or None.  Returns (list of quantised-dequantised weights, loss fp32 [n])."""
    import ctypes

    n = len(weights)
    w0 = weights[0]
    _require_gpu(w0, U)
    R, K = w0.shape
    keep = []

    def ptrs(ts, dtype=None):
        if ts is None:
            return None
        arr = (ctypes.c_void_p * n)()
        for i, t in enumerate(ts):
            t = t.contiguous() if dtype is None else t.to(dtype).contiguous()
            keep.append(t)
            arr[i] = t.data_ptr()
        return arr

    for w in weights:
        assert w.shape == (R, K) and w.dtype == w0.dtype and w.stride(1) == 1 and w.stride(0) == w0.stride(0)
    assert U.shape == (n, K, K) and U.dtype == torch.float32 and U.is_contiguous()
    for s_ in scales:
        assert s_.dtype == scales[0].dtype and s_.numel() == scales[0].numel()
    if perms is not None:
        perms = perms.to(torch.int32).contiguous()
    outs = [torch.empty((R, K), dtype=w0.dtype, device=w0.device) for _ in range(n)]
    loss = torch.empty(n, dtype=torch.float32, device=w0.device)
    nbytes = _lib.lib().llmc_gptq_quantize_grouped_workspace_bytes(n, R, K, int(form))
    ws = _workspace(w0.device, nbytes)
    wp = (ctypes.c_void_p * n)(*[w.data_ptr() for w in weights])
    op = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
    sp, zp = ptrs(scales), ptrs(zero_points)
    gp, ip = ptrs(global_scales, torch.float32), ptrs(g_idxs, torch.int32)
    with torch.cuda.device(w0.device):
        rc = _lib.lib().llmc_gptq_quantize_grouped(
            wp, _dt(w0), n, R, K, w0.stride(0), U.data_ptr(), K, K * K, _ptr(perms), _ptr(dead), sp, _dt(keep[0]),
            zp, gp, ip, row_div, scale_row_stride, fmt, bits, blocksize, int(form), op, K, loss.data_ptr(),
            ws.data_ptr(), ws.numel(), _stream(w0))
    _lib.check(rc, "llmc_gptq_quantize_grouped")
    return outs, loss


def sparsegpt_sparsify(weight, U, sparsity: float, prune_n: int = 0, prune_m: int = 0, dead=None,
                       blocksize: int = 128, preserve_sparsity_mask: bool = False, form: int = FACTOR_INVERSE):
    """The SparseGPT column loop on the factor U of gptq_hinv_ (of the given form).  Returns (pruned weight in
    weight.dtype, loss fp32 [1])."""
    _require_gpu(weight, U)
    assert weight.ndim == 2 and weight.stride(1) == 1 and U.stride(1) == 1
    R, K = weight.shape
    if prune_n:
        if prune_m not in (2, 4, 8) or not 0 < prune_n <= prune_m or blocksize % prune_m or blocksize > 128:
            raise ValueError(f"sparsegpt_sparsify: unsupported mask structure {prune_n}:{prune_m} for block size "
                             f"{blocksize} (M must be 2, 4 or 8 and divide the block size, which is at most 128)")
    elif not (0.0 <= sparsity < 1.0) or not 32 <= blocksize <= 128:
        raise ValueError(f"sparsegpt_sparsify: sparsity {sparsity} must lie in [0, 1) and the block size "
                         f"{blocksize} in [32, 128]")
    out = torch.empty((R, K), dtype=weight.dtype, device=weight.device)
    loss = torch.empty(1, dtype=torch.float32, device=weight.device)
    nbytes = _lib.lib().llmc_sparsegpt_workspace_bytes(R, K, int(form))
    ws = _workspace(weight.device, nbytes)
    with torch.cuda.device(weight.device):
        rc = _lib.lib().llmc_sparsegpt_sparsify(
            weight.data_ptr(), _dt(weight), R, K, weight.stride(0), U.data_ptr(), U.stride(0), _ptr(dead),
            float(sparsity), int(prune_n), int(prune_m), int(blocksize), int(form),
            1 if preserve_sparsity_mask else 0, out.data_ptr(), K, loss.data_ptr(), ws.data_ptr(), ws.numel(),
            _stream(weight))
    _lib.check(rc, "llmc_sparsegpt_sparsify")
    return out, loss


def _mse_common(maxshrink, grid, patience, norm, expand):
    steps = int(maxshrink * grid)
    if steps > 256:
        raise ValueError(f"MSE observer: int(maxshrink*grid)={steps} search steps exceed the supported 256")
    return steps, float(grid), int(patience), float(norm), float(expand)


def mse_observe_groups(w, group: int, fmt: int, bits: int, symmetric: bool, scale_mode: int = SCALE_PLAIN,
                       maxshrink=0.20, patience=5, grid=100.0, norm=2.4, expand=1.0):
    """MSE grid search per run of `group` columns of w [R,K] -> (min, max) [R, K/group]."""
    _require_gpu(w)
    assert w.ndim == 2 and w.stride(1) == 1
    R, K = w.shape
    steps, grid, patience, norm, expand = _mse_common(maxshrink, grid, patience, norm, expand)
    n = R * (K // group)
    mn = torch.empty((R, K // group), dtype=w.dtype, device=w.device)
    mx = torch.empty_like(mn)
    ws = _workspace(w.device, _lib.lib().llmc_mse_workspace_bytes(n))
    with torch.cuda.device(w.device):
        rc = _lib.lib().llmc_mse_observe_groups(
            w.data_ptr(), _dt(w), R, K, w.stride(0), group, fmt, bits, 1 if symmetric else 0, scale_mode, steps,
            grid, patience, norm, expand, mn.data_ptr(), mx.data_ptr(), ws.data_ptr(), ws.numel(), _stream(w))
    _lib.check(rc, "llmc_mse_observe_groups")
    return mn, mx


def sumsq_accumulate_(total: torch.Tensor, x: torch.Tensor):
    """total[K] (fp32, in place) += sum over the rows of x [T, K] of x^2."""
    _require_gpu(total, x)
    assert total.dtype == torch.float32 and total.ndim == 1 and x.ndim == 2 and x.shape[1] == total.shape[0]
    if x.stride(1) != 1:
        x = x.contiguous()
    ws = _workspace(x.device, _lib.lib().llmc_sumsq_workspace_bytes(x.shape[1]))
    with torch.cuda.device(x.device):
        rc = _lib.lib().llmc_sumsq_accumulate(x.data_ptr(), _dt(x), x.shape[0], x.shape[1], x.stride(0),
                                              total.data_ptr(), ws.data_ptr(), ws.numel(), _stream(x))
    _lib.check(rc, "llmc_sumsq_accumulate")
    return total


SUMSQ_NOALLOC_MAX_K = 16384  # LLMC_SUMSQ_NOALLOC_MAX_K


def sumsq_accumulate_noalloc_(total: torch.Tensor, x: torch.Tensor):
    """sumsq_accumulate_ without any allocation: the partial sums use a device array inside the library.
    x must already be [T, K] with unit column stride and K <= SUMSQ_NOALLOC_MAX_K; calls on one GPU must not
    overlap in time."""
    _require_gpu(total, x)
    assert total.dtype == torch.float32 and total.ndim == 1 and x.ndim == 2 and x.shape[1] == total.shape[0]
    if x.stride(1) != 1:
        raise ValueError("sumsq_accumulate_noalloc_: x needs unit column stride (making it contiguous would allocate)")
    if x.shape[1] > SUMSQ_NOALLOC_MAX_K:
        raise ValueError(f"sumsq_accumulate_noalloc_: K={x.shape[1]} exceeds the library's device array "
                         f"(K <= {SUMSQ_NOALLOC_MAX_K}); use sumsq_accumulate_ with a workspace")
    with torch.cuda.device(x.device):
        rc = _lib.lib().llmc_sumsq_accumulate_noalloc(x.data_ptr(), _dt(x), x.shape[0], x.shape[1], x.stride(0),
                                                      total.data_ptr(), _stream(x))
    _lib.check(rc, "llmc_sumsq_accumulate_noalloc")
    return total


def imatrix_observe_groups(w, group: int, fmt: int, bits: int, symmetric: bool, scale_mode: int = SCALE_PLAIN,
                           importance=None, maxshrink=0.95, patience=5, grid=20, norm=3.0, expand=1.0):
    """Importance-weighted grid search per run of `group` columns of w [R,K] -> (min, max) [R, K/group]."""
    _require_gpu(w)
    assert w.ndim == 2 and w.stride(1) == 1
    R, K = w.shape
    steps = max(1, int(maxshrink * grid)) + 1
    if steps > 256:
        raise ValueError(f"imatrix_observe_groups: {steps} candidates exceed the 256 this build records")
    if importance is not None:
        importance = importance.to(device=w.device, dtype=torch.float32).contiguous()
        assert importance.numel() == K
    n = R * (K // group)
    mn = torch.empty((R, K // group), dtype=w.dtype, device=w.device)
    mx = torch.empty_like(mn)
    ws = _workspace(w.device, _lib.lib().llmc_mse_workspace_bytes(n))
    with torch.cuda.device(w.device):
        rc = _lib.lib().llmc_imatrix_observe_groups(
            w.data_ptr(), _dt(w), R, K, w.stride(0), group, fmt, bits, 1 if symmetric else 0, scale_mode, steps,
            float(grid), int(patience), float(norm), float(expand), _ptr(importance), mn.data_ptr(), mx.data_ptr(),
            ws.data_ptr(), ws.numel(), _stream(w))
    _lib.check(rc, "llmc_imatrix_observe_groups")
    return mn, mx


def mse_observe_strided(x, n0: int, n1: int, group: int, s0: int, s1: int, fmt: int, bits: int, symmetric: bool,
                        scale_mode: int = SCALE_PLAIN, maxshrink=0.20, patience=5, grid=100.0, norm=2.4, expand=1.0):
    _require_gpu(x)
    steps, grid, patience, norm, expand = _mse_common(maxshrink, grid, patience, norm, expand)
    mn = torch.empty((n1,), dtype=x.dtype, device=x.device)
    mx = torch.empty_like(mn)
    ws = _workspace(x.device, _lib.lib().llmc_mse_workspace_bytes(n1))
    with torch.cuda.device(x.device):
        rc = _lib.lib().llmc_mse_observe_strided(
            x.data_ptr(), _dt(x), n0, n1, group, s0, s1, fmt, bits, 1 if symmetric else 0, scale_mode, steps, grid,
            patience, norm, expand, mn.data_ptr(), mx.data_ptr(), ws.data_ptr(), ws.numel(), _stream(x))
    _lib.check(rc, "llmc_mse_observe_strided")
    return mn, mx


def mse_observe_blocks(w, bh: int, bw: int, fmt: int, bits: int, symmetric: bool, scale_mode: int = SCALE_PLAIN,
                       maxshrink=0.20, patience=5, grid=100.0, norm=2.4, expand=1.0):
    _require_gpu(w)
    assert w.ndim == 2 and w.stride(1) == 1
    R, K = w.shape
    steps, grid, patience, norm, expand = _mse_common(maxshrink, grid, patience, norm, expand)
    shape = ((R + bh - 1) // bh, (K + bw - 1) // bw)
    mn = torch.empty(shape, dtype=w.dtype, device=w.device)
    mx = torch.empty_like(mn)
    ws = _workspace(w.device, _lib.lib().llmc_mse_workspace_bytes(shape[0] * shape[1]))
    with torch.cuda.device(w.device):
        rc = _lib.lib().llmc_mse_observe_blocks(
            w.data_ptr(), _dt(w), R, K, w.stride(0), bh, bw, fmt, bits, 1 if symmetric else 0, scale_mode, steps,
            grid, patience, norm, expand, mn.data_ptr(), mx.data_ptr(), ws.data_ptr(), ws.numel(), _stream(w))
    _lib.check(rc, "llmc_mse_observe_blocks")
    return mn, mx


def _imatrix_steps(maxshrink, grid):
    steps = max(1, int(maxshrink * grid)) + 1
    if steps > 256:
        raise ValueError(f"imatrix search: {steps} candidates exceed the 256 this build records")
    return steps


def imatrix_observe_strided(x, n0: int, n1: int, group: int, s0: int, s1: int, fmt: int, bits: int, symmetric: bool,
                            scale_mode: int = SCALE_PLAIN, maxshrink=0.95, patience=5, grid=20, norm=3.0, expand=1.0):
    """The uniform fp32-error search on an (n0, n1, group) strided view -> (min, max) [n1]."""
    _require_gpu(x)
    mn = torch.empty((n1,), dtype=x.dtype, device=x.device)
    mx = torch.empty_like(mn)
    ws = _workspace(x.device, _lib.lib().llmc_mse_workspace_bytes(n1))
    with torch.cuda.device(x.device):
        rc = _lib.lib().llmc_imatrix_observe_strided(
            x.data_ptr(), _dt(x), n0, n1, group, s0, s1, fmt, bits, 1 if symmetric else 0, scale_mode,
            _imatrix_steps(maxshrink, grid), float(grid), int(patience), float(norm), float(expand), mn.data_ptr(),
            mx.data_ptr(), ws.data_ptr(), ws.numel(), _stream(x))
    _lib.check(rc, "llmc_imatrix_observe_strided")
    return mn, mx


def imatrix_observe_blocks(w, bh: int, bw: int, fmt: int, bits: int, symmetric: bool, scale_mode: int = SCALE_PLAIN,
                           maxshrink=0.95, patience=5, grid=20, norm=3.0, expand=1.0):
    """The uniform fp32-error search on bh x bw blocks of w [R,K] -> (min, max) [ceil(R/bh), ceil(K/bw)]."""
    _require_gpu(w)
    assert w.ndim == 2 and w.stride(1) == 1
    R, K = w.shape
    shape = ((R + bh - 1) // bh, (K + bw - 1) // bw)
    mn = torch.empty(shape, dtype=w.dtype, device=w.device)
    mx = torch.empty_like(mn)
    ws = _workspace(w.device, _lib.lib().llmc_mse_workspace_bytes(shape[0] * shape[1]))
    with torch.cuda.device(w.device):
        rc = _lib.lib().llmc_imatrix_observe_blocks(
            w.data_ptr(), _dt(w), R, K, w.stride(0), bh, bw, fmt, bits, 1 if symmetric else 0, scale_mode,
            _imatrix_steps(maxshrink, grid), float(grid), int(patience), float(norm), float(expand), mn.data_ptr(),
            mx.data_ptr(), ws.data_ptr(), ws.numel(), _stream(w))
    _lib.check(rc, "llmc_imatrix_observe_blocks")
    return mn, mx


SGEMM_C_LOWER, SGEMM_A_LOWER_TRI, SGEMM_B_LOWER_TRI, SGEMM_FP32_MFMA = 1, 2, 4, 8


def sgemm_(C: torch.Tensor, A: torch.Tensor, B: torch.Tensor, alpha: float = 1.0, beta: float = 0.0,
           trans_b: bool = False, flags: int = 0):
    """C (fp32 [M,N], in place) = alpha * A @ (B.T if trans_b else B) + beta * C on the matrix cores."""
    _require_gpu(C, A, B)
    for t in (C, A, B):
        assert t.dtype == torch.float32 and t.ndim == 2 and t.stride(1) == 1
    M, Kc = A.shape
    N = B.shape[0] if trans_b else B.shape[1]
    assert C.shape == (M, N) and (B.shape[1] if trans_b else B.shape[0]) == Kc
    with torch.cuda.device(C.device):
        rc = _lib.lib().llmc_sgemm(A.data_ptr(), A.stride(0), B.data_ptr(), B.stride(0), C.data_ptr(), C.stride(0),
                                   M, N, Kc, float(alpha), float(beta), 1 if trans_b else 0, int(flags), _stream(C))
    _lib.check(rc, "llmc_sgemm")
    return C


GROUPED_LINEAR_ROWS = 128  # rows of one expert per entry of the tile table


def grouped_linear_tiles(counts, device) -> tuple[torch.Tensor, int]:
    """Tile table of ``grouped_linear`` for experts whose routed rows lie one after the other: per run of at most
    128 rows of one expert ``[expert, first row, rows, 0]`` (int32, on ``device``).  ``counts`` are the experts'
    row counts (host integers); an expert without rows gets no entry."""
    import numpy as np

    counts = np.asarray(counts, dtype=np.int64)
    per = (counts + GROUPED_LINEAR_ROWS - 1) // GROUPED_LINEAR_ROWS
    n = int(per.sum())
    table = np.zeros((max(n, 1), 4), dtype=np.int32)
    if n:
        expert = np.repeat(np.arange(counts.size), per)
        first_tile = np.cumsum(per) - per                       # index of each expert's first entry
        within = np.arange(n) - np.repeat(first_tile, per)      # entry number inside its expert
        start = np.repeat(np.cumsum(counts) - counts, per) + within * GROUPED_LINEAR_ROWS
        rows = np.minimum(np.repeat(counts, per) - within * GROUPED_LINEAR_ROWS, GROUPED_LINEAR_ROWS)
        table[:, 0], table[:, 1], table[:, 2] = expert, start, rows
    return torch.from_numpy(table).to(device), n


def grouped_linear_supported(N: int, K: int, dtype) -> bool:
    return dtype == torch.bfloat16 and N % 128 == 0 and K % 64 == 0


def weight_pointer_table(weights, device) -> torch.Tensor:
    """Device array of the data pointers of ``weights`` (each [N, K] bf16, unit column stride, one common row stride,
    16-byte aligned), in the order ``grouped_linear`` expects: split-major, expert-minor."""
    ptrs = [w.data_ptr() for w in weights]
    if any(p & 15 for p in ptrs):
        raise ValueError("weight_pointer_table: every weight must be 16-byte aligned")
    return torch.tensor(ptrs, dtype=torch.int64, device=device)


def grouped_linear_tiles_all(experts: int, rows: int, device) -> tuple[torch.Tensor, int]:
    """Tile table of ``grouped_linear`` for every expert on all ``rows`` rows of one input: expert e reads the
    rows 0 .. rows - 1 and writes the rows e * rows .. of the output (``out_rows = experts * rows``)."""
    import numpy as np

    per = (rows + GROUPED_LINEAR_ROWS - 1) // GROUPED_LINEAR_ROWS
    n = experts * per
    table = np.zeros((max(n, 1), 4), dtype=np.int32)
    if n:
        start = np.tile(np.arange(per) * GROUPED_LINEAR_ROWS, experts)
        expert = np.repeat(np.arange(experts), per)
        table[:, 0], table[:, 1] = expert, start
        table[:, 2] = np.minimum(rows - start, GROUPED_LINEAR_ROWS)
        table[:, 3] = expert * rows
    return torch.from_numpy(table).to(device), n


def grouped_linear(x: torch.Tensor, pointers: torch.Tensor, experts: int, splits: int, N: int, ldw: int,
                   tiles: torch.Tensor, ntiles: int, out_rows: int | None = None) -> torch.Tensor:
    """y [rows, splits * N] (bf16): the rows the tile table assigns to expert e times the transposed weights
    ``pointers[s * experts + e]`` ([N, K] bf16, row stride ldw) for every split s.  Every row of y must belong to
    a tile (the output is not cleared).  ``out_rows``: rows of y when the table's fourth entries move the tiles'
    results to other rows than their inputs' (default: as many as x has)."""
    _require_gpu(x, pointers, tiles)
    assert x.ndim == 2 and x.dtype == torch.bfloat16 and x.stride(1) == 1
    assert pointers.dtype == torch.int64 and pointers.numel() == experts * splits
    assert tiles.dtype == torch.int32 and tiles.ndim == 2 and tiles.shape[1] == 4 and tiles.shape[0] >= ntiles
    K = x.shape[1]
    y = torch.empty((x.shape[0] if out_rows is None else out_rows, splits * N), dtype=x.dtype, device=x.device)
    if x.shape[0] == 0 or ntiles == 0:
        return y
    with torch.cuda.device(x.device):
        rc = _lib.lib().llmc_grouped_linear(x.data_ptr(), _dt(x), x.stride(0), pointers.data_ptr(), ldw, experts,
                                            splits, y.data_ptr(), y.stride(0), tiles.data_ptr(), ntiles, N, K,
                                            _stream(x))
    _lib.check(rc, "llmc_grouped_linear")
    return y


DIAG_ORDER_MAX_K = 16384


def diag_argsort_desc(Hs) -> torch.Tensor:
    """int64 [n, K]: for each fp32 Hessian of ``Hs`` (one width, one row stride) its column numbers by descending
    diagonal entry, equal entries in column order -- ``torch.argsort(diag, descending=True, stable=True)`` in one
    launch for all of them."""
    import ctypes

    H0 = Hs[0]
    _require_gpu(H0)
    K = H0.shape[0]
    for H in Hs:
        assert H.dtype == torch.float32 and H.shape == (K, K) and H.stride(1) == 1 and H.stride(0) == H0.stride(0)
        assert H.device == H0.device
    out = torch.empty((len(Hs), K), dtype=torch.int64, device=H0.device)
    hp = (ctypes.c_void_p * len(Hs))(*[H.data_ptr() for H in Hs])
    with torch.cuda.device(H0.device):
        rc = _lib.lib().llmc_diag_argsort_desc(hp, H0.stride(0), len(Hs), K, out.data_ptr(), _stream(H0))
    _lib.check(rc, "llmc_diag_argsort_desc")
    return out
