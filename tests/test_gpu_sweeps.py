"""GPU parity sweeps: randomised shapes, dtypes, strategies and value distributions through the product's
seams (Observer registry -> get_qparams -> fake_quantize, and quantize_weight) against the CPU oracle.  Seeds are
fixed, so the cases are the same on every run."""
import random

import pytest
import torch

from oracle import gptq as G
from oracle import observers as O
from oracle import qformat as F

pytestmark = pytest.mark.gpu


def test_rtn_seam_sweep_is_bit_exact():
    """220 random round-to-nearest cases (int 2-8 bit group / channel / tensor / block, symmetric and not, FP8,
    NVFP4, MXFP4
    bf16 / f16 / f32 weights
    zero rows, outliers, tiny and large magnitudes): scales, zero points
    and fake-quantised weights equal the oracle's bit for bit."""
    from llmcompressor_amd.observers import Observer
    from llmcompressor_amd.quantization import QuantizationArgs, fake_quantize

    random.seed(0)
    torch.manual_seed(0)

    def same(a, b):
        a, b = a.cpu(), b.cpu()
        if a.dtype == torch.uint8 or b.dtype == torch.uint8:
            return a.shape == b.shape and torch.equal(a.view(torch.uint8) if a.dtype != torch.uint8 else a, b.view(torch.uint8) if b.dtype != torch.uint8 else b)
        return a.reshape(-1).shape == b.reshape(-1).shape and torch.equal(a.float().reshape(-1).nan_to_num(7e7), b.float().reshape(-1).nan_to_num(7e7))
    bad = 0
    n = 0
    for trial in range(220):
        dtype = random.choice([torch.bfloat16, torch.bfloat16, torch.float16, torch.float32])
        kind = random.choice(["int_group", "int_channel", "int_tensor", "int_block", "fp8_channel", "fp8_tensor", "fp8_block", "nvfp4", "mxfp4", "int_group_asym", "int_channel_asym", "int_tensor_asym"])
        R = random.choice([1, 3, 8, 33, 64, 100, 256])
        g = random.choice([8, 16, 32, 64, 128])
        K = g * random.choice([1, 2, 3, 5, 8])
        bits = random.choice([2, 3, 4, 5, 6, 8])
        spec = dict(num_bits=bits)
        if kind.startswith("int_group"): spec.update(strategy="group", group_size=g)
        elif kind.startswith("int_channel"): spec.update(strategy="channel")
        elif kind.startswith("int_tensor"): spec.update(strategy="tensor")
        elif kind == "int_block": spec.update(strategy="block", block_structure=[random.choice([2, 16, 128]), random.choice([8, 64, 128])])
        elif kind == "fp8_channel": spec.update(num_bits=8, type="float", strategy="channel")
        elif kind == "fp8_tensor": spec.update(num_bits=8, type="float", strategy="tensor")
        elif kind == "fp8_block": spec.update(num_bits=8, type="float", strategy="block", block_structure=[random.choice([16, 128]), random.choice([32, 128])])
        elif kind == "nvfp4":
            spec.update(num_bits=4, type="float", strategy="tensor_group", group_size=16, scale_dtype="float8_e4m3fn")
            K = 16 * random.choice([1, 3, 8, 20])
        elif kind == "mxfp4":
            spec.update(num_bits=4, type="float", strategy="group", group_size=32, scale_dtype="uint8")
            K = 32 * random.choice([1, 3, 8])
            dtype = torch.bfloat16
        if kind.endswith("asym"): spec["symmetric"] = False
        dist = random.choice(["normal", "small", "large", "zeros_rows", "positive", "outliers"])
        w = torch.randn(R, K)
        if dist == "small": w *= 1e-4
        if dist == "large": w *= 300
        if dist == "positive": w = w.abs() + 0.1
        if dist == "zeros_rows": w[::2] = 0
        if dist == "outliers": w[torch.rand(R, K) < 0.01] *= 50
        w = (w * 0.05).to(dtype)
        ospec = dict(spec)
        if "scale_dtype" in ospec: ospec["scale_dtype"] = getattr(torch, ospec["scale_dtype"])
        try:
            oargs = F.QArgs(**ospec)
            oobs = O.Observer("memoryless_minmax", "weight", oargs)
            oobs(w)
            oq = oobs.get_qparams()
            ofq = F.fake_quantize(w, oq["scale"], oq["zero_point"], oargs, global_scale=oq["global_scale"])
        except Exception as e:
            print("oracle error", kind, spec, type(e).__name__, str(e)[:100])
            continue
        n += 1
        try:
            args = QuantizationArgs(**spec)
            gobs = Observer.load_from_registry("memoryless_minmax", base_name="weight", args=args)
            gobs(w.cuda())
            gq = gobs.get_qparams()
            gfq = fake_quantize(w.cuda(), gq["scale"], gq["zero_point"], args, global_scale=gq["global_scale"])
            es = oq["scale"]
            gsx = gq["scale"]
            if gsx.dtype == torch.uint8: es = (torch.log2(es.float()) + 127).to(torch.uint8)
            ok_s = same(gsx, es)
            ok_z = True if args.symmetric else same(gq["zero_point"].float(), oq["zero_point"].float())
            ok_f = same(gfq, ofq.to(dtype))
            if not (ok_s and ok_z and ok_f):
                bad += 1
                print("MISMATCH", kind, spec, dtype, (R, K), dist, "scale", ok_s, "zp", ok_z, "fq", ok_f, flush=True)
        except Exception as e:
            bad += 1
            print("PRODUCT ERROR", kind, spec, dtype, (R, K), dist, type(e).__name__, str(e)[:160], flush=True)
    assert n >= 200 and bad == 0



def test_gptq_seam_sweep_matches_oracle():
    """70 random GPTQ cases through quantize_weight (all strategies and formats of the column loop, activation
    ordering none / weight / group, block sizes 32 / 48 / 128, dead columns, rank-deficient Hessians, two
    dampening fractions): at least 99.9 % identical weights in every case."""
    from llmcompressor_amd.modifiers.gptq import quantize_weight
    from llmcompressor_amd.modifiers.quantization.calibration import initialize_observer, observe
    from llmcompressor_amd.quantization import QuantizationArgs, QuantizationScheme

    random.seed(1)
    torch.manual_seed(1)
    worst = 1.0
    bad = 0
    for trial in range(70):
        kind = random.choice(["int_group", "int_group_asym", "int_channel", "int_tensor", "int_block", "fp8_channel", "nvfp4", "mxfp4"])
        actorder = random.choice([None, "weight", "weight", "group"])
        g = random.choice([16, 32, 64, 128])
        K = g * random.choice([1, 2, 3, 5])
        R = random.choice([1, 7, 32, 100, 130])
        bits = random.choice([3, 4, 8])
        spec = dict(num_bits=bits)
        if kind.startswith("int_group"): spec.update(strategy="group", group_size=g)
        elif kind == "int_channel": spec.update(strategy="channel")
        elif kind == "int_tensor": spec.update(strategy="tensor")
        elif kind == "int_block": spec.update(strategy="block", block_structure=[random.choice([2, 16]), g])
        elif kind == "fp8_channel": spec.update(num_bits=8, type="float", strategy="channel")
        elif kind == "nvfp4":
            spec.update(num_bits=4, type="float", strategy="tensor_group", group_size=16, scale_dtype="float8_e4m3fn")
            K = 16 * random.choice([2, 5, 12])
        elif kind == "mxfp4":
            spec.update(num_bits=4, type="float", strategy="group", group_size=32, scale_dtype="uint8")
            K = 32 * random.choice([1, 3, 6])
        if kind.endswith("asym"): spec["symmetric"] = False
        if actorder: spec["actorder"] = actorder
        blocksize = random.choice([128, 128, 32, 48])
        T = random.choice([K // 2, 2 * K, 4 * K])
        mix = torch.randn(K, K) * 0.3 + torch.eye(K)
        x = (torch.randn(T, K) @ mix).bfloat16()
        ndead = random.choice([0, 0, 1, 3])
        if ndead: x[:, torch.randperm(K)[:ndead]] = 0
        w0 = (torch.randn(R, K) * 0.05).bfloat16()
        ospec = dict(spec)
        if "scale_dtype" in ospec: ospec["scale_dtype"] = getattr(torch, ospec["scale_dtype"])
        oargs = F.QArgs(**ospec)
        oobs = O.Observer("memoryless_minmax", "weight", oargs)
        oobs(w0)
        Ho, n = G.make_empty_hessian(K), torch.zeros(())
        Ho, n = G.accumulate_hessian(x.unsqueeze(0), Ho, n)
        Hn = (Ho / n).clone()
        percdamp = random.choice([0.01, 0.1])
        _, exp, info = G.quantize_weight(w0, oobs, oargs, Hn.clone(), blocksize=blocksize, percdamp=percdamp)
        module = torch.nn.Linear(K, R, bias=False).cuda().to(torch.bfloat16)
        module.weight.data = w0.cuda()
        args = QuantizationArgs(**spec)
        module.quantization_scheme = QuantizationScheme(targets=["Linear"], weights=args)
        initialize_observer(module, "weight")
        observe(module, "weight")
        try:
            loss, q = quantize_weight(module=module, quant_args=args, hessian=Hn.clone().cuda(), blocksize=blocksize, percdamp=percdamp)
        except Exception as e:
            bad += 1
            print("PRODUCT ERROR", spec, (R, K, T), type(e).__name__, str(e)[:200], flush=True)
            continue
        agree = (q["weight"].cpu() == exp["weight"]).float().mean().item()
        worst = min(worst, agree)
        if agree < 0.999 or not info["ok"]:
            bad += (agree < 0.999)
            print(f"agree {agree:.4f} ok={info['ok']}", spec, (R, K, T), "blocksize", blocksize, "dead", ndead, "damp", percdamp, flush=True)
    assert bad == 0 and worst >= 0.999



def test_mse_observer_seam_sweep_is_bit_exact():
    """60 random MSE-observer cases from the registry (weights and multi-batch activations; int / FP8 / NVFP4 /
    MXFP4; bf16 / f16 / f32; search settings including the error exponents 2, 3, 0.5 and 1 for which the eager pow
    has closed forms with their own roundings): min / max of every group equal the oracle's."""
    from llmcompressor_amd.observers import Observer
    from llmcompressor_amd.quantization import QuantizationArgs

    random.seed(2)
    torch.manual_seed(2)
    bad = 0
    worst = 1.0
    for trial in range(60):
        dtype = random.choice([torch.bfloat16, torch.bfloat16, torch.float32, torch.float16])
        kind = random.choice(["int_group", "int_channel", "int_tensor", "int_block", "fp8_channel", "nvfp4", "mxfp4", "int_group_asym", "int_tensor_asym", "fp4_tg_noscale"])
        R = random.choice([1, 5, 32, 64])
        g = random.choice([16, 32, 128])
        K = g * random.choice([1, 2, 4])
        bits = random.choice([3, 4, 8])
        spec = dict(num_bits=bits)
        if kind.startswith("int_group"): spec.update(strategy="group", group_size=g)
        elif kind == "int_channel": spec.update(strategy="channel")
        elif kind.startswith("int_tensor"): spec.update(strategy="tensor")
        elif kind == "int_block": spec.update(strategy="block", block_structure=[random.choice([2, 16]), g])
        elif kind == "fp8_channel": spec.update(num_bits=8, type="float", strategy="channel")
        elif kind == "nvfp4":
            spec.update(num_bits=4, type="float", strategy="tensor_group", group_size=16, scale_dtype="float8_e4m3fn")
            K = 16 * random.choice([2, 8])
        elif kind == "fp4_tg_noscale":
            spec.update(num_bits=4, type="float", strategy="tensor_group", group_size=16)
            K = 16 * random.choice([2, 8])
        elif kind == "mxfp4":
            spec.update(num_bits=4, type="float", strategy="group", group_size=32, scale_dtype="uint8")
            K = 32 * random.choice([1, 4])
            dtype = torch.bfloat16
        if kind.endswith("asym"): spec["symmetric"] = False
        kw = random.choice([{}, {}, dict(maxshrink=0.8, patience=100), dict(norm=2.0), dict(grid=50.0, maxshrink=0.5, patience=3),
                            dict(norm=3.0, patience=1), dict(norm=0.5), dict(norm=1.0, maxshrink=0.4)])
        base = random.choice(["weight", "input"])
        name = "memoryless_mse" if base == "weight" else random.choice(["mse", "memoryless_mse"])
        if base == "input" and spec.get("strategy") in ("channel", "block"): base, name = "weight", "memoryless_mse"
        spec["observer_kwargs"] = dict(kw)
        ospec = dict(spec)
        if "scale_dtype" in ospec: ospec["scale_dtype"] = getattr(torch, ospec["scale_dtype"])
        oobs = O.Observer(name, base, F.QArgs(**ospec))
        gobs = Observer.load_from_registry(name, base_name=base, args=QuantizationArgs(**spec))
        ok = True
        frac = 1.0
        for step in range(1 if base == "weight" else 3):
            w = torch.randn(R, K) * random.choice([0.02, 1.0, 30.0])
            w[torch.rand(R, K) < 0.02] *= 8
            w = w.to(dtype)
            if base == "input": w = w.reshape(1, R, K)
            oobs(w)
            gobs(w.cuda())
            a, b = gobs.min_vals.cpu().float().reshape(-1), oobs.min_vals.float().reshape(-1)
            c, d = gobs.max_vals.cpu().float().reshape(-1), oobs.max_vals.float().reshape(-1)
            frac = min(frac, ((a == b) & (c == d)).float().mean().item())
        worst = min(worst, frac)
        if frac < 1.0:
            bad += 1
            print(f"identical groups {frac:.4f}", name, base, spec, dtype, (R, K), flush=True)
    assert bad == 0 and worst == 1.0



def test_dynamic_per_token_seam_sweep_is_bit_exact():
    """60 random dynamic per-token cases through forward_quantize (FP8 and int8 symmetric: the fused kernel;
    int8 asymmetric and int4: row min-max, qparams and fake-quant kernels; zero rows, outliers, 1 to 4096
    features): equal to the oracle bit for bit."""
    from llmcompressor_amd.quantization import QuantizationArgs, forward_quantize

    random.seed(5)
    torch.manual_seed(5)
    bad = 0
    # 1. dynamic per-token through forward_quantize vs oracle
    for trial in range(60):
        dtype = random.choice([torch.bfloat16, torch.float16])
        spec = random.choice([dict(num_bits=8, type="float", strategy="token", dynamic=True),
                              dict(num_bits=8, strategy="token", dynamic=True),
                              dict(num_bits=8, strategy="token", dynamic=True, symmetric=False),
                              dict(num_bits=4, strategy="token", dynamic=True)])
        B, T, K = random.choice([1, 2, 3]), random.choice([1, 7, 64, 130]), random.choice([8, 100, 512, 1000, 4096])
        x = torch.randn(B, T, K) * random.choice([0.01, 1.0, 100.0])
        x[torch.rand(B, T, K) < 0.01] *= 20
        if random.random() < 0.3: x[0, 0] = 0
        x = x.to(dtype)
        want, _ = F.forward_quantize_dynamic(x, F.QArgs(**spec))
        lin = torch.nn.Linear(K, 8, bias=False).cuda().to(dtype)
        args = QuantizationArgs(**spec)
        got = forward_quantize(lin, x.cuda(), "input", args).cpu()
        if not torch.equal(got.float().nan_to_num(9e9), want.float().nan_to_num(9e9)):
            bad += 1
            print("dynamic token mismatch", spec, dtype, (B, T, K), (got.float() != want.float()).float().mean().item(), flush=True)

    assert bad == 0


def test_checkpoint_tensor_round_trip_sweep():
    """60 random weight schemes (int 3/4/8 bit group / channel / tensor / block, with and without zero points,
    FP8, NVFP4, MXFP4) through observer, fake-quant, compress_module and decompress_weight: the decompressed
    weight equals the fake-quantised one."""
    from llmcompressor_amd.compressors import compress_module, decompress_weight, infer_format
    from llmcompressor_amd.modifiers.quantization.calibration import initialize_observer, observe, update_qparams
    from llmcompressor_amd.quantization import (QuantizationArgs, QuantizationScheme, fake_quantize,
                                                initialize_module_for_quantization)

    random.seed(6)
    torch.manual_seed(6)
    bad = 0
    # 2. compress_module -> decompress round trip equals fake-quantised weight; packed bytes equal oracle pack
    for trial in range(60):
        dtype = random.choice([torch.bfloat16, torch.float16])
        kind = random.choice(["w4g", "w4g_asym", "w8c", "w8t_asym", "fp8c", "nvfp4", "mxfp4", "w4c", "w3g", "w4block"])
        g = random.choice([16, 32, 128])
        K = g * random.choice([1, 2, 5])
        R = random.choice([1, 8, 33, 128])
        spec = {"w4g": dict(num_bits=4, strategy="group", group_size=g), "w4g_asym": dict(num_bits=4, strategy="group", group_size=g, symmetric=False),
                "w8c": dict(num_bits=8, strategy="channel"), "w8t_asym": dict(num_bits=8, strategy="tensor", symmetric=False),
                "fp8c": dict(num_bits=8, type="float", strategy="channel"), "w4c": dict(num_bits=4, strategy="channel"),
                "w3g": dict(num_bits=3, strategy="group", group_size=g), "w4block": dict(num_bits=4, strategy="block", block_structure=[8, g]),
                "nvfp4": dict(num_bits=4, type="float", strategy="tensor_group", group_size=16, scale_dtype="float8_e4m3fn"),
                "mxfp4": dict(num_bits=4, type="float", strategy="group", group_size=32, scale_dtype="uint8")}[kind]
        if kind == "nvfp4": K = 16 * random.choice([2, 6])
        if kind == "mxfp4":
            K = 32 * random.choice([1, 4])
            dtype = torch.bfloat16
        if kind == "w3g":
            g = 32
            spec = dict(num_bits=3, strategy="group", group_size=32)
            K = 32 * random.choice([1, 3])
        w = (torch.randn(R, K) * 0.05).to(dtype)
        w[torch.rand(R, K) < 0.02] *= 10
        lin = torch.nn.Linear(K, R, bias=False).cuda().to(dtype)
        lin.weight.data = w.cuda()
        args = QuantizationArgs(**spec)
        scheme = QuantizationScheme(targets=["Linear"], weights=args)
        try:
            initialize_module_for_quantization(lin, scheme)
            initialize_observer(lin, "weight")
            observe(lin, "weight")
            update_qparams(lin, "weight")
            fq = fake_quantize(lin.weight.data, lin.weight_scale.data, getattr(lin, "weight_zero_point", None), args, global_scale=getattr(lin, "weight_global_scale", None))
            lin.weight.data = fq
            fmt = infer_format(scheme)
            tensors = {k: v.cpu() for k, v in compress_module(lin).items()}
            deq = decompress_weight(tensors, args, fmt, dtype=dtype)
            differ = (deq.float() != fq.cpu().float()).float().mean().item()
            # 8-bit codes of 16-bit weights: re-quantising a fake-quantised value divides in the 16-bit dtype, whose
            # spacing near 127 is 0.5, so a few codes move by one (the reference's arithmetic does the same)
            if differ > (1e-3 if args.num_bits == 8 and args.type == "int" else 0.0):
                bad += 1
                print("round trip mismatch", kind, spec, dtype, (R, K), fmt, differ, flush=True)
        except Exception as e:
            bad += 1
            print("ERROR", kind, spec, dtype, (R, K), type(e).__name__, str(e)[:200], flush=True)

    assert bad == 0
