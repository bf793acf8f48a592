"""Host-side mirror of the reference interface: argument resolution, recipes, hooks, registry, C ABI surface.

Runs without a GPU.  Cases follow the reference's own unit tests (cited per test)."""
import ctypes
import os
import re
from contextlib import nullcontext

import pytest
import torch

from llmcompressor_amd import _lib
from llmcompressor_amd.compressors import CompressionFormat, infer_format
from llmcompressor_amd.modifiers.gptq import GPTQModifier
from llmcompressor_amd.modifiers.quantization import QuantizationModifier
from llmcompressor_amd.modifiers.utils.hooks import HooksMixin
from llmcompressor_amd.observers import Observer, flatten_for_calibration
from llmcompressor_amd.quantization import (
    QuantizationArgs,
    QuantizationScheme,
    initialize_module_for_quantization,
    preset_name_to_scheme,
)
from llmcompressor_amd.recipe import Recipe

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_c_abi_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "llmc_amd.h")).read()
    declared = set(re.findall(r"\b(llmc_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 15
    lib = ctypes.CDLL(_lib.LIB_PATH)
    missing = [n for n in sorted(declared) if not hasattr(lib, n)]
    assert not missing, missing
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    assert lib.llmc_version() >= 1


def test_ops_refuse_cpu_tensors_instead_of_falling_back():
    from llmcompressor_amd import ops

    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.hessian_accumulate_(torch.zeros(8, 8), torch.zeros(4, 8, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.minmax_groups(torch.zeros(4, 8), 8)


def _q_config_kwargs(config_0, config_1):
    def grp(actorder):
        return dict(targets=["Linear"], input_activations=dict(num_bits=8, symmetric=False, strategy="tensor"),
                    weights=dict(num_bits=4, symmetric=True, strategy="group", group_size=128, actorder=actorder))

    return dict(config_groups=dict(group_0=grp(config_0), group_1=grp(config_1)))


@pytest.mark.parametrize(
    "has_actorder,actorder,config_0,config_1,expected_0,expected_1",
    [
        (False, "N/A", None, None, "static", "static"),
        (True, "static", None, None, "static", "static"),
        (True, "group", None, None, "group", "group"),
        (True, None, None, None, None, None),
        (True, "group", None, "group", "group", "group"),
        (True, "group", "group", None, "group", "group"),
        (True, "static", None, "group", "error", "error"),
        (True, "static", "group", None, "error", "error"),
        (True, "group", None, "static", "error", "error"),
        (True, "group", "static", None, "error", "error"),
        (True, None, "static", None, "error", "error"),
        (False, "N/A", None, "static", "static", "static"),
        (False, "N/A", "static", None, "static", "static"),
        (False, "N/A", "static", "static", "static", "static"),
        (False, "N/A", None, "group", "static", "group"),
        (False, "N/A", "group", None, "group", "static"),
        (False, "N/A", "group", "group", "group", "group"),
    ],
)
def test_actorder_resolution(has_actorder, actorder, config_0, config_1, expected_0, expected_1):
    # reference: tests/llmcompressor/modifiers/gptq/test_base.py:60-113
    kwargs = _q_config_kwargs(config_0, config_1)
    with pytest.raises(ValueError) if expected_0 == "error" else nullcontext():
        modifier = GPTQModifier(**kwargs, actorder=actorder) if has_actorder else GPTQModifier(**kwargs)
        resolved = modifier.resolve_quantization_config()
    if expected_0 != "error":
        assert resolved.config_groups["group_0"].input_activations.actorder is None
        assert resolved.config_groups["group_0"].weights.actorder == expected_0
        assert resolved.config_groups["group_1"].input_activations.actorder is None
        assert resolved.config_groups["group_1"].weights.actorder == expected_1


def test_block_strategy_parsing_and_group_fallback():
    m = GPTQModifier(config_groups=dict(group_block=dict(
        targets=["Linear"], weights=dict(num_bits=8, symmetric=True, strategy="block", block_structure=[128, 128]))))
    w = m.resolve_quantization_config().config_groups["group_block"].weights
    assert w.strategy == "block" and w.block_structure == [128, 128]
    # actorder=group on an ungrouped strategy falls back to None
    m = GPTQModifier(actorder="group", config_groups=dict(g=dict(targets=["Linear"], weights=dict(strategy="channel"))))
    assert m.resolve_quantization_config().config_groups["g"].weights.actorder is None


def test_scheme_targets_and_serialisation():
    m = GPTQModifier(targets="Linear", scheme="W4A16", ignore=["lm_head"])
    cfg = m.resolve_quantization_config()
    w = cfg.config_groups["group_0"].weights
    assert (w.num_bits, w.group_size, w.symmetric, str(w.strategy.value)) == (4, 128, True, "group")
    assert m.resolved_targets == {"Linear"}
    assert m.model_dump()["actorder"] == "static"
    assert GPTQModifier(actorder=None).model_dump()["actorder"] is None
    with pytest.raises(ValueError):
        GPTQModifier(scheme="NOT_A_SCHEME")
    with pytest.raises(ValueError):
        GPTQModifier(scheme="W4A16", config_groups={"g": dict(targets=["Linear"])}).resolve_quantization_config()
    with pytest.raises(Exception):
        GPTQModifier(not_a_field=1)  # extra="forbid"
    assert GPTQModifier(scheme="W4A16").requires_calibration_data
    assert not QuantizationModifier(scheme="FP8_DYNAMIC").requires_calibration_data
    assert QuantizationModifier(scheme="FP8").requires_calibration_data  # static activation scales


def test_observer_overrides():
    m = QuantizationModifier(scheme="W4A16", weight_observer="mse")
    assert m.resolved_config.config_groups["group_0"].weights.observer == "mse"
    with pytest.raises(ValueError):
        QuantizationModifier(scheme="W4A16", weight_observer="mse", observer={"weights": "minmax"}).resolved_config


def test_recipe_round_trip_and_factory():
    # reference: tests/llmcompressor/recipe/test_recipe.py:21-72
    text = """
    test_stage:
      quant_modifiers:
        GPTQModifier:
          block_size: 64
          dampening_frac: 0.001
          actorder: static
          config_groups:
            group_0:
              targets: [Linear]
              weights: {num_bits: 4, type: int, symmetric: true, strategy: group, group_size: 128}
        QuantizationModifier:
          targets: [Linear]
          scheme: FP8_DYNAMIC
    """
    r = Recipe.create_instance(text)
    assert [type(m).__name__ for m in r.modifiers] == ["GPTQModifier", "QuantizationModifier"]
    assert r.modifiers[0].block_size == 64 and r.modifiers[0].group == "quant"
    r2 = Recipe.create_instance(r.yaml())
    assert r2.dict() == r.dict()
    r3 = Recipe.create_instance([GPTQModifier(scheme="W4A16")])
    assert Recipe.create_instance(r3.yaml()).modifiers[0].scheme == "W4A16"
    with pytest.raises(ValueError):
        Recipe.create_instance("test_stage:\n  x_modifiers:\n    NoSuchModifier: {}\n")


class _Dummy(HooksMixin):
    pass


def test_hooks_register_remove_disable_keep():
    # reference: tests/llmcompressor/modifiers/utils/test_hooks.py:40-120
    lin_a, lin_b = torch.nn.Linear(4, 4), torch.nn.Linear(4, 4)
    mod_a, mod_b = _Dummy(), _Dummy()
    calls = []
    ha = mod_a.register_hook(lin_a, lambda *a: calls.append("a"), "forward")
    hb = mod_b.register_hook(lin_b, lambda *a: calls.append("b"), "forward_pre")
    x = torch.zeros(1, 4)
    lin_a(x), lin_b(x)
    assert calls == ["a", "b"]
    with HooksMixin.disable_hooks():
        lin_a(x), lin_b(x)
    assert calls == ["a", "b"]
    with HooksMixin.disable_hooks(keep={hb}):
        lin_a(x), lin_b(x)
    assert calls == ["a", "b", "b"]
    mod_a.remove_hooks()
    lin_a(x), lin_b(x)
    assert calls == ["a", "b", "b", "b"]
    mod_b.remove_hooks({hb})
    lin_b(x)
    assert calls == ["a", "b", "b", "b"]
    assert ha not in mod_a._hooks


@pytest.mark.parametrize(
    "args",
    [
        QuantizationArgs(strategy="tensor"),
        QuantizationArgs(strategy="channel"),
        QuantizationArgs(strategy="group", group_size=4),
        QuantizationArgs(strategy="tensor_group", group_size=4),
        QuantizationArgs(strategy="block", block_structure=[5, 4]),
        QuantizationArgs(strategy="block", block_structure=[3, 3]),
    ],
)
def test_flatten_for_calibration_weights_matches_param_shapes(args):
    # reference: tests/llmcompressor/observers/test_helpers.py:37-59
    module = torch.nn.Linear(8, 10)
    initialize_module_for_quantization(module, QuantizationScheme(targets=[], weights=args))
    flat = flatten_for_calibration(module.weight, "weight", args)
    assert flat.shape[1:-1] == module.weight_scale.shape
    assert flat.shape[1:-1] == module.weight_zero_point.shape


@pytest.mark.parametrize("args", [QuantizationArgs(strategy="tensor"), QuantizationArgs(strategy="tensor_group", group_size=4)])
def test_flatten_for_calibration_input(args):
    module = torch.nn.Linear(8, 10)
    initialize_module_for_quantization(module, QuantizationScheme(targets=[], input_activations=args))
    flat = flatten_for_calibration(torch.empty((3, 5, 8)), "input", args)
    assert flat.shape[1:-1] == module.input_scale.shape


def test_flatten_errors_match_reference_messages():
    w = torch.empty(4, 8)
    with pytest.raises(ValueError, match="Token quantization cannot be applied to weights"):
        flatten_for_calibration(w, "weight", QuantizationArgs(strategy="token"))
    with pytest.raises(ValueError, match="Channel quantization cannot be applied to activations"):
        flatten_for_calibration(w, "input", QuantizationArgs(strategy="channel"))
    with pytest.raises(ValueError, match="Unknown quantization base name"):
        flatten_for_calibration(w, "bogus", QuantizationArgs())


def test_observer_registry_names():
    for name, cls in [("memoryless_minmax", "MemorylessMinMaxObserver"), ("static_minmax", "StaticMinMaxObserver"),
                      ("minmax", "MinMaxObserver"), ("memoryless_mse", "MemorylessMSEObserver"),
                      ("mse", "MovingAverageMSEObserver"), ("nvfp4_expanded_mse", "NVFP4ExpandedMSEObserver")]:
        obs = Observer.load_from_registry(name, base_name="weight", args=QuantizationArgs())
        assert type(obs).__name__ == cls
    with pytest.raises(AssertionError, match="No statistics available"):
        Observer.load_from_registry("minmax", base_name="weight", args=QuantizationArgs()).get_qparams()
    with pytest.raises(ValueError):
        Observer.load_from_registry("mse", base_name="weight", args=QuantizationArgs(), expand=0.5)


def test_group_size_validation_error():
    from llmcompressor_amd.core import State

    model = torch.nn.Sequential(torch.nn.Linear(200, 16))
    m = QuantizationModifier(scheme="W4A16")
    with pytest.raises(ValueError, match="not divisible by group_size"):
        m.on_initialize(State(model=model))
    QuantizationModifier(scheme="W4A16", bypass_divisibility_checks=True).on_initialize(State(model=torch.nn.Sequential(torch.nn.Linear(200, 16))))


@pytest.mark.parametrize(
    "preset,fmt",
    [("W8A8", CompressionFormat.int_quantized), ("W4A16", CompressionFormat.pack_quantized),
     ("W8A16", CompressionFormat.pack_quantized), ("FP8", CompressionFormat.float_quantized),
     ("FP8_DYNAMIC", CompressionFormat.float_quantized), ("NVFP4A16", CompressionFormat.nvfp4_pack_quantized),
     ("NVFP4", CompressionFormat.nvfp4_pack_quantized), ("MXFP4A16", CompressionFormat.mxfp4_pack_quantized)],
)
def test_format_inference(preset, fmt):
    # reference: tests/llmcompressor/transformers/compression/test_compress_tensor_utils.py:289-325
    assert infer_format(preset_name_to_scheme(preset, ["Linear"])) == fmt
    w8a16_float = QuantizationScheme(targets=["Linear"], weights=QuantizationArgs(num_bits=8, type="float"))
    assert infer_format(w8a16_float) == CompressionFormat.naive_quantized


def test_quantization_format_override():
    """``save_pretrained(..., quantization_format=...)``: the reference's W4AFP8 example stores its int4 codes
    packed on request (examples/quantization_w4a8_fp8/llama3_example.py:76-80); a format that cannot hold a
    scheme's codes is refused before anything is written."""
    from llmcompressor_amd.compressors import resolve_format

    w4afp8 = preset_name_to_scheme("W4AFP8", ["Linear"])
    assert w4afp8.weights.num_bits == 4 and w4afp8.weights.group_size == 128
    assert w4afp8.input_activations.type.value == "float" and w4afp8.input_activations.dynamic is True
    assert resolve_format(w4afp8) == CompressionFormat.int_quantized
    assert resolve_format(w4afp8, "pack-quantized") == CompressionFormat.pack_quantized
    assert resolve_format(w4afp8, "pack_quantized") == CompressionFormat.pack_quantized

    class _Enum:  # compressed_tensors.QuantizationFormat members carry the string in ``value``
        value = "pack-quantized"

    assert resolve_format(w4afp8, _Enum) == CompressionFormat.pack_quantized
    assert resolve_format(w4afp8, "dense") == CompressionFormat.dense
    with pytest.raises(ValueError, match="cannot hold"):
        resolve_format(w4afp8, "float-quantized")
    with pytest.raises(ValueError, match="cannot hold"):
        resolve_format(preset_name_to_scheme("FP8", ["Linear"]), "pack-quantized")
    with pytest.raises(ValueError, match="cannot hold"):
        resolve_format(preset_name_to_scheme("NVFP4A16", ["Linear"]), "mxfp4-pack-quantized")
    with pytest.raises(ValueError, match="unknown quantization_format"):
        resolve_format(w4afp8, "marlin-24")
    assert resolve_format(preset_name_to_scheme("W8A8", ["Linear"]), "naive-quantized") == "naive-quantized"


def test_oneshot_wraps_save_pretrained(tmp_path):
    """After ``oneshot`` the model's own ``save_pretrained`` takes ``save_compressed`` / ``quantization_format``
    (reference: entrypoints/utils.py:96, compressed_tensors_utils.py:86-190); wrapping twice changes nothing and
    an un-quantised model is written as transformers writes it, with no ``quantization_config``."""
    import json

    from safetensors import safe_open
    from transformers import LlamaConfig, LlamaForCausalLM

    import llmcompressor_amd
    from llmcompressor.transformers.compression.compressed_tensors_utils import modify_save_pretrained

    model = LlamaForCausalLM(LlamaConfig(vocab_size=64, hidden_size=32, intermediate_size=64, num_hidden_layers=1,
                                         num_attention_heads=2, num_key_value_heads=2))
    llmcompressor_amd.oneshot(model=model, recipe=None)
    first = model.save_pretrained
    assert getattr(first, "_overridden", False)
    modify_save_pretrained(model)
    assert model.save_pretrained is first
    model.save_pretrained(str(tmp_path / "a"), save_compressed=True)
    model.save_pretrained(str(tmp_path / "b"), save_compressed=False, quantization_format="dense")
    for sub in ("a", "b"):
        with open(tmp_path / sub / "config.json") as f:
            assert "quantization_config" not in json.load(f)
        with safe_open(str(tmp_path / sub / "model.safetensors"), "pt") as f:
            keys = set(f.keys())
        assert "model.layers.0.self_attn.q_proj.weight" in keys and not any("observer" in k for k in keys)
    plain = torch.nn.Linear(4, 4)
    modify_save_pretrained(plain)  # no ``save_pretrained``: left alone
    assert not hasattr(plain, "save_pretrained")


def test_moe_token_routing_counts():
    # reference: tests/llmcompressor/modeling/test_linear_experts.py:12-106 (hidden 16, inter 32, 4 experts, top-2)
    from llmcompressor_amd.modeling import LinearExperts2D, moe_calibration_context

    torch.manual_seed(0)
    E, H, I, T, k = 4, 16, 32, 16, 2
    experts = LinearExperts2D.from_fused(torch.randn(E, 2 * I, H), torch.randn(E, H, I))
    x = torch.randn(T, H)
    idx = torch.stack([torch.arange(T) % E, (torch.arange(T) + 1) % E], dim=1)
    wts = torch.full((T, k), 0.5)
    counts = {}
    for e, ex in enumerate(experts):
        ex.gate_proj.register_forward_hook(lambda m, a, o, e=e: counts.__setitem__(e, a[0].shape[0]))
    out_routed = experts(x, idx, wts)
    assert counts == {0: 8, 1: 8, 2: 8, 3: 8}
    with moe_calibration_context():
        out_all = experts(x, idx, wts)
    assert counts == {0: 16, 1: 16, 2: 16, 3: 16}
    assert torch.allclose(out_routed, out_all, atol=1e-5)
    # an expert without tokens is still called (with an empty batch)
    counts.clear()
    experts(x, torch.zeros(T, k, dtype=torch.long), wts)
    assert counts == {0: 32, 1: 0, 2: 0, 3: 0}  # both top-k slots of every token point at expert 0


def test_model_free_config_and_matching():
    """model_free_ptq host logic: scheme/config validation, ignore rules, first-match-wins targets
    (reference: entrypoints/model_free/validate.py:22-78, process.py:44-60)."""
    from llmcompressor_amd.entrypoints.model_free import _match_tensors_to_schemes, validate_config
    from llmcompressor_amd.quantization import QuantizationArgs, QuantizationConfig, QuantizationScheme

    with pytest.raises(ValueError, match="either `config` or `scheme`"):
        validate_config(None, None, [])
    with pytest.raises(ValueError, match="not both"):
        validate_config(QuantizationConfig(config_groups={}), "FP8_DYNAMIC", [])
    static_act = QuantizationScheme(targets=["Linear"], weights=QuantizationArgs(num_bits=8),
                                    input_activations=QuantizationArgs(num_bits=8, dynamic=False))
    with pytest.raises(ValueError, match="cannot calibrate activations"):
        validate_config(None, static_act, [])
    cfg = validate_config(None, "FP8_DYNAMIC", ["lm_head", "re:.*embed.*"])
    assert list(cfg.config_groups) == ["FP8_DYNAMIC"] and cfg.ignore == ["lm_head", "re:.*embed.*"]
    names = ["model.embed_tokens.weight", "model.layers.0.self_attn.q_proj.weight", "model.layers.0.self_attn.q_proj.bias",
             "model.layers.0.post_attention_layernorm.weight", "model.norm.weight", "lm_head.weight",
             "model.layers.0.mlp.down_proj.weight"]
    got = [m for m, _, _ in _match_tensors_to_schemes(names, cfg)]
    assert got == ["model.layers.0.self_attn.q_proj", "model.layers.0.mlp.down_proj"]
    # two groups: the first that matches a tensor wins
    a = QuantizationScheme(targets=["re:.*q_proj$"], weights=QuantizationArgs(num_bits=4, strategy="group", group_size=32))
    b = QuantizationScheme(targets=["Linear"], weights=QuantizationArgs(num_bits=8, strategy="channel"))
    cfg2 = validate_config(QuantizationConfig(config_groups={"a": a, "b": b}), None, ["lm_head", "model.embed_tokens"])
    got2 = {m: s.weights.num_bits for m, _, s in _match_tensors_to_schemes(names, cfg2)}
    assert got2 == {"model.layers.0.self_attn.q_proj": 4, "model.layers.0.mlp.down_proj": 8}


def test_intermediates_cache_interface():
    """IntermediatesCache (reference: pipelines/cache.py, tests/llmcompressor/pipelines/test_cache.py):
    fetch / update / delete / append / iter / size over nested containers; values stay on their device
    unless an offload device is given."""
    from dataclasses import dataclass

    from llmcompressor_amd.pipelines.cache import IntermediatesCache

    @dataclass
    class Out:
        a: torch.Tensor
        b: object = None

    loader = [{"input_ids": torch.arange(6).view(2, 3), "attention_mask": torch.ones(2, 3)} for _ in range(3)]
    cache = IntermediatesCache.from_dataloader(loader)
    assert len(cache) == 3 and isinstance(cache.batch_intermediates[0], dict)
    got = cache.fetch(0, ["input_ids"])
    assert set(got) == {"input_ids"} and torch.equal(got["input_ids"], loader[0]["input_ids"])
    nested = {"t": (torch.ones(2), [torch.zeros(3), 7, None]), "d": Out(torch.full((2,), 3.0), "x")}
    cache.update(0, {"hidden_states": nested, "logits": torch.randn(2, 3)})
    back = cache.fetch(0)["hidden_states"]
    assert torch.equal(back["t"][0], torch.ones(2)) and back["t"][1][1] == 7 and back["t"][1][2] is None
    assert isinstance(back["d"], Out) and torch.equal(back["d"].a, torch.full((2,), 3.0)) and back["d"].b == "x"
    cache.delete(0, ["hidden_states"])
    assert "hidden_states" not in cache.batch_intermediates[0] and "logits" in cache.batch_intermediates[0]
    cache.append({"input_ids": torch.zeros(1, 3)})
    assert len(cache) == 4
    assert [set(b) for b in cache.iter(["input_ids"])] == [{"input_ids"}] * 4
    a, b = list(cache.iter()), list(cache.iter_prefetch())
    assert len(a) == len(b) and all(set(x) == set(y) for x, y in zip(a, b))
    assert list(IntermediatesCache.empty(0).iter_prefetch()) == []
    sizes = cache.size()
    assert sizes[torch.device("cpu")] > 0
    # offloading keeps the fetch device
    off = IntermediatesCache.empty(1, offload_device="cpu")
    off.update(0, {"h": torch.ones(4)})
    assert off.batch_intermediates[0]["h"].value.device.type == "cpu" and off.fetch(0)["h"].device.type == "cpu"


def test_sparsegpt_modifier_fields_and_validation():
    """SparseGPTModifier keeps the reference's fields, validators and registry name
    (modifiers/pruning/sparsegpt/{base,sgpt_base}.py)."""
    import warnings

    from llmcompressor_amd.modifiers.factory import ModifierFactory
    from llmcompressor_amd.modifiers.pruning import SparseGPTModifier

    m = SparseGPTModifier(sparsity=0.5, mask_structure="2:4")
    assert (m._prune_n, m._prune_m) == (2, 4) and m.block_size == 128 and m.dampening_frac == 0.01
    assert m.targets == ["Linear"] and m.requires_calibration_data and not m.preserve_sparsity_mask
    assert (SparseGPTModifier(sparsity=0.3)._prune_n, SparseGPTModifier(sparsity=0.3)._prune_m) == (0, 0)
    with pytest.raises(ValueError):
        SparseGPTModifier(sparsity=0.5, sparsity_profile="owl")  # owl needs owl_m and owl_lmbda too
    with pytest.raises(ValueError):
        SparseGPTModifier(sparsity=0.5, sparsity_profile="other")
    ok = SparseGPTModifier(sparsity=0.5, sparsity_profile="OWL", owl_m=5, owl_lmbda=0.05)
    assert ok.sparsity_profile == "owl"
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        assert SparseGPTModifier(sparsity=0.5, sequential_update=False).sequential_update is True
        assert any(issubclass(x.category, DeprecationWarning) for x in w)
    made = ModifierFactory.create("SparseGPTModifier", sparsity=0.7, mask_structure="4:8", dampening_frac=0.001)
    assert isinstance(made, SparseGPTModifier) and made._prune_m == 8

    from llmcompressor_amd.recipe import Recipe

    recipe = Recipe.create_instance("""
    test_stage:
      obcq_modifiers:
        SparseGPTModifier:
          sparsity: 0.5
          mask_structure: "2:4"
          dampening_frac: 0.001
          block_size: 128
          targets: ['Linear']
          ignore: ['re:.*lm_head']
    """)
    (mod,) = recipe.modifiers
    assert isinstance(mod, SparseGPTModifier) and mod.ignore == ["re:.*lm_head"] and mod._prune_n == 2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("all_experts", [False, True])
def test_moe_forward_equals_the_per_expert_loop(dtype, all_experts):
    """LinearExperts2D.forward routes once for all experts; its output equals the reference's per-expert loop
    (oracle/moe.py) bit for bit, also with an idle expert and uneven counts, and the dense closed form in fp64."""
    from llmcompressor_amd.modeling import LinearExperts2D, moe_calibration_context
    from oracle.moe import experts_forward

    torch.manual_seed(3)
    E, H, I, T, k = 6, 16, 24, 40, 3
    experts = LinearExperts2D.from_fused(torch.randn(E, 2 * I, H) * 0.3, torch.randn(E, H, I) * 0.3).to(dtype)
    x = torch.randn(T, H).to(dtype)
    logits = torch.randn(T, E)
    logits[:, 4] = -1e9  # expert 4 idle
    wts, idx = torch.topk(torch.softmax(logits, -1), k, -1)
    wts = wts.to(dtype)
    seen = {}
    for e, ex in enumerate(experts):
        ex.down_proj.register_forward_hook(lambda m, a, o, e=e: seen.__setitem__(e, a[0].shape[0]))
    with torch.no_grad():
        if all_experts:
            with moe_calibration_context():
                got = experts(x, idx, wts)
        else:
            got = experts(x, idx, wts)
        want = experts_forward(list(experts), x, idx, wts, calibrate_all_experts=all_experts)
    assert torch.equal(got, want)
    assert seen[4] == (T if all_experts else 0) and len(seen) == E
    dense = torch.zeros(T, H, dtype=torch.float64)
    with torch.no_grad():
        for t in range(T):
            for j in range(k):
                dense[t] += wts[t, j].double() * experts[int(idx[t, j])].double()(x[t].double())
    experts.to(dtype)
    tol = 1e-5 if dtype == torch.float32 else 5e-2
    assert (got.double() - dense).abs().max() <= tol * dense.abs().max()


def test_sequential_partition_prefers_decoder_layers_over_nested_lists():
    """The layer list is the model's ``_no_split_modules`` classes when it names them, else the longest
    ModuleList that is not nested inside another list's element (an experts list is not the layer list)."""
    from llmcompressor_amd.pipelines import find_decoder_layers

    class Layer(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.experts = torch.nn.ModuleList([torch.nn.Linear(4, 4) for _ in range(8)])

    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = torch.nn.ModuleList([Layer() for _ in range(2)])

    m = Model()
    assert find_decoder_layers(m, None) == list(m.layers)
    m._no_split_modules = ["Layer"]
    assert find_decoder_layers(m, None) == list(m.layers)
    # explicit targets that are not the elements of one list cannot be run as a chain: the layers are used
    assert find_decoder_layers(m, ["Linear"]) == list(m.layers)
    assert find_decoder_layers(m, ["Layer"]) == list(m.layers)


@pytest.mark.parametrize("transposed,bias", [(False, False), (True, False), (False, True)])
def test_linearize_moe_keeps_the_function(transposed, bias):
    """A fused experts module (standard layout, transposed layout, with biases) and its per-expert replacement
    compute the same function (reference: modeling/moe/linear_experts.py:186-208, linearize.py:97-125)."""
    from llmcompressor_amd.modeling import LinearExperts2D, get_non_linearized_moes, linearize_moe

    E, H, I, T, k = 4, 8, 12, 10, 2
    torch.manual_seed(5)

    class Fused(torch.nn.Module):
        is_transposed = transposed

        def __init__(self):
            super().__init__()
            gu, dn = torch.randn(E, 2 * I, H), torch.randn(E, H, I)
            self.gate_up_proj = torch.nn.Parameter(gu.transpose(1, 2).contiguous() if transposed else gu)
            self.down_proj = torch.nn.Parameter(dn.transpose(1, 2).contiguous() if transposed else dn)
            if bias:
                self.gate_up_proj_bias = torch.nn.Parameter(torch.randn(E, 2 * I))
                self.down_proj_bias = torch.nn.Parameter(torch.randn(E, H))
            self.act_fn = torch.nn.GELU()

        def forward(self, x, idx, w):
            out = torch.zeros_like(x)
            for t in range(x.shape[0]):
                for j in range(idx.shape[1]):
                    e = int(idx[t, j])
                    gu = self.gate_up_proj[e].t() if transposed else self.gate_up_proj[e]
                    dn = self.down_proj[e].t() if transposed else self.down_proj[e]
                    h = gu @ x[t] + (self.gate_up_proj_bias[e] if bias else 0)
                    h = self.act_fn(h[:I]) * h[I:]
                    out[t] += w[t, j] * (dn @ h + (self.down_proj_bias[e] if bias else 0))
            return out

    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.block = torch.nn.ModuleDict({"experts": Fused()})

    model = Model()
    x = torch.randn(T, H)
    w, idx = torch.topk(torch.softmax(torch.randn(T, E), -1), k, -1)
    with torch.no_grad():
        want = model.block["experts"](x, idx, w)
        assert [n for n, _ in get_non_linearized_moes(model)] == ["block.experts"]
        linearize_moe(model)
        lin = model.block["experts"]
        assert isinstance(lin, LinearExperts2D) and get_non_linearized_moes(model) == []
        assert isinstance(lin[0].act_fn, torch.nn.GELU) and (lin[0].gate_proj.bias is not None) == bias
        got = lin(x, idx, w)
    assert torch.allclose(got, want, atol=1e-4, rtol=1e-4)


def test_gptq_job_planning():
    """compress_module_list plans lock-step sets by input width: at least ``group_min_modules`` Linears of one width
    form a set (split so that a set's work buffers stay within ``group_max_bytes``), the rest go one by one."""
    from llmcompressor_amd.modifiers.gptq import GPTQModifier
    from llmcompressor_amd.quantization import QuantizationArgs, QuantizationScheme

    class FakeCuda(torch.Tensor):
        """A CPU tensor that claims to live on the GPU, enough for the planner's eligibility checks."""

        @property
        def is_cuda(self):
            return True

    def lin(i, o):
        m = torch.nn.Linear(i, o, bias=False)
        m.weight = torch.nn.Parameter(torch.Tensor._make_subclass(FakeCuda, m.weight.data), requires_grad=False)
        m.quantization_scheme = QuantizationScheme(targets=["Linear"], weights=QuantizationArgs(
            num_bits=4, strategy="group", group_size=32))
        return m

    mods = [lin(64, 64), lin(64, 16), lin(64, 16), lin(64, 128), lin(128, 64), lin(96, 32), lin(96, 32)]
    mod = GPTQModifier(targets="Linear", scheme="W4A16")
    for m in mods:
        mod._hessians[m] = torch.Tensor._make_subclass(FakeCuda, torch.zeros(m.in_features, m.in_features))
    plan = mod._plan_jobs(list(mods))
    sets = [j for j in plan if isinstance(j, list)]
    singles = [j for j in plan if not isinstance(j, list)]
    assert len(sets) == 1 and sets[0] == mods[:4]            # four Linears of width 64
    assert singles == mods[4:]                               # width 128 alone; two of width 96 are below the minimum
    mod.group_min_modules = 2
    plan = mod._plan_jobs(list(mods))
    assert [len(j) for j in plan if isinstance(j, list)] == [4, 2]
    mod.group_max_bytes = 10 * 64 * 64 * 3                   # room for three width-64 problems per job
    plan = mod._plan_jobs(list(mods))
    assert [len(j) if isinstance(j, list) else 1 for j in plan][:2] == [3, 1]
    mod.group_min_modules = 0
    assert mod._plan_jobs(list(mods)) == mods


def test_observed_kv_cache_stand_in():
    """The stand-in for ``past_key_values`` shows keys and values to the module's observers and defers to the
    real cache when there is one."""
    from llmcompressor_amd.modifiers.quantization.quantization.mixin import _kv_cache_pre_hook, _ObservedKVCache

    seen = []

    class Attn(torch.nn.Module):
        def k_observer(self, x):
            seen.append(("k", x.shape))

        def v_observer(self, x):
            seen.append(("v", x.shape))

    class Real:
        marker = 7

        def update(self, k, v, layer_idx, cache_kwargs=None):
            return k + 1, v + 1

    attn = Attn()
    k, v = torch.zeros(1, 2, 5, 4), torch.ones(1, 2, 5, 4)
    _, kwargs = _kv_cache_pre_hook(attn, (), {"past_key_values": None, "x": 1})
    k2, v2 = kwargs["past_key_values"].update(k, v, 0)
    assert k2 is k and v2 is v and seen == [("k", k.shape), ("v", v.shape)] and kwargs["x"] == 1
    wrapped = _ObservedKVCache(attn, Real())
    k3, v3 = wrapped.update(k, v, 0, cache_kwargs={})
    assert torch.equal(k3, k + 1) and torch.equal(v3, v + 1) and wrapped.marker == 7 and len(seen) == 4
    _, kwargs = _kv_cache_pre_hook(attn, (), {})
    assert isinstance(kwargs["past_key_values"], _ObservedKVCache)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_lerp_equals_the_eager_expression_on_cpu(dtype):
    """The step-by-step lerp of the activation observers equals ``start * (1 - w) + end * w`` as eager CPU ops
    evaluate it (reference: observers/helpers.py:218-220)."""
    from llmcompressor_amd.observers.helpers import lerp

    torch.manual_seed(0)
    a, b = (torch.randn(50000) * 3).to(dtype), (torch.randn(50000) * 3).to(dtype)
    for w in (0.01, 0.1, 0.5):
        assert torch.equal(lerp(a, b, w), (a * (1.0 - w)) + (b * w))


def test_checkpoint_unpacking_helpers_match_the_oracle_pack():
    """_unpack_int32 inverts the oracle's pack_to_int32 for 2 to 8 bit fields and ragged widths; _expand_qparam lays
    scales out per strategy."""
    from oracle import pack as P

    from llmcompressor_amd.compressors import _expand_qparam, _unpack_int32
    from llmcompressor_amd.quantization import QuantizationArgs

    torch.manual_seed(0)
    for bits in (2, 3, 4, 8):
        for K in (1, 7, 32, 45):
            lo, hi = -(1 << (bits - 1)), (1 << (bits - 1)) - 1
            codes = torch.randint(lo, hi + 1, (5, K), dtype=torch.int8)
            packed = P.pack_to_int32(codes, bits)
            assert torch.equal(_unpack_int32(packed, bits, K).to(torch.int8), codes)
    s = torch.arange(6, dtype=torch.float32).reshape(2, 3)
    g = _expand_qparam(s, QuantizationArgs(num_bits=4, strategy="group", group_size=2), 2, 6)
    assert g.tolist() == [[0, 0, 1, 1, 2, 2], [3, 3, 4, 4, 5, 5]]
    b = _expand_qparam(s, QuantizationArgs(num_bits=4, strategy="block", block_structure=[2, 2]), 3, 5)
    assert b.shape == (3, 5) and b[2].tolist() == [3, 3, 4, 4, 5] and b[0].tolist() == [0, 0, 1, 1, 2]
    c = _expand_qparam(torch.tensor([[2.0], [3.0]]), QuantizationArgs(num_bits=8, strategy="channel"), 2, 4)
    assert c.shape == (2, 1)
    t = _expand_qparam(torch.tensor([5.0]), QuantizationArgs(num_bits=8, strategy="tensor"), 2, 4)
    assert t.shape == (1, 1)
    perm = torch.tensor([2, 0, 1, 1, 0, 2])
    gi = _expand_qparam(s, QuantizationArgs(num_bits=4, strategy="group", group_size=2), 2, 6, g_idx=perm)
    assert gi[0].tolist() == [2, 0, 1, 1, 0, 2]


def test_owl_outlier_percentage_and_sparsity_mapping():
    """The OWL profile's layer statistic against a brute-force count, and the mapping of the ratios to per-layer
    sparsities: mean of (1 - sparsity) equals the global keep ratio, spread equals 2 * lambda."""
    from llmcompressor_amd.modifiers.pruning.sparsegpt.owl import outlier_percentage

    torch.manual_seed(0)
    members = [(torch.randn(12, 16), torch.rand(16) + 0.1), (torch.randn(5, 16) * 3, torch.rand(16))]
    scores = torch.cat([(w.abs() * a[None, :]).flatten() for w, a in members])
    want = 100.0 * (scores > 3.0 * scores.mean()).sum().item() / scores.numel()
    assert abs(outlier_percentage(members, 3.0) - want) < 1e-9
    assert outlier_percentage([], 3.0) == 0.0
    d = torch.tensor([1.0, 4.0, 2.5], dtype=torch.float64)
    lmbda, target = 0.08, 0.6
    stretched = (d - d.min()) * (2 * lmbda / (d.max() - d.min()))
    keep = stretched - stretched.mean() + (1 - target)
    assert abs(keep.mean().item() - (1 - target)) < 1e-12 and abs((keep.max() - keep.min()).item() - 2 * lmbda) < 1e-12


def test_tail_pass_restores_instance_level_forwards_and_refuses_a_short_second_pass():
    """The pass that calibrates what follows the last sequential layer short-circuits the layers by assigning
    `forward` on the instances.  A layer that already carried an instance-level forward (a wrapper such as an
    offloading hook) must get it back, a layer without one must fall back to its class, and a dataloader that is
    exhausted after the first pass must raise instead of leaving the tail modules without samples."""
    import torch

    from llmcompressor_amd.pipelines import _calibrate_tail

    class Layer(torch.nn.Module):
        def forward(self, hidden_states):
            return hidden_states + 1

    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = torch.nn.ModuleList([Layer(), Layer()])
            self.head = torch.nn.Linear(4, 4, bias=False)

        def forward(self, x):
            for layer in self.layers:
                x = layer(x)
            return self.head(x)

    class Cache:
        def __init__(self, items):
            self.items = items

        def __len__(self):
            return len(self.items)

        def fetch(self, i):
            return {"args": (self.items[i],)}

    model = Model()
    calls = []
    original = model.layers[0].forward

    def wrapper(hidden_states):  # what accelerate's add_hook_to_module leaves on an instance
        calls.append(1)
        return original(hidden_states)

    model.layers[0].forward = wrapper
    seen = []
    model.head.register_forward_pre_hook(lambda m, a: seen.append(a[0].clone()))
    batches = [torch.zeros(1, 4), torch.ones(1, 4)]
    cache = Cache([torch.full((1, 4), 7.0), torch.full((1, 4), 9.0)])
    _calibrate_tail(model, list(model.layers), [model.head], batches, cache, torch.device("cpu"), returns_tuple=False)
    assert [t[0, 0].item() for t in seen] == [7.0, 9.0]  # the head saw the cached outputs of the last layer
    assert vars(model.layers[0])["forward"] is wrapper and not calls  # wrapper back in place, not called meanwhile
    assert "forward" not in vars(model.layers[1])  # back to the class's method
    assert model(torch.zeros(1, 4)).shape == (1, 4) and calls == [1]
    with pytest.raises(RuntimeError, match="re-iterable"):
        _calibrate_tail(model, list(model.layers), [model.head], iter(batches[:1]), cache, torch.device("cpu"),
                        returns_tuple=False)
    assert vars(model.layers[0])["forward"] is wrapper and "forward" not in vars(model.layers[1])


@pytest.mark.parametrize("shape", [(2, 3, 8, 8), (3, 8, 8)])
def test_conv2d_hessian_branch_fails_the_way_the_reference_does(shape):
    """/root/reference/src/llmcompressor/modifiers/gptq/gptq_quantize.py:36-56: every input is brought to three
    dimensions before the Conv2d branch, where ``Unfold`` then takes it for one unbatched image and returns a
    matrix, so the following three-axis ``permute`` raises.  The branch cannot succeed for any input in the
    reference; the mirror applies the same operations in the same order and fails at the same one, before any
    device call."""
    from llmcompressor_amd.modifiers.gptq.gptq_quantize import accumulate_hessian, make_empty_hessian

    conv = torch.nn.Conv2d(3, 8, 3, padding=1)
    H = make_empty_hessian(conv)
    assert H.shape == (3, 3)  # weight.shape[1], as in the reference (not in_channels * kernel area)
    with pytest.raises(RuntimeError, match="permute"):
        accumulate_hessian(torch.randn(*shape), conv, H, torch.zeros(1))


def test_calibration_dataloader_from_an_in_memory_dataset():
    """``oneshot(dataset=<datasets.Dataset>, num_calibration_samples=..., max_seq_length=...)`` as the reference's
    examples call it (datasets/utils.py:122-393): sampler, truncating collator, tokenisation of a text column,
    pass-through of ready loaders, refusal of hub names."""
    datasets = pytest.importorskip("datasets")
    from torch.utils.data import DataLoader

    from llmcompressor.datasets import LengthAwareSampler, get_calibration_dataloader

    lengths = [5, 9, 3, 12, 7, 8]
    ds = datasets.Dataset.from_dict({
        "input_ids": [list(range(1, n + 1)) for n in lengths],
        "attention_mask": [[1] * n for n in lengths],
    })
    # longest first without shuffling; the shortest samples are the ones left out
    loader = get_calibration_dataloader(ds, num_calibration_samples=4, shuffle_calibration_samples=False,
                                        max_seq_length=10)
    assert isinstance(loader, DataLoader) and len(loader) == 4
    batches = list(loader)
    assert [b["input_ids"].shape for b in batches] == [(1, 10), (1, 9), (1, 8), (1, 7)]
    assert batches[0]["input_ids"].dtype == torch.int64 and batches[0]["attention_mask"].shape == (1, 10)
    assert torch.equal(batches[1]["input_ids"][0], torch.arange(1, 10))
    assert list(LengthAwareSampler(ds, num_samples=3)) == [3, 1, 5]
    # a batch is cut to its shortest member
    loader = get_calibration_dataloader(ds, num_calibration_samples=6, shuffle_calibration_samples=False, batch_size=2)
    assert [tuple(b["input_ids"].shape) for b in loader] == [(2, 9), (2, 7), (2, 3)]
    # default: a random subset, each sample at most once
    torch.manual_seed(0)
    loader = get_calibration_dataloader(ds, num_calibration_samples=5)
    seen = sorted(int(b["input_ids"].shape[1]) for b in loader)
    assert len(seen) == 5 and len(set(seen)) == 5 and set(seen) <= set(lengths)
    # more samples requested than there are
    assert len(get_calibration_dataloader(ds, num_calibration_samples=512)) == 6
    # a DatasetDict falls back to its train split; a named split is taken as asked
    dd = datasets.DatasetDict({"train": ds, "test": ds.select(range(2))})
    assert len(get_calibration_dataloader(dd)) == 6
    assert len(get_calibration_dataloader(dd, splits="test")) == 2
    assert len(get_calibration_dataloader(dd, splits={"calibration": "test"})) == 2
    with pytest.raises(ValueError, match="train"):
        get_calibration_dataloader(datasets.DatasetDict({"validation": ds}))

    # a text column is tokenised with truncation and (by default) padding to max_seq_length
    class Tok:
        model_max_length = 16
        calls = []

        def __call__(self, text, padding=False, max_length=None, truncation=False):
            Tok.calls.append((padding, max_length, truncation))
            ids = [ord(c) % 50 + 1 for c in text][: max_length if truncation else None]
            mask = [1] * len(ids)
            if padding == "max_length":
                ids, mask = ids + [0] * (max_length - len(ids)), mask + [0] * (max_length - len(mask))
            return {"input_ids": ids, "attention_mask": mask}

    text = datasets.Dataset.from_dict({"text": ["hello world", "a much longer line of text than that"], "n": [1, 2]})
    loader = get_calibration_dataloader(text, Tok(), max_seq_length=8, shuffle_calibration_samples=False)
    got = list(loader)
    assert set(got[0].keys()) == {"input_ids", "attention_mask"} and got[0]["input_ids"].shape == (1, 8)
    assert Tok.calls[0] == ("max_length", 8, True)
    loader = get_calibration_dataloader(text, Tok(), max_seq_length=64, pad_to_max_length=False,
                                        shuffle_calibration_samples=False)
    assert [b["input_ids"].shape[1] for b in loader] == [16, 11]  # clipped to the tokenizer's model_max_length
    with pytest.raises(ValueError, match="tokenize"):
        get_calibration_dataloader(text)
    with pytest.raises(ValueError, match="text_column"):
        get_calibration_dataloader(text, Tok(), text_column="prompt")
    # pass-through and refusals
    ready = [{"input_ids": torch.ones(1, 4, dtype=torch.long)}]
    assert get_calibration_dataloader(ready) is ready
    dl = DataLoader(ready)
    assert get_calibration_dataloader(dl) is dl and get_calibration_dataloader(None) is None
    with pytest.raises(ValueError, match="network"):
        get_calibration_dataloader("open_platypus")
    with pytest.raises(ValueError, match="Unknown data collator"):
        get_calibration_dataloader(ds, data_collator="nope")
    custom = get_calibration_dataloader(ds, data_collator=lambda feats: {"n": len(feats)}, batch_size=3,
                                        shuffle_calibration_samples=False)
    assert [b["n"] for b in custom] == [3, 3]


def test_sequential_targets_that_are_not_a_layer_list_fall_back_to_the_layers(caplog):
    """The reference cuts its traced graph at any module class (``sequential_targets=["Attention", "ExpertMLP"]`` in
    its MoE examples); here targets that are not the elements of one layer list would not form a chain, so the
    model's decoder layers are used and a warning says so."""
    import logging

    from llmcompressor_amd.pipelines import find_decoder_layers

    class Attn(torch.nn.Module):
        pass

    class Mlp(torch.nn.Module):
        pass

    class Block(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.attn, self.mlp = Attn(), Mlp()

    class Model(torch.nn.Module):
        _no_split_modules = ["Block"]

        def __init__(self):
            super().__init__()
            self.layers = torch.nn.ModuleList([Block() for _ in range(3)])

    model = Model()
    assert find_decoder_layers(model, ["Block"]) == list(model.layers)
    assert find_decoder_layers(model, "Block") == list(model.layers)
    with caplog.at_level(logging.WARNING, logger="llmcompressor_amd"):
        got = find_decoder_layers(model, ["Attn", "Mlp"])
    assert got == list(model.layers)
    assert "not the elements of one layer list" in caplog.text
    assert find_decoder_layers(model, ["NoSuchClass"]) == list(model.layers)


class _ModelOptStyleConverter:
    """A user-side converter of the kind the reference's ``converter=`` argument takes: NVFP4 layers stored the
    ModelOpt way (``weight`` packed, ``weight_scale_2`` and ``input_scale`` as divisors) are renamed to the
    compressed-tensors names with the global scales inverted (the mapping table of the reference's
    docs/guides/entrypoints/convert.md)."""

    def __init__(self, targets):
        import re

        self.patterns = [re.compile(t[3:]) for t in targets]
        self.seen_meta = []

    def _hit(self, name):
        module = name.rsplit(".", 1)[0]
        return any(p.match(module) for p in self.patterns)

    def get_dependencies(self, name):
        if name.endswith(".weight") and self._hit(name):
            m = name[: -len("weight")]
            return [m + "weight_scale", m + "weight_scale_2", m + "input_scale"]
        return []

    def validate(self, tensors):
        for name, t in tensors.items():
            assert t.device.type == "meta"
            if name.endswith(".weight") and self._hit(name):
                self.seen_meta.append(name)
                if t.dtype != torch.uint8:
                    raise ValueError(f"{name} is not packed fp4")
                if name[: -len("weight")] + "weight_scale_2" not in tensors:
                    raise ValueError(f"{name} has no second-level scale beside it")

    def process(self, tensors):
        out = {}
        for name, t in tensors.items():
            module, leaf = name.rsplit(".", 1)
            if not self._hit(name):
                out[name] = t
            elif leaf == "weight":
                out[module + ".weight_packed"] = t
            elif leaf == "weight_scale_2":
                out[module + ".weight_global_scale"] = 1.0 / t
            elif leaf == "input_scale":
                out[module + ".input_global_scale"] = 1.0 / t
            else:
                out[name] = t
        return out

    def create_config(self):
        from llmcompressor_amd.quantization import QuantizationConfig, preset_name_to_scheme

        sch = preset_name_to_scheme("NVFP4", ["re:" + p.pattern for p in self.patterns])
        return QuantizationConfig(config_groups={"config_group_0": sch}, format="nvfp4-pack-quantized",
                                  ignore=["lm_head"])


def test_model_free_converter_config_merge_and_dependencies(tmp_path):
    """``converter=`` host logic (reference: entrypoints/model_free/__init__.py:101,126, save_utils.py:64-126):
    the converter's config is the starting point and this run's groups are appended to it; tensors a converter
    needs together are planned into one job; validation hands the converter meta tensors."""
    import json

    from safetensors.torch import save_file

    from llmcompressor_amd.entrypoints.model_free import (_build_jobs, _validate_converted, update_config,
                                                          validate_config)

    conv = _ModelOptStyleConverter(["re:.*mlp\\.(gate|up|down)_proj$"])
    cfg = validate_config(None, "FP8_DYNAMIC", ["lm_head"])
    (tmp_path / "config.json").write_text(json.dumps({"model_type": "toy"}))
    q = update_config(str(tmp_path), cfg, conv)
    assert list(q["config_groups"]) == ["config_group_0", "FP8_DYNAMIC"]
    assert q["config_groups"]["config_group_0"]["weights"]["group_size"] == 16
    assert q["config_groups"]["FP8_DYNAMIC"]["format"] == "float-quantized"
    assert q["format"] == "mixed-precision" and q["ignore"] == ["lm_head"]
    assert json.loads((tmp_path / "config.json").read_text())["quantization_config"] == q
    # a group name that is taken is not overwritten
    cfg0 = validate_config(None, "FP8_DYNAMIC", [])
    cfg0.config_groups = {"config_group_0": cfg0.config_groups["FP8_DYNAMIC"]}
    q0 = update_config(str(tmp_path), cfg0, conv)
    assert list(q0["config_groups"]) == ["config_group_0", "config_group_1"]
    assert q0["config_groups"]["config_group_1"]["weights"]["num_bits"] == 8
    # without a converter the checkpoint's own compressed-tensors config is the starting point (what the last call
    # left in config.json: the converter's group and the FP8 one), and a config of another method is dropped
    q1 = update_config(str(tmp_path), validate_config(None, "W8A16", []))
    assert list(q1["config_groups"]) == ["config_group_0", "config_group_1", "W8A16"] and q1["ignore"] == ["lm_head"]
    assert q1["format"] == "mixed-precision"
    (tmp_path / "config.json").write_text(json.dumps({"quantization_config": {"quant_method": "fp8"}}))
    assert list(update_config(str(tmp_path), cfg)["config_groups"]) == ["FP8_DYNAMIC"]
    (tmp_path / "config.json").write_text(json.dumps({"model_type": "toy"}))
    assert list(update_config(str(tmp_path), cfg)["config_groups"]) == ["FP8_DYNAMIC"]

    # the second-level scale of down_proj lives in the other shard: it is planned into the job of its weight
    src = tmp_path / "src"
    src.mkdir()
    a = {"m.mlp.down_proj.weight": torch.zeros(8, 16, dtype=torch.uint8),
         "m.mlp.down_proj.weight_scale": torch.ones(8, 2).to(torch.float8_e4m3fn),
         "m.self_attn.o_proj.weight": torch.zeros(8, 8, dtype=torch.bfloat16)}
    b = {"m.mlp.down_proj.weight_scale_2": torch.ones(1), "m.mlp.down_proj.input_scale": torch.ones(1)}
    save_file(a, str(src / "a.safetensors"))
    save_file(b, str(src / "b.safetensors"))
    files = {"a.safetensors": str(src / "a.safetensors"), "b.safetensors": str(src / "b.safetensors")}
    jobs, _ = _build_jobs(files, str(tmp_path / "dst"), cfg, conv)
    by_out = {os.path.basename(p): iwm for iwm, p in jobs}
    assert sorted(by_out["a.safetensors"][files["b.safetensors"]]) == ["m.mlp.down_proj.input_scale",
                                                                     "m.mlp.down_proj.weight_scale_2"]
    assert by_out["b.safetensors"][files["b.safetensors"]] == []
    _validate_converted(jobs, cfg, conv)
    assert conv.seen_meta == ["m.mlp.down_proj.weight"]
    # a converter that refuses a shard stops the run before anything is quantized
    jobs_split, _ = _build_jobs(files, str(tmp_path / "dst"), cfg, None)
    with pytest.raises(ValueError, match="no second-level scale"):
        _validate_converted(jobs_split, cfg, conv)
    from llmcompressor_amd import model_free_ptq

    with pytest.raises(TypeError, match="process"):
        model_free_ptq(str(src), str(tmp_path / "dst"), scheme="FP8_DYNAMIC", converter=object())


def test_sequential_pipeline_pass_structure_on_the_host():
    """The sequential pipeline's passes with a recording modifier on a CPU model (no kernel involved; reference:
    pipelines/sequential/pipeline.py:136-181): by default every layer runs twice per batch (hooks live, then hooks
    off on the layer the epoch-end event has just changed) and the next layer is fed the second pass's outputs;
    ``propagate_error=False`` runs the first pass only and feeds its outputs on;
    ``sequential_targets_per_subgraph=2`` hands two layers to one epoch-end event."""
    from llmcompressor_amd.core import active_session
    from llmcompressor_amd.modifiers import Modifier
    from llmcompressor_amd.pipelines import CalibrationPipeline

    class Layer(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.lin = torch.nn.Linear(4, 4, bias=False)
            with torch.no_grad():
                self.lin.weight.copy_(torch.eye(4))

        def forward(self, x):
            return self.lin(x)

    class Model(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.layers = torch.nn.ModuleList([Layer() for _ in range(3)])

        def forward(self, x):
            for layer in self.layers:
                x = layer(x)
            return x

    class Recorder(Modifier):
        requires_calibration_data: bool = True
        log: list = []

        def on_initialize(self, state, **kwargs):
            self.log.clear()
            return True

        def on_calibration_start(self, state, event, **kwargs):
            for i, layer in enumerate(state.model.layers):
                self.register_hook(layer.lin, lambda m, args, out, i=i: self.log.append(("seen", i, args[0].sum().item())),
                                   "forward")

        def on_sequential_epoch_end(self, state, event, modules=(), **kwargs):
            lins = [m for m in modules if isinstance(m, torch.nn.Linear)]
            if lins:
                self.log.append(("epoch_end", len(lins)))
            for lin in lins:  # "compress": the layer doubles its input from now on
                lin.weight.data.mul_(2.0)

        def on_calibration_end(self, state, event, **kwargs):
            self.remove_hooks()

        def on_finalize(self, state, **kwargs):
            return True

    class Args:
        sequential_targets = None

    data = [torch.ones(1, 4), 2 * torch.ones(1, 4)]

    def run(**kw):
        model, mod = Model(), Recorder()
        session = active_session()
        session.reset()
        session.initialize(model=model, recipe=mod)
        args = Args()
        for k, v in kw.items():
            setattr(args, k, v)
        forwards = [0, 0, 0]
        handles = [l.register_forward_pre_hook(lambda m, a, i=i: forwards.__setitem__(i, forwards[i] + 1))
                   for i, l in enumerate(model.layers)]
        CalibrationPipeline.load_from_registry("sequential")(model, data, args)
        for h in handles:
            h.remove()
        session.finalize()
        session.reset()
        return list(mod.log), forwards

    log, forwards = run()
    # layer 0 is also entered once per batch by the pass that captures its inputs
    assert forwards == [6, 4, 4]
    # layer 1 sees layer 0's compressed (doubled) outputs, layer 2 the twice-doubled ones
    assert log == [("seen", 0, 4.0), ("seen", 0, 8.0), ("epoch_end", 1), ("seen", 1, 8.0), ("seen", 1, 16.0),
                   ("epoch_end", 1), ("seen", 2, 16.0), ("seen", 2, 32.0), ("epoch_end", 1)]
    log, forwards = run(propagate_error=False)
    assert forwards == [4, 2, 2]
    assert log == [("seen", 0, 4.0), ("seen", 0, 8.0), ("epoch_end", 1), ("seen", 1, 4.0), ("seen", 1, 8.0),
                   ("epoch_end", 1), ("seen", 2, 4.0), ("seen", 2, 8.0), ("epoch_end", 1)]
    log, forwards = run(sequential_targets_per_subgraph=2)
    assert forwards == [6, 4, 4]
    assert log == [("seen", 0, 4.0), ("seen", 1, 4.0), ("seen", 0, 8.0), ("seen", 1, 8.0), ("epoch_end", 2),
                   ("seen", 2, 16.0), ("seen", 2, 32.0), ("epoch_end", 1)]


def test_experts_block_tells_input_reading_hooks_from_the_rest():
    """What lets an experts block call a Linear's hooks itself instead of the Linear (``moe_grouped_calibration``):
    every live hook is a plain forward hook that declares it only reads the module's input, as GPTQ's Hessian hook
    does; anything else (an undeclared hook, a pre-hook, a hook taking keyword arguments) keeps the per-expert
    calls, and hooks that ``disable_hooks`` has switched off do not count."""
    from llmcompressor_amd.modeling.moe import _input_hooks
    from llmcompressor_amd.modifiers.gptq import GPTQModifier
    from llmcompressor_amd.modifiers.utils.hooks import HooksMixin, hook_is_inert

    assert GPTQModifier.calibrate_module._llmc_input_only is True
    lin = torch.nn.Linear(4, 4)
    assert _input_hooks(lin, hook_is_inert) == []
    owner = HooksMixin()
    seen = []

    def reads_input(module, args, output):
        seen.append(args[0].shape)

    reads_input._llmc_input_only = True
    handle = owner.register_hook(lin, reads_input, "forward")
    live = _input_hooks(lin, hook_is_inert)
    assert len(live) == 1
    live[0](lin, (torch.zeros(3, 4),), None)  # the call an experts block makes
    assert seen == [torch.Size([3, 4])]
    with HooksMixin.disable_hooks():
        assert _input_hooks(lin, hook_is_inert) == []
    with HooksMixin.disable_hooks(keep={handle}):
        assert len(_input_hooks(lin, hook_is_inert)) == 1
    plain = lin.register_forward_hook(lambda m, a, o: None)  # says nothing about itself
    assert _input_hooks(lin, hook_is_inert) is None
    plain.remove()
    pre = lin.register_forward_pre_hook(lambda m, a: None)
    assert _input_hooks(lin, hook_is_inert) is None
    pre.remove()
    kw = lin.register_forward_hook(lambda m, a, k, o: None, with_kwargs=True)
    assert _input_hooks(lin, hook_is_inert) is None
    kw.remove()
    assert len(_input_hooks(lin, hook_is_inert)) == 1
    owner.remove_hooks()
    assert _input_hooks(lin, hook_is_inert) == []


def test_shared_inputs_do_not_pair_up_neighbouring_experts_without_tokens():
    """``share_identical_inputs``: two experts that receive no token in a batch are handed empty row ranges that
    start at one address and have one shape; they are two inputs all the same (only the very same tensor object
    counts when it is empty), so neither becomes the other's follower -- and an expert's up_proj, which is handed
    the very object its gate_proj got, still follows it, empty or not."""
    from llmcompressor_amd.modifiers.gptq import GPTQModifier

    mod = GPTQModifier(targets="Linear", scheme="W4A16")
    gate = [torch.nn.Linear(8, 4, bias=False) for _ in range(2)]
    up = [torch.nn.Linear(8, 4, bias=False) for _ in range(2)]
    routed = torch.randn(6, 8)

    def batch(rows_of_expert):
        followed = []
        for e, (lo, hi) in enumerate(rows_of_expert):
            x = routed[lo:hi]
            for lin in (gate[e], up[e]):
                follows = mod._follows_recent_input(lin, x)
                followed.append(follows)
                if not follows and lin not in mod._num_samples:  # what the hook does for a module of its own
                    mod._num_samples[lin] = 0
        return followed

    # both experts without tokens: the ranges routed[3:3] and routed[3:3] are equal in every respect but identity
    assert batch([(3, 3), (3, 3)]) == [False, True, False, True]
    assert mod._leader == {up[0]: gate[0], up[1]: gate[1]}
    # later they get different rows: nobody raises, everybody still follows its own gate_proj
    assert batch([(0, 2), (2, 6)]) == [False, True, False, True]
    assert batch([(0, 0), (0, 6)]) == [False, True, False, True]
