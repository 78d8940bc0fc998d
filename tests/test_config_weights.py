"""Configuration, registry, weights: what is read, what is refused, and what the one error lists."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

import sparseengine_amd  # noqa: F401
from sparseengine_amd.config.method_registry import normalize_sparse_method, resolve_prefill_schedule_policy
from sparseengine_amd.config.registry import resolve_architecture, supported_architectures
from sparseengine_amd.config.runtime import Config
from sparseengine_amd.config.specs import AttentionSpec, ModelSpec, MoESpec, ScheduleEntry
from sparseengine_amd.models.minimax_m2 import MiniMaxM2Config, build_spec
from sparseengine_amd.parts import build_model
from sparseengine_amd.weights import loader
from sparseengine_amd.weights.random_weights import write_model_folder
from tests.helpers import CONFIGS, TINY_A, TINY_B, make_folder

OFFICIAL = dict(   # the values the reference's test holds (tests/test_minimax_m2_config.py:25-52)
    architectures=["MiniMaxM2ForCausalLM"], model_type="minimax_m2", vocab_size=200064, hidden_size=3072,
    intermediate_size=1536, num_hidden_layers=62, num_attention_heads=48, num_key_value_heads=8, head_dim=128,
    rotary_dim=64, num_local_experts=256, num_experts_per_tok=8, max_position_embeddings=204800,
    shared_intermediate_size=0, mtp_transformer_layers=1, num_mtp_modules=3, hidden_act="silu",
    qk_norm_type="per_layer", scoring_func="sigmoid", use_qk_norm=True, use_routing_bias=True, use_mtp=True,
    tie_word_embeddings=False, rms_norm_eps=1e-6, rope_theta=5000000)


def test_official_config_becomes_parts():
    cfg = MiniMaxM2Config.from_dict(OFFICIAL)
    spec = build_spec(cfg)
    assert len(spec.layers) == 62 and [e.layer for e in spec.schedule] == list(range(62))
    att, moe = spec.layers[0].mixer, spec.layers[0].feed_forward
    assert isinstance(att, AttentionSpec) and isinstance(moe, MoESpec)
    assert (att.num_heads, att.num_kv_heads, att.head_dim, att.qk_norm) == (48, 8, 128, "flat")
    assert att.scale == 128 ** -0.5                       # of the full head size, not of the rotary part
    assert (att.position.rotary_dim, att.position.theta, att.position.max_position) == (64, 5e6, 204800)
    assert (moe.num_experts, moe.top_k, moe.intermediate_size, moe.scoring) == (256, 8, 1536, "sigmoid")
    assert att.window is None and spec.hidden_size == 3072 and spec.vocab_size == 200064
    assert cfg.extra["num_mtp_modules"] == 3              # carried, not used
    decls = build_model(spec).all_param_decls()
    assert decls["layers.0.mixer.qkv"].shape == ((48 + 16) * 128, 3072)      # head_dim is read, not hidden / heads
    assert decls["layers.61.ffn.w13"].shape == (256, 3072, 3072) and decls["layers.3.ffn.router"].policy == "float32"


@pytest.mark.parametrize("key,value,word", [
    ("qk_norm_type", "per_head", "qk_norm_type"), ("scoring_func", "softmax", "scoring_func"),
    ("hidden_act", "gelu", "hidden_act"), ("tie_word_embeddings", True, "tie_word_embeddings"),
    ("use_routing_bias", False, "use_routing_bias"), ("num_key_value_heads", 5, "kv heads"),
    ("rotary_dim", 7, "rotary_dim"), ("rotary_dim", 256, "rotary_dim"), ("num_experts_per_tok", 300, "num_experts_per_tok"),
    ("head_dim", 100, "head_dim"), ("shared_intermediate_size", 64, "shared"),
    ("quantization_config", {"quant_method": "fp8"}, "quantised")])
def test_fixed_semantics_are_checked(key, value, word):
    with pytest.raises(ValueError, match=word):
        MiniMaxM2Config.from_dict({**OFFICIAL, key: value})


def test_missing_keys_and_rope_sources():
    broken = {k: v for k, v in OFFICIAL.items() if k not in ("head_dim", "rms_norm_eps")}
    with pytest.raises(ValueError, match=r"head_dim.*rms_norm_eps|rms_norm_eps.*head_dim"):
        MiniMaxM2Config.from_dict(broken)
    assert MiniMaxM2Config.from_dict({k: v for k, v in OFFICIAL.items() if k != "rope_theta"}).rope_theta == 10000.0
    nested = MiniMaxM2Config.from_dict({**OFFICIAL, "rope_parameters": {"rope_theta": 123.0, "rope_type": "default"}})
    assert nested.rope_theta == 123.0 and nested.rope_scaling is None        # rope_parameters wins over rope_theta
    yarn = MiniMaxM2Config.from_dict({**OFFICIAL, "rope_scaling": {"type": "yarn", "factor": 4.0,
                                                                  "original_max_position_embeddings": 51200}})
    assert dict(yarn.rope_scaling)["rope_type"] == "yarn"
    with pytest.raises(ValueError, match="dynamic"):
        MiniMaxM2Config.from_dict({**OFFICIAL, "rope_scaling": {"type": "dynamic", "factor": 2.0}})
    assert not MiniMaxM2Config.from_dict({**TINY_B}).use_qk_norm


def test_registry_and_methods():
    # the product registers one architecture (another test of this session may have registered its toy)
    assert [a for a in supported_architectures() if a != "ToyForCausalLM"] == ["MiniMaxM2ForCausalLM"]
    assert resolve_architecture({"architectures": ["MiniMaxM2ForCausalLM"]}).name == "MiniMaxM2ForCausalLM"
    assert resolve_architecture({"model_type": "minimax_m2"}).name == "MiniMaxM2ForCausalLM"
    with pytest.raises(NotImplementedError, match="MiniMaxM2ForCausalLM"):
        resolve_architecture({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})
    assert normalize_sparse_method("vanilla") == "" == normalize_sparse_method("")
    with pytest.raises(ValueError, match="vanilla"):
        normalize_sparse_method("snapkv")
    assert resolve_prefill_schedule_policy("", "auto") == "all_chunked"
    with pytest.raises(ValueError):
        resolve_prefill_schedule_policy("", "layerwise")


def test_schedule_is_data():
    cfg = MiniMaxM2Config.from_dict(TINY_A)
    spec = build_spec(cfg)
    twice = ModelSpec(**{**spec.__dict__, "schedule": (ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1, cache_from=1))})
    requests = build_model(twice).cache_requests()
    assert sorted(requests) == [0, 1, 2]                  # position 3 reads position 1's cache
    with pytest.raises(ValueError, match="does not run before"):
        ModelSpec(**{**spec.__dict__, "schedule": (ScheduleEntry(0, cache_from=1), ScheduleEntry(1))})
    with pytest.raises(ValueError, match="names layer"):
        ModelSpec(**{**spec.__dict__, "schedule": (ScheduleEntry(5),)})


def test_runtime_config(tmp_path):
    folder = make_folder(tmp_path, "A")
    cfg = Config.from_kwargs(folder)
    assert cfg.max_model_len == 256 and cfg.max_decoding_seqs == cfg.max_num_seqs_in_batch == 32
    assert cfg.max_num_seqs_in_gpu == 96 and cfg.max_num_batched_tokens == 256 == cfg.engine_prefill_chunk_size
    assert cfg.sparse_method == "" and cfg.prefill_schedule_policy == "all_chunked" and cfg.dtype == "bfloat16"
    assert Config.from_kwargs(folder, sparse_method="vanilla", max_num_batched_tokens=64).engine_prefill_chunk_size == 64
    with pytest.raises(ValueError, match="unknown configuration keys.*enable_magic"):
        Config.from_kwargs(folder, enable_magic=True)
    with pytest.raises(ValueError, match="tensor_parallel_size"):
        Config.from_kwargs(folder, tensor_parallel_size=2)
    with pytest.raises(ValueError, match="max_model_len"):
        Config.from_kwargs(folder, max_model_len=9999)
    with pytest.raises(ValueError, match="dtype"):
        Config.from_kwargs(folder, dtype="float16")
    tiny = Config.from_kwargs(folder, tiny_random=True, tiny_random_config=json.dumps({"num_hidden_layers": 1}))
    assert tiny.model_config.num_hidden_layers == 1
    with pytest.raises(ValueError, match="does not have"):
        Config.from_kwargs(folder, tiny_random=True, tiny_random_config=json.dumps({"layers": 1}))


# ------------------------------------------------------------------------------- weights
def load(folder, dtype=torch.bfloat16):
    raw = json.load(open(os.path.join(folder, "config.json")))
    arch = resolve_architecture(raw)
    cfg = arch.parse_config(raw)
    decls = build_model(arch.build_spec(cfg)).all_param_decls()
    return loader.load_parameters(folder, arch, cfg, decls, dtype, "cpu"), cfg


def test_random_folder_is_seeded_by_name_and_loads_by_name(tmp_path):
    a = make_folder(tmp_path / "one", "A")
    b = make_folder(tmp_path / "two", "A")
    ta, tb = load_file(os.path.join(a, "model.safetensors")), load_file(os.path.join(b, "model.safetensors"))
    assert ta.keys() == tb.keys() and all(torch.equal(ta[k], tb[k]) for k in ta)
    other = write_model_folder(str(tmp_path / "three"), CONFIGS["A"][0], 99, CONFIGS["A"][1])
    assert not torch.equal(load_file(os.path.join(other, "model.safetensors"))["lm_head.weight"], ta["lm_head.weight"])
    assert ta["model.layers.0.block_sparse_moe.gate.weight"].dtype == torch.float32
    assert ta["model.layers.0.self_attn.q_proj.weight"].dtype == torch.bfloat16
    assert abs(float(ta["model.norm.weight"].float().mean()) - 1.0) < 0.1          # norm weights 1 + N(0, 0.1)
    params, cfg = load(a)
    q, kv, inter = 64, 32, 32
    qkv = params["layers.1.mixer.qkv"]
    assert qkv.dtype == torch.bfloat16
    assert torch.equal(qkv[:q], ta["model.layers.1.self_attn.q_proj.weight"])
    assert torch.equal(qkv[q:q + kv], ta["model.layers.1.self_attn.k_proj.weight"])
    assert torch.equal(qkv[q + kv:], ta["model.layers.1.self_attn.v_proj.weight"])
    w13 = params["layers.0.ffn.w13"]
    assert torch.equal(w13[5, :inter], ta["model.layers.0.block_sparse_moe.experts.5.w1.weight"])    # gate rows first
    assert torch.equal(w13[5, inter:], ta["model.layers.0.block_sparse_moe.experts.5.w3.weight"])
    assert torch.equal(params["layers.0.ffn.w2"][5], ta["model.layers.0.block_sparse_moe.experts.5.w2.weight"])
    assert params["layers.0.ffn.router"].dtype == torch.float32 and params["layers.0.ffn.router_bias"].dtype == torch.float32
    # a float32 engine upcasts exactly; a tensor stored in 32-bit stays 32-bit under bfloat16
    p32, _ = load(a, torch.float32)
    assert p32["embed.weight"].dtype == torch.float32 and torch.equal(p32["embed.weight"], ta["model.embed_tokens.weight"].float())
    ta["model.norm.weight"] = ta["model.norm.weight"].float() + 1e-4
    ta["table.of.ints"] = torch.arange(4, dtype=torch.int64)
    save_file({k: v for k, v in ta.items() if k != "table.of.ints"}, os.path.join(a, "model.safetensors"))
    kept, _ = load(a)
    assert kept["final_norm.weight"].dtype == torch.float32 and kept["layers.0.norm_mixer.weight"].dtype == torch.bfloat16


def test_one_error_lists_everything(tmp_path):
    folder = make_folder(tmp_path, "A")
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    del tensors["model.layers.1.self_attn.o_proj.weight"]
    del tensors["model.layers.0.block_sparse_moe.experts.3.w2.weight"]
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(4)
    tensors["lm_head.weight"] = tensors["lm_head.weight"][:, :32].contiguous()
    tensors["model.mtp.0.proj.weight"] = torch.zeros(2, 2)           # ignored: not part of the decoder
    save_file(tensors, path)
    with pytest.raises(loader.WeightLoadError) as err:
        load(folder)
    e = err.value
    assert e.missing == ["model.layers.0.block_sparse_moe.experts.3.w2.weight", "model.layers.1.self_attn.o_proj.weight"]
    assert e.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert len(e.wrong_shape) == 1 and "lm_head.weight" in e.wrong_shape[0] and "[512, 32]" in e.wrong_shape[0]
    text = str(e)
    assert "missing tensors (2)" in text and "unexpected tensors (1)" in text and "wrong shapes (1)" in text


def test_duplicates_quantised_and_empty_folders(tmp_path):
    folder = make_folder(tmp_path, "A")
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    save_file({"lm_head.weight": tensors["lm_head.weight"]}, os.path.join(folder, "model-extra.safetensors"))
    with pytest.raises(loader.WeightLoadError, match="duplicate tensor lm_head.weight"):
        load(folder)
    os.remove(os.path.join(folder, "model-extra.safetensors"))
    save_file({"model.layers.0.self_attn.q_proj.weight_scale_inv": torch.ones(1, 1)}, os.path.join(folder, "scales.safetensors"))
    with pytest.raises(loader.WeightLoadError, match="quantised checkpoints are not supported"):
        load(folder)
    empty = tmp_path / "empty"
    empty.mkdir()
    (empty / "config.json").write_text(json.dumps(TINY_A))
    with pytest.raises(FileNotFoundError, match="safetensors"):
        load(str(empty))


def test_sharded_checkpoint_loads(tmp_path):
    folder = make_folder(tmp_path, "B")
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    names = sorted(tensors)
    os.remove(path)
    save_file({n: tensors[n] for n in names[::2]}, os.path.join(folder, "model-00001-of-00002.safetensors"))
    save_file({n: tensors[n] for n in names[1::2]}, os.path.join(folder, "model-00002-of-00002.safetensors"))
    params, _ = load(folder)
    assert torch.equal(params["head.weight"], tensors["lm_head.weight"])
    assert "layers.0.mixer.q_norm" not in params            # use_qk_norm = false: no such parameter


def test_rope_scaling_tables():
    """Scaled tables against the reference's formulas written out for single frequencies
    (layers/rotary_embedding.py:26-101)."""
    from sparseengine_amd.parts.position import rotary_inverse_frequencies
    base = 1.0 / (10000.0 ** (torch.arange(0, 64, 2, dtype=torch.float32) / 64))
    inv, factor = rotary_inverse_frequencies(64, 10000.0, {"rope_type": "linear", "factor": 4.0})
    torch.testing.assert_close(inv, base / 4) and factor == 1.0
    inv, _ = rotary_inverse_frequencies(64, 10000.0, {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                                      "high_freq_factor": 4.0, "original_max_position_embeddings": 8192})
    wavelength = 2 * torch.pi / base
    assert torch.equal(inv[wavelength < 8192 / 4], base[wavelength < 8192 / 4])               # short waves untouched
    torch.testing.assert_close(inv[wavelength > 8192], base[wavelength > 8192] / 8)          # long waves slowed
    mid = (wavelength >= 8192 / 4) & (wavelength <= 8192)
    assert mid.any() and ((inv[mid] < base[mid]) & (inv[mid] > base[mid] / 8)).all()
    inv, factor = rotary_inverse_frequencies(64, 10000.0, {"rope_type": "yarn", "factor": 4.0,
                                                           "original_max_position_embeddings": 4096})
    assert factor == pytest.approx(0.1 * torch.log(torch.tensor(4.0)).item() + 1.0)
    assert torch.equal(inv[:8], base[:8]) and torch.allclose(inv[-4:], base[-4:] / 4)         # fast dims kept, slow dims scaled


def test_command_line_options_and_random_folder(tmp_path):
    """Every field of Config and SamplingParams is an option; the one name both have is told apart;
    ``random`` writes a folder that loads."""
    from sparseengine_amd.__main__ import _collect, build_parser, main
    from sparseengine_amd.sampling.params import SamplingParams
    parser = build_parser()
    args = parser.parse_args(["generate", "--model", "/x", "--prompt-ids", "[1, 2]", "--max-tokens", "6",
                              "--temperature", "0.8", "--top-k", "5", "--seed", "7", "--dtype", "float32",
                              "--eos-token-ids", "[3]", "--sampling-eos-token-ids", "[4, 5]", "--kv-page-size", "16",
                              "--no-ignore-eos", "--max-num-batched-tokens", "auto"])
    assert _collect(args, Config, skip=("model",)) == {"eos_token_ids": [3], "dtype": "float32", "kv_page_size": 16,
                                                       "max_num_batched_tokens": "auto"}
    assert _collect(args, SamplingParams, prefix="sampling_") == {
        "temperature": 0.8, "top_k": 5, "max_tokens": 6, "ignore_eos": False, "eos_token_ids": [4, 5], "seed": 7}
    SamplingParams(**_collect(args, SamplingParams, prefix="sampling_"))
    with pytest.raises(SystemExit):
        parser.parse_args(["generate", "--model", "/x", "--no-such-option", "1"])
    config_file = tmp_path / "config.json"
    config_file.write_text(json.dumps(TINY_A))
    out = tmp_path / "model"
    assert main(["random", "--config", str(config_file), "--out", str(out), "--seed", "3"]) == 0
    assert json.load(open(out / "config.json"))["hidden_size"] == TINY_A["hidden_size"]
    params, _ = load(str(out))            # the written folder loads, tensor for tensor
    assert params["embed.weight"].shape == (TINY_A["vocab_size"], TINY_A["hidden_size"])
