"""Configuration, registry, safetensors reading and the loader's errors (no GPU)."""
import json
import os

import pytest
import torch
from safetensors import safe_open
from safetensors.torch import save_file

from pico_vllm_amd.config import (ConfigError, EngineArgs, Qwen2Config, known_architectures,
                                  load_model_description, resolve_architecture)
from pico_vllm_amd.parts.model import model_param_specs
from pico_vllm_amd.parts.spec import ParamSpec
from pico_vllm_amd.weights.loader import WeightsError, load_checkpoint
from pico_vllm_amd.weights.random_init import write_random_model
from pico_vllm_amd.weights.safetensors_io import SafetensorsFile, write_safetensors
from tiny_configs import CONFIGS, TINY_A, TINY_B, model_dir


def test_config_reads_every_key_and_has_no_size_defaults():
    for raw in CONFIGS.values():
        cfg = Qwen2Config.from_dict(raw)
        for k in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                  "intermediate_size", "rms_norm_eps", "rope_theta", "tie_word_embeddings"):
            assert getattr(cfg, k) == raw[k]
        assert cfg.head_dim == raw.get("head_dim", raw["hidden_size"] // raw["num_attention_heads"])
    for k in ("vocab_size", "hidden_size", "num_hidden_layers", "intermediate_size", "rms_norm_eps", "rope_theta",
              "tie_word_embeddings", "num_key_value_heads"):
        bad = dict(TINY_A)
        del bad[k]
        with pytest.raises(ConfigError, match=k):
            Qwen2Config.from_dict(bad)


@pytest.mark.parametrize("patch,word", [
    ({"num_key_value_heads": 3}, "multiple"), ({"hidden_act": "gelu"}, "hidden_act"),
    ({"use_sliding_window": True}, "sliding"), ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"),
    ({"hidden_size": 66}, "head_dim"), ({"head_dim": 15}, "even"), ({"attention_bias": False}, "bias"),
    ({"vocab_size": 0}, "vocab_size"), ({"hidden_size": "64"}, "hidden_size must be an integer"),
    ({"vocab_size": 255.5}, "vocab_size must be an integer"), ({"num_hidden_layers": True}, "must be an integer"),
    ({"rms_norm_eps": "1e-6"}, "rms_norm_eps must be a number"), ({"tie_word_embeddings": "yes"}, "true or false"),
    ({"max_position_embeddings": 0}, "max_position_embeddings"), ({"eos_token_id": "3"}, "eos_token_id"),
    ({"architectures": "Qwen2ForCausalLM"}, "list of names"),
])
def test_config_rejects_what_the_engine_cannot_run(patch, word):
    with pytest.raises(ConfigError, match=word):
        Qwen2Config.from_dict({**TINY_A, **patch})


def test_a_config_file_that_is_missing_or_broken_and_the_way_back_to_a_file(tmp_path):
    from pico_vllm_amd.config.model_config import read_config_json
    with pytest.raises(ConfigError, match="does not exist"):
        read_config_json(str(tmp_path))
    (tmp_path / "config.json").write_text('{"vocab_size": 256,')
    with pytest.raises(ConfigError, match="not valid JSON"):
        read_config_json(str(tmp_path))
    cfg = Qwen2Config.from_dict({**TINY_A, "eos_token_id": [7, 9], "some_future_key": 1})
    assert cfg.eos_token_id == 7 and cfg.ignored_keys == ("some_future_key",) and cfg.num_kv_groups == 4
    assert Qwen2Config.from_dict({**TINY_A, "eos_token_id": []}).eos_token_id is None
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_dict()))
    assert Qwen2Config.from_dict(read_config_json(str(tmp_path))) == cfg      # what it writes, it reads
    for key, word in (("rms_norm_eps", "rms_norm_eps"), ("rope_theta", "rope_theta")):
        with pytest.raises(ConfigError, match=word):
            Qwen2Config.from_dict({**TINY_A, key: 0.0})


def test_registry_resolves_by_name_and_lists_known_names():
    assert "Qwen2ForCausalLM" in known_architectures()
    assert resolve_architecture(TINY_A).name == "Qwen2ForCausalLM"
    with pytest.raises(ConfigError, match="Qwen2ForCausalLM"):
        resolve_architecture({**TINY_A, "architectures": ["LlamaForCausalLM"]})
    with pytest.raises(ConfigError, match="architectures"):
        resolve_architecture({k: v for k, v in TINY_A.items() if k != "architectures"})


def test_spec_is_data_layer_by_layer():
    _, cfg, spec = load_model_description(model_dir("B"))
    assert len(spec.layers) == 3 and [e.layer for e in spec.run_order] == [0, 1, 2]
    attn = spec.layers[1].slots["mixer"][1]
    assert attn.kind == "gqa_attention" and attn.params["num_kv_heads"] == 3 and attn.params["head_dim"] == 32
    assert attn.params["position"].params["theta"] == 1e6
    assert spec.layers[0].slots["norm1"][1].params["eps"] == 1e-5
    assert spec.head_name == "lm_head.weight"
    names = {p.name for p in model_param_specs(spec)}
    assert "model.layers.2.self_attn.k_proj.bias" in names and "model.layers.0.mlp.gate_proj.weight" in names
    assert "lm_head.weight" in names and "model.norm.weight" in names
    _, _, spec_a = load_model_description(model_dir("A"))
    assert spec_a.head_name is None and "lm_head.weight" not in {p.name for p in model_param_specs(spec_a)}


def test_engine_args_validate():
    EngineArgs(model="x").validate()
    with pytest.raises(ValueError):
        EngineArgs(dtype="float16").validate()
    with pytest.raises(ValueError):
        EngineArgs(block_size=12).validate()
    for bad in (dict(prefill_chunk=0), dict(num_gpu_blocks=0), dict(kv_memory_fraction=0.0), dict(kv_memory_fraction=1.5)):
        with pytest.raises(ValueError, match=next(iter(bad))):
            EngineArgs(**bad).validate()
    EngineArgs(prefill_chunk=512, num_gpu_blocks=10, kv_memory_fraction=1.0).validate()


# ---- safetensors -----------------------------------------------------------
def test_own_reader_agrees_with_the_safetensors_package(tmp_path):
    t = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int32)}
    save_file(t, str(tmp_path / "x.safetensors"))
    with SafetensorsFile(str(tmp_path / "x.safetensors")) as sf:
        assert set(sf.entries) == set(t)
        for k, v in t.items():
            assert torch.equal(sf.tensor(k), v) and sf.tensor(k).dtype == v.dtype


def test_own_writer_is_read_by_the_safetensors_package(tmp_path):
    t = {"w": torch.randn(4, 6).to(torch.bfloat16), "n": torch.rand(6)}
    write_safetensors(str(tmp_path / "y.safetensors"), [(k, tuple(v.shape), v.dtype) for k, v in t.items()],
                      lambda name: t[name])
    with safe_open(str(tmp_path / "y.safetensors"), framework="pt") as f:
        assert set(f.keys()) == set(t)
        for k in t:
            assert torch.equal(f.get_tensor(k), t[k])


def test_random_model_is_seeded_and_typed():
    a1, a2, b = model_dir("A", 0), model_dir("A", 0), model_dir("A", 1)
    with SafetensorsFile(os.path.join(a1, "model.safetensors")) as f1, \
            SafetensorsFile(os.path.join(b, "model.safetensors")) as f2:
        q1, q2 = f1.tensor("model.layers.0.self_attn.q_proj.weight"), f2.tensor("model.layers.0.self_attn.q_proj.weight")
        assert q1.dtype == torch.bfloat16 and not torch.equal(q1, q2)
        n = f1.tensor("model.norm.weight")
        assert n.dtype == torch.float32 and float(n.min()) >= 0.9 and float(n.max()) <= 1.1
    with open(os.path.join(a1, "config.json")) as f:
        assert json.load(f)["vocab_size"] == 256
    assert a1 == a2


def test_random_model_distributions(tmp_path):
    d = write_random_model(str(tmp_path / "m"), TINY_B, seed=3)
    with SafetensorsFile(os.path.join(d, "model.safetensors")) as f:
        w = f.tensor("model.layers.1.mlp.gate_proj.weight").float()
        assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.001
        b = f.tensor("model.layers.1.self_attn.q_proj.bias").float()
        assert abs(float(b.std()) - 0.02) < 0.006


# ---- loader ----------------------------------------------------------------
def _specs(name):
    return model_param_specs(load_model_description(model_dir(name))[2])


def test_loader_keeps_bf16_and_widens_for_the_32_bit_engine():
    d = model_dir("A")
    t = load_checkpoint(d, _specs("A"), torch.bfloat16)
    assert t["model.layers.0.mlp.down_proj.weight"].dtype == torch.bfloat16
    assert t["model.norm.weight"].dtype == torch.float32               # norm weights are always 32 bit
    t32 = load_checkpoint(d, _specs("A"), torch.float32)
    assert all(v.dtype == torch.float32 for v in t32.values())
    assert torch.equal(t32["model.embed_tokens.weight"], t["model.embed_tokens.weight"].float())


def test_a_tensor_stored_in_32_bit_stays_so_and_tables_are_int32(tmp_path):
    save_file({"m": torch.randn(4, 4), "h": torch.randn(4, 4).half(), "t": torch.arange(4, dtype=torch.int64)},
              str(tmp_path / "model.safetensors"))
    specs = [ParamSpec("m", (4, 4)), ParamSpec("h", (4, 4)), ParamSpec("t", (4,), role="table")]
    out = load_checkpoint(str(tmp_path), specs, torch.bfloat16)
    assert out["m"].dtype == torch.float32 and out["h"].dtype == torch.bfloat16 and out["t"].dtype == torch.int32


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = model_dir("A")
    with safe_open(os.path.join(d, "model.safetensors"), framework="pt") as f:
        t = {k: f.get_tensor(k) for k in f.keys()}
    del t["model.layers.1.self_attn.v_proj.bias"]
    del t["model.norm.weight"]
    t["model.layers.0.mlp.up_proj.weight"] = torch.zeros(10, 64, dtype=torch.bfloat16)
    t["model.layers.7.extra.weight"] = torch.zeros(2)
    os.makedirs(tmp_path / "m")
    save_file(t, str(tmp_path / "m" / "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_checkpoint(str(tmp_path / "m"), _specs("A"), torch.bfloat16)
    err = e.value
    assert err.missing == ["model.layers.1.self_attn.v_proj.bias", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.extra.weight"]
    assert [(n, tuple(x), tuple(y)) for n, x, y in err.wrong_shape] == [("model.layers.0.mlp.up_proj.weight", (172, 64), (10, 64))]
    msg = str(err)
    for word in ("missing", "unexpected", "wrong shapes", "v_proj.bias", "extra.weight", "[172, 64]", "[10, 64]"):
        assert word in msg


def test_tied_model_ignores_a_stored_lm_head_and_untied_needs_it(tmp_path):
    d = model_dir("A")
    with safe_open(os.path.join(d, "model.safetensors"), framework="pt") as f:
        t = {k: f.get_tensor(k) for k in f.keys()}
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    os.makedirs(tmp_path / "m")
    save_file(t, str(tmp_path / "m" / "model.safetensors"))
    load_checkpoint(str(tmp_path / "m"), _specs("A"), torch.bfloat16, optional=["lm_head.weight"])
    # the model description names what a file may hold unasked: the tied configuration does, by name or by pattern
    from pico_vllm_amd.config.registry import resolve_architecture
    arch = resolve_architecture(CONFIGS["A"])
    assert arch.build_spec(arch.config_from_dict(CONFIGS["A"])).ignored_tensors == ("lm_head.weight",)
    assert arch.build_spec(arch.config_from_dict(CONFIGS["B"])).ignored_tensors == ()
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    save_file(t, str(tmp_path / "m" / "model.safetensors"))
    with pytest.raises(WeightsError) as e:
        load_checkpoint(str(tmp_path / "m"), _specs("A"), torch.bfloat16, optional=["lm_head.weight"])
    assert e.value.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    load_checkpoint(str(tmp_path / "m"), _specs("A"), torch.bfloat16, optional=["lm_head.weight", "*.rotary_emb.inv_freq"])
    with pytest.raises(WeightsError) as e:
        load_checkpoint(d, _specs("A") + [ParamSpec("lm_head.weight", (256, 64))], torch.bfloat16)
    assert e.value.missing == ["lm_head.weight"]


def test_a_tensor_stored_twice_or_as_the_wrong_kind_of_number(tmp_path):
    from pico_vllm_amd.weights.safetensors_io import write_safetensors
    specs = [ParamSpec("w", (2, 4)), ParamSpec("table", (3,), role="table")]
    made = {"w": torch.ones(2, 4, dtype=torch.bfloat16), "table": torch.arange(3, dtype=torch.int64)}

    def store(name, names, tensors=made):
        write_safetensors(str(tmp_path / name), [(n, tuple(tensors[n].shape), tensors[n].dtype) for n in names], tensors.__getitem__)

    store("model-1.safetensors", ["w", "table"])
    out = load_checkpoint(str(tmp_path), specs, torch.bfloat16)
    assert out["w"].dtype == torch.bfloat16 and out["table"].dtype == torch.int32 and out["table"].tolist() == [0, 1, 2]
    store("model-2.safetensors", ["w"])
    with pytest.raises(WeightsError, match="tensor w is stored twice"):
        load_checkpoint(str(tmp_path), specs, torch.bfloat16)
    (tmp_path / "model-2.safetensors").unlink()
    store("model-1.safetensors", ["w", "table"], {"w": torch.ones(2, 4, dtype=torch.int32), "table": torch.ones(3)})
    with pytest.raises(WeightsError) as e:
        load_checkpoint(str(tmp_path), specs, torch.bfloat16)
    assert "tensor w is stored as I32" in str(e.value) and "tensor table is stored as F32" in str(e.value)


def test_truncated_and_empty_folders(tmp_path):
    with pytest.raises(WeightsError, match="no .safetensors"):
        load_checkpoint(str(tmp_path), _specs("A"), torch.bfloat16)
    src = os.path.join(model_dir("A"), "model.safetensors")
    with open(src, "rb") as f:
        data = f.read()
    (tmp_path / "model.safetensors").write_bytes(data[:len(data) // 2])
    with pytest.raises(WeightsError, match="truncated"):
        load_checkpoint(str(tmp_path), _specs("A"), torch.bfloat16)


def test_a_malformed_header_is_one_clear_error_and_leaves_no_file_open(tmp_path):
    import struct
    import warnings

    def stored(header: bytes, body: bytes = b""):
        (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", len(header)) + header + body)

    cases = {
        b"[1, 2]": "not a JSON object",
        b"{not json": "not valid JSON",
        b'{"w": {"dtype": "BF16", "shape": [2, 2]}}': "needs dtype, shape and data_offsets",
        b'{"w": {"dtype": "BF16", "shape": [2, 2], "data_offsets": [-8, 0]}}': "shape .* needs 8",
        b'{"w": {"dtype": "BF16", "shape": [2, 2], "data_offsets": [0, 6]}}': "shape .* needs 8",
        b'{"w": {"dtype": "F8_E4M3", "shape": [2, 2], "data_offsets": [0, 4]}}': "unsupported dtype",
        b'{"w": {"dtype": "BF16", "shape": [2, 2], "data_offsets": [0, 8]}}': "truncated inside",
    }
    with warnings.catch_warnings():
        warnings.simplefilter("error", ResourceWarning)
        for header, message in cases.items():
            stored(header, b"\0" * 4)
            with pytest.raises(WeightsError, match=message):
                load_checkpoint(str(tmp_path), _specs("A"), torch.bfloat16)
        import gc
        gc.collect()


def test_named_configurations_parse_and_the_tiny_ones_differ_in_every_size():
    from pico_vllm_amd.config.model_config import Qwen2Config
    from pico_vllm_amd.config.presets import PRESETS, preset
    cfgs = {n: Qwen2Config.from_dict(preset(n)) for n in PRESETS}
    a, b = cfgs["tiny-a"], cfgs["tiny-b"]
    for f in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads", "head_dim",
              "intermediate_size", "rms_norm_eps", "rope_theta", "tie_word_embeddings"):
        assert getattr(a, f) != getattr(b, f), f
    big = cfgs["1.5b"]
    assert (big.hidden_size, big.num_attention_heads, big.num_key_value_heads, big.head_dim, big.vocab_size) == \
        (1536, 12, 2, 128, 151936)
    with pytest.raises(ValueError):
        preset("3b")



def test_the_command_line_writes_a_model_folder_from_a_named_size_or_a_config_file(tmp_path, capsys):
    from pico_vllm_amd import run
    from pico_vllm_amd.config.presets import preset
    from pico_vllm_amd.weights.safetensors_io import SafetensorsFile
    a, b = str(tmp_path / "a"), str(tmp_path / "b")
    assert run.main(["--write-random", a, "--random-config", "tiny-b", "--seed", "3"]) == 0
    (tmp_path / "cfg.json").write_text(json.dumps(preset("tiny-b")))
    assert run.main(["--write-random", b, "--config", str(tmp_path / "cfg.json"), "--seed", "3"]) == 0
    assert capsys.readouterr().out.splitlines() == [f"wrote {a}", f"wrote {b}"]
    with SafetensorsFile(os.path.join(a, "model.safetensors")) as fa, SafetensorsFile(os.path.join(b, "model.safetensors")) as fb:
        assert fa.entries == fb.entries and len(fa.entries) > 10
        assert all(torch.equal(fa.tensor(n), fb.tensor(n)) for n in fa.entries)
    load_checkpoint(a, model_param_specs(load_model_description(a)[2]), torch.bfloat16)
    for argv in (["--write-random", a], [], ["--random-config", "tiny-a"]):      # no size; no model; no prompt
        with pytest.raises(SystemExit) as e:
            run.main(argv)
        assert e.value.code == 2
    capsys.readouterr()


def test_parts_are_found_by_category_and_kind_and_unknown_ones_are_named():
    from pico_vllm_amd.parts.registry import CATEGORIES, part_class, register_part
    assert part_class("position", "none").__name__ == "NoPosition"
    assert {part_class(c, k).__name__ for c, k in (("mixer", "gqa_attention"), ("feed_forward", "swiglu_mlp"), ("norm", "rms_norm"),
                                                     ("position", "rotary_half"), ("block", "prenorm"))} \
        == {"GQAAttention", "SwiGLUMLP", "RMSNorm", "RotaryHalf", "PreNormBlock"}
    with pytest.raises(KeyError, match="no mixer part of kind 'mamba' is registered; known: .*gqa_attention"):
        part_class("mixer", "mamba")
    with pytest.raises(KeyError, match="unknown part category 'router'"):
        register_part("router", "top2")
    with pytest.raises(KeyError, match="no router part"):
        part_class("router", "top2")
    assert set(CATEGORIES) == {"mixer", "feed_forward", "norm", "position", "block", "stream"}


def test_parts_refuse_sizes_that_make_no_sense_when_they_are_built():
    from pico_vllm_amd.parts.attention import GQAAttention
    from pico_vllm_amd.parts.rotary import RotaryHalf
    from pico_vllm_amd.parts.spec import PartSpec
    none = PartSpec("none", {})
    GQAAttention(64, 4, 2, 16, True, none)
    for args, message in (((64, 4, 3, 16, True, none), "not a multiple"), ((64, 4, 2, 272, True, none), "head size"),
                          ((64, 4, 2, 0, True, none), "head size")):
        with pytest.raises(ValueError, match=message):
            GQAAttention(*args)
    with pytest.raises(ValueError, match="window must not be negative"):
        GQAAttention(64, 4, 2, 16, True, none, window=-1)
    with pytest.raises(ValueError, match="rotary_dim must be even"):
        RotaryHalf(15, 10000.0)


def test_a_description_that_does_not_hold_together_is_refused_when_the_model_is_built():
    import dataclasses
    from pico_vllm_amd.config.qwen2 import qwen2_spec
    from pico_vllm_amd.ops.linear import Linear
    from pico_vllm_amd.parts.model import DecoderModel, load_model
    from pico_vllm_amd.parts.spec import LayerSpec, PartSpec, RunEntry
    from tiny_configs import TINY_B
    spec = qwen2_spec(Qwen2Config.from_dict(TINY_B))
    assert len(spec.layers) == 3
    model = DecoderModel(spec, torch.float32, "cpu")               # building needs no GPU, only running does
    assert sorted(model.cache_specs()) == [0, 1, 2]

    def refused(message, **changes):
        with pytest.raises(ValueError, match=message):
            DecoderModel(dataclasses.replace(spec, **changes), torch.float32, "cpu")

    refused("run order names layer 5, the model has 3", run_order=[RunEntry(0), RunEntry(5)])
    refused("run entry 1: cache_of must name an earlier entry", run_order=[RunEntry(0), RunEntry(1, cache_of=1)])
    refused("run entry 2: cache_of must name an earlier entry that owns its cache",
            run_order=[RunEntry(0), RunEntry(1, cache_of=0), RunEntry(2, cache_of=1)])
    shared = DecoderModel(dataclasses.replace(spec, run_order=[RunEntry(0), RunEntry(1, cache_of=0), RunEntry(0)]), torch.float32, "cpu")
    assert sorted(shared.cache_specs()) == [0, 2]                  # the second run reads the first one's cache
    l1 = spec.layers[1]
    name, attn = l1.slots["mixer"]
    windowed = LayerSpec(l1.prefix, l1.block, {**l1.slots, "mixer": (name, PartSpec(attn.kind, dict(attn.params, window=8)))})
    refused("run entry 1 cannot use the cache of entry 0: different cache needs",
            layers=[spec.layers[0], windowed, spec.layers[2]], run_order=[RunEntry(0), RunEntry(1, cache_of=0), RunEntry(2)])
    no_ff = LayerSpec(l1.prefix, l1.block, {k: v for k, v in l1.slots.items() if k != "ff"})
    refused(r"layer model.layers.1: block 'prenorm' needs slots \['ff'\]", layers=[spec.layers[0], no_ff, spec.layers[2]])
    with pytest.raises(ValueError, match="dtype must be one of"):
        load_model(model_dir("A"), "float16", "cpu")
    # the matrix product's own refusals
    with pytest.raises(ValueError, match="a linear weight is a matrix"):
        Linear(torch.zeros(8))
    lin = Linear(torch.zeros(4, 8, dtype=torch.bfloat16), torch.zeros(4))
    assert (lin.out_features, lin.in_features) == (4, 8) and lin.bias.dtype == torch.bfloat16 and lin.bias_f32.dtype == torch.float32
    with pytest.raises(ValueError, match="input has 6 features, the weight wants 8"):
        lin(torch.zeros(2, 6, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="bfloat16 weights need bfloat16 activations"):
        lin(torch.zeros(2, 8))
