"""The benchmark asks the model's parts and the architecture's registry entry for sizes, bytes and flops: it reads no
key of any architecture's configuration, so another architecture can use it as it is."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_bench_names_no_configuration_key():
    from pico_vllm_amd.config.presets import PRESETS
    keys = {k for cfg in PRESETS.values() for k in cfg} - {"architectures"}
    with open(os.path.join(ROOT, "bench.py")) as f:
        text = f.read()
    found = sorted(k for k in keys if re.search(r"[\"']%s[\"']" % re.escape(k), text))
    assert not found, f"bench.py reads configuration keys {found}"


def test_the_registry_entry_gives_the_sizes_a_report_needs():
    from pico_vllm_amd.config.presets import preset
    from pico_vllm_amd.config.registry import resolve_architecture
    raw = preset("7b")
    arch = resolve_architecture(raw)
    sizes = arch.sizes(arch.config_from_dict(raw))
    assert sizes == {"layers": 28, "hidden": 3584, "q_heads": 28, "kv_heads": 4, "head_dim": 128, "intermediate": 18944,
                     "vocab": 152064, "tied": False}
    assert all(isinstance(v, (int, float, bool)) for v in sizes.values())        # flat: a record keeps nothing deeper
    fewer = arch.with_layers(raw, 3)
    assert arch.sizes(arch.config_from_dict(fewer))["layers"] == 3 and raw["num_hidden_layers"] == 28
    assert {k: v for k, v in arch.sizes(arch.config_from_dict(fewer)).items() if k != "layers"} == \
        {k: v for k, v in sizes.items() if k != "layers"}
