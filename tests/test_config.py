"""Configuration, registry and catalog (no GPU)."""
import json

import pytest

from rocml_amd.config import (AttentionSpec, ModelSpec, Qwen3Config, ScheduleEntry, architecture,
                              architecture_of, known_architectures)
from rocml_amd.config.catalog import CATALOG, catalog_names, resolve
from rocml_amd.errors import ConfigError, UnknownModelError, UnsupportedArchitectureError
from tests import helpers


def test_reads_every_size_from_config_json():
    for cfg in (helpers.TINY_A, helpers.TINY_B, helpers.TINY_C, helpers.TINY_D, helpers.TINY_E, helpers.TINY_F, helpers.TINY_G, helpers.TINY_H):
        c = Qwen3Config.from_dict(cfg)
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim", "rope_theta", "rms_norm_eps",
                    "max_position_embeddings", "tie_word_embeddings"):
            assert getattr(c, key) == cfg[key]
        assert Qwen3Config.from_dict(c.to_dict()) == c          # survives a round trip
    b = Qwen3Config.from_dict(helpers.TINY_B)
    assert b.q_dim == 192 and b.q_dim != b.hidden_size             # head_dim is its own key


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "num_key_value_heads", "head_dim", "rope_theta",
                                 "rms_norm_eps", "max_position_embeddings"])
def test_missing_key_is_named(key):
    cfg = dict(helpers.TINY_A)
    del cfg[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(cfg)


@pytest.mark.parametrize("change,word", [
    ({"num_attention_heads": 5}, "multiple"), ({"head_dim": 15}, "even"), ({"hidden_size": 0}, "positive"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"), ({"hidden_act": "gelu"}, "hidden_act"),
    ({"attention_bias": True}, "bias"), ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"),
    ({"layer_types": ["full_attention"]}, "layer_types"), ({"vocab_size": "big"}, "integer"),
    ({"layer_types": ["sliding_attention", "full_attention"]}, "sliding_window")])
def test_rules(change, word):
    with pytest.raises(ConfigError, match=word):
        Qwen3Config.from_dict(dict(helpers.TINY_A, **change))


def test_unknown_architecture_lists_known_ones():
    with pytest.raises(UnsupportedArchitectureError, match="Qwen3ForCausalLM"):
        architecture("LlamaForCausalLM")
    with pytest.raises(UnsupportedArchitectureError):
        Qwen3Config.from_dict(dict(helpers.TINY_A, architectures=["LlamaForCausalLM"]))
    assert architecture_of(helpers.TINY_A).name == "Qwen3ForCausalLM"
    assert "Qwen3ForCausalLM" in known_architectures()
    with pytest.raises(ConfigError):
        architecture_of({"hidden_size": 4})


def test_spec_carries_layer_by_layer_choices():
    spec = Qwen3Config.from_dict(helpers.TINY_D).to_model_spec()
    assert [b.mixer.window for b in spec.layers] == [None, 70, None, 70]
    m = spec.layers[0].mixer
    assert isinstance(m, AttentionSpec) and (m.n_heads, m.n_kv_heads, m.head_dim) == (4, 1, 64)
    assert m.scale == pytest.approx(1 / 8) and m.qk_norm.eps == 2e-5 and m.position.theta == 20000.0
    assert [e.layer for e in spec.schedule] == [0, 1, 2, 3]
    assert spec.tie_lm_head and spec.final_norm.size == 72
    old_style = dict(helpers.TINY_D, use_sliding_window=True, max_window_layers=2)
    del old_style["layer_types"]
    assert [b.mixer.window for b in Qwen3Config.from_dict(old_style).to_model_spec().layers] == [None, None, 70, 70]


def test_schedule_rules():
    spec = Qwen3Config.from_dict(helpers.TINY_A).to_model_spec()

    def with_schedule(*entries):
        return ModelSpec(**{**spec.__dict__, "schedule": tuple(entries)})

    with_schedule(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1), ScheduleEntry(0, reads_cache_of=0)).validate()
    with pytest.raises(ConfigError, match="names layer"):
        with_schedule(ScheduleEntry(2)).validate()
    with pytest.raises(ConfigError, match="does not run before"):
        with_schedule(ScheduleEntry(0, reads_cache_of=1), ScheduleEntry(1)).validate()
    with pytest.raises(ConfigError, match="no cache line"):
        with_schedule(ScheduleEntry(0), ScheduleEntry(1, reads_cache_of=0), ScheduleEntry(1, reads_cache_of=1)).validate()


def test_catalog_and_resolve(tmp_path):
    assert len(set(catalog_names())) == len(CATALOG)              # names are unique
    for e in CATALOG:
        Qwen3Config.from_dict(e.config)                            # every entry is a valid configuration
    assert resolve("qwen3-8b").entry.config["num_hidden_layers"] == 36
    assert resolve("qwen3-8b").entry.sampling.temperature == pytest.approx(0.6)
    with pytest.raises(UnknownModelError, match="qwen3-8b"):       # lists the known names
        resolve("qwen3-9b")
    with pytest.raises(UnknownModelError, match="config.json"):
        resolve(str(tmp_path))                                     # a folder without config.json
    (tmp_path / "config.json").write_text(json.dumps(helpers.TINY_A))
    assert resolve(str(tmp_path)).path == str(tmp_path)
    assert Qwen3Config.from_json(str(tmp_path)).hidden_size == 64
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        Qwen3Config.from_json(str(tmp_path))


def test_decode_splits_fill_the_chip_evenly():
    """Key-range splits of a decode step: about a block a CU for a few sequences; from eight
    sequences' worth of (token, kv head) pairs on, the count that leaves the busiest CU the least
    work when every block and every merge has a fixed price; never more than the pages there are."""
    from rocml_amd.ops import decode_splits
    assert [decode_splits(b * 8, 256, 64) for b in (1, 2, 4, 8, 16, 32, 64, 128)] == [32, 16, 8, 4, 2, 1, 1, 1]
    assert decode_splits(24 * 8, 256, 64) == 1          # 192 blocks, one a CU with two pieces on their way, no merge
    assert decode_splits(14 * 8, 256, 64) == 2          # not 9: 1,008 tiny blocks and a merge of nine
    assert decode_splits(18 * 8, 256, 64) == 3          # 432 blocks, under two a CU
    assert decode_splits(40 * 8, 256, 64) == 3          # 960 blocks: two rounds of two a CU
    assert decode_splits(48 * 8, 256, 64) == 2
    assert decode_splits(20 * 8, 256, 64) == 3          # 480 of 512 is near enough
    assert decode_splits(16 * 8, 256, 1) == 1           # one page in the table: nothing to split
    assert decode_splits(8, 256, 5) == 5 and decode_splits(4096, 256, 64) == 1
