"""Configuration, registry and command line (no GPU)."""
import argparse
import json

import pytest

from conftest import TINY_A, TINY_B, TINY_C
from ullm_amd.config import ConfigError, EngineConfig, Qwen3Config, read_config_json
from ullm_amd.models import MODEL_REGISTRY, build_model, resolve_architecture


def test_reads_every_size_from_the_config():
    for d in (TINY_A, TINY_B, TINY_C):
        c = Qwen3Config.from_dict(d)
        for key in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                    "head_dim", "intermediate_size", "max_position_embeddings", "rms_norm_eps", "rope_theta",
                    "tie_word_embeddings", "attention_bias"):
            assert getattr(c, key) == d[key], key


def test_defaults_follow_the_reference():
    d = {k: v for k, v in TINY_A.items() if k not in ("head_dim", "rope_theta", "attention_bias",
                                                      "tie_word_embeddings", "use_sliding_window")}
    c = Qwen3Config.from_dict(d)
    assert c.head_dim == d["hidden_size"] // d["num_attention_heads"]     # ullm/models/qwen3.py:78
    assert c.rope_theta == 1000000.0                                       # ullm/models/qwen3.py:144
    assert c.attention_bias is False and c.tie_word_embeddings is False
    assert all(c.window_of_layer(i) == 0 for i in range(c.num_hidden_layers))


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads", "intermediate_size",
                                 "vocab_size", "rms_norm_eps", "max_position_embeddings", "architectures"])
def test_missing_required_key_is_named(key):
    d = dict(TINY_B)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(d)


def test_bad_values_are_refused():
    with pytest.raises(ConfigError, match="multiple"):
        Qwen3Config.from_dict(dict(TINY_A, num_attention_heads=5))
    with pytest.raises(ConfigError, match="hidden_act"):
        Qwen3Config.from_dict(dict(TINY_A, hidden_act="gelu"))
    with pytest.raises(ConfigError, match="sliding_window"):
        Qwen3Config.from_dict(dict(TINY_A, use_sliding_window=True))
    with pytest.raises(ConfigError, match="expected int"):
        Qwen3Config.from_dict(dict(TINY_A, hidden_size="64"))


def test_window_is_chosen_layer_by_layer():
    c = Qwen3Config.from_dict(TINY_C)
    assert [c.window_of_layer(i) for i in range(3)] == [0, 24, 24]
    # a list of the layers' kinds wins over max_window_layers; without use_sliding_window it may name no window
    kinds = ["sliding_attention", "full_attention", "sliding_attention"]
    listed = Qwen3Config.from_dict(dict(TINY_C, layer_types=kinds))
    assert [listed.window_of_layer(i) for i in range(3)] == [24, 0, 24] and listed.to_dict()["layer_types"] == kinds
    plain = Qwen3Config.from_dict(dict(TINY_A, layer_types=["full_attention"] * TINY_A["num_hidden_layers"]))
    assert all(plain.window_of_layer(i) == 0 for i in range(plain.num_hidden_layers))
    with pytest.raises(ConfigError, match="layer_types"):
        Qwen3Config.from_dict(dict(TINY_C, layer_types=kinds[:2]))
    with pytest.raises(ConfigError, match="layer_types"):
        Qwen3Config.from_dict(dict(TINY_C, layer_types=["full_attention", "chunked", "full_attention"]))
    with pytest.raises(ConfigError, match="use_sliding_window"):
        Qwen3Config.from_dict(dict(TINY_C, use_sliding_window=False, layer_types=kinds))
    _, model = build_model(TINY_C)
    groups, cache_group, states = model.cache_layout()
    assert len(groups) == 2 and not states
    by_window = {g.window: g for g in groups}
    assert by_window[0].layers == ((0, 0),) and by_window[24].layers == ((1, 0), (2, 0))    # (cache id, need index)


def test_registry_maps_the_architecture_name():
    assert "Qwen3ForCausalLM" in MODEL_REGISTRY
    assert resolve_architecture(TINY_A).name == "Qwen3ForCausalLM"
    with pytest.raises(ConfigError, match="not supported"):
        resolve_architecture({"architectures": ["LlamaForCausalLM"]})
    cfg, model = build_model(TINY_B)
    assert len(model.blocks) == TINY_B["num_hidden_layers"]
    names = {d.name: d.shape for d in model.weight_decls()}
    assert names["model.layers.2.self_attn.q_proj.weight"] == (8 * 32, 96)     # heads*head_dim != hidden
    assert names["model.layers.0.self_attn.q_norm.weight"] == (32,)
    assert names["lm_head.weight"] == (503, 96)


def test_read_config_json_errors(tmp_path):
    with pytest.raises(ConfigError, match="no config.json"):
        read_config_json(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        read_config_json(str(tmp_path))


def test_engine_config_names_and_checks(tmp_path):
    ap = argparse.ArgumentParser()
    EngineConfig.add_cli_args(ap)
    args = ap.parse_args(["--model", str(tmp_path), "--max-bs", "7", "--context-len", "300", "--dtype", "fp32",
                          "--page-size", "32", "--enforce-eager", "--gpu-memory-utilization", "0.5"])
    ec = EngineConfig.from_args(args)
    assert (ec.max_bs, ec.context_len, ec.dtype, ec.page_size, ec.enforce_eager) == (7, 300, "float32", 32, True)
    # the reference's defaults (ullm/entrypoints/api_server.py:133-156)
    base = EngineConfig.from_args(ap.parse_args(["--model", "x"]))
    assert (base.gpu_memory_utilization, base.max_bs, base.context_len, base.tp_size, base.pp_size) == (0.9, 50, 2048, 1, 1)
    assert (base.nccl_port, base.device_ids, base.profile, base.profile_dir, base.disable_async_scheduling) == \
        (29500, None, False, "./profiles", False)
    other = EngineConfig.from_args(ap.parse_args(["--model", "x", "--device-ids", "3", "--profile", "--profile-dir", "/tmp/p",
                                                  "--disable-async-scheduling", "--nccl-port", "1234"]))
    assert other.device == "cuda:3" and other.profile and other.profile_dir == "/tmp/p" and other.disable_async_scheduling
    with pytest.raises(ConfigError, match="exactly one"):
        EngineConfig(model="x", device_ids=[0, 1])
    with pytest.raises(ConfigError):
        EngineConfig(model="x", tp_size=2)
    with pytest.raises(ConfigError):
        EngineConfig(model="x", page_size=12)
    with pytest.raises(ConfigError):
        EngineConfig(model="x", dtype="float16")
    (tmp_path / "generation_config.json").write_text(json.dumps({"temperature": 0.6, "top_k": 20, "top_p": 0.95}))
    assert EngineConfig(model=str(tmp_path)).generation_defaults() == {"temperature": 0.6, "top_k": 20, "top_p": 0.95}


def test_cli_parser_has_sampling_options():
    from ullm_amd.cli import build_parser
    a = build_parser().parse_args(["--model", "m", "--prompt-ids", "1,2,3", "--temperature", "0", "--top-k", "5",
                                   "--top-p", "0.9", "--min-p", "0.1", "--max-new-tokens", "4", "--ignore-eos"])
    assert a.prompt_ids == ["1,2,3"] and a.temperature == 0 and a.top_k == 5 and a.ignore_eos


def test_scaled_rotation_is_refused_not_ignored():
    """The engine builds its angles from rope_theta alone (as ullm/models/qwen3.py:97-102 does): a config that
    asks for anything else must not load."""
    for ok in (None, {"rope_type": "default"}, {"type": "default"}):
        assert Qwen3Config.from_dict(dict(TINY_A, rope_scaling=ok)).rope_theta == TINY_A["rope_theta"]
    for bad in ({"rope_type": "yarn", "factor": 4.0, "original_max_position_embeddings": 32768},
                {"type": "linear", "factor": 2.0}, {"rope_type": "dynamic", "factor": 2.0}, "yarn"):
        with pytest.raises(ConfigError, match="rope_scaling"):
            Qwen3Config.from_dict(dict(TINY_A, rope_scaling=bad))


def test_every_stop_id_of_the_config_is_kept():
    c = Qwen3Config.from_dict(dict(TINY_A, eos_token_id=[7, 9, 200]))
    assert c.eos_token_id == 7 and c.eos_token_ids == (7, 9, 200)
    c = Qwen3Config.from_dict(dict(TINY_A, eos_token_id=5))
    assert c.eos_token_id == 5 and c.eos_token_ids == (5,)
    c = Qwen3Config.from_dict(TINY_A)
    assert c.eos_token_id == -1 and c.eos_token_ids == ()
    with pytest.raises(ConfigError, match="eos_token_id"):
        Qwen3Config.from_dict(dict(TINY_A, eos_token_id="7"))


def test_random_weights_specification(tmp_path):
    """``--random-weights NAME[:SEED]`` or ``CONFIG.JSON[:SEED]`` stands in for ``--model``."""
    from ullm_amd.config import parse_random_weights, preset_names
    assert {"qwen3-0.6b", "qwen3-8b", "qwen3-14b", "qwen3-32b"} <= set(preset_names())
    cfg, seed = parse_random_weights("qwen3-8b")
    c = Qwen3Config.from_dict(cfg)
    assert seed == 0 and (c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.num_key_value_heads, c.head_dim,
                          c.intermediate_size, c.vocab_size) == (4096, 36, 32, 8, 128, 12288, 151936)
    cfg, seed = parse_random_weights("Qwen3-32B:7")
    c = Qwen3Config.from_dict(cfg)
    assert seed == 7 and (c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.intermediate_size) == (5120, 64, 64, 25600)
    path = tmp_path / "config.json"
    path.write_text(json.dumps(TINY_B))
    assert parse_random_weights(f"{path}:3") == (TINY_B, 3) and parse_random_weights(str(path)) == (TINY_B, 0)
    with pytest.raises(ConfigError, match="neither"):
        parse_random_weights("qwen3-9000b")
    ap = argparse.ArgumentParser()
    EngineConfig.add_cli_args(ap)
    ec = EngineConfig.from_args(ap.parse_args(["--random-weights", "qwen3-14b:2"]))
    assert ec.model is None and ec.random_weights == "qwen3-14b:2" and ec.generation_defaults() == {}
    with pytest.raises(ConfigError, match="either"):
        EngineConfig.from_args(ap.parse_args([]))
    with pytest.raises(ConfigError, match="either"):
        EngineConfig(model="x", random_weights="qwen3-8b")


def test_a_windowed_configuration_is_announced_as_this_engines_own_reading(caplog):
    """The reference reads none of the sliding-window keys (ullm/models/qwen3.py builds every layer with full
    attention), so a config that switches windows on gets logits no reference run pins: said once per model."""
    import logging
    with caplog.at_level(logging.WARNING, logger="ullm_amd"):
        build_model(TINY_A)
    assert not [r for r in caplog.records if "sliding-window" in r.getMessage()]
    with caplog.at_level(logging.WARNING, logger="ullm_amd"):
        build_model(TINY_C)
    said = [r.getMessage() for r in caplog.records if "sliding-window" in r.getMessage()]
    assert len(said) == 1 and "2 of 3 layers look back 24 keys" in said[0] and "the reference applies no window" in said[0]


def test_a_context_past_the_models_positions_is_refused(caplog):
    """The reference's rotary table has max_position_embeddings rows (ullm/models/qwen3.py:142,
    ullm/layers/rotary_embedding.py:69); an engine with a longer context is refused when it is built.  Trace
    replay, whose number is a pool's size and whose traces are given, says so once and goes on."""
    import logging
    from ullm_amd.engine.loading import context_within_model
    cfg, _ = build_model(TINY_A)                       # max_position_embeddings = 128
    assert context_within_model(cfg, 128) == 128 and context_within_model(cfg, 64) == 64
    with pytest.raises(ConfigError, match="max_position_embeddings=128"):
        context_within_model(cfg, 129)
    with caplog.at_level(logging.WARNING, logger="ullm_amd"):
        assert context_within_model(cfg, 512, strict=False) == 512
    assert any("max_position_embeddings=128" in r.getMessage() for r in caplog.records)
    assert context_within_model({"no": "such key"}, 10 ** 6) == 10 ** 6     # a configuration without the key has no limit


def test_projection_limits_come_from_the_table_or_from_the_size_rules(tmp_path, monkeypatch):
    """A matrix the table of measurements holds takes its limits from there (missing fields from the rules);
    any other matrix takes the rules, which speak of the matrix's size only."""
    import json
    from ullm_amd.kernels import dispatch
    small, large = dispatch.default_limits(1024, 1024), dispatch.default_limits(24576, 4096)
    assert (small.rows, small.fold_norm, small.stacked_from, small.f32_skinny) == (0, 16, 0, 16)
    assert (large.rows, large.fold_norm, large.silu_skinny, large.stacked_to) == (64, 8, 32, 256)
    assert dispatch.default_limits(151936, 4096).f32_skinny == 32 and dispatch.default_limits(51200, 5120).silu_skinny == 16
    table = tmp_path / "table.json"
    table.write_text(json.dumps({"matrices": {"777x64": {"skinny": 5, "rows": 9, "not a field": 1}}}))
    monkeypatch.setattr(dispatch, "TABLE_PATH", str(table))
    monkeypatch.setattr(dispatch, "_table", None)
    got = dispatch.limits(777, 64)
    assert (got.skinny, got.rows) == (5, 9) and got.fold_norm == dispatch.default_limits(777, 64).fold_norm
    assert dispatch.is_tuned(777, 64) and not dispatch.is_tuned(778, 64)
    assert dispatch.limits(778, 64) == dispatch.default_limits(778, 64)
    dispatch.write_entry(778, 64, {"skinny": 3})
    assert dispatch.limits(778, 64).skinny == 3 and dispatch.limits(777, 64).skinny == 5
    assert dispatch.limits(778, 64).rows == dispatch.default_limits(778, 64).rows
    with pytest.raises(KeyError):
        dispatch.write_entry(778, 64, {"no such limit": 3})
    monkeypatch.setattr(dispatch, "_table", None)             # the real table again for whoever comes next


def test_limits_are_derived_from_times_by_the_time_saved_in_total():
    """One measurement that is off by its noise does not end a kernel's range; a kernel that is never ahead gets
    none; the norm stays folded only while that beats the norm's own kernel plus the best unfolded product."""
    from ullm_amd.kernels.microbench import derive_limits
    rows = [1, 8, 16, 17, 32, 64, 128, 256]
    stream = {"library>norm": dict(zip(rows, [19, 19, 19, 17, 17, 19, 29, 27])),
              "partial sums>norm": dict(zip(rows, [13, 14, 14, 15, 17.2, 18, 22, 29]))}
    assert derive_limits(stream, {"stream"}, 0, 0) == {"stacked_from": 17, "stacked_to": 128}
    never = {"library>norm": {17: 5.0, 64: 5.0}, "partial sums>norm": {17: 6.0, 64: 9.0}}
    assert derive_limits(never, {"stream"}, 0, 0) == {"stacked_from": 0, "stacked_to": 0}
    store = {"norm": {1: 2.5, 8: 2.5, 16: 2.5, 32: 2.5}, "library": {1: 14, 8: 14, 16: 14, 32: 15},
             "skinny": {1: 10, 8: 10.5, 16: 13, 32: 19}, "rows": {1: 10.5, 8: 10.6, 16: 10.7, 32: 12},
             "skinny+norm": {1: 11.5, 8: 12.5, 16: 16}}
    assert derive_limits(store, {"store"}, 0, 0) == {"skinny": 8, "rows": 32, "fold_norm": 8, "sums_from": 0, "sums_to": 0}
    # above the rows the weight-streaming kernels take, partial sums and the kernel that adds them as far as they save time
    more = {"library": {32: 15, 64: 17, 65: 17, 128: 25, 256: 40, 512: 60}, "rows": {32: 12, 64: 16},
            "partial sums>sum": {32: 14, 64: 16.5, 65: 16, 128: 21, 256: 31, 512: 70}, "norm": {}}
    assert derive_limits(more, {"store"}, 0, 0) == {"skinny": 0, "rows": 64, "fold_norm": 0, "sums_from": 65, "sums_to": 256}
