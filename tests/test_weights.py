"""Weight binding by name, its one error, and the random-weights mode (no GPU)."""
import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from conftest import TINY_A, TINY_B
from ullm_amd.models import build_model
from ullm_amd.parts import PartEnv
from ullm_amd.weights.loader import WeightError, checkpoint_index, load_weights
from ullm_amd.weights.random_init import write_random_model

CPU32 = PartEnv(torch.device("cpu"), torch.float32, 64)
CPU16 = PartEnv(torch.device("cpu"), torch.bfloat16, 64)


def test_random_folder_is_complete_and_deterministic(tmp_path):
    a = write_random_model(TINY_B, str(tmp_path / "a"), seed=7)
    b = write_random_model(TINY_B, str(tmp_path / "b"), seed=7)
    c = write_random_model(TINY_B, str(tmp_path / "c"), seed=8)
    assert json.load(open(os.path.join(a, "config.json")))["hidden_size"] == 96
    wa, wb, wc = (load_file(os.path.join(d, "model.safetensors")) for d in (a, b, c))
    assert set(wa) == {d.name for d in build_model(TINY_B)[1].weight_decls()}
    assert all(torch.equal(wa[k], wb[k]) for k in wa)
    assert any(not torch.equal(wa[k], wc[k]) for k in wa)
    assert all(v.dtype == torch.bfloat16 for v in wa.values())
    # gains are 1 + N(0, s), matrices N(0, s) with s = initializer_range
    assert abs(wa["model.norm.weight"].float().mean() - 1.0) < 0.05
    assert abs(wa["model.layers.0.mlp.down_proj.weight"].float().std() - 0.05) < 0.005


def test_random_folder_from_the_command_line(tmp_path, capsys):
    from ullm_amd.weights import random_init
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(TINY_A))
    assert random_init.main(["--config", str(cfg_path), "--out", str(tmp_path / "m"), "--seed", "3", "--dtype", "float32"]) == 0
    assert capsys.readouterr().out.strip() == str(tmp_path / "m")
    same = write_random_model(TINY_A, str(tmp_path / "n"), seed=3, dtype="float32")
    wa, wb = load_file(str(tmp_path / "m" / "model.safetensors")), load_file(os.path.join(same, "model.safetensors"))
    assert set(wa) == set(wb) and all(torch.equal(wa[k], wb[k]) and wa[k].dtype == torch.float32 for k in wa)


def test_tied_model_stores_no_head_and_binds_the_embedding(tmp_path):
    d = write_random_model(TINY_A, str(tmp_path / "a"), seed=0)
    assert "lm_head.weight" not in checkpoint_index(d)
    _, model = build_model(TINY_A)
    load_weights(model, d, CPU16)
    assert model.head.data_ptr() == model.embedding.data_ptr()
    assert model.embedding.dtype == torch.bfloat16
    assert model.final_norm.gain.dtype == torch.float32            # gains stay 32-bit


def test_float32_mode_widens_exactly(tmp_path):
    d = write_random_model(TINY_A, str(tmp_path / "a"), seed=0)
    stored = load_file(os.path.join(d, "model.safetensors"))
    _, model = build_model(TINY_A)
    load_weights(model, d, CPU32)
    assert model.embedding.dtype == torch.float32
    assert torch.equal(model.embedding, stored["model.embed_tokens.weight"].float())
    attn = model.blocks[0].mixer
    want = torch.cat([stored[f"model.layers.0.self_attn.{n}_proj.weight"].float() for n in "qkv"])
    assert torch.equal(attn.w_qkv, want)                           # rows q | k | v (ullm/layers/linear.py:381-389)
    ffn = model.blocks[1].ffn
    want = torch.cat([stored["model.layers.1.mlp.gate_proj.weight"].float(),
                      stored["model.layers.1.mlp.up_proj.weight"].float()])
    assert torch.equal(ffn.w_gate_up, want)                        # rows gate | up (ullm/models/qwen3.py:307-308)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = write_random_model(TINY_B, str(tmp_path / "b"), seed=1)
    path = os.path.join(d, "model.safetensors")
    w = load_file(path)
    del w["model.layers.1.self_attn.k_norm.weight"]
    del w["lm_head.weight"]
    w["model.layers.0.mlp.down_proj.weight"] = torch.zeros(96, 100, dtype=torch.bfloat16)
    w["model.layers.9.mlp.down_proj.weight"] = torch.zeros(2, 2, dtype=torch.bfloat16)
    w["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)      # known and ignorable
    save_file(w, path)
    _, model = build_model(TINY_B)
    with pytest.raises(WeightError) as e:
        load_weights(model, d, CPU32)
    msg = str(e.value)
    assert "missing tensors (2)" in msg and "model.layers.1.self_attn.k_norm.weight" in msg and "lm_head.weight" in msg
    assert "unexpected tensors (1)" in msg and "model.layers.9.mlp.down_proj.weight" in msg
    assert "wrong shapes (1)" in msg and "[96, 100]" in msg and "[96, 224]" in msg
    assert "inv_freq" not in msg


def test_no_safetensors_file(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    _, model = build_model(TINY_A)
    with pytest.raises(WeightError, match="no \\*.safetensors"):
        load_weights(model, str(tmp_path), CPU32)


def test_tensors_may_be_spread_over_files_and_stored_in_32_bit(tmp_path):
    d = write_random_model(TINY_A, str(tmp_path / "a"), seed=3, dtype="float32")
    path = os.path.join(d, "model.safetensors")
    w = load_file(path)
    assert all(v.dtype == torch.float32 for v in w.values())
    names = sorted(w)
    save_file({k: w[k] for k in names[:10]}, os.path.join(d, "model-00001-of-00002.safetensors"))
    save_file({k: w[k] for k in names[10:]}, os.path.join(d, "model-00002-of-00002.safetensors"))
    os.unlink(path)
    _, model = build_model(TINY_A)
    load_weights(model, d, CPU32)
    assert torch.equal(model.final_norm.gain, w["model.norm.weight"])
    _, model16 = build_model(TINY_A)
    load_weights(model16, d, CPU16)
    assert model16.embedding.dtype == torch.bfloat16 and model16.final_norm.gain.dtype == torch.float32
    assert torch.equal(model16.final_norm.gain, w["model.norm.weight"])     # a 32-bit gain stays as stored


def test_a_checkpoint_may_hold_the_merged_matrices_whole(tmp_path):
    """q | k | v and gate | up already put together in the file, under the reference's own names
    (ullm/models/qwen3.py:300-310, split again by ullm/layers/linear.py:359-379,473-485): the same model."""
    d = write_random_model(TINY_B, str(tmp_path / "b"), seed=4)
    path = os.path.join(d, "model.safetensors")
    w = load_file(path)
    _, pieces = build_model(TINY_B)
    load_weights(pieces, d, CPU32)
    for i in range(TINY_B["num_hidden_layers"]):
        a, m = f"model.layers.{i}.self_attn", f"model.layers.{i}.mlp"
        w[f"{a}.qkv_proj.weight"] = torch.cat([w.pop(f"{a}.{n}_proj.weight") for n in "qkv"])
        if i != 1:                                               # layer 1 keeps gate and up apart: both forms in one file
            w[f"{m}.gate_up_proj.weight"] = torch.cat([w.pop(f"{m}.gate_proj.weight"), w.pop(f"{m}.up_proj.weight")])
    save_file(w, path)
    _, whole = build_model(TINY_B)
    load_weights(whole, d, CPU32)
    for b0, b1 in zip(pieces.blocks, whole.blocks):
        assert torch.equal(b0.mixer.w_qkv, b1.mixer.w_qkv) and torch.equal(b0.ffn.w_gate_up, b1.ffn.w_gate_up)
    # a merged matrix of the wrong height, and a merged matrix beside one of its pieces, are named in the error
    w["model.layers.0.self_attn.qkv_proj.weight"] = w["model.layers.0.self_attn.qkv_proj.weight"][:-1].contiguous()
    w["model.layers.2.mlp.up_proj.weight"] = torch.zeros(224, 96, dtype=torch.bfloat16)
    save_file(w, path)
    with pytest.raises(WeightError) as e:
        load_weights(build_model(TINY_B)[1], d, CPU32)
    msg = str(e.value)
    assert "wrong shapes (1)" in msg and "qkv_proj.weight" in msg and "[383, 96]" in msg and "[384, 96]" in msg
    assert "unexpected tensors (1)" in msg and "model.layers.2.mlp.gate_up_proj.weight" in msg and "up_proj.weight" in msg


def test_a_missing_piece_of_a_merged_matrix_is_named(tmp_path):
    d = write_random_model(TINY_A, str(tmp_path / "a"), seed=4)
    path = os.path.join(d, "model.safetensors")
    w = load_file(path)
    del w["model.layers.1.self_attn.k_proj.weight"]
    save_file(w, path)
    with pytest.raises(WeightError, match=r"missing tensors \(1\):\n  model.layers.1.self_attn.k_proj.weight  expected shape \[32, 64\]"):
        load_weights(build_model(TINY_A)[1], d, CPU32)


def test_random_weights_bound_in_place(tmp_path):
    """The mode every benchmark runs on: every declared tensor is there with its shape and dtype, a tied
    head is the embedding itself, the same seed gives the same tensors, and the 32-bit engine holds
    exactly the bfloat16 engine's weights."""
    from conftest import TINY_C
    from ullm_amd.weights.loader import merged_tensors, unique_decls
    from ullm_amd.weights.random_init import bind_random_weights

    def bound(cfg, env, seed):
        _, model = build_model(cfg)
        seen = {}
        inner = model.bind
        model.bind = lambda tensors, e: (seen.update(tensors), inner(tensors, e))
        bind_random_weights(model, env, seed)
        return model, seen

    for cfg in (TINY_A, TINY_C):                                  # tied head; biases and an untied head
        m16, t16 = bound(cfg, CPU16, 5)
        m32, t32 = bound(cfg, CPU32, 5)
        again, t16b = bound(cfg, CPU16, 5)
        other, t16c = bound(cfg, CPU16, 6)
        decls = unique_decls(m16.weight_decls())
        merged = merged_tensors(m16.weight_decls())
        want = {n: (d.shape, d.keep_fp32) for n, d in decls.items() if d.merged_into is None}
        want.update({n: (m.shape, m.pieces[0].keep_fp32) for n, m in merged.items()})
        assert set(t16) == set(want) == set(t32)
        for n, (shape, keep) in want.items():
            assert tuple(t16[n].shape) == tuple(shape) == tuple(t32[n].shape), n
            assert t16[n].dtype == (torch.float32 if keep else torch.bfloat16) and t32[n].dtype == torch.float32, n
            assert torch.equal(t16[n].float(), t32[n]), n             # widened exactly
            assert torch.equal(t16[n], t16b[n]), n
        assert any(not torch.equal(t16[n], t16c[n]) for n in want)
        if cfg["tie_word_embeddings"]:
            assert m16.head.data_ptr() == m16.embedding.data_ptr()
        else:
            assert m16.head.data_ptr() != m16.embedding.data_ptr()
        std = cfg["initializer_range"]
        assert abs(float(m32.blocks[0].ffn.w_gate_up.std()) - std) < 0.1 * std
        assert abs(float(m32.final_norm.gain.mean()) - 1.0) < 3 * std
        # the pieces of a merged matrix are different draws, not one draw repeated
        w = m32.blocks[0].mixer.w_qkv
        nq_rows = cfg["num_attention_heads"] * cfg["head_dim"]
        kv_rows = cfg["num_key_value_heads"] * cfg["head_dim"]
        assert not torch.equal(w[nq_rows:nq_rows + kv_rows], w[nq_rows + kv_rows:])
