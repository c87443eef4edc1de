"""Host-side pieces of Kekapel that need no GPU: configuration parsing (layer order with the loop, pool layout), the model
registry, token-level step planning, the checkpoint reader, and the plain implementation's own consistency."""
import json
import os

import numpy as np
import pytest
import torch

import kekapel_oracle as O


def test_layer_runs_follow_the_loop():
    from swiftllm_amd.model_config import KekapelModelConfig
    layers = [O.attention_layer(mlp=O.dense_mlp(32)) for _ in range(5)]
    cfg = KekapelModelConfig(O.make_config(layers=layers, loop=(2, 4, 3)))
    assert [(r.layer, r.pass_index) for r in cfg.layer_runs] == [
        (0, -1), (1, -1), (2, 0), (3, -1), (2, 1), (3, -1), (2, 2), (3, -1), (4, -1)]
    assert [r.index for r in cfg.layer_runs] == list(range(9))
    assert [(i, t if first else -1) for i, t, first in O.layer_runs(O.make_config(layers=layers, loop=(2, 4, 3)))] == \
        [(r.layer, r.pass_index) for r in cfg.layer_runs]
    # no loop, a loop of one pass (its step vector is still added), a loop over everything
    assert [r.pass_index for r in KekapelModelConfig(O.make_config(layers=layers)).layer_runs] == [-1] * 5
    one = KekapelModelConfig(O.make_config(layers=layers, loop=(2, 3, 1)))
    assert [(r.layer, r.pass_index) for r in one.layer_runs] == [(0, -1), (1, -1), (2, 0), (3, -1), (4, -1)]
    every = KekapelModelConfig(O.make_config(layers=layers, loop=(0, 5, 2)))
    assert [r.layer for r in every.layer_runs] == list(range(5)) * 2
    assert [r.pass_index for r in every.layer_runs] == [0, -1, -1, -1, -1, 1, -1, -1, -1, -1]
    with pytest.raises(ValueError):
        KekapelModelConfig(O.make_config(layers=layers, loop=(3, 2, 2)))


def test_config_reads_every_size_per_layer():
    from swiftllm_amd.model_config import KekapelModelConfig
    layers = [O.attention_layer(heads=6, kv_heads=3, dim=16, vdim=24, window=7, mlp=O.moe_mlp(40, 6, 1)),
              O.attention_layer(heads=3, kv_heads=1, dim=24, vdim=8, window=1, softcap=None, mlp=None)]
    cfg = KekapelModelConfig(O.make_config(width=48, vocab=80, layers=layers, loop=(0, 1, 2), eps=3e-6,
                                           residual_mult=0.25, embedding_scale=7.0))
    a, b = cfg.layers
    assert (a.mixer.num_q_heads, a.mixer.num_kv_heads, a.mixer.head_dim, a.mixer.value_dim, a.mixer.window) == (6, 3, 16, 24, 7)
    assert (a.mlp.kind, a.mlp.num_experts, a.mlp.top_k, a.mlp.ffn_inter_dim) == ("moe", 6, 1, 40)
    assert b.mlp is None and b.mixer.softcap == 0.0 and b.mixer.window == 1
    assert (cfg.norm_eps, cfg.residual_mult, cfg.embedding_scale) == (3e-6, 0.25, 7.0)
    # K and V of every layer run: layer 0 runs twice
    assert cfg.kv_elems_per_token() == 2 * (3 * 16 + 3 * 24) + (24 + 8)
    assert cfg.get_kvslot_size(torch.float32) == 4 * cfg.kv_elems_per_token()
    with pytest.raises(ValueError):
        KekapelModelConfig(O.make_config(layers=[O.attention_layer(heads=4, kv_heads=3)]))
    bad = O.make_config()
    bad["layers"][0]["type"] = "recurrent"
    with pytest.raises(ValueError):
        KekapelModelConfig(bad)


def test_registry_picks_the_class_by_config(tmp_path):
    from swiftllm_amd import registry
    from swiftllm_amd.model_config import KekapelModelConfig, LlamaModelConfig
    (tmp_path / "k").mkdir()
    (tmp_path / "l").mkdir()
    (tmp_path / "x").mkdir()
    json.dump(O.make_config(), open(tmp_path / "k" / "config.json", "w"))
    llama = dict(model_type="llama", hidden_act="silu", num_hidden_layers=2, num_attention_heads=4, hidden_size=64,
                 vocab_size=100, max_position_embeddings=128, intermediate_size=128, rms_norm_eps=1e-5)
    json.dump(llama, open(tmp_path / "l" / "config.json", "w"))
    json.dump({"architecture": "Unknown"}, open(tmp_path / "x" / "config.json", "w"))
    assert isinstance(registry.load_model_config(str(tmp_path / "k")), KekapelModelConfig)
    assert isinstance(registry.load_model_config(str(tmp_path / "l")), LlamaModelConfig)
    assert registry.model_class(str(tmp_path / "k")).__name__ == "KekapelModel"
    assert registry.model_class(str(tmp_path / "l")).__name__ == "LlamaModel"
    with pytest.raises(ValueError, match="no model registered"):
        registry.model_class(str(tmp_path / "x"))
    assert "float32" in registry.model_class(str(tmp_path / "k")).SUPPORTED_DTYPES


def test_plan_step_flattens_portions_and_tiles():
    from swiftllm_amd.worker.batch_plan import StepEntry, plan_step
    plan = plan_step([StepEntry(2, list(range(40)), 100, (0, 39)), StepEntry(0, [7], 5, (0,)), StepEntry(3, [1, 2], 0, ())],
                     vocab_size=50, max_positions=256)
    assert plan.num_tokens == 43 and plan.num_seqs == 3
    assert plan.seq_ids_list == [2, 0, 3] and plan.target_lens_list == [140, 6, 2]
    assert plan.tok_pos.tolist() == list(range(100, 140)) + [5, 0, 1]
    assert plan.tok_seq.tolist() == [2] * 40 + [0] + [3, 3]
    assert plan.want_rows.tolist() == [0, 39, 40]
    assert plan.tile_row0.tolist() == [0, 16, 32, 40, 41] and plan.tile_cnt.tolist() == [16, 16, 8, 1, 2]
    layout, total = plan.packed_layout()
    buf = np.zeros(total, dtype=np.int32)
    plan.pack_into(buf)
    for name, off, n in layout:
        assert off % 4 == 0 and buf[off:off + n].tolist() == getattr(plan, name).tolist()
    for bad in ([StepEntry(0, [50], 0)], [StepEntry(0, [1], 256)], [StepEntry(0, [], 0)], [StepEntry(0, [1], -1)],
                [StepEntry(0, [1], 0), StepEntry(0, [2], 1)], [StepEntry(0, [1, 2], 0, (2,))]):
        with pytest.raises((ValueError, RuntimeError)):
            plan_step(bad, vocab_size=50, max_positions=256)


def test_checkpoint_reader_fuses_and_stacks(tmp_path):
    from safetensors.torch import save_file
    from swiftllm_amd.model_config import KekapelModelConfig
    from swiftllm_amd.worker.kekapel_weight import load_kekapel_weights
    cfg = O.make_config(layers=[O.attention_layer(heads=4, kv_heads=2, dim=8, vdim=12, mlp=O.moe_mlp(10, 3, 2)),
                                O.attention_layer(mlp=O.dense_mlp(20)), O.attention_layer(mlp=None)], loop=(0, 2, 2))
    W = O.random_weights(cfg, seed=1)
    json.dump(cfg, open(tmp_path / "config.json", "w"))
    save_file(W, str(tmp_path / "model.safetensors"))
    mc = KekapelModelConfig(cfg)
    w = load_kekapel_weights(mc, torch.float32, str(tmp_path), device="cpu")
    l0, l1, l2 = w.layers
    assert torch.equal(l0.qkv, torch.cat((W["l0.mix.q"], W["l0.mix.k"], W["l0.mix.v"])).float())
    assert l0.qkv.shape == (4 * 8 + 2 * 8 + 2 * 12, 64)
    assert torch.equal(l0.gate_up[2], torch.cat((W["l0.mlp.e2.gate"], W["l0.mlp.e2.up"])).float())
    assert torch.equal(l0.down[1], W["l0.mlp.e1.down"].float()) and l0.router.dtype == torch.float32
    assert l1.act == [float(x) for x in W["l1.mlp.act"].float()] and not hasattr(l2, "norm2_w")
    assert w.loop_step.shape == (2, 64) and w.loop_step.dtype == torch.float32
    assert w.embed.dtype == torch.float32 and torch.equal(w.embed, W["embed"].float())
    bf = load_kekapel_weights(mc, torch.bfloat16, str(tmp_path), device="cpu")
    assert bf.layers[0].qkv.dtype == torch.bfloat16 and bf.layers[0].norm1_w.dtype == torch.float32
    # a wrong shape is refused before use
    W2 = dict(W)
    W2["l1.mlp.up"] = W["l1.mlp.up"][:-1].contiguous()
    save_file(W2, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError, match="l1.mlp.up"):
        load_kekapel_weights(mc, torch.float32, str(tmp_path), device="cpu")
    dummy = load_kekapel_weights(mc, torch.bfloat16, str(tmp_path), use_dummy=True, device="cpu")
    assert dummy.head.shape == (cfg["vocab"], 64)


def test_build_subset_names_existing_sources():
    from swiftllm_amd.csrc import build
    for name, srcs in build.MODEL_SOURCES.items():
        assert set(srcs) <= set(build.SOURCES), name
    assert "swap_blocks.hip" in build.MODEL_SOURCES["Kekapel"]      # (holds the ABI version and error strings)


def test_plain_implementation_is_causal_and_windowed():
    """The oracle itself: a token never sees later tokens, and with one attention layer and no loop a token never sees
    anything older than its window."""
    cfg = O.make_config(layers=[O.attention_layer(window=5, mlp=O.dense_mlp(32))], width=32, vocab=40, max_positions=64)
    W = O.random_weights(cfg, seed=2)
    toks = list(range(20))
    base = O.forward(cfg, W, toks)
    later = O.forward(cfg, W, toks[:12] + [39] + toks[13:])
    assert torch.equal(base[:12], later[:12]) and not torch.equal(base[12], later[12])
    assert not torch.allclose(base[16], later[16]) and torch.allclose(base[17:], later[17:], atol=0, rtol=0)
