"""Host-side pieces of the Lorulix worker (no GPU): the configuration reader, the registry, the state slot manager, the step
plan's per-portion arrays and the distance rows of the bias table."""
import numpy as np
import pytest

import lorulix_oracle as O
from swiftllm_amd import registry
from swiftllm_amd.model_config import LorulixModelConfig, distance_bias_rows
from swiftllm_amd.worker.batch_plan import StepEntry, plan_step
from swiftllm_amd.worker.state_slots import StateSlotManager


def test_config_reads_every_layer():
    layers = [O.delta_layer(heads=6, kv_heads=2, dim=8, vdim=24, conv=3, mlp=O.moe_mlp(16, 5, 2, scale=1.5, shared=12)),
              O.attention_layer(heads=4, kv_heads=1, dim=16, vdim=8, bias_max=77, temp=(0.3, 4), mlp=O.dense_mlp(40, 0.8)),
              O.attention_layer(heads=4, kv_heads=1, dim=16, vdim=8, bias_max=None, temp=None, kv_from=1, mlp=None)]
    cfg = LorulixModelConfig(O.make_config(width=32, vocab=50, layers=layers, taps=4, max_positions=99))
    assert (cfg.hidden_size, cfg.vocab_size, cfg.canon_taps, cfg.max_position_embeddings) == (32, 50, 4, 99)
    d, a, b = (l.mixer for l in cfg.layers)
    assert (d.qk_size, d.v_size, d.conv_channels, d.proj_size, d.state_elems) == (16, 144, 176, 332, 6 * 8 * 24)
    assert (a.q_size, a.k_size, a.v_size, a.bias_max, a.q_temp_coef, a.q_temp_every, a.kv_from) == (64, 16, 8, 77.0, 0.3, 4, -1)
    assert (b.bias_max, b.q_temp_coef, b.kv_from) == (0.0, 0.0, 1)
    m = cfg.layers[0].mlp
    assert (m.num_experts, m.top_k, m.router_scale, m.shared_ffn_inter_dim) == (5, 2, 1.5, 12)
    assert cfg.layers[1].mlp.limit == 0.8 and cfg.layers[2].mlp is None
    assert cfg.kv_elems_per_token() == 24          # only the layer with keys of its own


def test_config_refuses_bad_borrowing():
    layers = [O.attention_layer(kv_from=1), O.attention_layer()]
    with pytest.raises(ValueError):
        LorulixModelConfig(O.make_config(layers=layers))
    layers = [O.delta_layer(), O.attention_layer(kv_from=0)]
    with pytest.raises(ValueError):
        LorulixModelConfig(O.make_config(layers=layers))
    layers = [O.attention_layer(dim=16), O.attention_layer(dim=8, kv_from=0)]
    with pytest.raises(ValueError):
        LorulixModelConfig(O.make_config(layers=layers))


def test_registry_knows_the_design(tmp_path):
    import json
    (tmp_path / "config.json").write_text(json.dumps(O.make_config()))
    assert type(registry.load_model_config(str(tmp_path))).__name__ == "LorulixModelConfig"
    assert registry.architecture_of(registry.read_config(str(tmp_path))) == "Lorulix"


def test_distance_rows():
    assert distance_bias_rows(8, 64, 6) == [0, 1, 2, 3, 4, 4]
    rows = distance_bias_rows(12, 40, 300)
    assert rows[:7] == list(range(7)) and rows[8] == 6 and rows[29] == 10 and rows[40] == 11 and rows[-1] == 11
    assert all(b >= a for a, b in zip(rows, rows[1:]))
    assert rows == [O.distance_bucket(n, 12, 40) for n in range(300)]


def test_state_slots_are_reused_and_parity_alternates():
    mgr = StateSlotManager(2, device="cpu")
    a, b = mgr.add_region(10), mgr.add_region(3)
    assert (a, b) == (0, 12) and mgr.slot_floats == 16
    mgr.allocate()
    assert mgr.pool.shape == (2, 16)
    assert mgr.begin_step([5, 9], [0, 0]).tolist() == [0, 2]
    assert mgr.begin_step([9], [4]).tolist() == [3]                 # same slot, other tail buffer
    assert mgr.begin_step([5, 9], [7, 5]).tolist() == [1, 2]
    with pytest.raises(RuntimeError):
        mgr.begin_step([7], [0])                                    # no slot left
    with pytest.raises(RuntimeError):
        mgr.begin_step([7], [3])                                    # continues without ever having started
    mgr.release([5])
    assert mgr.num_free_slots == 1
    assert mgr.begin_step([7], [0]).tolist() == [0]                 # the freed slot, parity from the start
    mgr.pool[mgr.slot_of(9)] = 4.0
    mgr.swap_out([9])
    assert mgr.num_free_slots == 1
    assert mgr.begin_step([3], [0]).tolist() == [2]
    mgr.release([3, 7])
    mgr.swap_in([9])
    assert float(mgr.pool[mgr.slot_of(9)].min()) == 4.0 and mgr.begin_step([9], [6]).tolist() == [mgr.slot_of(9) * 2 + 1]


def test_plan_describes_the_portions():
    plan = plan_step([StepEntry(3, [1, 2, 3], 5, (2,)), StepEntry(0, [4], 9, (0,)), StepEntry(1, list(range(20)), 0, ())], 50, 64)
    assert plan.seq_row0.tolist() == [0, 3, 4] and plan.seq_cnt.tolist() == [3, 1, 20]
    assert plan.tok_start.tolist() == [5] * 3 + [9] + [0] * 20
    assert plan.tok_state.tolist() == [0] * 24
    layout, total = plan.packed_layout()
    buf = np.zeros(total, dtype=np.int32)
    plan.pack_into(buf)
    names = [n for n, _, _ in layout]
    assert names == list(plan.SEGMENTS) and all(off % 4 == 0 for _, off, _ in layout)
