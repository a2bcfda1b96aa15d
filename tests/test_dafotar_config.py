"""Dafotar's config.json reader, its plan of parts and what the cache manager is told (no GPU)."""
import copy

import numpy as np
import pytest

from dafotar_util import CFG_A, CFG_B, CFG_C, attention_layer, config, mlstm_layer, random_weights, tensor_shapes, write_model
from zse_amd.config import ConfigError, resolve_architecture
from zse_amd.engine.model import Model
from zse_amd.parts.base import PagedKV, StateNeed


def plan_of(cfg):
    arch = resolve_architecture(cfg)
    assert arch.name == "Dafotar"
    return arch.plan(arch.config_from_dict(cfg))


def test_the_architecture_is_found_by_its_name():
    assert resolve_architecture({"architecture": "Dafotar"}).name == "Dafotar"
    assert resolve_architecture({"architectures": ["Dafotar"]}).name == "Dafotar"
    assert resolve_architecture({"architectures": ["Gemma2ForCausalLM"]}).name == "Gemma2ForCausalLM"
    with pytest.raises(ConfigError):
        resolve_architecture({"architecture": "Nobody"})


@pytest.mark.parametrize("cfg", [CFG_A, CFG_B, CFG_C])
def test_the_model_asks_for_exactly_the_designs_tensors(cfg):
    model = Model(plan_of(cfg))
    want = tensor_shapes(cfg)
    got = {}
    for r in model.tensor_reqs():
        assert got.setdefault(r.name, tuple(r.shape)) == tuple(r.shape)
    assert got == want


def test_every_size_and_constant_comes_from_the_config():
    plan = plan_of(CFG_A)
    assert [c.cache_of for c in plan.order] == [None, None, 1, None, None]
    assert plan.embedding.copies == 3 and plan.final_norm.streams == 3 and plan.head.weight == plan.embedding.weight
    l1, l2, l4 = plan.layers[1].mixer, plan.layers[2].mixer, plan.layers[4].mixer
    assert (l1.num_heads, l1.num_kv_heads, l1.head_dim, l1.value_dim, l1.window) == (4, 2, 24, 16, 20)
    assert (l1.position.rotary_dim, l1.position.theta, l1.value_rotation, l1.scale) == (12, 500.0, 500.0, 0.3)
    assert "k" not in l2.names and l2.k_norm is None and l2.window == 33 and l2.scale == 0.25
    assert (l4.head_dim, l4.value_dim, l4.window, l4.position.rotary_dim) == (8, 40, 7, 8)
    m0 = plan.layers[0].mixer
    assert (m0.kind, m0.num_heads, m0.key_dim, m0.value_dim, m0.gate_cap, m0.eps) == ("mlstm", 2, 8, 16, 6.0, 1e-5)
    assert plan.layers[0].ffn.activation == "relu" and plan.layers[1].ffn is None
    assert plan.layers[0].conv.taps == 3 and plan.layers[0].norms["pre_mixer"].eps == 1e-5


def test_what_the_config_leaves_out_does_not_exist():
    plan = plan_of(CFG_B)
    assert plan.embedding.copies == 1 and plan.final_norm.streams == 1
    for b in plan.layers:
        assert b.streams is None and b.conv is None and b.names == {}
    a0, a2 = plan.layers[0].mixer, plan.layers[2].mixer
    assert a0.window is None and a0.value_rotation == 2000.0
    assert a2.position.kind == "none" and a2.value_rotation is None
    model = Model(plan)
    assert not any(hasattr(b, "state_needs") and b.state_needs() for b in model.blocks)


def test_keys_read_through_a_wider_window_are_kept_that_long():
    needs = Model(plan_of(CFG_A)).cache_needs()
    assert isinstance(needs[0], StateNeed) and needs[0].nbytes == 2 * (8 * 16 + 8 + 1) * 4
    assert needs[1] == PagedKV(2, 24, 33, 16)            # its own window is 20; layer 2 reads it through 33
    assert needs[2] is None
    assert needs[4] == PagedKV(1, 8, 7, 40)
    needs = Model(plan_of(CFG_C)).cache_needs()
    assert needs[0].window == 9 and needs[2] is None
    # a reader that sees every key keeps them for ever
    cfg = config([attention_layer(window=5), attention_layer(window=None, kv_from=0)])
    assert Model(plan_of(cfg)).cache_needs()[0].window is None
    # a reader with the narrower window changes nothing
    cfg = config([attention_layer(window=50), attention_layer(window=4, kv_from=0)])
    assert Model(plan_of(cfg)).cache_needs()[0].window == 50


def test_state_of_a_layer_is_the_mixers_and_the_convolutions():
    model = Model(plan_of(CFG_A))
    assert [b.state_needs() for b in model.blocks] == [[("conv", 2 * 48 * 4)]] * 5
    one_tap = Model(plan_of(config([mlstm_layer()], taps=1)))
    assert one_tap.blocks[0].state_needs() == []


def test_errors_name_the_layer_and_the_key():
    bad = copy.deepcopy(CFG_A)
    del bad["layers"][1]["mixer"]["scale"]
    bad["layers"][2]["mixer"]["kv_from"] = 0              # layer 0 is no attention
    bad["layers"][3]["type"] = "conv"
    bad["layers"][4]["mixer"]["heads"] = 3                 # not a multiple of kv_heads... 1 divides 3; make it fail otherwise
    bad["layers"][4]["mixer"]["kv_heads"] = 2
    with pytest.raises(ConfigError) as e:
        plan_of(bad)
    msg = str(e.value)
    assert "layer 1" in msg and "'scale'" in msg
    assert "layer 2" in msg and "kv_from" in msg
    assert "layer 3" in msg and "unknown type" in msg
    assert "layer 4" in msg and "multiple of kv_heads" in msg
    for key in ("vocab", "width", "norm", "layers"):
        c = copy.deepcopy(CFG_B)
        del c[key]
        with pytest.raises(ConfigError, match=key):
            plan_of(c)
    c = copy.deepcopy(CFG_A)
    c["layers"][2]["mixer"]["dim"] = 16                    # not the size of the keys it reads
    with pytest.raises(ConfigError, match="differ"):
        plan_of(c)


def test_a_written_folder_passes_the_loaders_check(tmp_path):
    from zse_amd.weights.loader import WeightError, check_folder
    folder = write_model(str(tmp_path / "m"), CFG_A, random_weights(CFG_A, 0))
    model = Model(plan_of(CFG_A))
    assert len(check_folder(folder, model.tensor_reqs(), (), model.plan.optional_prefixes)) == len(tensor_shapes(CFG_A))
    w = random_weights(CFG_A, 0)
    del w["l2.hc2.mix"]
    w["l2.mix.k"] = np.zeros((2, 2), np.float32)           # a layer that reads another's keys has none of its own
    folder = write_model(str(tmp_path / "bad"), CFG_A, w)
    with pytest.raises(WeightError) as e:
        check_folder(folder, model.tensor_reqs(), (), model.plan.optional_prefixes)
    assert e.value.missing == ["l2.hc2.mix"] and e.value.unexpected == ["l2.mix.k"]
