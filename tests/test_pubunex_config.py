"""Pubunex on the host: registry, configuration keys, the order of layer runs, the tensor list,
what a request keeps, and error messages."""
import copy

import numpy as np
import pytest

import zse_amd.models  # noqa: F401
from pubunex_util import CFG_A, CFG_B, CFG_C, attention_layer, config, delta_layer, latent_layer, moe, tensor_shapes
from zse_amd.config.base import ConfigError, resolve_architecture
from zse_amd.engine.model import Model
from zse_amd.parts.base import PagedKV, StateNeed


def model_of(cfg):
    arch = resolve_architecture(cfg)
    return Model(arch.plan(arch.config_from_dict(cfg)))


def test_the_registry_knows_the_design():
    assert resolve_architecture({"architecture": "Pubunex"}).name == "Pubunex"
    assert resolve_architecture({"model_type": "pubunex"}).name == "Pubunex"


@pytest.mark.parametrize("cfg", [CFG_A, CFG_B, CFG_C])
def test_the_model_asks_for_exactly_the_checkpoints_tensors(cfg):
    reqs = {r.name: tuple(r.shape) for r in model_of(cfg).tensor_reqs()}
    assert reqs == tensor_shapes(cfg)


def test_the_order_of_layer_runs():
    calls = lambda cfg: [(c.layer, c.add_embedding) for c in model_of(cfg).plan.order]
    assert calls(CFG_A) == [(0, False), (1, False), (0, True), (1, False), (2, False), (3, False)]
    assert calls(CFG_B) == [(0, False), (1, False), (2, False)]
    assert calls(CFG_C) == [(0, False), (1, False), (1, True), (1, True), (2, False)]
    once = copy.deepcopy(CFG_C)
    once["loop"]["times"] = 1
    assert calls(once) == [(0, False), (1, False), (2, False)]
    whole = copy.deepcopy(CFG_B)
    whole["loop"] = {"start": 0, "stop": 3, "times": 2}
    assert calls(whole) == [(0, False), (1, False), (2, False), (0, True), (1, False), (2, False)]


def test_every_run_of_a_layer_keeps_its_own_cache_or_state():
    m = model_of(CFG_A)
    needs = m.cache_needs()
    assert [type(n) for n in needs] == [StateNeed, PagedKV, StateNeed, PagedKV, PagedKV, StateNeed]
    # S [heads, dim, vdim] as floats, then taps - 1 rows of the q, k and v channels
    assert needs[0].nbytes == 4 * (4 * 16 * 24 + 2 * (2 * 2 * 16 + 4 * 24))
    assert needs[5].nbytes == 4 * (2 * 24 * 8 + 3 * (2 * 2 * 24 + 2 * 8))
    assert (needs[1].num_kv_heads, needs[1].head_dim, needs[1].value_dim, needs[1].window) == (2, 24, 16, None)
    # a latent layer caches one row of kv_rank + rot_dim a token and no values
    assert (needs[4].num_kv_heads, needs[4].head_dim, needs[4].value_dim, needs[4].values_in_keys) == (1, 24, 20, True)
    one_tap = model_of(CFG_C).cache_needs()
    assert one_tap[1].nbytes == 4 * 12 * 70


def test_scaled_frequencies_and_their_magnitude():
    from plain import pubunex_plain as P
    m = model_of(CFG_A)
    rot = m.blocks[1].mixer.position
    f, mag = P.rotary_frequencies(12, 500.0, {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0})
    assert np.allclose(rot.frequencies(), f.astype(np.float32), rtol=1e-6)
    assert abs(rot.magnitude() - mag) < 1e-12 and mag > 1.0
    plain = model_of(CFG_B).blocks[0].mixer.position
    assert plain.magnitude() == 1.0 and not plain.interleaved
    assert np.allclose(plain.frequencies(), 2000.0 ** (-np.arange(16) / 16.0), rtol=1e-6)
    assert model_of(CFG_A).blocks[2].mixer.position.interleaved
    # some frequencies are divided by the factor, some stay, some lie in between
    f0, _ = P.rotary_frequencies(12, 500.0, None)
    ratio = f / f0
    assert ratio.max() == 1.0 and abs(ratio.min() - 1 / 8.0) < 1e-12 and len(set(np.round(ratio, 6))) >= 3


def test_what_the_config_leaves_out_does_not_exist():
    cfg = config([attention_layer(mlp=None), delta_layer(mlp=moe(shared_ff=None))])
    m = model_of(cfg)
    assert m.blocks[0].ffn is None and m.blocks[1].ffn.shared is None
    assert all(not c.add_embedding for c in m.plan.order)
    names = {r.name for r in m.tensor_reqs()}
    assert not any(n.startswith("l0.mlp") or "shared" in n for n in names)


@pytest.mark.parametrize("change, message", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["layers"][0].update(type="conv"), "unknown type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple of kv_heads"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][2]["mixer"].update(rot_dim=5), "rot_dim"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "mlp.kind"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("fast"), "fast"),
])
def test_a_config_that_cannot_be_served_says_why(change, message):
    cfg = copy.deepcopy(CFG_A)
    change(cfg)
    with pytest.raises(ConfigError) as e:
        resolve_architecture(cfg).config_from_dict(cfg)
    assert message in str(e.value)
