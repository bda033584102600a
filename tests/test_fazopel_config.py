"""Fazopel without a GPU: its configuration (every key required, every error names its key), the specification built
from it (a layer that uses another's tensors is one more run of that layer with a cache or state of its own), the
frequencies the product hands its kernels, and the plain implementation against itself (a state carried over a cut,
a window of one sequence)."""
import copy

import pytest
import torch

import plain_fazopel as pf
from prelude_amd import models  # noqa: F401  (registers the architectures)
from prelude_amd.config.model_config import ConfigError, FazopelConfig
from prelude_amd.config.registry import resolve_architecture
from prelude_amd.models.causal_lm import CausalLM
from prelude_amd.parts.base import KVCacheSpec, StateSpec


def build(cfg):
    arch = resolve_architecture(cfg)
    assert arch.name == "fazopel"
    return CausalLM(arch.build_spec(arch.parse_config(cfg)))


@pytest.mark.parametrize("make", [pf.tiny_config_p, pf.tiny_config_q, pf.tiny_config_r])
def test_the_model_asks_for_the_tensors_a_file_holds(make):
    cfg = make()
    m = build(cfg)
    want = pf.tensor_shapes(cfg)
    got = {k: tuple(v.shape) for k, v in m.tensor_requests().items()}
    assert got == want
    assert m.spec.eos_token_ids == () and m.spec.vocab_size == cfg["vocab"]


def test_a_layer_that_uses_anothers_tensors_is_a_run_of_its_own():
    cfg = pf.tiny_config_p()
    m = build(cfg)
    assert [r.layer for r in m.spec.order] == [0, 1, 0, 2] and len(m.spec.layers) == 3
    assert m.run_cache == [0, 1, 2, 3], "every run keeps a cache or state of its own"
    kinds = [type(c.spec) for c in m.cache_slots]
    assert kinds == [StateSpec, KVCacheSpec, StateSpec, KVCacheSpec]
    assert m.cache_slots[0].spec == m.cache_slots[2].spec and m.needs_state
    assert m.graph_safe and m.graph_safe_portions and not m.atomic_prefill
    assert m.blocks[2].KIND == "branch_norm_mixer_only"
    q = build(pf.tiny_config_q())
    assert [r.layer for r in q.spec.order] == [0, 1, 0, 2]
    # the two attention runs share a group of pages (equal specifications), each with storage of its own
    assert q.cache_slots[0].spec == q.cache_slots[2].spec == KVCacheSpec(1, 64, 0)


def test_sizes_and_constants_come_from_the_configuration():
    c = FazopelConfig.from_dict(pf.tiny_config_q())
    a, l = c.layers[0].mixer, c.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.scale, a.rot_base, a.rot_dims) == (4, 1, 64, 0.11, 50000.0, 32)
    assert (a.rot_scaling.factor, a.rot_scaling.low, a.rot_scaling.high, a.rot_scaling.original) == (4.0, 1.0, 2.0, 128)
    assert (l.heads, l.dim, l.vdim, l.decay) == (2, 40, 72, (0.97, 1.0))
    f = c.layers[3].mlp
    assert (f.kind, f.experts, f.top, f.ff, f.limit, f.route_scale, f.shared_ff, f.shared_limit) == ("moe", 4, 1, 32, 0.8, 2.5, 24, 1.2)
    assert c.layers[0].mlp.shared_ff == 0 and c.layers[1].mlp.kind == "dense" and c.layers[2].weights_of == 0
    assert FazopelConfig.from_dict(pf.tiny_config_p()).layers[3].mixer.rot_scaling is None
    spec = build(pf.tiny_config_q()).spec
    ffn = spec.layers[2].parts["ffn"].params
    assert ffn["route_scale"] == 2.5 and ffn["limit"] == 0.8 and ffn["shared_limit"] == 1.2 and ffn["top"] == 1
    mixer = spec.layers[0].parts["mixer"].params
    assert mixer["values_from_keys"] and mixer["sink"] == "zero" and mixer["scale"] == 0.11 and mixer["rotary_dim"] == 32


def _without(cfg, path):
    c = copy.deepcopy(cfg)
    d = c
    for k in path[:-1]:
        d = d[k]
    del d[path[-1]]
    return c


def _with(cfg, path, value):
    c = copy.deepcopy(cfg)
    d = c
    for k in path[:-1]:
        d = d[k]
    d[path[-1]] = value
    return c


@pytest.mark.parametrize("path,key", [
    (("vocab",), "vocab"), (("width",), "width"), (("norm",), "norm"), (("norm", "eps"), "norm.eps"),
    (("layers", 0, "type"), "type"), (("layers", 0, "mixer"), "layers[0].mixer"),
    (("layers", 0, "mixer", "heads"), "layers[0].mixer.heads"), (("layers", 0, "mixer", "decay"), "layers[0].mixer.decay"),
    (("layers", 0, "mixer", "vdim"), "layers[0].mixer.vdim"),
    (("layers", 1, "mixer", "kv_heads"), "layers[1].mixer.kv_heads"), (("layers", 1, "mixer", "scale"), "layers[1].mixer.scale"),
    (("layers", 1, "mixer", "rot"), "layers[1].mixer.rot"), (("layers", 1, "mixer", "rot", "base"), "layers[1].mixer.rot.base"),
    (("layers", 1, "mixer", "rot", "scaling", "factor"), "layers[1].mixer.rot.scaling.factor"),
    (("layers", 0, "mlp", "router"), "layers[0].mlp.router"), (("layers", 0, "mlp", "router", "scale"), "layers[0].mlp.router.scale"),
    (("layers", 0, "mlp", "expert", "limit"), "layers[0].mlp.expert.limit"), (("layers", 0, "mlp", "shared", "ff"), "layers[0].mlp.shared.ff"),
    (("layers", 1, "mlp", "ff"), "layers[1].mlp.ff")])
def test_a_missing_key_is_named(path, key):
    cfg = pf.tiny_config_p()
    cfg["layers"][2] = _without(cfg["layers"][2], ("weights_of",)) if path[:2] != ("layers", 0) else cfg["layers"][2]
    broken = _without(cfg, path)
    if path[:2] == ("layers", 0):
        broken["layers"][2] = dict(copy.deepcopy(broken["layers"][0]), weights_of=0)
    with pytest.raises(ConfigError, match=key.replace("[", r"\[").replace("]", r"\]").replace(".", r"\.")):
        FazopelConfig.from_dict(broken)


@pytest.mark.parametrize("path,value,says", [
    (("layers", 0, "type"), "conv", "type"), (("layers", 0, "mixer", "decay"), [0.5, 0.9], "decay"),
    (("layers", 0, "mixer", "decay"), [0.5, 0.9, 1.5], "decay"), (("layers", 1, "mixer", "kv_heads"), 3, "kv_heads"),
    (("layers", 1, "mixer", "vdim"), 16, "vdim"), (("layers", 1, "mixer", "rot", "dims"), 15, "rot.dims"),
    (("layers", 1, "mixer", "rot", "dims"), 34, "rot.dims"), (("layers", 1, "mixer", "rot", "scaling", "high"), 0.5, "high"),
    (("layers", 0, "mlp", "router", "top"), 6, "router.top"), (("layers", 1, "mlp", "kind"), "gated", "kind"),
    (("layers", 2, "weights_of"), 2, "weights_of"), (("layers", 2, "weights_of"), 9, "weights_of"),
    (("layers", 1, "mixer", "heads"), 0, "heads")])
def test_a_value_that_cannot_be_is_refused(path, value, says):
    cfg = _with(pf.tiny_config_p(), path, value)
    if path[:2] == ("layers", 0):
        cfg["layers"][2] = dict(copy.deepcopy(cfg["layers"][0]), weights_of=0)
    with pytest.raises(ConfigError, match=says):
        FazopelConfig.from_dict(cfg)


def test_a_chain_of_layers_ends_at_the_one_with_tensors():
    cfg = pf.tiny_config_p()
    cfg["layers"].append(dict(copy.deepcopy(cfg["layers"][0]), weights_of=2))      # 4 -> 2 -> 0
    c = FazopelConfig.from_dict(cfg)
    assert c.layers[4].weights_of == 0 and c.layers[2].weights_of == 0
    m = build(cfg)
    assert [r.layer for r in m.spec.order] == [0, 1, 0, 2, 0] and len(m.cache_slots) == 5
    cfg["layers"][0]["weights_of"] = 4
    with pytest.raises(ConfigError, match="circle"):
        FazopelConfig.from_dict(cfg)


def test_a_layer_with_anothers_tensors_and_constants_of_its_own():
    """The same tensors under another decay and another router scale: parts of its own that ask for layer 0's tensors."""
    cfg = pf.tiny_config_p()
    cfg["layers"][2]["mixer"] = dict(cfg["layers"][2]["mixer"], decay=[0.1, 0.2, 0.3])
    cfg["layers"][2]["mlp"] = copy.deepcopy(cfg["layers"][2]["mlp"])
    cfg["layers"][2]["mlp"]["router"]["scale"] = 3.0
    m = build(cfg)
    assert [r.layer for r in m.spec.order] == [0, 1, 3, 2] and len(m.spec.layers) == 4
    assert m.spec.layers[3].parts["mixer"].params["decay"] == (0.1, 0.2, 0.3)
    assert m.spec.layers[3].parts["ffn"].params["route_scale"] == 3.0
    assert m.spec.layers[3].parts["mixer"].weights["q"] == "l0.mix.q" and m.spec.layers[3].parts["ffn_norm"].weights["weight"] == "l0.norm2"
    assert {k: tuple(v.shape) for k, v in m.tensor_requests().items()} == pf.tensor_shapes(pf.tiny_config_p())


def test_what_may_go_unsaid():
    cfg = pf.tiny_config_p()
    del cfg["layers"][1]["mixer"]["vdim"]                       # the attention's values are its keys
    cfg["layers"][0]["mixer"]["decay"] = 0.75                   # one decay for all heads
    cfg["layers"][2] = dict(copy.deepcopy(cfg["layers"][0]), weights_of=0)
    del cfg["layers"][3]["mlp"]                                 # no feed-forward: null or absent
    c = FazopelConfig.from_dict(cfg)
    assert c.layers[0].mixer.decay == (0.75, 0.75, 0.75) and c.layers[3].mlp is None
    assert build(cfg).cache_slots[1].spec == KVCacheSpec(2, 32, 0)


def test_long_wavelengths_are_slowed_down():
    """The frequencies the product hands its kernels, for wavelengths on both sides of both borders and between."""
    from prelude_amd.parts.rope import RotaryFrequencies
    for base, dims, sc in ((1000.0, 16, (8.0, 1.0, 4.0, 64)), (50000.0, 32, (4.0, 1.0, 2.0, 128)), (100.0, 24, None),
                           (20000.0, 64, (2.0, 0.5, 8.0, 4096)), (10.0, 8, (3.0, 2.0, 3.0, 16))):
        rot = {"base": base, "dims": dims}
        kw = {}
        if sc is not None:
            rot["scaling"] = dict(zip(("factor", "low", "high", "original"), sc))
            kw = dict(long_wave_factor=sc[0], long_wave_low=sc[1], long_wave_high=sc[2], long_wave_original=sc[3])
        got = RotaryFrequencies(dims, base, **kw).frequencies()
        want = pf.scaled_frequencies(rot)
        assert torch.allclose(got, want, rtol=1e-12, atol=0), (base, dims, sc)
        if sc is not None:
            assert not torch.allclose(got, pf.scaled_frequencies({"base": base, "dims": dims}), rtol=1e-3), "the case scales something"


# ---- the plain implementation against itself ---------------------------------------------------------------------
def test_the_plain_state_carries_over_a_cut():
    cfg = pf.tiny_config_q()
    w = {k: v.double() for k, v in pf.random_weights(cfg, 5).items()}
    m = cfg["layers"][1]["mixer"]
    h = torch.randn(30, cfg["width"], dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    whole, S = pf.decaying_state_mixer(h, w, "l1.mix.", m, 1e-6)
    a, Sa = pf.decaying_state_mixer(h[:11], w, "l1.mix.", m, 1e-6)
    b, Sb = pf.decaying_state_mixer(h[11:], w, "l1.mix.", m, 1e-6, state=Sa)
    assert torch.allclose(torch.cat([a, b]), whole, rtol=1e-12, atol=1e-12) and torch.allclose(Sb, S, rtol=1e-12, atol=1e-14)


def test_the_plain_sink_takes_its_share():
    s = torch.tensor([[0.0, -1e9], [2.0, 1.0]], dtype=torch.float64)
    p = pf.softmax_with_empty_sink(s)
    assert torch.allclose(p[0], torch.tensor([0.5, 0.0], dtype=torch.float64))
    e = torch.exp(s[1])
    assert torch.allclose(p[1], e / (1 + e.sum())) and float(p[1].sum()) < 1.0


def test_the_plain_router_weighs_by_the_score_alone():
    w = {"m.router": torch.eye(4, dtype=torch.float64) * 3, "m.correction": torch.tensor([0.0, 0.0, 5.0, 0.0], dtype=torch.float64)}
    h = torch.tensor([[1.0, 0.5, 0.0, 0.0]], dtype=torch.float64)
    chosen, ws = pf.route(h, w, "m.", 2, 2.0)
    assert sorted(chosen[0].tolist()) == [0, 2], "the correction brings expert 2 in"
    s = torch.softmax(h @ w["m.router"].T, dim=-1)[0]
    got = dict(zip(chosen[0].tolist(), ws[0].tolist()))
    assert abs(got[0] - 2.0 * float(s[0] / (s[0] + s[2]))) < 1e-12 and abs(got[0] + got[2] - 2.0) < 1e-12
