"""Libodra without a GPU: the configuration's reader, the specification built from it, random tables, and the
plain implementation against itself (the latent kept and the maps moved to the query side give the same scores)."""
import copy

import pytest
import torch

import plain_libodra as pl
from prelude_amd import models  # noqa: F401
from prelude_amd.config import ConfigError, resolve_architecture
from prelude_amd.models.causal_lm import CausalLM
from prelude_amd.weights.random_init import random_tensors


def build(raw):
    a = resolve_architecture(raw)
    return CausalLM(a.build_spec(a.parse_config(raw)))


@pytest.mark.parametrize("make", [pl.tiny_config_p, pl.tiny_config_q, pl.tiny_config_r])
def test_the_model_asks_for_the_tensors_the_design_names(make):
    raw = make()
    m = build(raw)
    want = pl.tensor_shapes(raw)
    got = {k: tuple(v.shape) for k, v in m.tensor_requests().items()}
    assert got == want
    kinds = [type(b).KIND for b in m.blocks]
    assert kinds == ["prenorm" if l["mlp"] is not None else "prenorm_mixer_only" for l in raw["layers"]]
    assert not m.needs_state and m.graph_safe and m.graph_safe_portions
    assert len({c.spec for c in m.cache_slots}) == len({(l["mixer"]["kv_rank"], l["mixer"]["rot_dim"]) for l in raw["layers"]})


def test_every_size_and_constant_comes_from_the_configuration():
    raw = pl.tiny_config_p()
    m = build(raw)
    for blk, l in zip(m.blocks, raw["layers"]):
        mx, c = blk.mixer, l["mixer"]
        assert (mx.num_heads, mx.head_dim, mx.rot_dim, mx.value_dim, mx.kv_rank, mx.q_rank) == \
            (c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"], c["q_rank"])
        assert mx.scale == c["scale"] and mx.rotary_dim == c["rot"]["dims"] and mx.rope.theta == c["rot"]["base"]
        assert mx.norm_eps == raw["norm"]["eps"] and blk.input_norm.eps == raw["norm"]["eps"]
        f = l["mlp"]
        if f and f["kind"] == "dense":
            assert (blk.ffn.intermediate_size, blk.ffn.limit) == (f["ff"], f["limit"])
        elif f:
            assert (blk.ffn.num_experts, blk.ffn.top, blk.ffn.expert_size) == (f["router"]["experts"], f["router"]["top"], f["expert"]["ff"])
            assert blk.ffn.shared_size == (f["shared"]["ff"] if f.get("shared") else 0)


@pytest.mark.parametrize("path,value,word", [
    (("vocab",), None, "vocab"), (("layers", 0, "type"), "other", "type"), (("layers", 0, "mixer", "heads"), 0, "heads"),
    (("layers", 0, "mixer", "rot", "dims"), 7, "rot.dims"), (("layers", 2, "mlp", "kind"), "gated", "kind"),
    (("layers", 0, "mlp", "router", "top"), 9, "top"), (("norm",), None, "norm"), (("layers",), [], "layers")])
def test_a_wrong_configuration_is_named(path, value, word):
    raw = copy.deepcopy(pl.tiny_config_p())
    at = raw
    for k in path[:-1]:
        at = at[k]
    if value is None:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    with pytest.raises(ConfigError, match=word.replace(".", r"\.")):
        build(raw)


def test_random_weights_give_tables_of_distinct_experts():
    raw = pl.tiny_config_p()
    t = random_tensors(raw, seed=3, device="cpu")
    table = t["l0.mlp.table"]
    assert table.dtype == torch.int32 and tuple(table.shape) == (raw["vocab"], 2)
    assert int(table.min()) >= 0 and int(table.max()) < 6 and bool((table[:, 0] != table[:, 1]).all())
    assert len(set(table.reshape(-1).tolist())) == 6
    assert abs(float(t["l0.norm1"].float().mean())) < 0.1, "norm weights lie around zero"


def test_the_latent_alone_gives_the_expanded_keys_scores():
    """(W_uk^T q) . c = q . (W_uk c), and the sum of weighted latents through W_uv is the sum of weighted values."""
    g = torch.Generator().manual_seed(0)
    d, rank, vd, n = 12, 20, 7, 9
    uk, uv = torch.randn(d, rank, generator=g, dtype=torch.float64), torch.randn(vd, rank, generator=g, dtype=torch.float64)
    q, c = torch.randn(d, generator=g, dtype=torch.float64), torch.randn(n, rank, generator=g, dtype=torch.float64)
    assert torch.allclose((uk.T @ q) @ c.T, q @ (c @ uk.T).T)
    p = pl.sink_softmax((q @ (c @ uk.T).T)[None, :], torch.tensor(0.3, dtype=torch.float64))[0]
    assert float(p.sum()) < 1.0
    assert torch.allclose(uv @ (p @ c), p @ (c @ uv.T))


def test_plain_prefix_logits_do_not_depend_on_what_follows():
    raw = pl.tiny_config_p()
    w = pl.random_weights(raw, 5)
    toks = list(range(3, 40))
    full = pl.forward(raw, w, toks)
    assert torch.allclose(pl.forward(raw, w, toks[:11]), full[:11], atol=1e-9)
