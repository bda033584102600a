"""Fazopel: from its typed configuration to a model specification.

A decoder whose layers are listed one by one in the configuration.  A layer norms each branch's output before adding
it, x <- x + norm1(mixer(x)) and, where it has a feed-forward, x <- x + norm2(ff(x)), with plain RMS norms and a
32-bit stream (``branch_norm``).  The mixer is linear attention with a decaying state per request
(``lightning_attention``) or grouped-query attention whose values are its keys as projected, with per-head
query/key norm, a partly rotated head, long wavelengths slowed down, a given score scale and an empty sink in the
softmax (``gqa_attention``).  The feed-forward is two products around the square of relu (``squared_relu_mlp``) or
routed experts with an optional gated shared one (``routed_experts``).  A layer that names another's tensors runs
as one more entry of the run order on that layer, with a cache or state of its own.
Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.model_config import FazopelConfig
from ..config.registry import Architecture, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, RunSpec

# the design fixes these
EXPERT_ALPHA = 1.702         # the sigmoid's slope in an expert's gate
# no longest position is part of the design (angles are computed from the position, there is no table); the engine's
# bookkeeping wants a bound, and positions are 32-bit integers
MAX_POSITIONS = 1 << 24


def _layer_spec(cfg: FazopelConfig, lc, p: str, positions) -> LayerSpec:
    """One layer's parts with the constants of its own entry ``lc`` and the tensors named under the prefix ``p``."""
    h = cfg.width
    norm = lambda name: PartSpec("rms_norm", dict(size=h, eps=cfg.norm_eps, residual_float32=True), {"weight": name})
    m = lc.mixer
    if lc.type == "lightning":
        mixer = PartSpec("lightning_attention", dict(
            hidden_size=h, num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, decay=m.decay, norm_eps=cfg.norm_eps,
            activation="silu"), {n: f"{p}mix.{n}" for n in ("q", "k", "v", "g", "o", "norm")})
    else:
        pos = None
        if m.rot_dims:
            sc = m.rot_scaling
            pos = f"rot{m.rot_dims}@{m.rot_base!r}/{sc!r}"
            params = dict(rotary_dim=m.rot_dims, theta=m.rot_base)
            if sc is not None:
                params.update(long_wave_factor=sc.factor, long_wave_low=sc.low, long_wave_high=sc.high,
                              long_wave_original=sc.original)
            positions.setdefault(pos, PartSpec("rotary_frequencies", params))
        mixer = PartSpec("gqa_attention", dict(
            hidden_size=h, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, norm_eps=cfg.norm_eps,
            qk_norm=True, position=pos, rotary_dim=m.rot_dims, scale=m.scale, values_from_keys=True, sink="zero"),
            {"q_proj.weight": p + "mix.q", "k_proj.weight": p + "mix.k", "o_proj.weight": p + "mix.o",
             "q_norm.weight": p + "mix.q.norm", "k_norm.weight": p + "mix.k.norm"})
    f = lc.mlp
    if f is None:
        return LayerSpec("branch_norm_mixer_only", {"mixer": mixer, "mixer_norm": norm(p + "norm1")})
    if f.kind == "dense":
        ffn = PartSpec("squared_relu_mlp", dict(hidden_size=h, intermediate_size=f.ff),
                       {"up": p + "mlp.up", "down": p + "mlp.down"})
    else:
        w = {"router": p + "mlp.router", "correction": p + "mlp.correction"}
        for e in range(f.experts):
            for n in ("gate", "up", "down"):
                w[f"e{e}.{n}"] = f"{p}mlp.e{e}.{n}"
        if f.shared_ff:
            for n in ("gate", "up", "down", "sg"):
                w[f"shared.{n}"] = f"{p}mlp.shared.{n}"
        ffn = PartSpec("routed_experts", dict(
            hidden_size=h, num_experts=f.experts, top=f.top, expert_size=f.ff, limit=f.limit, route_scale=f.route_scale,
            alpha=EXPERT_ALPHA, correction=True, shared_size=f.shared_ff, shared_limit=f.shared_limit), w)
    return LayerSpec("branch_norm", {"mixer": mixer, "mixer_norm": norm(p + "norm1"), "ffn": ffn,
                                     "ffn_norm": norm(p + "norm2")})


def fazopel_spec(cfg: FazopelConfig) -> ModelSpec:
    import dataclasses
    h = cfg.width
    positions = {}
    layers, order, index_of = [], [], {}
    for i, lc in enumerate(cfg.layers):
        if lc.weights_of is None:
            index_of[i] = len(layers)
            layers.append(_layer_spec(cfg, lc, f"l{i}.", positions))
    for i, lc in enumerate(cfg.layers):
        j = lc.weights_of
        if j is None:
            order.append(RunSpec(index_of[i]))
        elif dataclasses.replace(lc, weights_of=None) == cfg.layers[j]:
            order.append(RunSpec(index_of[j]))        # layer j once more: the same parts, a cache or state of its own
        else:
            # layer j's tensors under constants of this entry's own (a decay, a scale, a clamp that differ): parts
            # of its own that ask for the same tensors
            order.append(RunSpec(len(layers)))
            layers.append(_layer_spec(cfg, lc, f"l{j}.", positions))
    norm = PartSpec("rms_norm", dict(size=h, eps=cfg.norm_eps, residual_float32=True), {"weight": "final.norm"})
    return ModelSpec(
        architecture="Fazopel", vocab_size=cfg.vocab, hidden_size=h, max_positions=MAX_POSITIONS, eos_token_ids=(),
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab, hidden_size=h), {"weight": "embed"}),
        layers=layers, order=order, final_norm=norm,
        head=PartSpec("linear_head", dict(vocab_size=cfg.vocab, hidden_size=h), {"weight": "head"}),
        positions=positions)


FAZOPEL = register_architecture(Architecture(
    name="fazopel", architecture_aliases=("Fazopel",), model_type_aliases=("fazopel",),
    parse_config=FazopelConfig.from_dict, build_spec=fazopel_spec))
