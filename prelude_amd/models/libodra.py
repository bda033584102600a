"""Libodra: from its typed configuration to a model specification.

A decoder whose layers are listed one by one in the configuration.  A layer is pre-norm, x <- x + mixer(norm1(x))
and, where it has a feed-forward, x <- x + ff(norm2(x)); the norms are RMS norms whose stored weight lies around
zero (gain 1 + w).  The mixer attends through a latent with a learned sink per head (``latent_attention``); the
feed-forward is a clamped gated pair (``clamped_gated_mlp``) or experts chosen by token id from a table, with an
optional shared expert (``table_experts``).  The residual stream is 32-bit whatever the engine's element type.
Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.model_config import LibodraConfig
from ..config.registry import Architecture, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, RunSpec

# the design fixes these
GATE_ALPHA = 1.702           # the sigmoid's slope in the dense feed-forward
# no longest position is part of the design (angles are computed from the position, there is no table); the engine's
# bookkeeping wants a bound, and positions are 32-bit integers
MAX_POSITIONS = 1 << 24


def libodra_spec(cfg: LibodraConfig) -> ModelSpec:
    h = cfg.width
    positions = {}
    layers = []
    for i, lc in enumerate(cfg.layers):
        p = f"l{i}."
        m = lc.mixer
        pos = None
        if m.rot_dims:
            pos = f"rot{m.rot_dims}@{m.rot_base!r}"
            positions.setdefault(pos, PartSpec("rotary_frequencies", dict(rotary_dim=m.rot_dims, theta=m.rot_base)))
        names = ("dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "sink", "o")
        mixer = PartSpec("latent_attention", dict(
            hidden_size=h, num_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, value_dim=m.vdim, kv_rank=m.kv_rank,
            q_rank=m.q_rank, norm_eps=cfg.norm_eps, scale=m.scale, position=pos, rotary_dim=m.rot_dims, sink=True),
            {n: f"{p}mix.{n}" for n in names})
        norm = lambda name: PartSpec("rms_norm", dict(size=h, eps=cfg.norm_eps, weight_offset=1.0, residual_float32=True),
                                     {"weight": name})
        f = lc.mlp
        if f is None:
            layers.append(LayerSpec("prenorm_mixer_only", {"input_norm": norm(p + "norm1"), "mixer": mixer}))
            continue
        if f.kind == "dense":
            ffn = PartSpec("clamped_gated_mlp", dict(hidden_size=h, intermediate_size=f.ff, limit=f.limit, alpha=GATE_ALPHA),
                           {n: f"{p}mlp.{n}" for n in ("gate", "up", "down")})
        else:
            w = {"table": p + "mlp.table"}
            for e in range(f.experts):
                w[f"e{e}.up"] = f"{p}mlp.e{e}.up"
                w[f"e{e}.down"] = f"{p}mlp.e{e}.down"
            if f.shared_ff:
                w["shared.up"], w["shared.down"] = p + "mlp.shared.up", p + "mlp.shared.down"
            ffn = PartSpec("table_experts", dict(hidden_size=h, vocab_size=cfg.vocab, num_experts=f.experts, top=f.top,
                                                 expert_size=f.ff, shared_size=f.shared_ff), w)
        layers.append(LayerSpec("prenorm", {"input_norm": norm(p + "norm1"), "mixer": mixer,
                                            "post_mixer_norm": norm(p + "norm2"), "ffn": ffn}))
    return ModelSpec(
        architecture="Libodra", vocab_size=cfg.vocab, hidden_size=h, max_positions=MAX_POSITIONS, eos_token_ids=(),
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab, hidden_size=h), {"weight": "embed"}),
        layers=layers, order=[RunSpec(i) for i in range(len(layers))],
        final_norm=PartSpec("rms_norm", dict(size=h, eps=cfg.norm_eps, weight_offset=1.0, residual_float32=True),
                            {"weight": "final.norm"}),
        head=PartSpec("linear_head", dict(vocab_size=cfg.vocab, hidden_size=h), {"weight": "head"}),
        positions=positions)


LIBODRA = register_architecture(Architecture(
    name="libodra", architecture_aliases=("Libodra",), model_type_aliases=("libodra",),
    parse_config=LibodraConfig.from_dict, build_spec=libodra_spec))
