"""Libodra, plainly: every mechanism as one slow function on CPU tensors, written from the design's equations.

Nothing here is shared with the product path, and nothing is rearranged for speed: keys and values are
expanded per head from the latent (the product keeps the latent and moves the maps to the query side), a
sequence is always run whole, and the experts are visited token by token.  ``dtype`` float64 by default.

    norm(x; w)      = x / sqrt(mean(x^2) + eps) * (1 + w)
    layer           x <- x + mixer(norm(x; w1));  x <- x + ff(norm(x; w2))   (the second only with a feed-forward)
    output          logits = head . norm(x; w_final)
"""
import math

import torch


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    return unit_rms(x, eps) * (1.0 + w)


def turn_pairs(x, positions, base, dims):
    """x [T, ..., D]: of the first ``dims`` dimensions, (2i, 2i+1) is turned by the angle p * base^(-2i/dims)."""
    out = x.clone()
    for i in range(dims // 2):
        ang = positions.to(x.dtype) * (float(base) ** (-2.0 * i / dims))
        c, s = torch.cos(ang), torch.sin(ang)
        while c.dim() < x.dim() - 1:
            c, s = c.unsqueeze(-1), s.unsqueeze(-1)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def sink_softmax(scores, sink):
    """Softmax over the last axis whose denominator also holds exp(sink); scores may hold -inf."""
    m = torch.maximum(scores.max(dim=-1, keepdim=True).values, sink)
    e = torch.exp(scores - m)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - m))


def latent_mixer(h, w, pre, m, eps, positions=None, window=0):
    """h [T, width]; ``m``: the layer's mixer sizes as in the configuration; ``w[pre + name]`` its tensors."""
    n = h.shape[0]
    H, d, r, vd, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(n) if positions is None else positions
    cq = unit_rms(h @ w[pre + "dq"].T, eps) * w[pre + "dq.norm"]
    q = (cq @ w[pre + "uq"].T).reshape(n, H, d + r)
    low = h @ w[pre + "dkv"].T
    c = unit_rms(low[:, :rank], eps) * w[pre + "dkv.norm"]
    shared = turn_pairs(low[:, rank:], pos, m["rot"]["base"], m["rot"]["dims"])          # [T, r], one for all heads
    k_plain = (c @ w[pre + "uk"].T).reshape(n, H, d)
    val = (c @ w[pre + "uv"].T).reshape(n, H, vd)
    q_plain = q[..., :d]
    q_turn = turn_pairs(q[..., d:], pos, m["rot"]["base"], m["rot"]["dims"])
    out = torch.zeros(n, H, vd, dtype=h.dtype)
    for head in range(H):
        s = (q_plain[:, head] @ k_plain[:, head].T + q_turn[:, head] @ shared.T) * m["scale"]
        seen = pos[:, None] >= pos[None, :]
        if window:
            seen = seen & (pos[None, :] > pos[:, None] - window)
        s = s.masked_fill(~seen, -math.inf)
        out[:, head] = sink_softmax(s, w[pre + "sink"][head].to(h.dtype)) @ val[:, head]
    return out.reshape(n, H * vd) @ w[pre + "o"].T


def clamped_pair_ff(h, w, pre, limit, alpha=1.702):
    g = torch.clamp(h @ w[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ w[pre + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)) @ w[pre + "down"].T


def squared_relu_expert(h, w, pre):
    return (torch.relu(h @ w[pre + "up"].T) ** 2) @ w[pre + "down"].T


def table_experts_ff(h, tokens, w, pre, f):
    """Each token's experts are the row of the table at its id; each counts 1/top; a shared expert is added."""
    top = f["router"]["top"]
    out = torch.zeros_like(h)
    for t, tok in enumerate(tokens):
        for j in range(top):
            e = int(w[pre + "table"][tok, j])
            out[t] += squared_relu_expert(h[t:t + 1], w, f"{pre}e{e}.")[0] / top
    if f.get("shared"):
        out = out + squared_relu_expert(h, w, pre + "shared.")
    return out


def forward(cfg, w, tokens, dtype=torch.float64, layers_out=None):
    """Logits [T, vocab] for one sequence run whole from position 0."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        x = x + latent_mixer(offset_norm(x, w[p + "norm1"], eps), w, p + "mix.", layer["mixer"], eps)
        f = layer["mlp"]
        if f is not None:
            hn = offset_norm(x, w[p + "norm2"], eps)
            if f["kind"] == "dense":
                x = x + clamped_pair_ff(hn, w, p + "mlp.", f["limit"])
            else:
                x = x + table_experts_ff(hn, tokens, w, p + "mlp.", f)
        if layers_out is not None:
            layers_out.append(x.clone())
    return offset_norm(x, w["final.norm"], eps) @ w["head"].T


# ---- configurations and weights of the tests' own ------------------------------------------------------------
def mixer_cfg(heads, dim, rot_dim, vdim, kv_rank, q_rank, base=10000.0, rot_dims=None, scale=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
            "rot": {"base": base, "dims": rot_dim if rot_dims is None else rot_dims},
            "scale": (dim + rot_dim) ** -0.5 if scale is None else scale}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(experts, top, ff, shared_ff=None):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared_ff:
        f["shared"] = {"ff": shared_ff}
    return f


def config(vocab, width, layers, eps=1e-5):
    return {"architecture": "Libodra", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "layers": [{"type": "latent_attention", "mixer": m, "mlp": f} for m, f in layers]}


def tiny_config_p():
    """Odd sizes: three heads, a latent that is no multiple of 16, values wider than keys, two experts a token,
    a part of the rotated dimensions left unturned, a layer without a feed-forward, experts without a shared one."""
    a = mixer_cfg(3, 24, 16, 40, 48, 40, base=1000.0, rot_dims=8, scale=0.21)
    b = mixer_cfg(5, 16, 8, 16, 72, 24, base=300.0)
    return config(97, 80, [(a, moe(6, 2, 24, 56)), (b, None), (a, dense(112, 0.9)), (b, moe(5, 3, 40))], eps=3e-5)


def tiny_config_q():
    """Sizes in steps of 64, one expert a token, every layer alike but the feed-forward."""
    a = mixer_cfg(8, 32, 32, 32, 128, 64, base=50000.0)
    return config(300, 128, [(a, dense(256, 2.5)), (a, moe(4, 1, 64, 64)), (a, dense(256, 2.5))], eps=1e-6)


def tiny_config_r():
    """Sizes that fit no 16-byte piece: a width of 100, one and two heads, a latent of 20, all experts for every
    token, layers that differ in every size."""
    a = mixer_cfg(1, 10, 6, 12, 20, 12, base=77.0, rot_dims=2, scale=0.4)
    b = mixer_cfg(2, 6, 4, 10, 28, 20, base=5000.0)
    return config(50, 100, [(a, dense(50, 1.1)), (b, moe(3, 3, 30, 18)), (b, None), (a, moe(2, 1, 14))], eps=1e-4)


def tensor_shapes(cfg):
    V, W = cfg["vocab"], cfg["width"]
    out = {"embed": (V, W), "final.norm": (W,), "head": (V, W)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        H, d, r, vd, rank, qr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        out.update({p + "norm1": (W,), p + "mix.dq": (qr, W), p + "mix.dq.norm": (qr,), p + "mix.uq": (H * (d + r), qr),
                    p + "mix.dkv": (rank + r, W), p + "mix.dkv.norm": (rank,), p + "mix.uk": (H * d, rank),
                    p + "mix.uv": (H * vd, rank), p + "mix.sink": (H,), p + "mix.o": (W, H * vd)})
        f = layer["mlp"]
        if f is None:
            continue
        out[p + "norm2"] = (W,)
        if f["kind"] == "dense":
            out.update({p + "mlp.gate": (f["ff"], W), p + "mlp.up": (f["ff"], W), p + "mlp.down": (W, f["ff"])})
        else:
            for e in range(f["router"]["experts"]):
                out.update({f"{p}mlp.e{e}.up": (f["expert"]["ff"], W), f"{p}mlp.e{e}.down": (W, f["expert"]["ff"])})
            out[p + "mlp.table"] = (V, f["router"]["top"])
            if f.get("shared"):
                out.update({p + "mlp.shared.up": (f["shared"]["ff"], W), p + "mlp.shared.down": (W, f["shared"]["ff"])})
    return out


def random_weights(cfg, seed=0, gain=1.0):
    """Weights large enough that every mechanism moves the logits: projections of unit-order outputs, norm weights
    and sinks of order one half, tables of distinct experts.  Rounded to bfloat16 (what a model file holds)."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith("table"):
            layer = cfg["layers"][int(name[1:name.index(".")])]["mlp"]
            n = layer["router"]["experts"]
            w[name] = torch.stack([torch.randperm(n, generator=g)[:shape[1]] for _ in range(shape[0])]).to(torch.int32)
        elif len(shape) == 1:
            scale = 1.0 if name.endswith("sink") else (0.3 if name.endswith(("norm1", "norm2", "final.norm")) else 0.0)
            t = torch.randn(shape, generator=g) * scale
            w[name] = (t if scale else 1.0 + 0.2 * torch.randn(shape, generator=g)).to(torch.bfloat16).float()
        else:
            std = gain / math.sqrt(shape[1]) if name not in ("embed",) else 1.0
            w[name] = (torch.randn(shape, generator=g) * std).to(torch.bfloat16).float()
    return w
