"""Fazopel, plainly: every mechanism as one slow function on CPU tensors, written from the design's equations.

Nothing here is shared with the product path and nothing is arranged for speed: the recurrent mixer walks a
sequence token by token, the attention builds the whole score matrix, the experts are visited token by token.
``dtype`` float64 by default.  ``cfg`` is a config.json's content, ``w`` name -> tensor.

    unit(x)         = x / sqrt(mean(x^2) + eps)
    layer           x <- x + unit(mixer(x)) * w1;  x <- x + unit(ff(x)) * w2      (the sublayers read x itself)
    output          logits = head . (unit(x) * w_final)
"""
import math

import torch


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(x):
    return x * torch.sigmoid(x)


# ---- the recurrent mixer ---------------------------------------------------------------------------------------
def decaying_state_mixer(h, w, pre, m, eps, state=None):
    """h [T, width] of one sequence.  Per head S_t = a S_(t-1) + k_t v_t^T and o_t = S_t^T q_t, with q, k, v
    passed through SiLU; the heads side by side are brought to unit RMS together, scaled, gated and projected.
    ``state`` [heads, dim, vdim] is where the sequence stands (None: zero); returns (output, state after)."""
    n = h.shape[0]
    H, d, vd = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[pre + "q"].T).reshape(n, H, d)
    k = silu(h @ w[pre + "k"].T).reshape(n, H, d)
    v = silu(h @ w[pre + "v"].T).reshape(n, H, vd)
    S = torch.zeros(H, d, vd, dtype=h.dtype) if state is None else state.clone()
    a = torch.tensor(m["decay"], dtype=h.dtype)
    out = torch.zeros(n, H, vd, dtype=h.dtype)
    for t in range(n):
        S = a[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    o = unit_rms(out.reshape(n, H * vd), eps) * w[pre + "norm"]
    o = o * torch.sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T, S


# ---- attention ---------------------------------------------------------------------------------------------------
def scaled_frequencies(rot, dtype=torch.float64):
    """f_i = base^(-2i/dims); with a scaling, by each frequency's wavelength lambda = 2 pi / f_i: short waves
    (lambda < original / high) keep f_i, long ones (lambda > original / low) get f_i / factor, and a wave between the
    two a mixture of both, weighted t and 1 - t with t = (original / lambda - low) / (high - low)."""
    dims = rot["dims"]
    f = torch.tensor([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=dtype)
    sc = rot.get("scaling")
    if not sc:
        return f
    out = f.clone()
    for i in range(dims // 2):
        l = 2.0 * math.pi / float(f[i])
        if l < sc["original"] / sc["high"]:
            continue
        if l > sc["original"] / sc["low"]:
            out[i] = f[i] / sc["factor"]
        else:
            s = (sc["original"] / l - sc["low"]) / (sc["high"] - sc["low"])
            out[i] = (1.0 - s) * f[i] / sc["factor"] + s * f[i]
    return out


def turn_halves(x, positions, freqs):
    """x [T, heads, D]: dimension i < n is paired with i + n (n = len(freqs)) and the pair turned by p * f_i; the
    dimensions from 2n on pass through."""
    n = freqs.shape[0]
    ang = positions.to(x.dtype)[:, None] * freqs.to(x.dtype)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :n], x[..., n:2 * n]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * n:]], dim=-1)


def softmax_with_empty_sink(scores):
    """p_j = exp(s_j) / (1 + sum exp(s_j)): one more term of score 0 in the denominator that brings no value."""
    m = torch.clamp(scores.max(dim=-1, keepdim=True).values, min=0.0)
    e = torch.exp(scores - m)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(-m))


def keys_as_values_attention(h, w, pre, m, eps, positions=None):
    """h [T, width] of one sequence.  Grouped queries; the values are the keys as projected (before norm and turn)."""
    n = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    pos = torch.arange(n) if positions is None else positions
    q = (h @ w[pre + "q"].T).reshape(n, H, d)
    k = (h @ w[pre + "k"].T).reshape(n, G, d)
    val = k
    q = unit_rms(q, eps) * w[pre + "q.norm"]
    k = unit_rms(k, eps) * w[pre + "k.norm"]
    f = scaled_frequencies(m["rot"], h.dtype)
    q, k = turn_halves(q, pos, f), turn_halves(k, pos, f)
    out = torch.zeros(n, H, d, dtype=h.dtype)
    seen = pos[:, None] >= pos[None, :]
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        s = s.masked_fill(~seen, -math.inf)
        out[:, head] = softmax_with_empty_sink(s) @ val[:, g]
    return out.reshape(n, H * d) @ w[pre + "o"].T


# ---- feed-forward ------------------------------------------------------------------------------------------------
def squared_relu_ff(h, w, pre):
    return (torch.relu(h @ w[pre + "up"].T) ** 2) @ w[pre + "down"].T


def clamped_expert(h, w, pre, limit, alpha=1.702):
    g = torch.clamp(h @ w[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ w[pre + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)) @ w[pre + "down"].T


def route(h, w, pre, top, scale):
    """(chosen experts [T, top], their weights [T, top]): scores softmax(W_router h); chosen by score + correction,
    weighted by the score alone, over the chosen ones' sum, times ``scale``."""
    s = torch.softmax(h @ w[pre + "router"].T, dim=-1)
    chosen = torch.topk(s + w[pre + "correction"], top, dim=-1).indices
    ws = torch.gather(s, 1, chosen)
    return chosen, ws / (ws.sum(dim=-1, keepdim=True) + 1e-20) * scale


def routed_experts_ff(h, w, pre, f):
    chosen, ws = route(h, w, pre, f["router"]["top"], f["router"]["scale"])
    out = torch.zeros(h.shape[0], w[pre + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t].tolist(), ws[t]):
            out[t] += a * clamped_expert(h[t:t + 1], w, f"{pre}e{e}.", f["expert"]["limit"])[0]
    if f.get("shared"):
        gate = torch.sigmoid(h @ w[pre + "shared.sg"].T)            # [T, 1]
        out = out + gate * clamped_expert(h, w, pre + "shared.", f["shared"]["limit"])
    return out


# ---- the model ---------------------------------------------------------------------------------------------------
def forward(cfg, w, tokens, dtype=torch.float64, layers_out=None):
    """Logits [T, vocab] of one whole sequence; ``layers_out`` (a list) receives the stream after every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{lc.get('weights_of', i)}."
        if lc["type"] == "lightning":
            y, _ = decaying_state_mixer(x, w, p + "mix.", lc["mixer"], eps)
        elif lc["type"] == "attention":
            y = keys_as_values_attention(x, w, p + "mix.", lc["mixer"], eps)
        else:
            raise ValueError(lc["type"])
        x = x + unit_rms(y, eps) * w[p + "norm1"]
        f = lc.get("mlp")
        if f is not None:
            y = squared_relu_ff(x, w, p + "mlp.") if f["kind"] == "dense" else routed_experts_ff(x, w, p + "mlp.", f)
            x = x + unit_rms(y, eps) * w[p + "norm2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    return (unit_rms(x, eps) * w["final.norm"]) @ w["head"].T


# ---- configurations and weights of the tests' own --------------------------------------------------------------------
def _lightning(heads, dim, vdim, decay):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}}


def _attention(heads, kv_heads, dim, scale, base, dims, scaling=None):
    rot = {"base": base, "dims": dims}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "rot": rot}}


def _moe(experts, top, ff, limit, scale, shared=None):
    f = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top, "scale": scale}}
    if shared is not None:
        f["shared"] = {"ff": shared[0], "limit": shared[1]}
    return f


def tiny_config_p():
    """Three heads of unequal decay, a layer run twice, a layer without a feed-forward, heads of 32 and 16."""
    first = dict(_lightning(3, 16, 24, (0.5, 0.9, 0.995)), mlp=_moe(5, 2, 24, 1.5, 1.5, shared=(40, 0.7)))
    return {"architecture": "Fazopel", "vocab": 97, "width": 64, "norm": {"eps": 1e-5}, "layers": [
        first,
        dict(_attention(4, 2, 32, 0.2, 1000.0, 16, scaling=(8.0, 1.0, 4.0, 64)), mlp={"kind": "dense", "ff": 96}),
        dict(first, weights_of=0),
        dict(_attention(6, 3, 16, 0.3, 10000.0, 16), mlp=None)]}


def tiny_config_q():
    """Attention first; one KV head under four query heads; odd state sizes; a decay of 1; experts without a shared one."""
    first = dict(_attention(4, 1, 64, 0.11, 50000.0, 32, scaling=(4.0, 1.0, 2.0, 128)), mlp=_moe(8, 3, 16, 2.0, 1.0))
    return {"architecture": "Fazopel", "vocab": 211, "width": 128, "norm": {"eps": 1e-6}, "layers": [
        first,
        dict(_lightning(2, 40, 72, (0.97, 1.0)), mlp={"kind": "dense", "ff": 160}),
        dict(first, weights_of=0),
        dict(_lightning(4, 32, 32, (0.6, 0.8, 0.9, 0.99)), mlp=_moe(4, 1, 32, 0.8, 2.5, shared=(24, 1.2)))]}


def tiny_config_r():
    """Ones: one head, one KV head, every expert chosen, a decay of 0; a head size the matrix cores do not take; the
    whole head rotated; value columns beyond two tiles."""
    return {"architecture": "Fazopel", "vocab": 61, "width": 48, "norm": {"eps": 1e-5}, "layers": [
        dict(_lightning(1, 8, 130, (0.9,)), mlp=_moe(3, 3, 8, 1.0, 1.0, shared=(8, 1.0))),
        dict(_attention(1, 1, 24, 0.25, 100.0, 24), mlp={"kind": "dense", "ff": 40}),
        dict(_lightning(2, 8, 8, (0.0, 0.75)), mlp=None)]}


def tensor_shapes(cfg):
    """name -> shape of every tensor a model of this configuration stores."""
    h, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"]), "final.norm": (cfg["width"],), "head": (cfg["vocab"], cfg["width"])}
    for i, lc in enumerate(cfg["layers"]):
        if "weights_of" in lc:
            continue
        p, m = f"l{i}.", lc["mixer"]
        out[p + "norm1"] = (h,)
        if lc["type"] == "lightning":
            qk, vv = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            out.update({p + "mix.q": (qk, h), p + "mix.k": (qk, h), p + "mix.v": (vv, h), p + "mix.g": (vv, h),
                        p + "mix.o": (h, vv), p + "mix.norm": (vv,)})
        else:
            out.update({p + "mix.q": (m["heads"] * m["dim"], h), p + "mix.k": (m["kv_heads"] * m["dim"], h),
                        p + "mix.q.norm": (m["dim"],), p + "mix.k.norm": (m["dim"],), p + "mix.o": (h, m["heads"] * m["dim"])})
        f = lc.get("mlp")
        if f is None:
            continue
        out[p + "norm2"] = (h,)
        if f["kind"] == "dense":
            out.update({p + "mlp.up": (f["ff"], h), p + "mlp.down": (h, f["ff"])})
            continue
        e = f["router"]["experts"]
        out.update({p + "mlp.router": (e, h), p + "mlp.correction": (e,)})
        for j in range(e):
            ff = f["expert"]["ff"]
            out.update({f"{p}mlp.e{j}.gate": (ff, h), f"{p}mlp.e{j}.up": (ff, h), f"{p}mlp.e{j}.down": (h, ff)})
        if f.get("shared"):
            ff = f["shared"]["ff"]
            out.update({p + "mlp.shared.gate": (ff, h), p + "mlp.shared.up": (ff, h), p + "mlp.shared.down": (h, ff),
                        p + "mlp.shared.sg": (1, h)})
    return out


def random_weights(cfg, seed):
    """Weights as a file would hold them: values of bfloat16, here as float32.  Matrices ~ N(0, 1 / in) (the gates'
    and the experts' a little larger, so that clamps bite), norm weights around one, corrections of the size of the
    scores' differences."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, shape in tensor_shapes(cfg).items():
        if len(shape) == 1 and name.endswith(("norm1", "norm2", ".norm")):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif name.endswith("correction"):
            t = 0.2 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            boost = 2.0 if (".mlp.e" in name or ".shared." in name or name.endswith("router")) else 1.0
            t = torch.randn(shape, generator=g) * boost / math.sqrt(shape[-1])
        w[name] = t.to(torch.bfloat16).to(torch.float32)
    return w
