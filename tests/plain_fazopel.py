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
    """f_i = base^(-2i/dims), then long wavelengths slowed down: wavelength l = 2 pi / f; l < original / high keeps
    f, l > original / low gives f / factor, and between them the two are blended by
    s = (original / l - low) / (high - low): (1 - s) f / factor + s f."""
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
