"""Libodra on the GPU against the plain implementation (``plain_libodra``): every mechanism's kernels alone, then
the engine under schedules (whole, token by token, portions down to two tokens, unequal requests in one batch,
pages used again, long decoding) and greedy generation through ``LLM``.  Configurations and weights are the
tests' own."""
import functools
import json
import math
import os
import tempfile

import numpy as np
import pytest
import torch

import plain_libodra as pl
from helpers import check

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}
_keep = []


def close(got, want, dtype, what, scale=None):
    got, want = got.double().cpu(), want.double()
    bound = (2e-5 if dtype == "float32" else 2e-2) * (float(want.abs().max()) if scale is None else scale)
    err = float((got - want).abs().max())
    assert err <= bound, f"{what}: {err:.3e} > {bound:.3e}"


def rnd(shape, seed, dtype, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(TD[dtype])


# ---- the mechanisms' kernels alone ------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [80, 256, 1000, 2560, 9000])
def test_norm_with_a_32_bit_residual(gpu, dtype, hidden):
    from prelude_amd.ops import kernels as K
    x = rnd((7, hidden), 1, dtype)
    res = torch.randn((7, hidden), generator=torch.Generator().manual_seed(2)) * 3
    w = torch.randn(hidden, generator=torch.Generator().manual_seed(3)) * 0.3
    s = x.double() + res.double()
    want = pl.offset_norm(s, w.double(), 1e-5)
    r = res.to(gpu)
    out = K.rmsnorm_wide(x.to(gpu), (1 + w).to(gpu), 1e-5, residual=r)
    close(out, want, dtype, "normed")
    assert r.dtype == torch.float32
    close(r, s, "float32", "the residual keeps the unrounded sum")
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=gpu)
    r2 = res.to(gpu)
    out = K.rmsnorm_wide(x.to(gpu), (1 + w).to(gpu), 1e-5, residual=r2, rows=rows)
    close(out, want[[5, 0, 5]], dtype, "chosen rows")
    assert torch.equal(r2.cpu(), res), "chosen rows leave the residual alone"
    parts = torch.randn((3, 7, hidden), generator=torch.Generator().manual_seed(4))
    r3 = res.to(gpu)
    out = K.rmsnorm_wide(K.SliceSums(parts.to(gpu), TD[dtype]), (1 + w).to(gpu), 1e-5, residual=r3)
    close(out, pl.offset_norm(parts.double().sum(0) + res.double(), w.double(), 1e-5), dtype, "from partial sums")


@pytest.mark.parametrize("dtype", DTYPES)
def test_clamped_pair_and_squared_relu(gpu, dtype):
    from prelude_amd.ops import kernels as K
    for rows, inter in ((9, 37), (8, 40)):       # (the second: whole 16-byte pieces, the vector kernels' case)
        gu = rnd((rows, 2 * inter), 5, dtype, 2.0)
        g, u = gu[:, 0::2].double(), gu[:, 1::2].double()
        for limit, alpha in ((1.5, 1.702), (0.4, 1.0), (7.0, 2.5)):
            gc, uc = torch.clamp(g, max=limit), torch.clamp(u, -limit, limit)
            close(K.clamped_gate(gu.to(gpu), limit, alpha), gc * torch.sigmoid(alpha * gc) * (uc + 1), dtype, f"limit {limit}")
        x = rnd((rows, inter), 6, dtype)
        close(K.relu_squared(x.to(gpu)), torch.relu(x.double()) ** 2, dtype, "squared relu")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_rank,rank,rot,dims", [(40, 48, 16, 8), (64, 128, 32, 32), (24, 72, 8, 8), (16, 20, 0, 0)])
def test_latent_prep_norms_rotates_and_caches(gpu, dtype, q_rank, rank, rot, dims):
    from prelude_amd.ops import kernels as K
    T, page, pages, eps, base = 11, 4, 6, 1e-5, 300.0
    down = rnd((T, q_rank + rank + rot), 7, dtype, 2.0)
    wq, wc = 1 + 0.3 * torch.randn(q_rank), 1 + 0.3 * torch.randn(rank)
    pos = torch.tensor([0, 1, 2, 3, 100, 101, 5000, 7, 8, 9, 65537], dtype=torch.int32)
    slots = torch.randperm(page * pages)[:T].to(torch.int32)
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float32) if dims else None
    cache = torch.zeros((pages, page, rank + rot), dtype=TD[dtype], device=gpu)
    cache_t = torch.zeros((pages, rank, page), dtype=TD[dtype], device=gpu)
    cq = K.latent_prep(down.to(gpu), wq.to(gpu), wc.to(gpu), None if freq is None else freq.to(gpu), pos.to(gpu), slots.to(gpu),
                       cache, q_rank, rank, rot, dims, eps, cache_t=cache_t)
    assert torch.equal(cache_t.transpose(1, 2), cache[:, :, :rank]), "the transposed copy holds the same latents"
    d = down.double()
    close(cq, pl.unit_rms(d[:, :q_rank], eps) * wq.double(), dtype, "query latent")
    got = cache.reshape(-1, rank + rot)[slots.long().to(gpu)]
    close(got[:, :rank], pl.unit_rms(d[:, q_rank:q_rank + rank], eps) * wc.double(), dtype, "latent")
    if rot:
        # angles of large positions: the 32-bit product p * f decides, so the comparison is against that product
        want = pl.turn_pairs(d[:, q_rank + rank:], pos, base, dims)
        close(got[:, rank:], want, dtype, "shared key part", scale=float(d.abs().max()) * (50 if dtype == "float32" else 1))
    untouched = torch.ones(pages * page, dtype=torch.bool)
    untouched[slots.long()] = False
    assert float(cache.reshape(-1, rank + rot)[untouched.to(gpu)].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
def test_rotation_of_a_part_of_every_head(gpu, dtype):
    from prelude_amd.ops import kernels as K
    T, H, d, r, dims, rank, base = 6, 3, 24, 16, 8, 48, 1000.0
    q = rnd((T, H, d + r), 8, dtype)
    pos = torch.tensor([0, 1, 17, 63, 64, 900], dtype=torch.int32)
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float32)
    out = torch.zeros((T, H, rank + r), dtype=TD[dtype], device=gpu)
    K.rotate_pairs(q.to(gpu), out, freq.to(gpu), pos.to(gpu), d, rank, r, dims)
    close(out[..., rank:], pl.turn_pairs(q.double()[..., d:], pos, base, dims), dtype, "rotated part")
    assert float(out[..., :rank].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,H,k,n", [(1, 3, 24, 48), (19, 5, 72, 16), (40, 2, 130, 300), (150, 4, 128, 512)])
def test_a_product_per_head(gpu, dtype, T, H, k, n):
    from prelude_amd.ops import kernels as K
    x = rnd((T, H, k + 5), 9, dtype)
    w = rnd((H, n, k), 10, dtype, 1 / math.sqrt(k))           # [head, out, in]
    out = torch.zeros((T, H, n + 3), dtype=TD[dtype], device=gpu)
    K.head_linear(x.to(gpu), K.GroupedWeight(w.to(gpu)), out, x_off=5, out_off=3)
    want = torch.einsum("thk,hnk->thn", x.double()[..., 5:], w.double())
    close(out[..., 3:], want, dtype, "per-head product")
    assert float(out[..., :3].abs().max()) == 0.0
    if k % 8 == 0:       # rows of whole 16-byte pieces: in bfloat16 the matrix cores take it
        x8 = rnd((T, H, k + 8), 11, dtype)
        out = torch.zeros((T, H, n + 3), dtype=TD[dtype], device=gpu)
        K.head_linear(x8.to(gpu), K.GroupedWeight(w.to(gpu)), out, x_off=8, out_off=3)
        close(out[..., 3:], torch.einsum("thk,hnk->thn", x8.double()[..., 8:], w.double()), dtype, "per-head product, aligned")


def _paged(latents, page, gpu, dtype, seed=0):
    """Scatter sequences' cached vectors [n_i, width] over shuffled pages; returns (cache, block table)."""
    need = [-(-len(x) // page) for x in latents]
    total = sum(need) + 3
    perm = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
    cache = torch.full((total, page, latents[0].shape[1]), 77.0, dtype=TD[dtype])       # stale pages hold rubbish
    table = torch.full((len(latents), max(need)), -1, dtype=torch.int32)
    for i, x in enumerate(latents):
        for j in range(need[i]):
            pg = perm.pop()
            table[i, j] = pg
            part = x[j * page:(j + 1) * page]
            cache[pg, :len(part)] = part.to(TD[dtype])
    return cache.to(gpu), table.to(gpu)


def _plain_latent_attention(q, lat, sink, rank, scale, pos, window=0):
    """q [n, H, width] at positions ``pos`` over cached vectors lat [ctx, width]; returns [n, H, rank]."""
    out = torch.zeros(q.shape[0], q.shape[1], rank, dtype=torch.float64)
    keys = torch.arange(lat.shape[0])
    for h in range(q.shape[1]):
        s = (q[:, h].double() @ lat.double().T) * scale
        seen = keys[None, :] <= pos[:, None]
        if window:
            seen = seen & (keys[None, :] > pos[:, None] - window)
        s = s.masked_fill(~seen, -math.inf)
        out[:, h] = pl.sink_softmax(s, sink[h].double()) @ lat.double()[:, :rank]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,rank,rot,page", [(3, 48, 16, 4), (8, 128, 32, 16), (5, 72, 8, 8), (1, 512, 64, 16)])
def test_latent_attention_over_pages(gpu, dtype, H, rank, rot, page):
    """Two sequences in one launch: a portion of a long one (keys hundreds back, one of them made to stand out)
    and a single token of a short one; sinks of both signs."""
    from prelude_amd.ops import kernels as K
    width, scale = rank + rot, 0.11
    ctx = [333, 130]
    lat = [rnd((n, width), 20 + i, dtype) for i, n in enumerate(ctx)]
    qa, qb = rnd((37, H, width), 30, dtype), rnd((1, H, width), 31, dtype)
    far = 5                                          # a key far back: the last query of the portion points at it
    qa[-1] = (lat[0][far].float() * 3.0).to(TD[dtype])[None, :].expand(H, width)
    sink = torch.linspace(-2.0, 3.0, H)
    cache, table = _paged(lat, page, gpu, dtype)
    pos = torch.cat([torch.arange(ctx[0] - 37, ctx[0]), torch.tensor([ctx[1] - 1])]).to(torch.int32)
    seq = torch.tensor([0] * 37 + [1], dtype=torch.int32)
    q = torch.cat([qa, qb]).to(gpu)
    for window in (0, 64, 7):
        out = K.latent_attention_generic(q, cache, sink.to(gpu), table, seq.to(gpu), pos.to(gpu), rank, window, scale)
        want = torch.cat([_plain_latent_attention(qa, lat[0], sink, rank, scale, pos[:37].long(), window),
                          _plain_latent_attention(qb, lat[1], sink, rank, scale, pos[37:].long(), window)])
        close(out, want, dtype, f"window {window}", scale=1.0)
    # the far key carries the last query's output when nothing hides it
    full = _plain_latent_attention(qa[-1:], lat[0], sink, rank, scale, pos[36:37].long())
    cut = _plain_latent_attention(qa[-1:], lat[0][far + 1:], sink, rank, scale, pos[36:37].long() - far - 1)
    assert float((full - cut).abs().max()) > 0.2
    # without its sink a head's weights add up to one: the sink must make a difference the bound would catch
    no_sink = _plain_latent_attention(qb, lat[1], torch.full((H,), -1e30), rank, scale, pos[37:].long())
    assert float((no_sink - want[37:]).abs().max()) > 0.05


@pytest.mark.parametrize("H,rank,rot,page", [(3, 48, 16, 8), (8, 128, 32, 16), (5, 72, 8, 8), (16, 512, 64, 16), (40, 256, 64, 32), (2, 64, 0, 24)])
def test_latent_attention_on_the_matrix_cores(gpu, H, rank, rot, page):
    """The bfloat16 kernel: portions of unequal length (one starting at position 0, one deep in its context, with a
    far key made to stand out), then every sequence feeding one token with its keys in splits."""
    from prelude_amd.ops import kernels as K
    assert K.latent_attention_mfma_supported(rank, rot, page)
    dtype, width, scale = "bfloat16", rank + rot, 0.09
    ctx = [700, 45, 300, 1]
    qn = [70, 45, 2, 1]
    lat = [rnd((n, width), 60 + i, dtype) for i, n in enumerate(ctx)]
    qs = [rnd((n, H, width), 70 + i, dtype) for i, n in enumerate(qn)]
    qs[0][-1] = (lat[0][9].float() * 3.0).to(torch.bfloat16)[None, :].expand(H, width)
    sink = torch.linspace(-3.0, 2.0, H)
    cache, table = _paged(lat, page, gpu, dtype, seed=5)
    cache_t = cache[:, :, :rank].transpose(1, 2).contiguous()          # [pages, rank, page]: the copy the cache keeps
    cu = torch.tensor([0] + list(np.cumsum(qn)), dtype=torch.int32, device=gpu)
    cl = torch.tensor(ctx, dtype=torch.int32, device=gpu)
    q = torch.cat(qs).to(gpu)
    for window in (0, 40):
        out = torch.zeros((q.shape[0], H, rank), dtype=torch.bfloat16, device=gpu)
        K.latent_attention_mfma(q, cache, cache_t, sink.to(gpu), table, None, 4, cu, cl, out, max(qn), rank, window, scale)
        want = torch.cat([_plain_latent_attention(qs[i], lat[i], sink, rank, scale, torch.arange(ctx[i] - qn[i], ctx[i]), window)
                          for i in range(4)])
        close(out, want, dtype, f"portions, window {window}", scale=1.0)
    # a chosen list of sequences leaves the other rows alone
    out = torch.zeros((q.shape[0], H, rank), dtype=torch.bfloat16, device=gpu)
    K.latent_attention_mfma(q, cache, cache_t, sink.to(gpu), table, torch.tensor([2, 0], dtype=torch.int32, device=gpu), 2, cu, cl, out,
                            70, rank, 0, scale)
    assert float(out[70:115].abs().max()) == 0.0 and float(out[:70].abs().max()) > 0
    # single tokens, keys in splits (and one context within a single split)
    ql = [rnd((1, H, width), 80 + i, dtype) for i in range(4)]
    ql[0][0] = (lat[0][300].float() * 3.0).to(torch.bfloat16)[None, :].expand(H, width)
    cu1 = torch.arange(5, dtype=torch.int32, device=gpu)
    out = torch.zeros((4, H, rank), dtype=torch.bfloat16, device=gpu)
    for window in (0, 290):
        want = torch.cat([_plain_latent_attention(ql[i], lat[i], sink, rank, scale, torch.tensor([ctx[i] - 1]), window) for i in range(4)])
        for per_wave in (False, True):      # a split a workgroup that stages its keys; a split a wavefront that reads the cache
            out.zero_()
            K.latent_attention_mfma(torch.cat(ql).to(gpu), cache, cache_t, sink.to(gpu), table, None, 4, cu1, cl, out, 1, rank, window,
                                    scale, max_context=768, per_wave=per_wave)
            close(out, want, dtype, f"single tokens in splits, window {window}, per wavefront {per_wave}", scale=1.0)
    # a chosen list of sequences, the other rows left alone, both ways
    for per_wave in (False, True):
        out.zero_()
        K.latent_attention_mfma(torch.cat(ql).to(gpu), cache, cache_t, sink.to(gpu), table, torch.tensor([2, 0], dtype=torch.int32, device=gpu),
                                2, cu1, cl, out, 1, rank, 0, scale, max_context=768, per_wave=per_wave)
        want = torch.cat([_plain_latent_attention(ql[i], lat[i], sink, rank, scale, torch.tensor([ctx[i] - 1]), 0) for i in (0, 2)])
        close(out[[0, 2]], want, dtype, f"chosen sequences, per wavefront {per_wave}", scale=1.0)
        assert float(out[[1, 3]].abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
def test_keys_at_page_borders_and_first_tokens(gpu, dtype):
    """Every query position of a sequence from 0 on, one launch a token, against the whole: position p sees keys 0..p,
    whatever page border p stands at."""
    from prelude_amd.ops import kernels as K
    H, rank, rot, page, n, scale = 2, 32, 8, 4, 70, 0.3
    lat = rnd((n, rank + rot), 40, dtype)
    q = rnd((n, H, rank + rot), 41, dtype)
    sink = torch.tensor([0.5, -1.0])
    cache, table = _paged([lat], page, gpu, dtype, seed=3)
    want = _plain_latent_attention(q, lat, sink, rank, scale, torch.arange(n))
    zeros = torch.zeros(1, dtype=torch.int32, device=gpu)
    for p in range(n):
        out = K.latent_attention_generic(q[p:p + 1].to(gpu), cache, sink.to(gpu), table, zeros,
                                         torch.tensor([p], dtype=torch.int32, device=gpu), rank, 0, scale)
        close(out, want[p:p + 1], dtype, f"position {p}", scale=1.0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("E,top,T,ff", [(6, 2, 50, 24), (5, 3, 1, 24), (4, 1, 33, 20), (9, 2, 300, 136), (3, 2, 400, 24),
                                        (130, 4, 40, 24), (130, 4, 300, 24), (70, 1, 5, 40)])   # more experts than a wavefront has lanes
def test_experts_by_table(gpu, dtype, E, top, T, ff):
    from prelude_amd.ops import kernels as K
    V, Wd = 31, 80
    g = torch.Generator().manual_seed(E * 100 + T)
    table = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(V)]).to(torch.int32)
    if top == 1 and E < 64:
        table[table == E - 1] = 0                                          # an expert nobody uses
    ids = torch.randint(0, V, (T,), generator=g).to(torch.int32)
    x = rnd((T, Wd), 50, dtype)
    up, down = rnd((E, ff, Wd), 51, dtype, Wd ** -0.5), rnd((E, Wd, ff), 52, dtype, ff ** -0.5)
    base = rnd((T, Wd), 53, dtype)
    choice = K.moe_choices_by_table(ids.to(gpu), table.to(gpu), E)
    assert torch.equal(choice.cpu().reshape(T, top), table[ids.long()])
    eo = K.moe_order(choice, E, top)
    order, place, offsets = eo.order.cpu().long(), eo.place.cpu().long(), eo.offsets.cpu().long()
    flat = table[ids.long()].reshape(-1).long()
    assert torch.equal(order[place], torch.arange(T * top)) and offsets[0] == 0 and offsets[-1] == T * top
    assert torch.equal(flat[order], torch.sort(flat, stable=True).values), "entries lie in the order of their experts"
    for e in range(E):
        mine = order[offsets[e]:offsets[e + 1]]
        assert torch.equal(mine, torch.sort(mine).values), "and within an expert in their own order"
    mid = K.moe_linear(x.to(gpu), K.GroupedWeight(up.to(gpu)), eo, True, relu_squared_epilogue=True)
    y = K.moe_linear(mid, K.GroupedWeight(down.to(gpu)), eo, False, out_dtype=torch.float32)
    out = K.moe_combine(y, eo, 1.0 / top, base.to(gpu), TD[dtype])
    want = base.double().clone()
    for t in range(T):
        for j in range(top):
            e = int(table[ids[t], j])
            want[t] += (torch.relu(up[e].double() @ x[t].double()) ** 2) @ down[e].double().T / top
    close(out, want, dtype, "experts")


# ---- the engine -------------------------------------------------------------------------------------------------
# (configuration, seed, page size)
CONFIGS = {"p": (pl.tiny_config_p, 11, 8), "q": (pl.tiny_config_q, 12, 16), "r": (pl.tiny_config_r, 13, 4)}


@functools.lru_cache(maxsize=None)
def folder(name):
    from prelude_amd.weights import write_safetensors
    make, seed, _ = CONFIGS[name]
    cfg = make()
    w = pl.random_weights(cfg, seed)
    tmp = tempfile.TemporaryDirectory(prefix=f"prelude_amd_libodra_{name}_")
    _keep.append(tmp)
    with open(os.path.join(tmp.name, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(tmp.name, "model.safetensors"),
                      {k: (v.to(torch.bfloat16) if v.is_floating_point() else v) for k, v in w.items()})
    return tmp.name, cfg, w


@functools.lru_cache(maxsize=None)
def plain_logits(name, seed, length):
    _, cfg, w = folder(name)
    toks = torch.randint(0, cfg["vocab"], (length,), generator=torch.Generator().manual_seed(500 + seed)).tolist()
    return toks, pl.forward(cfg, w, toks)


def runner(name, dtype, max_tokens, **kw):
    from prelude_amd.trace import TraceRunner
    return TraceRunner(folder(name)[0], dtype, max_tokens, page_size=CONFIGS[name][2], **kw)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["p", "q", "r"])
def test_whole_prompt_every_position(gpu, name, dtype):
    toks, ref = plain_logits(name, 0, 150)
    r = runner(name, dtype, 256)
    got = r.step([{"id": "x", "tokens": toks, "want": list(range(len(toks)))}], ["x"])
    check(got, ref, dtype, f"{name} whole")
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["p", "q", "r"])
def test_prefill_then_token_by_token(gpu, name, dtype):
    toks, ref = plain_logits(name, 1, 140)
    r = runner(name, dtype, 256)
    n = 40
    outs = [r.step([{"id": 0, "tokens": toks[:n], "want": list(range(n))}])]
    for i in range(n, len(toks)):          # a hundred single tokens: page borders, and in bfloat16 replays of a captured step
        outs.append(r.step([{"id": 0, "tokens": [toks[i]], "want": [0]}]))
    check(np.concatenate(outs), ref, dtype, f"{name} decode")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["p", "q", "r"])
def test_from_the_first_token_one_by_one(gpu, name, dtype):
    toks, ref = plain_logits(name, 2, 40)
    r = runner(name, dtype, 64)
    outs = [r.step([{"id": 0, "tokens": [t], "want": [0]}]) for t in toks]
    check(np.concatenate(outs), ref, dtype, f"{name} one by one")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["p", "q", "r"])
def test_portions_of_changing_size(gpu, name, dtype):
    toks, ref = plain_logits(name, 3, 170)
    sizes = [7, 2, 13, 2, 1, 31, 2, 9, 16, 3, 8, 2, 64, 5]
    r = runner(name, dtype, 256)
    outs, i, k = [], 0, 0
    while i < len(toks):
        n = min(sizes[k % len(sizes)], len(toks) - i)
        k += 1
        outs.append(r.step([{"id": "p", "tokens": toks[i:i + n], "want": list(range(n))}]))
        i += n
    check(np.concatenate(outs), ref, dtype, f"{name} portions")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["p", "q", "r"])
def test_unequal_requests_in_one_batch_and_pages_used_again(gpu, name, dtype):
    """Six requests of unequal length through a pool that holds three of them: portions of some beside single
    tokens of others, a request ends as soon as it is fed and its pages go to the next."""
    lengths = [90, 17, 64, 33, 120, 5]
    seqs = [plain_logits(name, 10 + i, n) for i, n in enumerate(lengths)]
    r = runner(name, dtype, 3 * 128)
    rng = np.random.default_rng(7)
    fed, waiting, live = [0] * len(seqs), list(range(len(seqs))), []
    got = [[] for _ in seqs]
    while waiting or live:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, end = [], []
        for i in live:
            left = lengths[i] - fed[i]
            n = 1 if (fed[i] > 0 and rng.random() < 0.5) else int(min(left, rng.choice([2, 3, 16, 29, 40])))
            entries.append({"id": f"r{i}", "tokens": seqs[i][0][fed[i]:fed[i] + n], "want": list(range(n))})
            fed[i] += n
            if fed[i] == lengths[i]:
                end.append(f"r{i}")
        out = r.step(entries, end)
        k = 0
        for e in entries:
            i = int(e["id"][1:])
            got[i].append(out[k:k + len(e["tokens"])])
            k += len(e["tokens"])
        live = [i for i in live if fed[i] < lengths[i]]
    for i, (toks, ref) in enumerate(seqs):
        check(np.concatenate(got[i]), ref, dtype, f"{name} request {i}")
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_token_far_back_moves_the_last_logits(gpu, dtype):
    """Hundreds of keys: the engine follows the plain implementation when one early token changes, and that
    change is one the bound would not let pass."""
    name = "q"
    toks, ref = plain_logits(name, 20, 600)
    _, cfg, w = folder(name)
    other = list(toks)
    other[3] = (toks[3] + 1) % cfg["vocab"]
    ref2 = pl.forward(cfg, w, other)
    r = runner(name, dtype, 1280)
    want = list(range(590, 600))
    a = r.step([{"id": "a", "tokens": toks[:512], "want": []}, ])
    assert a is None
    a = r.step([{"id": "a", "tokens": toks[512:], "want": [w_ - 512 for w_ in want]}], ["a"])
    b = r.step([{"id": "b", "tokens": other, "want": want}], ["b"])
    check(a, ref[want], dtype, "as it is")
    check(b, ref2[want], dtype, "with token 3 changed")


def test_greedy_generation_through_the_scheduler(gpu):
    """``LLM.generate`` with temperature 0 gives the plain implementation's greedy tokens, for prompts of unequal
    length in one call (32-bit, so that no rounding decides between neighbours)."""
    from prelude_amd.llm import LLM
    name = "p"
    path, cfg, w = folder(name)
    llm = LLM(path, dtype="float32", page_size=8, max_cache_tokens=512)
    prompts = [plain_logits(name, 30, 9)[0], plain_logits(name, 31, 31)[0], plain_logits(name, 32, 2)[0]]
    res = llm.generate(prompts, max_tokens=12, temperature=0.0)
    for p, out in zip(prompts, res):
        seq = list(p)
        for _ in range(12):
            seq.append(int(pl.forward(cfg, w, seq)[-1].argmax()))
        assert out.token_ids == seq[len(p):], f"prompt of {len(p)}"


def test_command_line_with_the_pools_sized_from_free_memory(gpu, capsys):
    """``python -m prelude_amd`` on a Libodra folder, nothing given but the model: the pools take what the device has
    left after a measured step, steps are replayed from graphs, and the greedy tokens are the same as with weights
    drawn again from the folder's own values in 32-bit."""
    from prelude_amd import cli
    name = "q"
    path, cfg, w = folder(name)
    prompt = plain_logits(name, 40, 11)[0]
    assert cli.main(["--model", path, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "6", "--temperature", "0"]) == 0
    rec = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert rec["finish_reason"] == "length" and len(rec["token_ids"]) == 6
    # bfloat16 may part from the plain greedy path where two logits are close; the first token's margin is checked instead
    ref = pl.forward(cfg, w, prompt)[-1]
    top2 = torch.topk(ref, 2).values
    if float(top2[0] - top2[1]) > 0.2 * float(ref.std()):
        assert rec["token_ids"][0] == int(ref.argmax())
    assert cli.main(["--model", path, "--random-weights", "--prompt-len", "5", "--max-tokens", "3", "--max-cache-tokens", "256"]) == 0
    rec = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert len(rec["token_ids"]) == 3 and all(0 <= t < cfg["vocab"] for t in rec["token_ids"])
