"""Each mechanism of the Vipalorn decoder alone on the GPU against its plain formula: the layer norm (also
with a sum added on the way), the short convolution with its state, the delta rule in one piece, in
portions and token by token over slots that are used again, the gated norm a head, the latent rows'
write and the attention over them (plain and matrix cores; a far key that holds the weight, keys at
the edges of pages), routing, the experts' products and their weighted sum."""
import math

import numpy as np
import pytest
import torch

from herbert_rs_amd.cache import Cache, KVNeed, StateNeed
from herbert_rs_amd.engine import batch as batching
from herbert_rs_amd.engine.batch import StepEntry
from herbert_rs_amd.kernels import latent, moe, ops, recurrent

from .plain import vipalorn as plain

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def step_meta(cache, slots, counts):
    entries = [StepEntry(s, [0] * n, []) for s, n in zip(slots, counts)]
    starts = [cache.length(s) for s in slots]
    cache.reserve_all([(s, n) for s, n in zip(slots, counts)])
    meta = batching.pack(entries, starts, torch.device(DEV))
    for s, n in zip(slots, counts):
        cache.commit(s, n)
    return meta


@pytest.mark.parametrize("H", [24, 100, 1536])
def test_layer_norm_and_the_sum_it_adds(H):
    x, w, d = rand(7, H, seed=1), 1 + 0.1 * rand(H, seed=2), rand(7, H, seed=3)
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 1.6e-2)):
        xg, y = x.to(DEV).clone(), torch.empty(7, H, dtype=dtype, device=DEV)
        ops.layernorm(xg, w.to(DEV), y, 1e-5)
        assert torch.allclose(y.float().cpu(), plain.layer_norm(x, w, 1e-5), atol=tol * 4, rtol=tol)
        ops.layernorm(xg, w.to(DEV), y, 1e-5, delta=d.to(DEV), mult=0.3)
        assert torch.allclose(xg.cpu(), x + 0.3 * d, atol=1e-6)
        assert torch.allclose(y.float().cpu(), plain.layer_norm(x + 0.3 * d, w, 1e-5), atol=tol * 4, rtol=tol)
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    y = torch.empty(3, H, device=DEV)
    ops.layernorm(x.to(DEV), w.to(DEV), y, 1e-5, rows)
    assert torch.allclose(y.cpu(), plain.layer_norm(x[[5, 0, 5]], w, 1e-5), atol=1e-5)
    xg = x.to(DEV).clone()
    ops.layernorm(xg, w.to(DEV), xg, 1e-5)                      # in place
    assert torch.allclose(xg.cpu(), plain.layer_norm(x, w, 1e-5), atol=1e-5)


def delta_reference(proj, taps, a_log, dt_bias, kv_heads, heads, D, V, b_off, a_off):
    """q, k, v after convolution, silu and unit vectors, and the recurrence's outputs, by the plain formulas."""
    T, C = proj.shape[0], 2 * kv_heads * D + heads * V
    y = plain.silu(plain.short_conv(proj[:, :C], taps))
    q = plain.unit_vectors(y[:, :kv_heads * D].view(T, kv_heads, D)) * D ** -0.5
    k = plain.unit_vectors(y[:, kv_heads * D:2 * kv_heads * D].view(T, kv_heads, D))
    v = y[:, 2 * kv_heads * D:].view(T, heads, V)
    beta = plain.sigmoid(proj[:, b_off:b_off + heads])
    decay = torch.exp(-torch.exp(a_log) * plain.softplus(proj[:, a_off:a_off + heads] + dt_bias))
    group = heads // kv_heads
    out = torch.stack([plain.delta_rule(q[:, n // group], k[:, n // group], v[:, n], beta[:, n], decay[:, n])
                       for n in range(heads)], 1)
    return torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1), out.reshape(T, heads * V)


@pytest.mark.parametrize("kv_heads,heads,D,V,K", [(1, 1, 8, 5, 1), (2, 6, 24, 70, 3), (3, 3, 48, 33, 4), (1, 2, 128, 64, 2),
                                                  (1, 1, 200, 12, 5)])
def test_convolution_and_delta_rule_whole_in_portions_and_token_by_token(kv_heads, heads, D, V, K):
    C = 2 * kv_heads * D + heads * V
    ld = C + heads * V + 2 * heads + 3
    b_off, a_off = C + heads * V + 1, C + heads * V + 1 + heads
    lengths = [41, 3, 18]
    taps = (1.0 / K + 0.3 * rand(C, K, seed=5))
    a_log, dt_bias = torch.tensor([-3.0, 0.2, -1.0, 0.5, -5.0, 0.0])[:heads], 0.3 * rand(heads, seed=7)
    projs = [rand(n, ld, seed=10 + i, scale=1.5) for i, n in enumerate(lengths)]
    refs = [delta_reference(p, taps, a_log, dt_bias, kv_heads, heads, D, V, b_off, a_off) for p in projs]
    needs = {0: (StateNeed((heads, D, V)), StateNeed((max(K - 1, 1), C)))}
    cache = Cache(needs, 64 * 8, 4096, torch.float32, DEV, max_slots=4)
    state, conv_state = cache.state_views(0)
    for cuts in ([], [1, 2, 3, 9, 17, 40], list(range(1, 41))):
        slots = [cache.alloc_slot() for _ in lengths]           # (slots that the round before has used: cleared)
        got_qkv = [[] for _ in lengths]
        got_out = [[] for _ in lengths]
        edges = sorted(set([0] + cuts + [max(lengths)]))
        for a, b in zip(edges[:-1], edges[1:]):
            live = [i for i, n in enumerate(lengths) if a < n]
            counts = [min(b, lengths[i]) - a for i in live]
            meta = step_meta(cache, [slots[i] for i in live], counts)
            proj = torch.cat([projs[i][a:a + c] for i, c in zip(live, counts)]).to(DEV).contiguous()
            T = proj.shape[0]
            qkv = torch.empty(T, C, device=DEV)
            recurrent.conv_silu(proj, taps.to(DEV), conv_state, meta, qkv, 2 * kv_heads, D, kv_heads, D ** -0.5, 1e-6, heads, V)
            out = torch.empty(T, heads * V, device=DEV)
            recurrent.gated_delta(qkv, proj, b_off, a_off, a_log.to(DEV), dt_bias.to(DEV), state, meta, out, kv_heads, heads, D, V)
            at = 0
            for i, c in zip(live, counts):
                got_qkv[i].append(qkv[at:at + c].cpu())
                got_out[i].append(out[at:at + c].cpu())
                at += c
        for i in range(len(lengths)):
            assert torch.allclose(torch.cat(got_qkv[i]), refs[i][0], atol=2e-6), f"convolution, cuts {cuts[:4]}"
            assert torch.allclose(torch.cat(got_out[i]), refs[i][1], atol=3e-6), f"delta rule, cuts {cuts[:4]}"
        for s in slots:
            cache.free_slot(s)


def test_gated_norm_a_head():
    T, heads, V = 5, 3, 70
    o, proj, w = rand(T, heads * V, seed=1), rand(T, heads * V + 9, seed=2), 1 + 0.1 * rand(V, seed=3)
    want = (plain.rms_scale(o.view(T, heads, V), 1e-5) * w * plain.silu(proj[:, 4:4 + heads * V].view(T, heads, V))).reshape(T, -1)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        y = torch.empty(T, heads * V, dtype=dtype, device=DEV)
        recurrent.gated_head_norm(o.to(DEV), proj.to(DEV), 4, w.to(DEV), y, heads, V, 1e-5)
        assert torch.allclose(y.float().cpu(), want, atol=tol, rtol=tol)


def latent_reference(proj, positions, norm_w, uk, uv, H, qd, rank, rot, rot_dims, base, scale, eps, gate_off):
    T = proj.shape[0]
    q = proj[:, :H * (qd + rot)].view(T, H, qd + rot)
    down = proj[:, H * (qd + rot):H * (qd + rot) + rank + rot]
    c = plain.rms_scale(down[:, :rank], eps) * norm_w
    r = plain.rotate_half_layout(down[:, rank:], positions, base, rot_dims) if rot else down[:, rank:]
    qr = plain.rotate_half_layout(q[..., qd:], positions, base, rot_dims) if rot else q[..., qd:]
    gate = plain.sigmoid(proj[:, gate_off:gate_off + H])
    pos = torch.as_tensor(positions)
    outs = []
    for n in range(H):
        s = (q[:, n, :qd] @ uk[n].T @ c.T + qr[:, n] @ r.T) * scale        # uk [H, rank, qd]
        s = s.masked_fill(pos[None, :] > pos[:, None], -math.inf)
        outs.append(torch.softmax(s, -1) @ c * gate[:, n:n + 1])
    return torch.cat([c, r], 1), torch.stack(outs, 1).reshape(T, H * rank)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,qd,rank,rot,rot_dims", [(3, 8, 24, 8, 4), (16, 32, 96, 32, 32), (20, 16, 128, 64, 64), (2, 8, 40, 0, 0)])
def test_latent_rows_and_attention_with_a_far_key(dtype, H, qd, rank, rot, rot_dims):
    """A prompt of 200 tokens, then tokens one by one to 330 (past the pages' edges at 64, 128, ...), beside a
    short sequence in the same steps. The query of every token is made to point at the latent of one far
    key (position 5, or the key at the last page's first place), so that this key holds most of the weight."""
    base, scale, eps = 5000.0, 0.25, 1e-5
    row, qw = rank + rot, H * (qd + rot)
    ld = qw + row + H
    L = 330
    proj = rand(L, ld, seed=3)
    uk, uv = rand(H, rank, qd, seed=4, scale=0.3), None
    norm_w = 1 + 0.1 * rand(rank, seed=5)
    if dtype == torch.bfloat16:
        proj, uk, norm_w = proj.bfloat16().float(), uk.bfloat16().float(), norm_w
    positions = list(range(L))
    rows_ref, out_ref = latent_reference(proj, positions, norm_w, uk, uv, H, qd, rank, rot, rot_dims, base, scale, eps, qw + row)
    short = 70
    rows_short, out_short = latent_reference(proj[:short] * 0.5, positions[:short], norm_w, uk, uv, H, qd, rank, rot, rot_dims,
                                             base, scale, eps, qw + row)
    store = dtype
    cache = Cache({0: KVNeed(1, row, None, values=False)}, 64 * 8, 4096, store, DEV, max_slots=3)
    kv = cache.kv_view(0)
    inv_freq = (base ** (-2.0 * torch.arange(rot_dims // 2, dtype=torch.float32) / max(rot_dims, 1))).to(DEV) if rot_dims else None
    use_cores = latent.mfma_takes(kv, rank, rot)
    buffers = {}

    def buffer(name, shape, dt):
        return buffers.setdefault((name, tuple(shape)), torch.empty(tuple(shape), dtype=dt, device=DEV))
    a, b = cache.alloc_slot(), cache.alloc_slot()
    got, got_short = [], []
    steps = [(200, short)] + [(1, 0)] * (L - 200)
    done = 0
    for n_long, n_short in steps:
        slots, counts = ([a, b], [n_long, n_short]) if n_short else ([a], [n_long])
        meta = step_meta(cache, slots, counts)
        p = torch.cat([proj[done:done + n_long]] + ([proj[:short] * 0.5] if n_short else [])).to(DEV).contiguous()
        T = p.shape[0]
        q_full = torch.zeros(T, H * row, device=DEV)
        latent.latent_write(p, 0, qw, norm_w.to(DEV), q_full, inv_freq, meta, kv, H, qd, rank, rot, rot_dims, eps)
        ops.gemm_plain_batched(p, uk.to(DEV), q_full, T, rank, qd, ld, qd, H * row, H, qd + rot, rank * qd, row)
        out = torch.empty(T, H * rank, dtype=store, device=DEV)
        if use_cores:
            latent.latent_attention_mfma(q_full, meta, kv, out, p, qw + row, H, rank, rot, scale, buffer)
        else:
            latent.latent_attention_plain(q_full, meta, kv, out, p, qw + row, H, rank, rot, scale)
        got.append(out[:n_long].float().cpu())
        if n_short:
            got_short.append(out[n_long:].float().cpu())
        done += n_long
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert torch.allclose(torch.cat(got), out_ref, atol=tol, rtol=tol)
    assert torch.allclose(torch.cat(got_short), out_short, atol=tol, rtol=tol)
    # the cached rows themselves
    table = kv.page_table[a].cpu().tolist()
    stored = torch.cat([kv.k[table[p // 64], 0, p % 64].float().cpu()[None] for p in range(L)])
    assert torch.allclose(stored, rows_ref, atol=1e-5 if dtype == torch.float32 else 2e-2, rtol=1e-2)


def test_a_single_far_key_holds_the_weight():
    """One key among hundreds has a score far above the others: the output is that key's latent (times the gate),
    whichever page it lies in, in the prompt and for single tokens; with one position less the key is unseen."""
    H, rank, rot = 16, 64, 32
    row = rank + rot
    for dtype in (torch.float32, torch.bfloat16):
        cache = Cache({0: KVNeed(1, row, None, values=False)}, 64 * 8, 4096, dtype, DEV, max_slots=2)
        kv = cache.kv_view(0)
        slot = cache.alloc_slot()
        L = 300
        meta = step_meta(cache, [slot], [L])
        rows = rand(L, row, seed=1, scale=0.1).to(dtype)
        table = kv.page_table[slot].cpu().tolist()
        for far in (0, 63, 64, 191, 299):
            rows_far = rows.clone()
            rows_far[far, :rank] = 1.0
            for p in range(L):
                kv.k[table[p // 64], 0, p % 64] = rows_far[p].to(DEV)
            q_full = torch.zeros(L, H * row, device=DEV)
            q_full.view(L, H, row)[:, :, :rank] = 2.0                      # score 2 * 64 * 0.25 = 32 against the far key
            out = torch.empty(L, H * rank, dtype=dtype, device=DEV)
            if latent.mfma_takes(kv, rank, rot):
                latent.latent_attention_mfma(q_full, meta, kv, out, None, 0, H, rank, rot, 0.25, None)
            else:
                latent.latent_attention_plain(q_full, meta, kv, out, None, 0, H, rank, rot, 0.25)
            out = out.float().cpu().view(L, H, rank)
            assert torch.allclose(out[far:], torch.ones(L - far, H, rank), atol=2e-2), f"far key {far} in {dtype}"
            if far:
                assert float(out[far - 1].abs().max()) < 0.5              # just before it: unseen


@pytest.mark.parametrize("T,E,top", [(1, 3, 3), (9, 5, 2), (300, 16, 4), (70, 130, 7)])
def test_routing_groups_and_products(T, E, top):
    W, F = 64, 96                                          # (K in steps of 32: what the matrix-core product takes)
    y, wr, br = rand(T, W, seed=1), rand(E, W, seed=2, scale=0.3), 0.1 * rand(E, seed=3)
    logits = (y @ wr.T).to(DEV).contiguous()
    routing = moe.Routing(torch.empty(moe.Routing.ints_needed(T, E, top), dtype=torch.int32, device=DEV),
                          torch.empty(T, top, device=DEV), T, E, top)
    moe.route(logits, br.to(DEV), routing)
    chosen, weight = plain.route(y, wr, br, top)
    got_chosen = routing.chosen.view(T, top).cpu()
    assert torch.equal(got_chosen.sort(-1).values, chosen.sort(-1).values.int())
    assert torch.allclose(routing.weight.cpu().sort(-1).values, weight.sort(-1).values, atol=1e-6)
    # every pair once, an expert's rows together, the tiles cover them
    order, row_of = routing.order.cpu(), routing.row_of.cpu()
    assert sorted(order.tolist()) == list(range(T * top)) and torch.equal(order[row_of.long()], torch.arange(T * top, dtype=torch.int32))
    experts_in_order = got_chosen.flatten()[order.long()]
    assert torch.equal(experts_in_order, experts_in_order.sort().values)
    gate_up, down = rand(E, 2 * F, W, seed=4, scale=0.2), rand(E, W, F, seed=5, scale=0.2)
    want = torch.zeros(T, W)
    for t in range(T):
        for j in range(top):
            e = int(got_chosen[t, j])
            want[t] += routing.weight[t, j].cpu() * plain.expert(y[t:t + 1], gate_up[e, :F], gate_up[e, F:], down[e], 1.5)[0]
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 4e-2)):
        yg, gu_w, down_w = y.to(DEV).to(dtype), gate_up.to(DEV).to(dtype), down.to(DEV).to(dtype)
        act = torch.empty(T * top, F, dtype=dtype, device=DEV)
        out = torch.empty(T * top, W, device=DEV)
        x = torch.zeros(T, W, device=DEV)
        if dtype == torch.bfloat16:
            moe.grouped_mfma(yg, W, 0, moe.pack_grouped(gu_w), act, F, 0, moe.EPI_GLU, routing, gather=True, limit=1.5, alpha=1.702)
            moe.grouped_mfma(act, F, 0, moe.pack_grouped(down_w), out, W, 0, moe.EPI_F32, routing)
        else:
            gu = torch.empty(T * top, 2 * F, device=DEV)
            moe.gemm_plain(yg, gu_w, gu, routing, gather=True)
            moe.activate(gu, act, 1.5, 1.702)
            moe.gemm_plain(act, down_w, out, routing, gather=False)
        moe.combine(out, routing, x)
        assert torch.allclose(x.cpu(), want, atol=tol, rtol=tol), f"{dtype}"
