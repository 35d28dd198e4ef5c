"""Each mechanism of the Modasun decoder alone on the GPU against its plain formula: the norm after a sum
with its copies, the per-head norm without weights and the query's factor at the positions where it
steps up (prompts, single tokens, the fused decode kernel), one far key that holds the weight at the
edges of pages, the decay a key channel and the delta rule under it (whole, in portions, token by
token, over slots that are used again), the sigmoid-gated norm a head, the choice of experts by scores
within groups (random, and cases made so that a group's edge or a masked expert shows), the shared
expert's gated sum, and the squared relu."""
import math

import pytest
import torch

from herbert_rs_amd.cache import Cache, StateNeed
from herbert_rs_amd.kernels import mfma, moe, ops, recurrent

from .plain import modasun as plain
from .test_kernels_gpu import paged_case
from .test_vipalorn_kernels_gpu import step_meta

pytestmark = pytest.mark.gpu
DEV = "cuda"


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


# ---------------------------------------------------------------- the norm after a sum
@pytest.mark.parametrize("H", [24, 72, 1536])
def test_norm_after_the_sum_and_its_copies(H):
    src, w = rand(9, H, seed=1, scale=3.0), 0.2 * rand(H, seed=2)
    want = plain.offset_norm(src, w, 1e-5)
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 8e-3)):
        acc = src.to(DEV).clone()
        x, y = torch.empty(9, H, device=DEV), torch.empty(9, H, dtype=dtype, device=DEV)
        ops.postnorm(acc, (1.0 + w).to(DEV), x, y, 1e-5, 1.75)
        assert torch.allclose(x.cpu(), want, atol=3e-6, rtol=2e-6)
        assert torch.allclose(y.float().cpu(), want, atol=tol * 4, rtol=tol)
        assert torch.allclose(acc.cpu(), 1.75 * want, atol=1e-5, rtol=2e-6)       # what the next part adds to
    # the first step of a stack: no norm, the copy and alpha x only
    x0 = src.to(DEV).clone()
    acc, y = torch.empty(9, H, device=DEV), torch.empty(9, H, dtype=torch.bfloat16, device=DEV)
    ops.postnorm(x0, None, None, y, 0.0, 1.7, acc=acc)
    assert torch.equal(x0.cpu(), src) and torch.allclose(acc.cpu(), 1.7 * src, rtol=1e-6)
    assert torch.allclose(y.float().cpu(), src, rtol=8e-3)


def test_squared_relu():
    z = rand(5, 77, seed=3, scale=2.0)
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 8e-3)):
        out = torch.empty(5, 77, dtype=dtype, device=DEV)
        ops.relu_squared(z.to(DEV), out)
        assert torch.allclose(out.float().cpu(), plain.relu_squared(z), atol=1e-6, rtol=tol)


# ---------------------------------------------------------------- attention
def attention_reference(qkv, positions, seq_of, firsts, nq, nkv, hd, eps, scale, q_temp, dtype):
    """Outputs [T, nq hd] of the step's tokens by the plain formulas; every sequence's tokens are all of it
    (positions from 0). Queries, keys and values are rounded to `dtype` where the kernels store them."""
    T = qkv.shape[0]
    x = qkv.view(T, nq + 2 * nkv, hd)
    temp = plain.query_temperature(positions, q_temp[0], q_temp[1]).float()
    q = (plain.rms_scale(x[:, :nq], eps) * temp[:, None, None]).to(dtype).float()
    k = plain.rms_scale(x[:, nq:nq + nkv], eps).to(dtype).float()
    v = x[:, nq + nkv:].to(dtype).float()
    out = torch.zeros(T, nq, hd)
    for s, first in enumerate(firsts):
        rows = (seq_of == s).nonzero().flatten()
        for h in range(nq):
            g = h // (nq // nkv)
            out[rows, h] = plain.softmax_attention(q[rows, h], k[rows, g], v[rows, g], scale)
    return out.view(T, nq * hd)


def run_attention(qkv, meta, kv, nq, nkv, hd, eps, scale, q_temp, dtype):
    T = qkv.shape[0]
    ones = torch.ones(hd, device=DEV)
    q = torch.empty(T, nq * hd, dtype=dtype, device=DEV)
    ops.qk_norm_rope_write(qkv.to(DEV), ones, ones, None, None, 0, meta, kv, q, nq, nkv, hd, eps, q_temp=q_temp)
    out = torch.full_like(q, 9.0)
    if mfma.attention_supported(q, kv, nq, nkv, hd):
        mfma.attention(q, meta, kv, out, nq, nkv, hd, scale, 0)
    else:
        ops.attention_plain(q, meta, kv, out, nq, nkv, hd, scale, 0)
    return out.float().cpu()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,hd,coef,every", [(4, 2, 64, 0.5, 16), (3, 1, 48, 0.8, 1), (2, 2, 128, 0.4, 64),
                                                  (6, 3, 32, 1.0, 7), (2, 1, 160, 0.3, 50)])
def test_plain_head_norm_and_the_growing_query_in_prompts(nq, nkv, hd, coef, every, dtype):
    """Whole prompts that cross pages and the positions at which the factor steps up: a factor that steps one
    position early or late changes every score of that position by a fifth or more."""
    lengths = [150, 70, 2 * every + 1]
    meta, kv, _ = paged_case(lengths, lengths, nkv, hd, dtype, seed=hd)
    qkv = rand(sum(lengths), (nq + 2 * nkv) * hd, seed=60, scale=1.3)
    scale, eps = 1.7 * hd ** -0.5, 1e-5
    got = run_attention(qkv, meta, kv, nq, nkv, hd, eps, scale, (coef, every), dtype)
    positions, seq_of = meta.positions.cpu().long(), meta.seq_of.cpu().long()
    want = attention_reference(qkv, positions, seq_of, [0] * 3, nq, nkv, hd, eps, scale, (coef, every), dtype)
    tol = 2e-5 if dtype == torch.float32 else 2 ** -6
    err = (got - want).abs().max(-1).values
    assert float(err.max()) <= tol * float(want.abs().max()), f"worst at row {int(err.argmax())}, position {int(positions[err.argmax()])}"
    # and the factor itself at the steps' edges (every - 2, every - 1, every, 2 every - 1): the last sequence's queries
    if dtype == torch.float32:
        ones = torch.ones(hd, device=DEV)
        q = torch.empty(sum(lengths), nq * hd, device=DEV)
        ops.qk_norm_rope_write(qkv.to(DEV), ones, ones, None, None, 0, meta, kv, q, nq, nkv, hd, eps, q_temp=(coef, every))
        x = plain.rms_scale(qkv.view(-1, nq + 2 * nkv, hd)[:, :nq], eps)
        first = lengths[0] + lengths[1]
        for p in (0, max(every - 2, 0), every - 1, every, 2 * every - 2, 2 * every - 1, 2 * every):
            factor = 1.0 + coef * math.log((p + 1) // every + 1)
            assert torch.allclose(q[first + p].cpu().view(nq, hd), x[first + p] * factor, atol=2e-6, rtol=2e-6), p


@pytest.mark.parametrize("nq,nkv,hd,coef,every", [(4, 2, 64, 0.5, 16), (8, 8, 128, 0.3, 32), (6, 2, 32, 1.0, 1)])
def test_the_growing_query_in_the_fused_decode_kernel(nq, nkv, hd, coef, every):
    """One token a sequence at the positions around a step of the factor: the kernel that norms, writes the
    cache and attends in one against the separate kernels and the plain formula."""
    from herbert_rs_amd.cache.paged import LayerKV
    lengths = [every - 1, every, every + 1, 2 * every, 2 * every + 1, 300, 64, 65]
    lengths = [max(n, 1) for n in lengths]
    B = len(lengths)
    meta, kv, dense = paged_case(lengths, [1] * B, nkv, hd, torch.bfloat16, seed=nq, n_pages=40)
    kv2 = LayerKV(kv.k.clone(), kv.v.clone(), kv.page_table, 64, 0)
    qkv = rand(B, (nq + 2 * nkv) * hd, seed=61, scale=1.5)
    scale, eps = hd ** -0.5, 1e-5
    ones = torch.ones(hd, device=DEV)
    assert mfma.decode_fusable(meta, kv, nq, nkv, hd, 0, torch.bfloat16)
    got = torch.full((B, nq * hd), 7.0, dtype=torch.bfloat16, device=DEV)
    mfma.attention_decode_fused(qkv.to(DEV), ones, ones, None, None, meta, kv, got, nq, nkv, hd, eps, scale, 0,
                                q_temp=(coef, every))
    separate = run_attention(qkv, meta, kv2, nq, nkv, hd, eps, scale, (coef, every), torch.bfloat16)
    x = qkv.view(B, nq + 2 * nkv, hd)
    want = torch.zeros(B, nq, hd)
    for b, n in enumerate(lengths):
        K, V = dense[b][0].clone(), dense[b][1].clone()
        K[n - 1] = plain.rms_scale(x[b, nq:nq + nkv], eps).bfloat16().float()
        V[n - 1] = x[b, nq + nkv:].bfloat16().float()
        factor = float(plain.query_temperature(torch.tensor([n - 1]), coef, every)[0])
        q = (plain.rms_scale(x[b, :nq], eps) * factor).bfloat16().float()
        for h in range(nq):
            g = h // (nq // nkv)
            s = (K[:, g] @ q[h]) * scale
            want[b, h] = torch.softmax(s.double(), 0).float() @ V[:, g]
    want = want.view(B, nq * hd)
    bound = 2 ** -6 * float(want.abs().max())
    assert float((got.float().cpu() - want).abs().max()) <= bound
    assert float((separate - want).abs().max()) <= bound


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hd", [64, 48])
def test_one_far_key_holds_the_weight_at_the_edges_of_pages(hd, dtype):
    """All queries and one key far back point the same way: after the norm their score is hd times the scale
    times the factor, far above the rest, and the output from that position on is that key's value; one position
    earlier the key is unseen."""
    nq, nkv, L = 4, 2, 260
    direction = rand(hd, seed=5)
    for far in (0, 63, 64, 191, 259):
        meta, kv, _ = paged_case([L], [L], nkv, hd, dtype, seed=far + 1)
        qkv = rand(L, (nq + 2 * nkv) * hd, seed=62).view(L, nq + 2 * nkv, hd)
        qkv[:, :nq] = 3.0 * direction
        qkv[far, nq:nq + nkv] = 0.5 * direction
        qkv = qkv.reshape(L, -1).contiguous()
        got = run_attention(qkv, meta, kv, nq, nkv, hd, 1e-5, 0.5, (0.2, 64), dtype).view(L, nq, hd)
        value = qkv.view(L, nq + 2 * nkv, hd)[far, nq + nkv:].to(dtype).float().repeat_interleave(nq // nkv, 0)
        assert float((got[far:] - value).abs().max()) < 0.03, f"far key at {far} in {dtype}"
        if far:
            assert float((got[far - 1] - value).abs().max()) > 0.3, f"the key at {far} seen a position early"


# ---------------------------------------------------------------- the delta rule with a decay a key channel
def channel_delta_reference(proj, taps, z, a_log, dt_bias, kv_heads, heads, D, V, b_off):
    T, C = proj.shape[0], 2 * kv_heads * D + heads * V
    y = plain.silu(plain.short_conv(proj[:, :C], taps))
    q = plain.unit_vectors(y[:, :kv_heads * D].view(T, kv_heads, D)) * D ** -0.5
    k = plain.unit_vectors(y[:, kv_heads * D:2 * kv_heads * D].view(T, kv_heads, D))
    v = y[:, 2 * kv_heads * D:].view(T, heads, V)
    beta = plain.sigmoid(proj[:, b_off:b_off + heads])
    decay = torch.exp(-torch.exp(a_log)[None, :, None] * plain.softplus(z + dt_bias).view(T, heads, D))
    group = heads // kv_heads
    out = torch.stack([plain.channel_delta_rule(q[:, n // group], k[:, n // group], v[:, n], beta[:, n], decay[:, n])
                       for n in range(heads)], 1)
    return decay.reshape(T, heads * D), out.reshape(T, heads * V)


@pytest.mark.parametrize("kv_heads,heads,D,V,K", [(1, 1, 8, 5, 1), (2, 6, 24, 70, 3), (3, 3, 48, 33, 4), (1, 2, 128, 64, 2),
                                                  (2, 4, 32, 32, 3), (1, 2, 10, 12, 2), (2, 2, 34, 21, 3), (1, 3, 6, 7, 2),
                                                  (1, 1, 160, 24, 2), (2, 2, 256, 16, 4)])
def test_channel_decay_and_delta_rule_whole_in_portions_and_token_by_token(kv_heads, heads, D, V, K):
    C = 2 * kv_heads * D + heads * V
    ld = C + heads + 5
    b_off = C + 2
    lengths = [41, 3, 18]
    taps = 1.0 / K + 0.3 * rand(C, K, seed=5)
    # rates from slow (a state that remembers the start) to fast, channel by channel different
    a_log, dt_bias = torch.tensor([-4.0, 0.3, -1.0, 0.6, -6.0, 0.0])[:heads], 0.5 * rand(heads * D, seed=7)
    projs = [rand(n, ld, seed=10 + i, scale=1.5) for i, n in enumerate(lengths)]
    zs = [rand(n, heads * D, seed=20 + i, scale=2.0) for i, n in enumerate(lengths)]
    refs = [channel_delta_reference(p, taps, z, a_log, dt_bias, kv_heads, heads, D, V, b_off) for p, z in zip(projs, zs)]
    needs = {0: (StateNeed((heads, D, V)), StateNeed((max(K - 1, 1), C)))}
    cache = Cache(needs, 64 * 8, 4096, torch.float32, DEV, max_slots=4)
    state, conv_state = cache.state_views(0)
    for cuts in ([], [1, 2, 3, 9, 17, 40], [2, 4, 20], list(range(1, 41))):
        slots = [cache.alloc_slot() for _ in lengths]           # (slots that the pass before has used: cleared)
        got_decay = [[] for _ in lengths]
        got_out = [[] for _ in lengths]
        edges = sorted(set([0] + cuts + [max(lengths)]))
        for a, b in zip(edges[:-1], edges[1:]):
            live = [i for i, n in enumerate(lengths) if a < n]
            counts = [min(b, lengths[i]) - a for i in live]
            meta = step_meta(cache, [slots[i] for i in live], counts)
            proj = torch.cat([projs[i][a:a + c] for i, c in zip(live, counts)]).to(DEV).contiguous()
            z = torch.cat([zs[i][a:a + c] for i, c in zip(live, counts)]).to(DEV).contiguous()
            T = proj.shape[0]
            qkv = torch.empty(T, C, device=DEV)
            recurrent.conv_silu(proj, taps.to(DEV), conv_state, meta, qkv, 2 * kv_heads, D, kv_heads, D ** -0.5, 1e-6, heads, V)
            recurrent.channel_decay(z, 0, a_log.to(DEV), dt_bias.to(DEV), z, heads, D)          # in place, as the part does
            out = torch.empty(T, heads * V, device=DEV)
            recurrent.gated_delta(qkv, proj, b_off, 0, None, None, state, meta, out, kv_heads, heads, D, V, decay=z)
            at = 0
            for i, c in zip(live, counts):
                got_decay[i].append(z[at:at + c].cpu())
                got_out[i].append(out[at:at + c].cpu())
                at += c
        for i in range(len(lengths)):
            assert torch.allclose(torch.cat(got_decay[i]), refs[i][0], atol=2e-6, rtol=2e-6), f"decay, cuts {cuts[:4]}"
            assert torch.allclose(torch.cat(got_out[i]), refs[i][1], atol=3e-6), f"delta rule, cuts {cuts[:4]}"
        for s in slots:
            cache.free_slot(s)


def test_a_channel_that_does_not_decay_remembers_the_first_token():
    """Two key channels: one keeps what it holds (decay 1), one forgets at once (decay ~0). The first token writes
    to both, 300 tokens later a query reads each: the value comes back from the first and nothing from the second.
    A decay a head instead of a channel, or the rows of the state mixed up with its columns, gives another answer."""
    D, V, T = 2, 3, 300
    qkv = torch.zeros(T, 2 * D + V)
    proj = torch.zeros(T, 1)
    proj[:, 0] = -30.0                       # beta = sigmoid(-30) ~ 0: the later tokens write nothing
    proj[0, 0] = 30.0                        # the first writes all of its value
    qkv[0, D:2 * D] = torch.tensor([0.6, 0.8])
    qkv[0, 2 * D:] = torch.tensor([1.0, -2.0, 3.0])
    qkv[1:, D] = 1.0                         # later keys: unit vectors that beta switches off
    qkv[-2, :D] = torch.tensor([1.0, 0.0])   # reads the first channel
    qkv[-1, :D] = torch.tensor([0.0, 1.0])   # reads the second
    decay = torch.ones(T, D)
    decay[1:, 1] = 1e-3
    cache = Cache({0: (StateNeed((1, D, V)),)}, 64 * 8, 4096, torch.float32, DEV, max_slots=2)
    state = cache.state_views(0)[0]
    for cuts in ([T], [1, 150, T], list(range(1, T + 1))):
        slot = cache.alloc_slot()
        outs, at = [], 0
        for end in cuts:
            meta = step_meta(cache, [slot], [end - at])
            out = torch.empty(end - at, V, device=DEV)
            recurrent.gated_delta(qkv[at:end].to(DEV).contiguous(), proj[at:end].to(DEV).contiguous(), 0, 0, None, None,
                                  state, meta, out, 1, 1, D, V, decay=decay[at:end].to(DEV).contiguous())
            outs.append(out.cpu())
            at = end
        out = torch.cat(outs)
        assert torch.allclose(out[-2], 0.6 * torch.tensor([1.0, -2.0, 3.0]), atol=1e-5), cuts[:3]
        assert float(out[-1].abs().max()) < 1e-6, cuts[:3]
        cache.free_slot(slot)


def test_sigmoid_gated_norm_a_head():
    T, heads, V = 5, 3, 70
    o, proj, w = rand(T, heads * V, seed=1), rand(T, heads * V + 9, seed=2, scale=2.0), 1 + 0.1 * rand(V, seed=3)
    want = (plain.rms_scale(o.view(T, heads, V), 1e-5) * w * plain.sigmoid(proj[:, 4:4 + heads * V].view(T, heads, V))).reshape(T, -1)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        y = torch.empty(T, heads * V, dtype=dtype, device=DEV)
        recurrent.gated_head_norm(o.to(DEV), proj.to(DEV), 4, w.to(DEV), y, heads, V, 1e-5, gate="sigmoid")
        assert torch.allclose(y.float().cpu(), want, atol=tol, rtol=tol)


# ---------------------------------------------------------------- experts chosen by scores within groups
def routed(logits, correction, E, top, groups, keep, width=None):
    T = logits.shape[0]
    rows = logits
    if width:                                  # rows wider than the experts: the further columns do not count
        rows = torch.full((T, width), 50.0)
        rows[:, :E] = logits
    routing = moe.Routing(torch.empty(moe.Routing.ints_needed(T, E, top), dtype=torch.int32, device=DEV),
                          torch.empty(T, top, device=DEV), T, E, top)
    moe.route(rows.to(DEV).contiguous(), correction.to(DEV), routing, scores=True, groups=groups, keep=keep)
    return routing


@pytest.mark.parametrize("T,E,top,groups,keep,shift", [(200, 8, 4, 2, 1, 0.0), (150, 12, 3, 3, 2, -1.5), (90, 6, 2, 6, 3, 0.0),
                                                       (40, 16, 16, 1, 1, -2.0), (70, 130, 7, 13, 4, -1.2), (1, 3, 3, 3, 3, 0.0),
                                                       (33, 9, 5, 3, 2, 0.7)])
def test_choice_by_scores_within_groups(T, E, top, groups, keep, shift):
    """Against the plain choice, token by token. With a correction around -1.5 every selection value is negative: an
    expert outside the kept groups that counted as 0 instead of as minus infinity would then win."""
    logits, correction = rand(T, E, seed=E, scale=1.5), shift + 0.3 * rand(E, seed=top)
    routing = routed(logits, correction, E, top, groups, keep, width=E + 5)
    got, weight = routing.chosen.view(T, top).cpu(), routing.weight.cpu()
    scores = plain.sigmoid(logits)
    for t in range(T):
        want = plain.choose_experts(scores[t], correction, top, groups, keep)
        assert sorted(got[t].tolist()) == sorted(want), f"token {t}"
        s = scores[t][got[t].long()]
        assert torch.allclose(weight[t], s / (s.sum() + 1e-20), atol=1e-6)
    order, row_of = routing.order.cpu(), routing.row_of.cpu()
    assert sorted(order.tolist()) == list(range(T * top))
    assert torch.equal(order[row_of.long()], torch.arange(T * top, dtype=torch.int32))


def test_a_group_is_worth_its_two_best_and_the_correction_only_chooses():
    logit = lambda s: torch.log(torch.tensor(s) / (1 - torch.tensor(s)))
    zero = torch.zeros(4)
    # the best expert (0.9) lies in the group whose two best sum to 1.0; the other group's sum to 1.15
    r = routed(logit([[0.9, 0.1, 0.6, 0.55]]), zero, 4, 1, 2, 1)
    assert r.chosen.cpu().tolist() == [2] and abs(float(r.weight[0, 0]) - 1.0) < 1e-6
    # by the largest alone, or by the sum of all of a group of three, the other group would win
    r = routed(logit([[0.8, 0.1, 0.1, 0.5, 0.45, 0.4]]), torch.zeros(6), 6, 2, 2, 1)
    assert sorted(r.chosen.cpu().tolist()) == [3, 4]
    r = routed(logit([[0.5, 0.45, 0.05, 0.4, 0.35, 0.34]]), torch.zeros(6), 6, 2, 2, 1)
    assert sorted(r.chosen.cpu().tolist()) == [0, 1]
    # the correction moves the choice (group and expert) and stays out of the weights
    r = routed(logit([[0.9, 0.1, 0.6, 0.55]]), torch.tensor([0.0, 0.5, 0.0, 0.0]), 4, 2, 2, 1)
    assert sorted(r.chosen.cpu().tolist()) == [0, 1]
    w = dict(zip(r.chosen.cpu().tolist(), r.weight.cpu()[0].tolist()))
    assert abs(w[0] - 0.9) < 1e-6 and abs(w[1] - 0.1) < 1e-6
    # two groups kept of three, every selection value negative: the third group's experts are never taken
    r = routed(logit([[0.3, 0.2, 0.6, 0.1, 0.5, 0.45]]), torch.full((6,), -2.0), 6, 4, 3, 2)
    assert sorted(r.chosen.cpu().tolist()) == [2, 3, 4, 5]


def test_experts_products_and_the_shared_experts_gated_sum():
    T, E, top, W, F = 50, 8, 3, 64, 96
    y, logits = rand(T, W, seed=1), rand(T, E + 1, seed=2, scale=1.5)
    routing = routed(logits[:, :E], 0.2 * rand(E, seed=3), E, top, 4, 2)
    rows = torch.zeros(T, 16)
    rows[:, :E + 1] = logits
    got_chosen = routing.chosen.view(T, top).cpu()
    gate, up, down = rand(E, F, W, seed=4, scale=0.2), rand(E, F, W, seed=5, scale=0.2), rand(E, W, F, seed=6, scale=0.2)
    shared = rand(T, W, seed=7)
    start = rand(T, W, seed=8)
    want = start.clone()
    for t in range(T):
        for j in range(top):
            e = int(got_chosen[t, j])
            want[t] += routing.weight[t, j].cpu() * plain.glu_expert(y[t], gate[e], up[e], down[e])
        want[t] += plain.sigmoid(logits[t, E]) * shared[t]
    gate_up = torch.cat([gate, up], 1)
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 4e-2)):
        yg, gu_w, down_w = y.to(DEV).to(dtype), gate_up.to(DEV).to(dtype), down.to(DEV).to(dtype)
        act = torch.empty(T * top, F, dtype=dtype, device=DEV)
        out = torch.empty(T * top, W, device=DEV)
        x = start.to(DEV).clone()
        if dtype == torch.bfloat16:
            moe.grouped_mfma(yg, W, 0, moe.pack_grouped(gu_w), act, F, 0, moe.EPI_GLU, routing, gather=True,
                             limit=math.inf, alpha=1.0, shift=0.0)
            moe.grouped_mfma(act, F, 0, moe.pack_grouped(down_w), out, W, 0, moe.EPI_F32, routing)
        else:
            gu = torch.empty(T * top, 2 * F, device=DEV)
            moe.gemm_plain(yg, gu_w, gu, routing, gather=True)
            moe.activate(gu, act, math.inf, 1.0, 0.0)
            moe.gemm_plain(act, down_w, out, routing, gather=False)
        moe.combine(out, routing, x, shared=shared.to(DEV), gate=(rows.to(DEV).contiguous(), E))
        assert torch.allclose(x.cpu(), want, atol=tol, rtol=tol), f"{dtype}"


# ---------------------------------------------------------------- the second product of a pair through a narrow middle
@pytest.mark.parametrize("M,N,K,col0,ld", [(1, 128, 32, 0, 32), (8, 2048, 128, 260, 400), (32, 48, 64, 4, 72), (7, 50, 96, 8, 104),
                                           (33, 64, 32, 0, 32), (5, 40, 24, 0, 24), (6, 32, 32, 3, 40)])
def test_product_of_some_columns_with_a_short_k(M, N, K, col0, ld):
    """Few rows of bfloat16 weights take a kernel of their own (k in steps of 32, rows on 16-byte borders);
    more rows, another k or columns off those borders take the tiled one: both against the plain product."""
    a, w = rand(M, ld, seed=M), rand(N, K, seed=N, scale=0.3)
    for dtype, tol in ((torch.bfloat16, 2e-5), (torch.float32, 2e-5)):
        wd = w.to(dtype)
        c = torch.full((M, N), 9.0, device=DEV)
        ops.gemm_plain_columns(a.to(DEV), col0, K, wd.to(DEV), c)
        want = a[:, col0:col0 + K].double() @ wd.double().T
        assert torch.allclose(c.cpu().double(), want, atol=tol, rtol=tol), dtype
        # the same product leaving the decays of which its sums are the pre-activations, for every size of a head
        # that divides the columns: exp(-exp(A_log[head]) softplus(sum + dt_bias[column]))
        for D in {1, 8, N // 2, N}:
            if N % D:
                continue
            rate, bias = rand(N // D, seed=D + 1), rand(N, seed=D + 2, scale=2.0)
            g = torch.full((M, N), 9.0, device=DEV)
            ops.gemm_plain_columns(a.to(DEV), col0, K, wd.to(DEV), g, decay=(rate.to(DEV), bias.to(DEV), D))
            want_g = torch.exp(-torch.exp(rate.double()).repeat_interleave(D) * plain.softplus(want + bias.double()))
            assert torch.allclose(g.cpu().double(), want_g, atol=tol, rtol=tol), (dtype, D)
