"""The plain Vipalorn formulas pinned by library routines, by special cases that can be worked out by hand
and by invariants; the configuration and the cache's needs of the family, on the CPU."""
import math

import pytest
import torch

from herbert_rs_amd.cache import Cache, KVNeed, StateNeed
from herbert_rs_amd.config.registry import resolve_architecture
from herbert_rs_amd.engine.model import Model
from herbert_rs_amd.errors import ConfigError

from .plain import vipalorn as plain
from .vipalorn_tiny import VIP_P, VIP_Q, VIP_R


def rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


def test_layer_norm_against_the_library():
    x, w = rand(5, 33), rand(33, seed=1)
    want = torch.nn.functional.layer_norm(x, (33,), w, None, 1e-5)
    assert torch.allclose(plain.layer_norm(x, w, 1e-5), want, atol=1e-12)


def test_short_convolution_against_the_library_and_by_hand():
    x, taps = rand(9, 4), rand(4, 3, seed=2)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (2, 0)), taps[:, None, :], groups=4)[0].T
    assert torch.allclose(plain.short_conv(x, taps), want, atol=1e-12)
    one = plain.short_conv(torch.tensor([[1.0], [0.0], [0.0], [0.0]], dtype=torch.float64), torch.tensor([[5.0, 7.0, 11.0]], dtype=torch.float64))
    assert one[:, 0].tolist() == [11.0, 7.0, 5.0, 0.0]          # the last tap weighs the current token


def test_delta_rule_special_cases():
    T, D, V = 6, 4, 3
    q, k, v = rand(T, D), rand(T, D, seed=1), rand(T, V, seed=2)
    ones, zeros = torch.ones(T, dtype=torch.float64), torch.zeros(T, dtype=torch.float64)
    # no decay, full step, orthonormal keys: token t's value is stored along its key and read back exactly
    eye = torch.eye(D, dtype=torch.float64)[[0, 1, 2, 3, 0, 1]]
    out = plain.delta_rule(eye, eye, v, ones, ones)
    assert torch.allclose(out, v, atol=1e-12)                  # o_t is read after token t has been written
    # beta 0 writes nothing: the state stays zero
    assert torch.equal(plain.delta_rule(q, k, v, zeros, ones), torch.zeros(T, V, dtype=torch.float64))
    # decay 0 forgets everything before the token: o_t = beta (k_t . q_t) v_t
    half = 0.5 * ones
    want = (half * (k * q).sum(-1))[:, None] * v
    assert torch.allclose(plain.delta_rule(q, k, v, half, zeros), want, atol=1e-12)
    # cutting the sequence anywhere and carrying S gives the same (checked by unrolling two tokens by hand)
    g, b = torch.tensor([0.9, 0.8], dtype=torch.float64), torch.tensor([0.3, 0.6], dtype=torch.float64)
    S = b[0] * torch.outer(k[0], v[0])
    S2 = g[1] * S
    S2 = S2 + torch.outer(k[1], b[1] * (v[1] - S2.T @ k[1]))
    assert torch.allclose(plain.delta_rule(q[:2], k[:2], v[:2], b, g)[1], S2.T @ q[1], atol=1e-12)


def test_rotation_keeps_lengths_and_turns_by_differences():
    x = rand(7, 2, 10)
    pos = [0, 1, 2, 3, 10, 100, 1000]
    y = plain.rotate_half_layout(x, pos, 250.0, 6)
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.allclose(y[0], x[0], atol=1e-12)
    assert torch.allclose(y[..., :6].norm(dim=-1), x[..., :6].norm(dim=-1), atol=1e-9)
    # a dot product of two rotated vectors depends on the difference of their positions only
    a, b = rand(1, 6, seed=3), rand(1, 6, seed=4)
    d1 = (plain.rotate_half_layout(a, [5], 250.0, 6) * plain.rotate_half_layout(b, [2], 250.0, 6)).sum()
    d2 = (plain.rotate_half_layout(a, [105], 250.0, 6) * plain.rotate_half_layout(b, [102], 250.0, 6)).sum()
    assert abs(float(d1 - d2)) < 1e-9
    # the pair (i, i + dims / 2) at angle p * base^(-2 i / dims)
    e = torch.zeros(1, 6, dtype=torch.float64)
    e[0, 1] = 1.0
    r = plain.rotate_half_layout(e, [3], 250.0, 6)
    ang = 3 * 250.0 ** (-2.0 / 6)
    assert abs(float(r[0, 1]) - math.cos(ang)) < 1e-12 and abs(float(r[0, 4]) - math.sin(ang)) < 1e-12


def test_routing_and_experts():
    h, wr, br = rand(6, 8), rand(5, 8, seed=1), rand(5, seed=2)
    chosen, weight = plain.route(h, wr, br, 2)
    z = h @ wr.T + br
    for t in range(6):
        order = sorted(range(5), key=lambda e: -float(z[t, e]))
        assert sorted(chosen[t].tolist()) == sorted(order[:2])
        assert abs(float(weight[t].sum()) - 1.0) < 1e-12
        a, b = float(z[t, order[0]]), float(z[t, order[1]])
        assert abs(float(weight[t].max()) - 1.0 / (1.0 + math.exp(b - a))) < 1e-12
    # the expert's clamps: a gate beyond the limit is cut from above only, the linear part on both sides
    one = torch.ones(1, 1, dtype=torch.float64)
    big = plain.expert(one, 10.0 * one, -10.0 * one, one, 2.0)
    assert abs(float(big) - 2.0 / (1.0 + math.exp(-1.702 * 2.0)) * (-2.0 + 1.0)) < 1e-12
    low = plain.expert(one, -10.0 * one, 0.5 * one, one, 2.0)
    assert abs(float(low) - (-10.0) / (1.0 + math.exp(17.02)) * 1.5) < 1e-12


def test_latent_attention_with_the_matrices_taken_to_the_other_side():
    """Scores and sums on the latents themselves (the query through W_uk^T first, W_uv last) give what the
    heads' own keys and values give: what the engine's kernels rely on."""
    m = {"heads": 3, "dim": 8, "rot_dim": 4, "vdim": 6, "kv_rank": 10, "scale": 0.3, "rot": {"base": 100.0, "dims": 4}}
    p, T, W = "x.", 9, 16
    w = {p + "q": rand(3 * 12, W), p + "dkv": rand(14, W, seed=1), p + "dkv.norm": rand(10, seed=2),
         p + "uk": rand(24, 10, seed=3), p + "uv": rand(18, 10, seed=4), p + "g": rand(3, W, seed=5),
         p + "o": rand(W, 18, seed=6)}
    h = rand(T, W, seed=7)
    want = plain.latent_attention_mixer(h, list(range(T)), w, p, m, 1e-5)
    q = (h @ w[p + "q"].T).view(T, 3, 12)
    down = h @ w[p + "dkv"].T
    c = plain.rms_scale(down[:, :10], 1e-5) * w[p + "dkv.norm"]
    r = plain.rotate_half_layout(down[:, 10:], list(range(T)), 100.0, 4)
    qr = plain.rotate_half_layout(q[..., 8:], list(range(T)), 100.0, 4)
    gate = plain.sigmoid(h @ w[p + "g"].T)
    outs = []
    for n in range(3):
        uk, uv = w[p + "uk"][8 * n:8 * n + 8], w[p + "uv"][6 * n:6 * n + 6]
        s = ((q[:, n, :8] @ uk) @ c.T + qr[:, n] @ r.T) * 0.3
        s = s.masked_fill(torch.triu(torch.ones(T, T, dtype=torch.bool), 1), -math.inf)
        outs.append((torch.softmax(s, -1) @ c) @ uv.T * gate[:, n:n + 1])
    assert torch.allclose(torch.cat(outs, -1) @ w[p + "o"].T, want, atol=1e-10)


@pytest.mark.parametrize("raw", [VIP_P, VIP_Q, VIP_R])
def test_configuration_spec_and_needs(raw):
    arch = resolve_architecture(raw)
    cfg = arch.config_class.from_dict(raw)
    assert arch.name == "Vipalorn" and cfg.to_dict() == raw
    model = Model(arch.build_spec(cfg))
    needs = model.tensor_needs()
    assert needs["embed"].shape == (raw["vocab"], raw["width"]) and "final.norm" in needs and "embed.norm" in needs
    for i, layer in enumerate(raw["layers"]):
        assert (f"l{i}.mlp.router" in needs) == (layer["mlp"] is not None)
        if layer["type"] == "delta":
            m = layer["mixer"]
            assert needs[f"l{i}.mix.q.conv"].shape == (m["kv_heads"] * m["dim"], m["conv"])
            assert needs[f"l{i}.mix.v"].shape == (m["heads"] * m["vdim"], raw["width"])
        else:
            m = layer["mixer"]
            assert needs[f"l{i}.mix.dkv"].shape == (m["kv_rank"] + m["rot_dim"], raw["width"])
            assert needs[f"l{i}.mix.uk"].shape == (m["heads"] * m["dim"], m["kv_rank"])
    cache_needs = model.cache_needs()
    for i, layer in enumerate(raw["layers"]):
        if layer["type"] == "latent_attention":
            assert cache_needs[i] == KVNeed(1, layer["mixer"]["kv_rank"] + layer["mixer"]["rot_dim"], None, values=False)


def test_configuration_errors():
    arch = resolve_architecture(VIP_R)
    for path, value in ((("layers", 0, "type"), "conv"), (("layers", 1, "mlp", "kind"), "dense"),
                        (("layers", 1, "mlp", "router", "top"), 9), (("layers", 1, "mixer", "rot", "dims"), 3),
                        (("layers", 0, "mixer", "kv_heads"), 0), (("norm",), None), (("vocab",), None)):
        import copy
        raw = copy.deepcopy(VIP_R)
        at = raw
        for key in path[:-1]:
            at = at[key]
        if value is None:
            del at[path[-1]]
        else:
            at[path[-1]] = value
        with pytest.raises(ConfigError):
            arch.config_class.from_dict(raw)
    with pytest.raises(ConfigError):
        resolve_architecture({"architecture": "Vipalorm"})


def test_rows_of_keys_alone_and_states_in_the_mixers_order():
    a, b = StateNeed((2, 3, 4)), StateNeed((1, 10))
    c = StateNeed((2, 5, 4))
    needs = {0: (a, b), 1: KVNeed(1, 12, None, values=False), 2: (c, b), 3: KVNeed(2, 12, None)}
    cache = Cache(needs, 64 * 4, 1 << 20, torch.float32, "cpu")
    view = cache.kv_view(1)
    assert view.v is None and tuple(view.k.shape[1:]) == (1, 64, 12)
    assert cache.kv_view(3).v is not None
    # a table no wider than the pool has pages, however many positions the model allows
    assert view.page_table.shape[1] == 4
    # entry 2's first state is its own, its second the group it shares with entry 0
    assert [tuple(v.shape[1:]) for v in cache.state_views(2)] == [(2, 5, 4), (1, 10)]
    assert [tuple(v.shape[1:]) for v in cache.state_views(0)] == [(2, 3, 4), (1, 10)]
    assert Cache.bytes_needed(needs, 64 * 4, torch.float32) > 0
    slot = cache.alloc_slot()
    cache.reserve_all([(slot, 200)])
    cache.commit(slot, 200)
    cache.check()
    cache.free_slot(slot)
    cache.check()
