"""The plain Modasun formulas pinned by library routines, by special cases that can be worked out by hand and by
invariants; the configuration, the parts' description and the cache's needs of the family, on the CPU."""
import copy
import json
import math

import pytest
import torch

from herbert_rs_amd.cache import KVNeed, StateNeed
from herbert_rs_amd.config.registry import resolve_architecture
from herbert_rs_amd.engine.model import Model
from herbert_rs_amd.errors import ConfigError

from .modasun_tiny import CONFIGS
from .plain import modasun as plain


def rand(*shape, seed=0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


def test_norm_with_its_weight_around_zero():
    x, w = rand(5, 33), 0.1 * rand(33, seed=1)
    want = torch.nn.functional.rms_norm(x, (33,), 1.0 + w, 1e-5)
    assert torch.allclose(plain.offset_norm(x, w, 1e-5), want, atol=1e-12)
    assert torch.allclose(plain.offset_norm(x, torch.zeros(33, dtype=torch.float64), 0.0).pow(2).mean(-1), torch.ones(5, dtype=torch.float64))
    # eps lies inside the root
    assert math.isclose(float(plain.rms_scale(torch.tensor([3.0, 4.0], dtype=torch.float64), 2.0)[0]), 3.0 / math.sqrt(12.5 + 2.0))


def test_the_querys_factor_steps_at_multiples_of_every():
    f = plain.query_temperature(torch.arange(200), 0.3, 64)
    assert f[0] == f[62] == 1.0                                    # floor((p + 1) / 64) = 0 up to p = 62
    assert math.isclose(float(f[63]), 1 + 0.3 * math.log(2)) and f[63] == f[126]
    assert math.isclose(float(f[127]), 1 + 0.3 * math.log(3)) and math.isclose(float(f[191]), 1 + 0.3 * math.log(4))
    g = plain.query_temperature(torch.arange(5), 1.0, 1)           # every position a step
    assert torch.allclose(g, 1 + torch.log(torch.arange(5, dtype=torch.float64) + 2))


def test_attention_against_the_library_and_its_causality():
    T, H, G, D, V, W = 11, 4, 2, 6, 10, 16
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.37, "q_temp": {"coef": 0.5, "every": 4}}
    w = {"q": rand(H * D, W, seed=1), "k": rand(G * D, W, seed=2), "v": rand(G * V, W, seed=3), "o": rand(W, H * V, seed=4)}
    h = rand(T, W, seed=5)
    got = plain.attention_mixer(h, w, m, 1e-5)
    q = plain.rms_scale((h @ w["q"].T).view(T, H, D), 1e-5) * plain.query_temperature(torch.arange(T), 0.5, 4)[:, None, None]
    k = plain.rms_scale((h @ w["k"].T).view(T, G, D), 1e-5).repeat_interleave(H // G, 1)
    v = (h @ w["v"].T).view(T, G, V).repeat_interleave(H // G, 1)
    lib = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1),
                                                           is_causal=True, scale=0.37)
    assert torch.allclose(got, lib.transpose(0, 1).reshape(T, H * V) @ w["o"].T, atol=1e-10)
    h2 = h.clone()
    h2[7] += 1.0                                                   # a later token changes nothing before it
    assert torch.allclose(plain.attention_mixer(h2, w, m, 1e-5)[:7], got[:7], atol=1e-12)


def test_short_convolution_against_the_library_and_by_hand():
    x, taps = rand(9, 4), rand(4, 3, seed=2)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (2, 0)), taps[:, None, :], groups=4)[0].T
    assert torch.allclose(plain.short_conv(x, taps), want, atol=1e-12)
    one = plain.short_conv(torch.tensor([[1.0], [0.0], [0.0], [0.0]], dtype=torch.float64),
                           torch.tensor([[5.0, 7.0, 11.0]], dtype=torch.float64))
    assert one[:, 0].tolist() == [11.0, 7.0, 5.0, 0.0]          # the last tap weighs the current token
    assert torch.equal(plain.short_conv(x, torch.ones(4, 1, dtype=torch.float64)), x)      # one tap: no convolution


def test_delta_rule_with_a_decay_a_channel_special_cases():
    T, D, V = 6, 4, 3
    q, k, v = rand(T, D), rand(T, D, seed=1), rand(T, V, seed=2)
    ones, zeros = torch.ones(T, dtype=torch.float64), torch.zeros(T, dtype=torch.float64)
    keep, forget = torch.ones(T, D, dtype=torch.float64), torch.zeros(T, D, dtype=torch.float64)
    # no decay, full step, orthonormal keys: a token's value is stored along its key and read back in the same step
    eye = torch.eye(D, dtype=torch.float64)[[0, 1, 2, 3, 0, 1]]
    assert torch.allclose(plain.channel_delta_rule(eye, eye, v, ones, keep), v, atol=1e-12)
    assert torch.equal(plain.channel_delta_rule(q, k, v, zeros, keep), torch.zeros(T, V, dtype=torch.float64))
    # decay 0 in every channel forgets everything before the token: o_t = beta (k_t . q_t) v_t
    half = 0.5 * ones
    assert torch.allclose(plain.channel_delta_rule(q, k, v, half, forget), (half * (k * q).sum(-1))[:, None] * v, atol=1e-12)
    # the decay scales the rows of S that belong to key channels: channel 0 keeps, the others forget
    mixed = forget.clone()
    mixed[:, 0] = 1.0
    S = torch.zeros(D, V, dtype=torch.float64)
    for t in range(3):
        S = mixed[t][:, None] * S
        S = S + torch.outer(k[t], half[t] * (v[t] - S.T @ k[t]))
    assert torch.allclose(plain.channel_delta_rule(q[:3], k[:3], v[:3], half[:3], mixed[:3])[2], S.T @ q[2], atol=1e-12)
    # a decay that is the same in every channel is the decay a head
    g = torch.tensor([0.9, 0.8, 0.7, 0.6, 0.5, 0.4], dtype=torch.float64)
    S = torch.zeros(D, V, dtype=torch.float64)
    outs = []
    for t in range(T):
        S = g[t] * S
        S = S + torch.outer(k[t], half[t] * (v[t] - S.T @ k[t]))
        outs.append(S.T @ q[t])
    assert torch.allclose(plain.channel_delta_rule(q, k, v, half, g[:, None].expand(T, D)), torch.stack(outs), atol=1e-12)


def test_the_choice_of_experts():
    t = lambda *v: torch.tensor(v, dtype=torch.float64)
    zero4 = torch.zeros(4, dtype=torch.float64)
    # the best expert lies in the group that loses on the sum of its two best
    assert plain.choose_experts(t(0.9, 0.1, 0.6, 0.55), zero4, 1, 2, 1) == [2]
    assert plain.choose_experts(t(0.9, 0.1, 0.6, 0.55), zero4, 2, 2, 2) == [0, 2]
    # two best, not all of a group and not the best alone
    assert sorted(plain.choose_experts(t(0.8, 0.1, 0.1, 0.5, 0.45, 0.4), torch.zeros(6, dtype=torch.float64), 2, 2, 1)) == [3, 4]
    assert sorted(plain.choose_experts(t(0.5, 0.45, 0.05, 0.4, 0.35, 0.34), torch.zeros(6, dtype=torch.float64), 2, 2, 1)) == [0, 1]
    # the correction chooses; negative selection values: the experts of other groups are out, not worth 0
    assert sorted(plain.choose_experts(t(0.9, 0.1, 0.6, 0.55), t(0.0, 0.5, 0.0, 0.0), 2, 2, 1)) == [0, 1]
    assert sorted(plain.choose_experts(t(0.3, 0.2, 0.6, 0.1, 0.5, 0.45), torch.full((6,), -2.0, dtype=torch.float64), 4, 3, 2)) == [2, 3, 4, 5]
    # groups of one expert are worth that expert
    assert plain.choose_experts(t(0.2, 0.7, 0.4), torch.zeros(3, dtype=torch.float64), 1, 3, 1) == [1]


def test_mixture_of_experts_weights_and_the_shared_expert():
    W, F, Fs, E, T = 8, 6, 5, 4, 7
    m = {"router": {"experts": E, "top": 2, "groups": {"count": 2, "keep": 2}}, "shared": {"ff": Fs}}
    w = {"router": rand(E, W, seed=1), "correction": 0.1 * rand(E, seed=2), "shared.gate": rand(Fs, W, seed=3),
         "shared.up": rand(Fs, W, seed=4), "shared.down": rand(W, Fs, seed=5), "shared.sg": rand(1, W, seed=6)}
    for e in range(E):
        w.update({f"e{e}.gate": rand(F, W, seed=10 + e), f"e{e}.up": rand(F, W, seed=20 + e), f"e{e}.down": rand(W, F, seed=30 + e)})
    h = rand(T, W, seed=7)
    got = plain.moe_ff(h, w, m)
    s = torch.sigmoid(h @ w["router"].T)
    top = torch.topk(s + w["correction"], 2, -1).indices        # every group kept: the choice is the plain top two
    want = torch.zeros(T, W, dtype=torch.float64)
    for t in range(T):
        a, b = int(top[t, 0]), int(top[t, 1])
        for e, other in ((a, b), (b, a)):
            y = torch.nn.functional.silu(h[t] @ w[f"e{e}.gate"].T) * (h[t] @ w[f"e{e}.up"].T)
            want[t] += s[t, e] / (s[t, e] + s[t, other]) * (y @ w[f"e{e}.down"].T)
    shared = (torch.nn.functional.silu(h @ w["shared.gate"].T) * (h @ w["shared.up"].T)) @ w["shared.down"].T
    bare = plain.moe_ff(h, w, {"router": {"experts": E, "top": 2}})       # one group, no shared expert
    assert torch.allclose(bare, want, atol=1e-10)
    want += torch.sigmoid(h @ w["shared.sg"].T) * shared
    assert torch.allclose(got, want, atol=1e-10)
    x = rand(4, W, seed=8)
    assert torch.allclose(plain.dense_ff(x, {"up": w["e0.up"], "down": w["e0.down"]}),
                          torch.relu(x @ w["e0.up"].T).pow(2) @ w["e0.down"].T, atol=1e-12)


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_configuration_spec_and_needs(name):
    raw = CONFIGS[name][0]
    arch = resolve_architecture(raw)
    cfg = arch.config_class.from_dict(raw)
    assert arch.name == "Modasun" and arch.config_class.from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()
    if name != "N":                      # (N leaves sections out, which are written back with what they default to)
        assert cfg.to_dict() == raw
    model = Model(arch.build_spec(cfg))
    needs = model.tensor_needs()
    W = raw["width"]
    assert needs["embed"].shape == (raw["vocab"], W) and needs["final.norm"].shape == (W,)
    cache_needs = model.cache_needs()
    assert sorted(cache_needs) == list(range(len(raw["layers"])))          # a cache entry a run, also of another layer's weights
    for i, layer in enumerate(raw["layers"]):
        m, p = layer["mixer"], f"l{i}."
        if "weights_of" in layer:
            assert not any(k.startswith(p) for k in needs)
            assert cache_needs[i] == cache_needs[layer["weights_of"]]
            continue
        assert (p + "norm2" in needs) == (layer["mlp"] is not None)
        if layer["type"] == "attention":
            assert needs[p + "mix.q"].shape == (m["heads"] * m["dim"], W) and needs[p + "mix.k"].shape == (m["kv_heads"] * m["dim"], W)
            assert needs[p + "mix.v"].shape == (m["kv_heads"] * m["vdim"], W) and needs[p + "mix.o"].shape == (W, m["heads"] * m["vdim"])
            assert cache_needs[i] == KVNeed(m["kv_heads"], max(m["dim"], m["vdim"]), None)
        else:
            qk, v = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
            assert needs[p + "mix.q.conv"].shape == (qk, m["conv"]) and needs[p + "mix.v.conv"].shape == (v, m["conv"])
            assert needs[p + "mix.a2"].shape == (m["heads"] * m["dim"], m["low_rank"]["decay"])
            assert needs[p + "mix.g2"].shape == (v, m["low_rank"]["gate"]) and needs[p + "mix.dt_bias"].shape == (m["heads"] * m["dim"],)
            assert needs[p + "mix.A_log"].shape == (m["heads"],) and needs[p + "mix.norm"].shape == (m["vdim"],)
            states = [StateNeed((m["heads"], m["dim"], m["vdim"]), torch.float32)]
            if m["conv"] > 1:
                states.append(StateNeed((m["conv"] - 1, 2 * qk + v), torch.float32))
            assert cache_needs[i] == tuple(states)
        mlp = layer["mlp"]
        if mlp is not None and mlp["kind"] == "moe":
            E = mlp["router"]["experts"]
            assert needs[p + "mlp.router"].shape == (E, W) and needs[p + "mlp.correction"].shape == (E,)
            assert needs[p + f"mlp.e{E - 1}.down"].shape == (W, mlp["expert"]["ff"]) and p + f"mlp.e{E}.down" not in needs
            if "shared" in mlp:
                assert needs[p + "mlp.shared.up"].shape == (mlp["shared"]["ff"], W) and needs[p + "mlp.shared.sg"].shape == (1, W)
            else:
                assert not any(k.startswith(p + "mlp.shared") for k in needs)
        elif mlp is not None:
            assert needs[p + "mlp.up"].shape == (mlp["ff"], W) and needs[p + "mlp.down"].shape == (W, mlp["ff"])


def test_a_run_of_a_run_ends_at_the_layer_that_has_the_tensors():
    raw = copy.deepcopy(CONFIGS["Q"][0])
    raw["layers"][3]["weights_of"] = 2                  # layer 2 runs layer 0's itself
    cfg = resolve_architecture(raw).config_class.from_dict(raw)
    assert [l.weights_of for l in cfg.layers] == [None, None, 0, 0]
    later = copy.deepcopy(CONFIGS["Q"][0])              # the tensors may belong to a later layer
    later["layers"] = [dict(later["layers"][0], weights_of=1)] + later["layers"][:2]
    arch = resolve_architecture(later)
    spec = arch.build_spec(arch.config_class.from_dict(later))
    assert [e.layer for e in spec.schedule] == [0, 0, 1] and "l1.mix.q" in Model(spec).tensor_needs()


def test_configuration_errors():
    base = CONFIGS["P"][0]
    arch = resolve_architecture(base)
    for path, value in ((("layers", 0, "type"), "conv"), (("layers", 0, "mlp", "kind"), "glu"),
                        (("layers", 0, "mlp", "router", "top"), 7), (("layers", 0, "mlp", "router", "groups", "count"), 4),
                        (("layers", 0, "mlp", "router", "groups", "keep"), 1), (("layers", 0, "mixer", "kv_heads"), 3),
                        (("layers", 1, "mixer", "q_temp", "every"), 0), (("layers", 1, "mixer", "scale"), None),
                        (("layers", 3, "weights_of"), 3), (("layers", 3, "weights_of"), 9), (("layers", 3, "mixer", "conv"), 2),
                        (("norm",), None), (("vocab",), None), (("postln_alpha",), None), (("embedding", "scale"), None)):
        raw = json.loads(json.dumps(base))           # (a copy in which no two layers share an object)
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
        resolve_architecture({"architecture": "Modasum"})


def test_sections_that_a_configuration_may_leave_out():
    """No "q_temp": queries that do not grow; no "groups": one group of all experts; no "shared": no shared expert."""
    raw = json.loads(json.dumps(CONFIGS["P"][0]))
    del raw["layers"][1]["mixer"]["q_temp"]
    del raw["layers"][2]["mixer"]["q_temp"]
    del raw["layers"][0]["mlp"]["router"]["groups"]
    del raw["layers"][0]["mlp"]["shared"]
    del raw["layers"][3]["mlp"]["router"]["groups"]
    del raw["layers"][3]["mlp"]["shared"]
    arch = resolve_architecture(raw)
    cfg = arch.config_class.from_dict(raw)
    assert cfg.layers[1].mixer.q_temp_coef == 0.0 and cfg.layers[0].mlp.groups == cfg.layers[0].mlp.keep == 1
    assert cfg.layers[0].mlp.shared_ff is None
    needs = Model(arch.build_spec(cfg)).tensor_needs()
    assert "l0.mlp.router" in needs and not any(k.startswith("l0.mlp.shared") for k in needs)
