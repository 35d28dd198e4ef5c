"""Plain, slow, whole-sequence formulas of the Modasun decoder: one function a mechanism.

A model of this design is a stack of layers whose norm comes after the sum:

    x <- norm1(alpha x + mixer(x));  x <- norm2(alpha x + ff(x))

with norm(x) = x / sqrt(mean(x^2) + eps) (1 + w). A mixer is a causal softmax attention without a
rotation (queries and keys are divided by their root mean square a head, and a query grows with the
logarithm of its position), or a gated delta rule whose state decays channel by channel. A
feed-forward is dense (squared relu) or a mixture of experts chosen by sigmoid scores within the
best groups, beside a gated shared expert. Layers may run another layer's weights. Nothing here has
a cache, a batch or code in common with the engine; everything runs on the CPU in the dtype of its
inputs (float32, or float64 to judge rounding).
"""
import json
import math
import os

import torch
from safetensors import safe_open


# ---------------------------------------------------------------- small pieces
def rms_scale(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """The design's norm: the stored weight is an offset from one."""
    return rms_scale(x, eps) * (1.0 + w)


def linear(x, weight):
    return x @ weight.T


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    return torch.where(x > 20.0, x, torch.log1p(torch.exp(torch.minimum(x, torch.full_like(x, 20.0)))))


def relu_squared(x):
    r = torch.clamp(x, min=0.0)
    return r * r


# ---------------------------------------------------------------- attention
def query_temperature(positions, coef, every):
    """1 + coef ln(floor((p + 1) / every) + 1) for every position p (a tensor of integers)."""
    steps = torch.div(positions + 1, every, rounding_mode="floor")
    return 1.0 + coef * torch.log(steps.to(torch.float64) + 1.0)


def softmax_attention(q, k, v, scale):
    """One head over T tokens, causal: row i attends to rows 0 .. i. q, k [T, D]; v [T, V]."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=q.dtype)
    for i in range(T):
        s = (k[: i + 1] @ q[i]) * scale
        p = torch.exp(s - s.max())
        out[i] = (p / p.sum()) @ v[: i + 1]
    return out


def attention_mixer(h, w, m, eps):
    """h [T, W]; w: q, k, v, o; m: heads, kv_heads, dim, vdim, scale, q_temp {coef, every} (or none: the
    queries stay as they are)."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_scale(linear(h, w["q"]).view(T, H, D), eps)
    k = rms_scale(linear(h, w["k"]).view(T, G, D), eps)
    v = linear(h, w["v"]).view(T, G, V)
    if m.get("q_temp") is not None:
        temp = query_temperature(torch.arange(T), m["q_temp"]["coef"], m["q_temp"]["every"]).to(h.dtype)
        q = q * temp[:, None, None]
    heads = []
    for head in range(H):
        g = head // (H // G)
        heads.append(softmax_attention(q[:, head], k[:, g], v[:, g], m["scale"]))
    return linear(torch.cat(heads, -1), w["o"])


# ---------------------------------------------------------------- gated delta rule with a decay a channel
def short_conv(x, taps):
    """y[t, c] = sum_j taps[c, j] x[t - (K - 1) + j, c], zeros before the start; x [T, C], taps [C, K]."""
    T, C = x.shape
    K = taps.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        for j in range(K):
            s = t - (K - 1) + j
            if s >= 0:
                out[t] += taps[:, j] * x[s]
    return out


def unit_vectors(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def channel_delta_rule(q, k, v, beta, decay):
    """One head over T tokens. q, k, decay [T, D]; v [T, V]; beta [T]. S (D x V) starts at zero;
    S <- decay (a factor a row) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, D = q.shape
    S = torch.zeros(D, v.shape[1], dtype=q.dtype)
    out = []
    for t in range(T):
        S = decay[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out)


def channel_delta_mixer(h, w, m, eps):
    """w: q, k, v, q.conv, k.conv, v.conv, b, A_log, dt_bias, a1, a2, g1, g2, norm, o."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(linear(h, w["q"]), w["q.conv"])).view(T, G, D)
    k = silu(short_conv(linear(h, w["k"]), w["k.conv"])).view(T, G, D)
    v = silu(short_conv(linear(h, w["v"]), w["v.conv"])).view(T, H, V)
    q = unit_vectors(q) * D ** -0.5
    k = unit_vectors(k)
    beta = sigmoid(linear(h, w["b"]))                                          # [T, H]
    step = softplus(linear(linear(h, w["a1"]), w["a2"]) + w["dt_bias"]).view(T, H, D)
    decay = torch.exp(-torch.exp(w["A_log"])[None, :, None] * step)
    gate = sigmoid(linear(linear(h, w["g1"]), w["g2"])).view(T, H, V)
    heads = []
    for head in range(H):
        g = head // (H // G)
        o = channel_delta_rule(q[:, g], k[:, g], v[:, head], beta[:, head], decay[:, head])
        heads.append(rms_scale(o, eps) * w["norm"] * gate[:, head])
    return linear(torch.cat(heads, -1), w["o"])


# ---------------------------------------------------------------- feed-forwards
def dense_ff(h, w):
    return linear(relu_squared(linear(h, w["up"])), w["down"])


def glu_expert(h, gate, up, down):
    return linear(silu(linear(h, gate)) * linear(h, up), down)


def choose_experts(scores, correction, top, groups, keep):
    """For one token: the indices of the chosen experts, best first. Selection values are the scores plus
    the correction; a run of adjacent experts is worth the two highest of its selection values, added (its only
    one, if it has one expert); outside the `keep` best groups nothing can be chosen."""
    E = scores.shape[0]
    choice = scores + correction
    size = E // groups
    worth = []
    for g in range(groups):
        part = torch.sort(choice[g * size:(g + 1) * size], descending=True).values
        worth.append(float(part[:2].sum()))
    best = sorted(range(groups), key=lambda g: (-worth[g], g))[:keep]
    masked = torch.full_like(choice, -math.inf)
    for g in best:
        masked[g * size:(g + 1) * size] = choice[g * size:(g + 1) * size]
    order = sorted(range(E), key=lambda e: (-float(masked[e]), e))
    return order[:top]


def moe_ff(h, w, m):
    """w: router, correction, e<i>.gate/up/down, shared.gate/up/down/sg; m: the layer's 'mlp' entry (without
    'groups': one group of all experts; without 'shared': no shared expert)."""
    r = m["router"]
    E, top = r["experts"], r["top"]
    groups, keep = (r["groups"]["count"], r["groups"]["keep"]) if r.get("groups") is not None else (1, 1)
    scores = sigmoid(linear(h, w["router"]))
    out = torch.zeros(h.shape[0], w["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        chosen = choose_experts(scores[t], w["correction"], top, groups, keep)
        total = sum(scores[t, e] for e in chosen) + 1e-20
        for e in chosen:
            out[t] += scores[t, e] / total * glu_expert(h[t], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])
    if m.get("shared") is None:
        return out
    shared = glu_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"])
    return out + sigmoid(linear(h, w["shared.sg"])) * shared


# ---------------------------------------------------------------- the model
def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg, tensors, tokens, dtype=torch.float32, layers_out=None, rows=None):
    """Logits [T, vocab] of one sequence of token ids (of the positions `rows` only, if given).
    layers_out: a list that receives the residual stream after every layer run."""
    t = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in tensors.items()}
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of", i)
        p = f"l{src}."
        m = layer["mixer"]
        if layer["type"] == "attention":
            mixed = attention_mixer(x, sub(t, p + "mix."), m, eps)
        elif layer["type"] == "channel_delta":
            mixed = channel_delta_mixer(x, sub(t, p + "mix."), m, eps)
        else:
            raise ValueError(layer["type"])
        x = offset_norm(alpha * x + mixed, t[p + "norm1"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                ff = dense_ff(x, sub(t, p + "mlp."))
            else:
                ff = moe_ff(x, sub(t, p + "mlp."), mlp)
            x = offset_norm(alpha * x + ff, t[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    if rows is not None:
        x = x[list(rows)]
    x = offset_norm(x, t["final.norm"], eps)
    return linear(x, t["embed"])


def greedy(cfg, tensors, prompt, n):
    """n tokens after the prompt, each the first of the largest logits of the sequence so far."""
    seq, out = list(prompt), []
    for _ in range(n):
        logits = forward(cfg, tensors, seq, rows=[len(seq) - 1])[0]
        out.append(int(torch.argmax(logits)))
        seq.append(out[-1])
    return out


def load_folder(folder):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name)
    return cfg, tensors
