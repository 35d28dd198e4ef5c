"""Plain, slow, whole-sequence formulas of the Vipalorn decoder: one function a mechanism.

A model of this design is a stack of layers, each a token mixer beside a routed feed-forward
that both read one layer norm of the residual stream x:

    h = layernorm(x);  x <- x + m * (mixer(h) + experts(h))

with two kinds of mixer: a gated delta rule (a matrix of state a head, written and read once a
token) and an attention over one shared low-rank latent a token. Nothing here has a cache, a
batch or code in common with the engine; everything runs on the CPU in the dtype of its inputs
(float32, or float64 to judge rounding).
"""
import json
import math
import os

import torch
from safetensors import safe_open


# ---------------------------------------------------------------- small pieces
def layer_norm(x, weight, eps):
    """(x - mean) / sqrt(var + eps) * w over the last axis; var = mean of squared deviations."""
    mean = x.mean(-1, keepdim=True)
    dev = x - mean
    var = (dev * dev).mean(-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * weight


def rms_scale(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def linear(x, weight):
    """y = W x for every row of x; weights are [out, in]."""
    return x @ weight.T


def sigmoid(x):
    return 1.0 / (1.0 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def softplus(x):
    """log(1 + e^x), written so that large x does not overflow."""
    return torch.where(x > 20.0, x, torch.log1p(torch.exp(torch.minimum(x, torch.full_like(x, 20.0)))))


# ---------------------------------------------------------------- short convolution
def short_conv(x, taps):
    """y[t, c] = sum_j taps[c, j] * x[t - (K - 1) + j, c] with x = 0 at negative times, so taps[:, K - 1]
    belongs to token t itself. x [T, C], taps [C, K]."""
    T, C = x.shape
    K = taps.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        for j in range(K):
            s = t - (K - 1) + j
            if s >= 0:
                out[t] += taps[:, j] * x[s]
    return out


# ---------------------------------------------------------------- gated delta rule
def unit_vectors(x):
    """x / sqrt(sum(x^2) + 1e-6) over the last axis."""
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def delta_rule(q, k, v, beta, decay):
    """The recurrence of one head over T tokens. q, k [T, D]; v [T, V]; beta, decay [T].
    S (D x V) starts at zero;  S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, D = q.shape
    S = torch.zeros(D, v.shape[1], dtype=q.dtype)
    out = []
    for t in range(T):
        S = decay[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out)


def delta_mixer(h, w, p, mixer, eps):
    """The whole 'delta' mixer on h [T, width]; `p` is the tensors' prefix ('l3.mix.')."""
    heads, kv_heads, D, V = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    T = h.shape[0]
    q = silu(short_conv(linear(h, w[p + "q"]), w[p + "q.conv"])).view(T, kv_heads, D)
    k = silu(short_conv(linear(h, w[p + "k"]), w[p + "k.conv"])).view(T, kv_heads, D)
    v = silu(short_conv(linear(h, w[p + "v"]), w[p + "v.conv"])).view(T, heads, V)
    q = unit_vectors(q) * D ** -0.5
    k = unit_vectors(k)
    beta = sigmoid(linear(h, w[p + "b"]))                                              # [T, heads]
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(linear(h, w[p + "a"]) + w[p + "dt_bias"]))
    gate = silu(linear(h, w[p + "g"])).view(T, heads, V)
    group = heads // kv_heads
    outs = []
    for n in range(heads):
        o = delta_rule(q[:, n // group], k[:, n // group], v[:, n], beta[:, n], decay[:, n])
        outs.append(rms_scale(o, eps) * w[p + "norm"] * gate[:, n])
    return linear(torch.stack(outs, 1).reshape(T, heads * V), w[p + "o"])


# ---------------------------------------------------------------- rotation
def rotate_half_layout(x, positions, base, dims):
    """The first `dims` entries of the last axis rotated: entry i pairs with i + dims/2; the pair
    (a, b) at position p becomes (a cos - b sin, b cos + a sin), angle p * base^(-2i/dims).
    x [T, ..., n >= dims]; entries from `dims` on are copied."""
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    freq = torch.as_tensor(base, dtype=x.dtype) ** (-2.0 * i / dims)
    angle = torch.as_tensor(positions, dtype=x.dtype)[:, None] * freq[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    cos, sin = torch.cos(angle).view(shape), torch.sin(angle).view(shape)
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * cos - b * sin, b * cos + a * sin, x[..., dims:]], -1)


# ---------------------------------------------------------------- latent attention
def latent_attention_mixer(h, positions, w, p, mixer, eps):
    """Attention with the heads' own keys [W_uk c | r] and values W_uv c built from a token's latent c and the
    rotated part r that all heads use; causal softmax; every head's output times a sigmoid gate."""
    H, D, R, V, rank = mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"], mixer["kv_rank"]
    rot = mixer["rot"]
    T = h.shape[0]
    q = linear(h, w[p + "q"]).view(T, H, D + R)
    q_plain, q_rot = q[..., :D], q[..., D:]
    down = linear(h, w[p + "dkv"])
    c = rms_scale(down[:, :rank], eps) * w[p + "dkv.norm"]
    k_rot = rotate_half_layout(down[:, rank:], positions, rot["base"], rot["dims"])       # [T, R]
    q_rot = rotate_half_layout(q_rot, positions, rot["base"], rot["dims"])
    k_plain = linear(c, w[p + "uk"]).view(T, H, D)
    value = linear(c, w[p + "uv"]).view(T, H, V)
    gate = sigmoid(linear(h, w[p + "g"]))                                              # [T, H]
    pos = torch.as_tensor(positions)
    seen = pos[None, :] <= pos[:, None]
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for n in range(H):
        score = (q_plain[:, n] @ k_plain[:, n].T + q_rot[:, n] @ k_rot.T) * mixer["scale"]
        score = torch.where(seen, score, torch.full_like(score, -math.inf))
        weight = torch.exp(score - score.max(-1, keepdim=True).values)
        weight = weight / weight.sum(-1, keepdim=True)
        out[:, n] = (weight @ value[:, n]) * gate[:, n:n + 1]
    return linear(out.reshape(T, H * V), w[p + "o"])


# ---------------------------------------------------------------- routed feed-forward
def expert(h, gate_w, up_w, down_w, limit):
    g = torch.clamp(linear(h, gate_w), max=limit)
    u = torch.clamp(linear(h, up_w), -limit, limit)
    return linear(g * sigmoid(1.702 * g) * (u + 1.0), down_w)


def route(h, router_w, router_b, top):
    """(chosen experts [T, top], their weights [T, top]): the largest logits, softmax over them only."""
    z = linear(h, router_w) + router_b
    best = torch.topk(z, top, dim=-1)
    weight = torch.exp(best.values - best.values.max(-1, keepdim=True).values)
    return best.indices, weight / weight.sum(-1, keepdim=True)


def routed_experts(h, w, p, mlp):
    top, limit = mlp["router"]["top"], mlp["expert"]["limit"]
    chosen, weight = route(h, w[p + "router"], w[p + "router.b"], top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(chosen[t, j])
            q = f"{p}e{e}."
            out[t] += weight[t, j] * expert(h[t:t + 1], w[q + "gate"], w[q + "up"], w[q + "down"], limit)[0]
    return out


# ---------------------------------------------------------------- the model
def read_folder(folder, dtype=torch.float32):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            tensors[name] = t.to(dtype) if t.is_floating_point() else t
    return cfg, tensors


def layer(x, positions, cfg, w, i):
    spec = cfg["layers"][i]
    eps = cfg["norm"]["eps"]
    h = layer_norm(x, w[f"l{i}.norm1"], eps)
    if spec["type"] == "delta":
        mixed = delta_mixer(h, w, f"l{i}.mix.", spec["mixer"], eps)
    elif spec["type"] == "latent_attention":
        mixed = latent_attention_mixer(h, positions, w, f"l{i}.mix.", spec["mixer"], eps)
    else:
        raise ValueError(f"unknown layer type {spec['type']!r}")
    if spec.get("mlp") is not None:
        mixed = mixed + routed_experts(h, w, f"l{i}.mlp.", spec["mlp"])
    return x + cfg["residual_mult"] * mixed


def forward(cfg, w, tokens, rows=None, residuals=None):
    """Logits [T, vocab] (or at `rows`) of a whole sequence from position 0; `residuals`, a list,
    receives the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    positions = list(range(len(tokens)))
    x = layer_norm(w["embed"][torch.as_tensor(tokens, dtype=torch.long)], w["embed.norm"], eps)
    for i in range(len(cfg["layers"])):
        x = layer(x, positions, cfg, w, i)
        if residuals is not None:
            residuals.append(x.clone())
    if rows is not None:
        x = x[torch.as_tensor(rows, dtype=torch.long)]
    return linear(layer_norm(x, w["final.norm"], eps), w["embed"]) * cfg["logit_scale"]


def greedy(cfg, w, prompt, max_new):
    seq, out = list(prompt), []
    for _ in range(max_new):
        logits = forward(cfg, w, seq, rows=[len(seq) - 1])[0]
        tok = int(torch.argmax(logits))
        out.append(tok)
        seq.append(tok)
    return out
