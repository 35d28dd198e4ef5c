"""Small Vipalorn configurations for the tests, their model folders, and the plain logits.

The configurations differ from each other in every size and option: which mixer comes first, heads
that share keys or not, taps, a rotation over a part of the rotated entries only, a layer without a
feed-forward, one expert a token, constants that are neither 1 nor equal to each other.
"""
import json
import os

import numpy as np
import torch
from safetensors import safe_open
from safetensors.torch import save_file

import herbert_rs_amd as hb

from .plain import vipalorn as plain


def delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base=10000.0, dims=None):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "rot": {"base": base, "dims": rot_dim if dims is None else dims}}}


def moe(experts, top, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def model(vocab, width, layers, eps=1e-5, mult=1.0, logit_scale=1.0):
    return {"architecture": "Vipalorn", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
            "residual_mult": mult, "logit_scale": logit_scale}


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


# P: attention first, three heads on three key heads in the delta layer, four taps, a rotation over half of
#    the rotated entries, sizes that no kernel's blocks divide
VIP_P = model(200, 72, [
    with_mlp(latent(3, 24, 12, 20, 40, 0.3, base=5000.0, dims=6), moe(5, 2, 40, 1.5)),
    with_mlp(delta(3, 3, 24, 40, 4), moe(5, 2, 40, 1.5)),
    with_mlp(latent(3, 24, 12, 20, 40, 0.3, base=5000.0, dims=6), None),
], eps=3e-6, mult=0.7, logit_scale=1.3)
# Q: delta layers around one attention layer, six heads on two key heads, two taps, one expert a token, widths
#    in steps of 32 (the matrix-core products take them)
VIP_Q = model(384, 128, [
    with_mlp(delta(6, 2, 16, 32, 2), moe(8, 1, 64, 3.0)),
    with_mlp(latent(4, 32, 32, 48, 96, 0.125, base=1.0e6), moe(8, 3, 64, 3.0)),
    with_mlp(delta(6, 2, 16, 32, 2), moe(8, 3, 64, 3.0)),
], eps=1e-6, mult=0.4, logit_scale=0.25)
# R: one head each, no convolution, values wider than a wave, a latent without a rotated part's rest
VIP_R = model(96, 64, [
    with_mlp(delta(1, 1, 48, 80, 1), None),
    with_mlp(latent(1, 16, 8, 16, 24, 0.5, base=100.0), moe(3, 3, 24, 0.75)),
], eps=1e-5, mult=1.0, logit_scale=1.0)
# S: attention first and last around two delta layers, heads that share keys in pairs, three taps, a latent
#    row that is no multiple of 32 (the plain attention kernel in either mode), three of twelve experts
VIP_S = model(320, 192, [
    with_mlp(latent(6, 24, 8, 40, 72, 0.2, base=40000.0), moe(12, 3, 80, 2.5)),
    with_mlp(delta(4, 2, 40, 48, 3), moe(12, 3, 80, 2.5)),
    with_mlp(delta(4, 2, 40, 48, 3), moe(12, 3, 80, 2.5)),
    with_mlp(latent(6, 24, 8, 40, 72, 0.2, base=40000.0), moe(12, 3, 80, 2.5)),
], eps=2e-5, mult=0.6, logit_scale=0.75)
# W: the widths of a larger model's layers at a small depth: keys of 128 a head, a latent of 256 + 64
VIP_W = model(1024, 512, [
    with_mlp(delta(8, 4, 128, 128, 4), moe(16, 4, 256, 7.0)),
    with_mlp(latent(8, 64, 64, 64, 256, 0.09), moe(16, 4, 256, 7.0)),
], eps=1e-6, mult=0.5, logit_scale=0.5)

CONFIGS = {"S": (VIP_S, 15, 0.08), "P": (VIP_P, 11, 0.12), "Q": (VIP_Q, 12, 0.09), "R": (VIP_R, 13, 0.15), "W": (VIP_W, 14, 0.05)}


def make_folder(root, name, dtype="float32", scale=None, set_to=None, tag=""):
    """Write the random model `name` into root/<name>_<dtype><tag> once. `scale` {tensor name suffix: factor}
    multiplies tensors afterwards, `set_to` {suffix: value} fills them: to make a far key, a long memory
    or a saturated gate show where random weights would hide it."""
    raw, seed, std = CONFIGS[name]
    folder = os.path.join(str(root), f"vip_{name}_{dtype}{tag}")
    if os.path.exists(os.path.join(folder, "model.safetensors")):
        return folder
    hb.write_random_model(folder, raw, seed=seed, dtype=dtype, std=std, norm_std=0.1)
    if scale or set_to:
        path = os.path.join(folder, "model.safetensors")
        tensors = {}
        with safe_open(path, framework="pt") as f:
            for k in f.keys():
                tensors[k] = f.get_tensor(k)
        for k in tensors:
            for suffix, factor in (scale or {}).items():
                if k.endswith(suffix):
                    tensors[k] = (tensors[k].float() * factor).to(tensors[k].dtype)
            for suffix, value in (set_to or {}).items():
                if k.endswith(suffix):
                    tensors[k] = torch.full_like(tensors[k], value)
        save_file(tensors, path)
    return folder


_folders, _logits = {}, {}


def plain_folder(folder):
    if folder not in _folders:
        _folders[folder] = plain.read_folder(folder, torch.float32)
    return _folders[folder]


def plain_logits(folder, tokens):
    """float32 [len(tokens), vocab] of the plain whole-sequence implementation, computed once."""
    key = (folder, tuple(tokens))
    if key not in _logits:
        cfg, w = plain_folder(folder)
        _logits[key] = plain.forward(cfg, w, list(tokens)).numpy().astype(np.float32)
    return _logits[key]


def random_tokens(vocab, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
