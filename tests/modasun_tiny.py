"""Small Modasun configurations for the tests, their model folders, and the plain logits.

The configurations differ from each other in every size and option: which mixer comes first, keys and
values of different sizes, heads that share keys or not, taps (also none), groups of one expert, every
expert chosen, a layer without a feed-forward, layers that run another layer's weights (an attention's
and a delta rule's), constants that are neither 1 nor equal to each other, and one where they are 1.
"""
import os

import numpy as np
import torch
from safetensors import safe_open
from safetensors.torch import save_file

import herbert_rs_amd as hb

from .plain import modasun as plain


def attention(heads, kv_heads, dim, vdim, scale, coef, every):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                                           "q_temp": {"coef": coef, "every": every}}}


def delta(heads, kv_heads, dim, vdim, conv, decay_rank, gate_rank):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                                               "low_rank": {"decay": decay_rank, "gate": gate_rank}}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, groups, keep, ff, shared_ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}},
            "shared": {"ff": shared_ff}}


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


def again(layers, source):
    """A further run of layer `source`'s weights."""
    return dict(layers[source], weights_of=source)


def model(vocab, width, layers, eps=1e-5, alpha=1.0, embed_scale=1.0):
    return {"architecture": "Modasun", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
            "postln_alpha": alpha, "embedding": {"scale": embed_scale}}


def _p():
    # P: the delta rule first, keys of 24 and values of 40 in both mixers, six heads on two key heads, four
    #    taps, three of six experts out of two of three groups, a layer without a feed-forward, a second run
    #    of the delta layer, sizes that no kernel's blocks divide
    layers = [with_mlp(delta(4, 2, 24, 40, 4, 10, 7), moe(6, 3, 3, 2, 40, 24)),
              with_mlp(attention(6, 2, 24, 40, 0.3, 0.5, 16), dense(100)),
              with_mlp(attention(6, 2, 24, 40, 0.3, 0.5, 16), None)]
    layers.append(again(layers, 0))
    return model(200, 72, layers, eps=3e-6, alpha=1.7, embed_scale=5.0)


def _q():
    # Q: sizes that the matrix cores take as they are (heads of 64, widths in steps of 32), constants that are 1,
    #    two taps, two of eight experts out of two of four groups, three runs of one attention layer
    layers = [with_mlp(attention(4, 2, 64, 64, 0.125, 0.2, 32), moe(8, 2, 4, 2, 64, 32)),
              with_mlp(delta(6, 2, 32, 32, 2, 32, 32), dense(256))]
    layers += [again(layers, 0), again(layers, 0)]
    return model(384, 128, layers, eps=1e-6, alpha=1.0, embed_scale=1.0)


def _r():
    # R: one head each, no convolution, values wider than a wave, keys of 48 (the matrix cores run them at
    #    128 with the values), groups of one expert, every expert chosen
    return model(96, 64, [with_mlp(delta(1, 1, 48, 80, 1, 5, 3), moe(3, 3, 3, 3, 24, 16)),
                          with_mlp(attention(1, 1, 48, 80, 0.06, 1.0, 1), moe(3, 3, 3, 3, 24, 16))],
                 eps=1e-5, alpha=0.8, embed_scale=3.0)


def _s():
    # S: heads beyond 128 (the plain attention kernel in either mode), a query that grows at every position,
    #    four of twelve experts in one group, heads that share keys in pairs, three taps, a second run of a
    #    delta layer between two attention layers
    layers = [with_mlp(attention(2, 1, 160, 144, 0.08, 0.3, 1), moe(12, 4, 1, 1, 80, 48)),
              with_mlp(delta(4, 2, 40, 48, 3, 12, 20), moe(12, 4, 1, 1, 80, 48))]
    layers += [again(layers, 1), with_mlp(attention(6, 3, 32, 16, 0.2, 0.1, 50), dense(96))]
    return model(320, 192, layers, eps=2e-5, alpha=2.25, embed_scale=9.0)


def _n():
    # N: the sections that a configuration may leave out: an attention whose queries do not grow, routers
    #    without groups, feed-forwards without a shared expert (one of the two routed layers keeps its own)
    bare = {"kind": "moe", "expert": {"ff": 48}, "router": {"experts": 5, "top": 2}}
    plain_attention = {"type": "attention", "mixer": {"heads": 3, "kv_heads": 3, "dim": 32, "vdim": 48, "scale": 0.25}}
    grouped = {"kind": "moe", "expert": {"ff": 32}, "router": {"experts": 6, "top": 2, "groups": {"count": 2, "keep": 1}}}
    layers = [with_mlp(plain_attention, bare), with_mlp(delta(2, 2, 32, 48, 3, 8, 8), grouped),
              with_mlp(attention(3, 1, 32, 48, 0.2, 0.4, 8), dict(bare, shared={"ff": 40}))]
    layers.append(again(layers, 0))
    return model(160, 96, layers, eps=4e-6, alpha=1.3, embed_scale=4.0)


def _w():
    # W: the widths of a larger model's layers at a small depth: heads of 128, sixteen experts
    return model(1024, 512, [with_mlp(attention(8, 2, 128, 128, 0.09, 0.25, 128), moe(16, 4, 4, 2, 256, 256)),
                             with_mlp(delta(8, 4, 128, 128, 4, 64, 64), moe(16, 4, 4, 2, 256, 256))],
                 eps=1e-6, alpha=2.0, embed_scale=12.0)


def _f():
    # F: for keys far back and long memories: sharper scores than a random model's, every expert chosen (no
    #    choice that rounding could turn), a second run of the attention layer
    layers = [with_mlp(attention(4, 2, 64, 64, 0.4, 0.2, 32), moe(4, 4, 2, 2, 64, 32)),
              with_mlp(delta(4, 2, 32, 32, 2, 16, 16), dense(256))]
    layers.append(again(layers, 0))
    return model(384, 128, layers, eps=1e-6, alpha=1.5, embed_scale=2.0)


CONFIGS = {"F": (_f(), 26, 0.09), "P": (_p(), 21, 0.12), "Q": (_q(), 22, 0.09), "R": (_r(), 23, 0.15), "S": (_s(), 24, 0.08), "N": (_n(), 27, 0.1), "W": (_w(), 25, 0.05)}


def make_folder(root, name, dtype="float32", scale=None, set_to=None, tag=""):
    """Write the random model `name` into root/<name>_<dtype><tag> once. `scale` {tensor name suffix: factor}
    multiplies tensors afterwards, `set_to` {suffix: value} fills them: to make a far key, a long memory
    or a group's edge show where random weights would hide it."""
    raw, seed, std = CONFIGS[name]
    folder = os.path.join(str(root), f"mod_{name}_{dtype}{tag}")
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
        _folders[folder] = plain.load_folder(folder)
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
