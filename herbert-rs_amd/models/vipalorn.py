"""Vipalorn as data: which parts each layer has and what its tensors are called.

A layer is the "parallel" arrangement: one layer norm (a weight, no bias), a mixer and a
feed-forward of routed experts that both read it, their sum times `residual_mult` joining the
residual stream. The mixer is a gated delta rule ("delta") or an attention over one shared latent a
token ("latent_attention"), layer by layer as the configuration lists them. The embedding's rows
pass a layer norm before they are the residual stream; the logits are the embedding table times the
normed last rows, times `logit_scale`. Tensors are stored under short names: `l<i>.norm1`,
`l<i>.mix.<name>`, `l<i>.mlp.<name>`, `embed`, `embed.norm`, `final.norm`.
"""
from ..config import register_architecture
from ..config.vipalorn import VipalornConfig
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def _delta(cfg, m, p):
    names = {k: p + k for k in ("q", "k", "v", "b", "a", "A_log", "dt_bias", "g", "norm", "o")}
    names.update(q_conv=p + "q.conv", k_conv=p + "k.conv", v_conv=p + "v.conv")
    return PartSpec("gated_delta", {"hidden_size": cfg.hidden_size, "heads": m.heads, "kv_heads": m.kv_heads,
                                    "dim": m.dim, "vdim": m.vdim, "conv": m.conv, "eps": cfg.norm_eps, "names": names})


def _latent(cfg, m, p):
    # the rotation's angles are computed from the positions, so no table bounds them
    position = PartSpec("rope", {"theta": m.rot_base, "rotary_dims": m.rot_dims,
                                 "max_positions": cfg.max_position_embeddings, "tables": False})
    names = {"q": p + "q", "dkv": p + "dkv", "dkv_norm": p + "dkv.norm", "uk": p + "uk", "uv": p + "uv",
             "g": p + "g", "o": p + "o"}
    return PartSpec("latent_attention", {"hidden_size": cfg.hidden_size, "heads": m.heads, "dim": m.dim,
                                         "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank,
                                         "scale": m.scale, "eps": cfg.norm_eps, "position": position, "names": names})


MIXER_SPECS = {"delta": _delta, "latent_attention": _latent}


def _experts(cfg, m, p):
    names = {"router": p + "router", "router_bias": p + "router.b", "gate": p + "e{e}.gate", "up": p + "e{e}.up",
             "down": p + "e{e}.down"}
    return PartSpec("routed_experts", {"hidden_size": cfg.hidden_size, "intermediate_size": m.ff,
                                       "experts": m.experts, "top": m.top, "limit": m.limit, "names": names})


def _norm(cfg, weight):
    return PartSpec("layernorm", {"size": cfg.hidden_size, "eps": cfg.norm_eps, "weight": weight})


def build_spec(cfg):
    layers = []
    for i, layer in enumerate(cfg.layers):
        mixer = MIXER_SPECS[layer.type](cfg, layer.mixer, f"l{i}.mix.")
        ffn = None if layer.mlp is None else _experts(cfg, layer.mlp, f"l{i}.mlp.")
        layers.append(LayerSpec(PartSpec("parallel", {"mult": cfg.residual_mult}), mixer, ffn,
                                {"input": _norm(cfg, f"l{i}.norm1")}))
    return ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size, max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("table", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size, "weight": "embed",
                                     "norm": _norm(cfg, "embed.norm")}),
        layers=layers, schedule=[ScheduleEntry(i) for i in range(len(layers))],
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size, "weight": "embed",
                                 "tied_to_embedding": True, "logit_scale": cfg.logit_scale}),
        eos_token_id=cfg.eos_token_id)


ARCHITECTURE = register_architecture("Vipalorn", VipalornConfig, build_spec, model_types=("vipalorn",))
