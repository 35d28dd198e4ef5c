"""Modasun as data: which parts each layer has and what its tensors are called.

A layer is the "postnorm" arrangement: x <- norm1(alpha x + mixer(x)), x <- norm2(alpha x + ff(x)), the norms
RMS norms whose stored weights are offsets from one. The mixer is a softmax attention without a rotation
("attention": queries and keys divided by their root mean square a head, a query growing with the logarithm
of its position, values of a size of their own) or a gated delta rule with a decay a key channel
("channel_delta": two-step projections for the decay and the sigmoid gate); the feed-forward is dense
(squared relu), a mixture of experts chosen by sigmoid scores within the best groups beside a gated shared
expert, or absent. A layer with `weights_of` is a second run of that layer's parts in the schedule, with a
cache entry of its own. The embedding's rows are scaled; the logits are the table itself times the normed
last rows. Tensors are stored under short names: `l<i>.norm1`, `l<i>.norm2`, `l<i>.mix.<name>`,
`l<i>.mlp.<name>`, `embed`, `final.norm`.
"""
from ..config import register_architecture
from ..config.modasun import DenseConfig, ModasunConfig
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def _attention(cfg, m, p):
    names = {k: p + k for k in ("q", "k", "v", "o")}
    return PartSpec("attention", {"hidden_size": cfg.hidden_size, "num_heads": m.heads, "num_kv_heads": m.kv_heads,
                                  "head_dim": m.dim, "value_dim": m.vdim, "eps": cfg.norm_eps,
                                  "position": PartSpec("none"), "names": names, "qk_norm": "plain",
                                  "scale": m.scale, "q_temp": (m.q_temp_coef, m.q_temp_every)})


def _channel_delta(cfg, m, p):
    names = {k: p + k for k in ("q", "k", "v", "b", "a1", "a2", "A_log", "dt_bias", "g1", "g2", "norm", "o")}
    names.update(q_conv=p + "q.conv", k_conv=p + "k.conv", v_conv=p + "v.conv")
    return PartSpec("gated_delta", {"hidden_size": cfg.hidden_size, "heads": m.heads, "kv_heads": m.kv_heads,
                                    "dim": m.dim, "vdim": m.vdim, "conv": m.conv, "eps": cfg.norm_eps, "names": names,
                                    "decay": "channel", "low_rank": (m.decay_rank, m.gate_rank), "gate": "sigmoid"})


MIXER_SPECS = {"attention": _attention, "channel_delta": _channel_delta}


def _feed_forward(cfg, m, p):
    if isinstance(m, DenseConfig):
        return PartSpec("squared_relu", {"hidden_size": cfg.hidden_size, "intermediate_size": m.ff,
                                         "names": {"up": p + "up", "down": p + "down"}})
    names = {"router": p + "router", "router_bias": p + "correction", "gate": p + "e{e}.gate", "up": p + "e{e}.up",
             "down": p + "e{e}.down"}
    shared = None
    if m.shared_ff is not None:
        shared = {"intermediate_size": m.shared_ff, "names": {k: p + "shared." + k for k in ("gate", "up", "down", "sg")}}
    return PartSpec("routed_experts", {"hidden_size": cfg.hidden_size, "intermediate_size": m.ff,
                                       "experts": m.experts, "top": m.top, "names": names, "routing": "scores",
                                       "groups": m.groups, "keep": m.keep, "activation": "silu",
                                       "shared_expert": shared})


def _norm(cfg, weight):
    return PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.norm_eps, "weight": weight, "offset": 1.0})


def build_spec(cfg):
    layers, spec_of = [], {}
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue
        mixer = MIXER_SPECS[layer.type](cfg, layer.mixer, f"l{i}.mix.")
        norms = {"post_mixer": _norm(cfg, f"l{i}.norm1")}
        ffn = None
        if layer.mlp is not None:
            ffn = _feed_forward(cfg, layer.mlp, f"l{i}.mlp.")
            norms["post_ff"] = _norm(cfg, f"l{i}.norm2")
        spec_of[i] = len(layers)
        layers.append(LayerSpec(PartSpec("postnorm", {"alpha": cfg.postln_alpha}), mixer, ffn, norms))
    # every listed layer is one run of the schedule, with a cache entry of its own, whoever's tensors it runs
    schedule = [ScheduleEntry(spec_of[i if layer.weights_of is None else layer.weights_of])
                for i, layer in enumerate(cfg.layers)]
    return ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size, max_positions=cfg.max_position_embeddings,
        embedding=PartSpec("table", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size, "weight": "embed",
                                     "scale": cfg.embedding_scale}),
        layers=layers, schedule=schedule,
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size, "weight": "embed",
                                 "tied_to_embedding": True}),
        eos_token_id=cfg.eos_token_id)


ARCHITECTURE = register_architecture("Modasun", ModasunConfig, build_spec, model_types=("modasun",))
