"""A mixer with a matrix of state a head instead of keys and values: the gated delta rule.

From the normed rows h:  q = W_q h, k = W_k h (kv_heads x dim), v = W_v h (heads x vdim), each filtered
along time, channel by channel, over the token and the K - 1 tokens before it (taps [channels, K], column
K - 1 weighs the token itself; nothing precedes a sequence's first token) and then through silu; q and k then unit vectors a head
(x / sqrt(sum x^2 + 1e-6)), q times dim^-1/2. A head h (on q/k head h / (heads / kv_heads)) keeps
S [dim, vdim], zero at the start, and for every token
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
with beta = sigmoid(W_b h) and g = exp(-exp(A_log) softplus(W_a h + dt_bias)) a head. o is divided by
its root mean square over vdim, multiplied by a weight [vdim] that the heads share and by
silu(W_g h), and goes through W_o. The recurrence and everything that enters it but the
projections is float32 in either mode. What a sequence carries from step to step: S, and the last
K - 1 inputs of the convolution.

Variants, each a parameter: `decay="channel"`: g is a factor a head and key channel (it scales the rows
of S), g = exp(-exp(A_log[h]) softplus(a + dt_bias)) with a and dt_bias of size heads x dim; `low_rank`:
the decay's pre-activation a and the gate's are each two products, W_2 (W_1 h), through a narrow
middle (names a1, a2, g1, g2 in place of a, g); `gate="sigmoid"`: the output is gated by
sigmoid(.) instead of silu(.).
"""
import torch

from ..cache import StateNeed
from ..kernels import ops, recurrent
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register

UNIT_EPS = 1e-6


def _taps_init(shape, gen, device, std, norm_std):
    """Taps near an average of the window, so that a random model's convolution passes its input on."""
    return 1.0 / shape[1] + 0.3 * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


def _rate_init(shape, gen, device, std, norm_std):
    """log decay rates and step biases of a random model: around zero, so that decays lie well inside (0, 1)."""
    return 0.5 * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


def _second_init(shape, gen, device, std, norm_std):
    """The second of two products through a narrow middle: drawn so that the pair's output is about as
    large as one full-width product's with the model's deviation would be (the middle's entries are sums
    of `width` terms of deviation std each; 1 / sqrt(middle) brings their sum back to one entry's size)."""
    return torch.randn(shape, generator=gen, device=device, dtype=torch.float32) / shape[1] ** 0.5


@register("mixer", "gated_delta")
class GatedDelta(Part):
    graph_safe = True
    stores_fresh_rows = True     # its output projection stores into rows that hold nothing yet (StepContext.adds_to)

    def __init__(self, hidden_size, heads, kv_heads, dim, vdim, conv, eps, names, unit_eps=UNIT_EPS, shared=None,
                 decay="head", low_rank=None, gate="silu"):
        """names: q, k, v, q_conv, k_conv, v_conv, b, a, A_log, dt_bias, g, norm, o -> tensor names
        (with low_rank: a1, a2, g1, g2 in place of a and g).
        conv: the taps of the convolution (1: none). eps: of the norm a head. decay: "head" or "channel".
        low_rank: None, or (the middle's size of the decay, of the gate); None for one of them: read from
        the stored tensor's shape. gate: "silu" or "sigmoid"."""
        if decay not in ("head", "channel") or gate not in ("silu", "sigmoid"):
            raise ValueError(f"the delta rule's decay is 'head' or 'channel' and its gate 'silu' or 'sigmoid', "
                             f"not {decay!r} and {gate!r}")
        self.decay, self.gate = decay, gate
        self.low_rank = None if low_rank is None else tuple(low_rank)
        if heads % kv_heads:
            raise ValueError("heads must be divisible by kv_heads")
        self.hidden_size, self.heads, self.kv_heads = int(hidden_size), int(heads), int(kv_heads)
        self.dim, self.vdim, self.taps = int(dim), int(vdim), int(conv)
        self.eps, self.unit_eps = float(eps), float(unit_eps)
        self.names = dict(names)
        if not 1 <= self.taps <= recurrent.MAX_TAPS or not 0 < self.dim <= recurrent.MAX_KEY_DIM:
            raise ValueError(f"the delta rule's kernels take 1 to {recurrent.MAX_TAPS} taps and keys of up to "
                             f"{recurrent.MAX_KEY_DIM}, not {self.taps} and {self.dim}")
        self.proj = self.o = None

    @property
    def channels(self):
        """Channels that pass the convolution: queries, keys, values."""
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    @property
    def decay_width(self):
        """Pre-activations of the decay a token: one a head, or one a head and key channel."""
        return self.heads * (self.dim if self.decay == "channel" else 1)

    def tensor_needs(self):
        n, W = self.names, self.hidden_size
        qk, v = self.kv_heads * self.dim, self.heads * self.vdim
        needs = {n["q"]: TensorNeed((qk, W)), n["k"]: TensorNeed((qk, W)), n["v"]: TensorNeed((v, W)),
                 n["q_conv"]: TensorNeed((qk, self.taps), "taps", _taps_init),
                 n["k_conv"]: TensorNeed((qk, self.taps), "taps", _taps_init),
                 n["v_conv"]: TensorNeed((v, self.taps), "taps", _taps_init),
                 n["b"]: TensorNeed((self.heads, W)),
                 n["A_log"]: TensorNeed((self.heads,), "rate", _rate_init),
                 n["dt_bias"]: TensorNeed((self.decay_width,), "rate", _rate_init),
                 n["norm"]: TensorNeed((self.vdim,), "scale"),
                 n["o"]: TensorNeed((W, v))}
        if self.low_rank is None:
            needs[n["a"]] = TensorNeed((self.decay_width, W))
            needs[n["g"]] = TensorNeed((v, W))
        else:
            ra, rg = self.low_rank
            # (a middle's size that the configuration does not give is whatever the stored tensor has)
            needs[n["a1"]] = TensorNeed((ra, W))
            needs[n["a2"]] = TensorNeed((self.decay_width, ra), "matrix", _second_init)
            needs[n["g1"]] = TensorNeed((rg, W))
            needs[n["g2"]] = TensorNeed((v, rg), "matrix", _second_init)
        return needs

    def cache_need(self):
        needs = [StateNeed((self.heads, self.dim, self.vdim), torch.float32)]
        if self.taps > 1:
            needs.append(StateNeed((self.taps - 1, self.channels), torch.float32))
        return tuple(needs)

    def load(self, tensors, rt):
        n = self.names
        # one projection [q | k | v | g | b | a]: the rows are read once; its float32 sums feed the
        # convolution, the gate and the recurrence's two scalars a head (with low_rank, g and a are the
        # narrow middles, and a second product each widens them)
        first = ("q", "k", "v", "g", "b", "a") if self.low_rank is None else ("q", "k", "v", "g1", "b", "a1")
        rows = [tensors[n[k]].to(rt.device) for k in first]
        self.proj = Linear(rt.weight(torch.cat(rows, 0)), scratch=rt.scratch)
        C = self.channels
        g_width, a_width = rows[3].shape[0], rows[5].shape[0]
        self.g_off, self.b_off, self.a_off = C, C + g_width, C + g_width + self.heads
        self.width = C + g_width + self.heads + a_width
        self.g_width, self.a_width = g_width, a_width
        if self.low_rank is not None:
            self.a2, self.g2 = rt.weight(tensors[n["a2"]]), rt.weight(tensors[n["g2"]])
        self.conv_w = torch.cat([rt.weight(tensors[n[k]], matrix=False) for k in ("q_conv", "k_conv", "v_conv")], 0).contiguous()
        self.a_log = rt.weight(tensors[n["A_log"]], matrix=False)
        self.dt_bias = rt.weight(tensors[n["dt_bias"]], matrix=False)
        self.norm_w = rt.weight(tensors[n["norm"]], matrix=False)
        self.o = Linear(rt.weight(tensors[n["o"]]), scratch=rt.scratch)

    def forward(self, ctx, y, x):
        rt = ctx.rt
        T = y.shape[0]
        views = ctx.cache.state_views(ctx.cache_entry)
        state = views[0]
        proj = rt.buffer("delta_proj", (T, self.width), torch.float32)
        self.proj.forward(y, proj)
        qkv = rt.buffer("delta_qkv", (T, self.channels), torch.float32)
        conv_state = views[1] if self.taps > 1 else rt.buffer("delta_no_conv", (1, 1, self.channels), torch.float32)
        recurrent.conv_silu(proj, self.conv_w, conv_state, ctx.meta, qkv, 2 * self.kv_heads, self.dim, self.kv_heads,
                            self.dim ** -0.5, self.unit_eps, self.heads, self.vdim)
        o = rt.buffer("delta_o", (T, self.heads * self.vdim), torch.float32)
        gate_rows, gate_off, decay_rows, decay_off = proj, self.g_off, proj, self.a_off
        if self.low_rank is not None:
            # the second products, float32 sums of the float32 middles
            gate_rows, gate_off = rt.buffer("delta_gate", (T, self.heads * self.vdim), torch.float32), 0
            ops.gemm_plain_columns(proj, self.g_off, self.g_width, self.g2, gate_rows)
            decay_rows, decay_off = rt.buffer("delta_decay", (T, self.decay_width), torch.float32), 0
            # (a decay a channel leaves this product as the decay itself: softplus and exponentials where the sum is stored)
            ops.gemm_plain_columns(proj, self.a_off, self.a_width, self.a2, decay_rows,
                                   decay=(self.a_log, self.dt_bias, self.dim) if self.decay == "channel" else None)
        if self.decay == "channel":
            factors = decay_rows
            if self.low_rank is None:
                factors = rt.buffer("delta_decay", (T, self.decay_width), torch.float32)
                recurrent.channel_decay(decay_rows, decay_off, self.a_log, self.dt_bias, factors, self.heads, self.dim)
            recurrent.gated_delta(qkv, proj, self.b_off, 0, None, None, state, ctx.meta, o,
                                  self.kv_heads, self.heads, self.dim, self.vdim, decay=factors)
        else:
            recurrent.gated_delta(qkv, decay_rows, self.b_off, decay_off, self.a_log, self.dt_bias, state, ctx.meta, o,
                                  self.kv_heads, self.heads, self.dim, self.vdim)
        gated = rt.buffer("delta_gated", (T, self.heads * self.vdim))
        recurrent.gated_head_norm(o, gate_rows, gate_off, self.norm_w, gated, self.heads, self.vdim, self.eps,
                                  gate=self.gate)
        adds = ctx.adds_to(x)
        left = ctx.leave_norm(self.o, x) if adds else None
        self.o.forward(gated, x, accumulate=adds, leave=None if left is None else left.leave())
