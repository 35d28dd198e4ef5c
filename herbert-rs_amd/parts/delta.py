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
"""
import torch

from ..cache import StateNeed
from ..kernels import recurrent
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


@register("mixer", "gated_delta")
class GatedDelta(Part):
    graph_safe = True
    stores_fresh_rows = True     # its output projection stores into rows that hold nothing yet (StepContext.adds_to)

    def __init__(self, hidden_size, heads, kv_heads, dim, vdim, conv, eps, names, unit_eps=UNIT_EPS, shared=None):
        """names: q, k, v, q_conv, k_conv, v_conv, b, a, A_log, dt_bias, g, norm, o -> tensor names.
        conv: the taps of the convolution (1: none). eps: of the norm a head."""
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

    def tensor_needs(self):
        n, W = self.names, self.hidden_size
        qk, v = self.kv_heads * self.dim, self.heads * self.vdim
        return {n["q"]: TensorNeed((qk, W)), n["k"]: TensorNeed((qk, W)), n["v"]: TensorNeed((v, W)),
                n["q_conv"]: TensorNeed((qk, self.taps), "taps", _taps_init),
                n["k_conv"]: TensorNeed((qk, self.taps), "taps", _taps_init),
                n["v_conv"]: TensorNeed((v, self.taps), "taps", _taps_init),
                n["b"]: TensorNeed((self.heads, W)), n["a"]: TensorNeed((self.heads, W)),
                n["A_log"]: TensorNeed((self.heads,), "rate", _rate_init),
                n["dt_bias"]: TensorNeed((self.heads,), "rate", _rate_init),
                n["g"]: TensorNeed((v, W)), n["norm"]: TensorNeed((self.vdim,), "scale"),
                n["o"]: TensorNeed((W, v))}

    def cache_need(self):
        needs = [StateNeed((self.heads, self.dim, self.vdim), torch.float32)]
        if self.taps > 1:
            needs.append(StateNeed((self.taps - 1, self.channels), torch.float32))
        return tuple(needs)

    def load(self, tensors, rt):
        n = self.names
        # one projection [q | k | v | g | b | a]: the rows are read once; its float32 sums feed the
        # convolution, the gate and the recurrence's two scalars a head
        rows = [tensors[n[k]].to(rt.device) for k in ("q", "k", "v", "g", "b", "a")]
        self.proj = Linear(rt.weight(torch.cat(rows, 0)), scratch=rt.scratch)
        C, V = self.channels, self.heads * self.vdim
        self.g_off, self.b_off, self.a_off = C, C + V, C + V + self.heads
        self.width = C + V + 2 * self.heads
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
        recurrent.gated_delta(qkv, proj, self.b_off, self.a_off, self.a_log, self.dt_bias, state, ctx.meta, o,
                              self.kv_heads, self.heads, self.dim, self.vdim)
        gated = rt.buffer("delta_gated", (T, self.heads * self.vdim))
        recurrent.gated_head_norm(o, proj, self.g_off, self.norm_w, gated, self.heads, self.vdim, self.eps)
        adds = ctx.adds_to(x)
        left = ctx.leave_norm(self.o, x) if adds else None
        self.o.forward(gated, x, accumulate=adds, leave=None if left is None else left.leave())
