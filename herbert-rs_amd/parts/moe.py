"""A feed-forward of many small experts, of which each token uses a few.

Router: z = W_r y + b in float32. A token goes to the `top` experts whose z is largest, and weighs them by
exp(z) normalised over those experts alone (not over all of them). An expert: g = min(W_gate y, limit), u = clamp(W_up y, -limit,
limit), out = W_down (g sigmoid(alpha g) (u + 1)), no biases. The part's output is the weighted sum
of the chosen experts' outputs. The routing never reaches the host: the (token, expert) pairs are put
in the order of their experts on the GPU and the experts' products run over a list of row tiles of
fixed length, so a step's grid depends on its size only.
"""
import torch

from ..kernels import moe, ops
from ..weights import TensorNeed
from .base import Part
from .linear import Linear
from .registry import register

GATE_ALPHA = 1.702


def _bias_init(shape, gen, device, std, norm_std):
    return 0.1 * torch.randn(shape, generator=gen, device=device, dtype=torch.float32)


@register("feed_forward", "routed_experts")
class RoutedExperts(Part):
    graph_safe = True

    def __init__(self, hidden_size, intermediate_size, experts, top, limit, names, alpha=GATE_ALPHA, shared=None):
        """names: router, router_bias (None: none), and gate, up, down as patterns with {e} for the
        expert's number."""
        self.hidden_size, self.inter = int(hidden_size), int(intermediate_size)
        self.experts, self.top = int(experts), int(top)
        self.limit, self.alpha = float(limit), float(alpha)
        self.names = dict(names)
        if not 0 < self.top <= self.experts or self.experts > moe.MAX_EXPERTS:
            raise ValueError(f"{self.top} of {self.experts} experts (the router takes up to {moe.MAX_EXPERTS})")

    def tensor_needs(self):
        n, W, F = self.names, self.hidden_size, self.inter
        needs = {n["router"]: TensorNeed((self.experts, W))}
        if n.get("router_bias"):
            needs[n["router_bias"]] = TensorNeed((self.experts,), "bias", _bias_init)
        for e in range(self.experts):
            needs[n["gate"].format(e=e)] = TensorNeed((F, W))
            needs[n["up"].format(e=e)] = TensorNeed((F, W))
            needs[n["down"].format(e=e)] = TensorNeed((W, F))
        return needs

    def load(self, tensors, rt):
        n = self.names
        self.router = Linear(rt.weight(tensors[n["router"]]), scratch=rt.scratch)
        self.router_bias = rt.weight(tensors[n["router_bias"]], matrix=False) if n.get("router_bias") else None
        # [E, 2 F, W]: an expert's gate rows, then its up rows; [E, W, F]
        self.gate_up = torch.stack([torch.cat([rt.weight(tensors[n["gate"].format(e=e)]),
                                               rt.weight(tensors[n["up"].format(e=e)])], 0)
                                    for e in range(self.experts)]).contiguous()
        self.down = torch.stack([rt.weight(tensors[n["down"].format(e=e)]) for e in range(self.experts)]).contiguous()
        # bfloat16 with sizes the matrix cores take: the matrices are kept in their operands' order
        W, F = self.hidden_size, self.inter
        self.cores = (rt.dtype == torch.bfloat16 and moe.mfma_takes(W, W, 0, 2 * F) and moe.mfma_takes(F, F, 0, W)
                      and F % 16 == 0)
        if self.cores:
            self.gate_up, self.down = moe.pack_grouped(self.gate_up), moe.pack_grouped(self.down)

    def forward(self, ctx, y, x):
        rt = ctx.rt
        T, E, top, F = y.shape[0], self.experts, self.top, self.inter
        logits = rt.buffer("moe_logits", (T, E), torch.float32)
        self.router.forward(y, logits)          # float32 sums of the rows' products with the router's matrix
        routing = moe.Routing(rt.buffer("moe_ints", (moe.Routing.ints_needed(T, E, top),), torch.int32),
                              rt.buffer("moe_weight", (T, top), torch.float32), T, E, top)
        moe.route(logits, self.router_bias, routing)
        act = rt.buffer("moe_act", (T * top, F))
        out = rt.buffer("moe_out", (T * top, self.hidden_size), torch.float32)
        if self.cores:
            # matrix cores; the activation is the first product's epilogue
            moe.grouped_mfma(y, self.hidden_size, 0, self.gate_up, act, F, 0, moe.EPI_GLU, routing, gather=True,
                             limit=self.limit, alpha=self.alpha)
            moe.grouped_mfma(act, F, 0, self.down, out, self.hidden_size, 0, moe.EPI_F32, routing)
        else:
            gu = rt.buffer("moe_gate_up", (T * top, 2 * F), torch.float32)
            moe.gemm_plain(y, self.gate_up, gu, routing, gather=True)
            moe.activate(gu, act, self.limit, self.alpha)
            moe.gemm_plain(act, self.down, out, routing, gather=False)
        moe.combine(out, routing, x)
