"""A feed-forward of routed experts: every token goes through the ``top`` experts with the
largest router logits, weighted by the softmax over those logits only, plus an optional shared
expert that every token takes.  An expert is the gated feed-forward down(silu(gate x) * up x)
without biases.  Router logits are float32 sums.

The experts' matrices are stacked at load ([experts, 2 ff, width] with an expert's gate rows
before its up rows, and [experts, width, ff]); the kernel table sorts the step's (token,
choice) pairs by expert on the device and runs one grouped product over all experts, so a step
is a fixed list of launches whatever the routing.
"""
import torch

from .base import FeedForward, ParamSpec
from .feedforward import GatedMLP


class RoutedExperts(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size, experts, top, ff, shared_ff=0, names=None):
        if not 1 <= top <= experts:
            raise ValueError("top must be between 1 and the number of experts")
        self.hidden_size, self.experts, self.top, self.ff = int(hidden_size), int(experts), int(top), int(ff)
        self.names = dict({"router": "router", "expert": "e{}.", "shared": "shared.",
                           "gate": "gate", "up": "up", "down": "down"}, **(names or {}))
        n = self.names
        self.shared = GatedMLP(hidden_size, shared_ff, names=(n["gate"], n["up"], n["down"])) \
            if shared_ff else None

    def param_specs(self):
        n, h, f = self.names, self.hidden_size, self.ff
        specs = {}
        for e in range(self.experts):
            p = n["expert"].format(e)
            specs[p + n["gate"]] = ParamSpec((f, h))
            specs[p + n["up"]] = ParamSpec((f, h))
            specs[p + n["down"]] = ParamSpec((h, f))
        specs[n["router"]] = ParamSpec((self.experts, h))
        if self.shared is not None:
            for name, spec in self.shared.param_specs().items():
                specs[n["shared"] + name] = spec
        return specs

    def load(self, tensors, rt):
        from .base import prefixed
        self.rt = rt
        n = self.names
        router = tensors(n["router"])
        extra = -router.shape[0] % 8
        if extra:
            router = torch.cat([router, router.new_zeros(extra, router.shape[1])], 0)
        self.w_router = rt.linear_weight(router)
        gate_up, down = [], []
        for e in range(self.experts):
            p = n["expert"].format(e)
            gate_up.append(torch.cat([tensors(p + n["gate"]), tensors(p + n["up"])], 0))
            down.append(tensors(p + n["down"]))
        prepare = getattr(rt.ops, "prepare_expert_matrices", lambda w, gated=False: w)   # (the kernel table's layout)
        self.w_gate_up = prepare(rt.matrix(torch.stack(gate_up)), gated=True)            # [E, 2 ff, width]
        self.w_down = prepare(rt.matrix(torch.stack(down)))                 # [E, width, ff]
        if self.shared is not None:
            self.shared.load(prefixed(n["shared"], tensors), rt)

    def forward(self, x):
        ops = self.rt.ops
        logits = ops.linear(x, self.w_router, None, out_f32=True)
        routing = ops.route_tokens(logits, self.experts, self.top)
        base = ops.materialize(self.shared.forward(x)) if self.shared is not None else None
        return ops.routed_experts(x, routing, self.w_gate_up, self.w_down, base)
