"""Feed-forwards: dense (gated or not) and routed."""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from .base import ParamSource, Part, PendingProduct, PendingScale, as_tensor, place, register_part
from .linear import LINEAR_LIBRARIES, decode_copy, linear


@register_part("feed_forward", "swiglu")
class SwiGLU(Part):
    """down(silu(gate(x)) * up(x)), three matrices without bias
    (lite_llama/models/llama.py:107-120, lite_llama/kernels/swiglu.py:44-67).
    gate and up are concatenated at load into one [2I, hidden] matrix (rows
    gate | up) so that one product feeds the SiLU-multiply kernel."""
    kernel_libraries = ("activation", "norm") + LINEAR_LIBRARIES
    takes_pending_scale = True
    can_defer_output = True

    def __init__(self, hidden_size: int, intermediate_size: int,
                 gate_name: str = "gate_proj.weight", up_name: str = "up_proj.weight",
                 down_name: str = "down_proj.weight"):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.names = (gate_name, up_name, down_name)
        self.gate_up: Optional[torch.Tensor] = None
        self.down: Optional[torch.Tensor] = None
        self.gate_up_blocked: Optional[torch.Tensor] = None      # decode copies (make_decode_copies)
        self.down_blocked: Optional[torch.Tensor] = None

    def param_sources(self) -> List[ParamSource]:
        g, u, d = self.names
        return [ParamSource(g, (self.intermediate_size, self.hidden_size)),
                ParamSource(u, (self.intermediate_size, self.hidden_size)),
                ParamSource(d, (self.hidden_size, self.intermediate_size))]

    def load(self, tensors, dtype, device) -> None:
        g, u, d = self.names
        self.gate_up = place(torch.cat([tensors[g], tensors[u]], dim=0), "matrix", dtype, device)
        self.down = place(tensors[d], "matrix", dtype, device)

    def make_decode_copies(self) -> int:
        self.gate_up_blocked, self.down_blocked = decode_copy(self.gate_up), decode_copy(self.down)
        return sum(t.numel() * t.element_size() for t in (self.gate_up_blocked, self.down_blocked)
                   if t is not None)

    def forward(self, x, defer_output: bool = False):
        scale = None
        if isinstance(x, PendingScale) and ops.gate_up_silu_fits(x.values, self.gate_up):
            x, scale = x.values, x.scale
        x = as_tensor(x)
        if ops.gate_up_silu_fits(x, self.gate_up, self.gate_up_blocked):
            # the few rows of a decode step: product and SiLU-multiply in one kernel
            a = ops.gate_up_silu(x, self.gate_up, scale, blocked=self.gate_up_blocked)
            if defer_output:
                return PendingProduct(a, self.down, self.down_blocked)
            return linear(a, self.down, blocked=self.down_blocked)
        a = ops.silu_mul(linear(x, self.gate_up, blocked=self.gate_up_blocked))
        if defer_output:                    # (the norm that follows picks the kernels by the rows)
            return PendingProduct(a, self.down, self.down_blocked)
        return linear(a, self.down, blocked=self.down_blocked)


@register_part("feed_forward", "gated_mlp")
class GatedMLP(Part):
    """down(act(gate(x), up(x))) with the activation as a parameter: "silu" (silu(g) * u) or
    "clamped" (g' = min(g, limit), u' = clamp(u, -limit, limit), g' * sigmoid(1.702 g') * (u' + 1)).
    No biases. gate and up are one [2I, hidden] matrix at run time."""
    kernel_libraries = ("moe",) + LINEAR_LIBRARIES

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu",
                 limit: float = 0.0, gate_name: str = "gate", up_name: str = "up", down_name: str = "down"):
        if activation not in ("silu", "clamped"):
            raise ValueError(f"unknown gated activation {activation!r}")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.act = ops.ACT_CLAMPED if activation == "clamped" else ops.ACT_SILU
        self.limit = float(limit)
        self.names = (gate_name, up_name, down_name)
        self.gate_up = self.down = self.gate_up_blocked = self.down_blocked = None

    def param_sources(self) -> List[ParamSource]:
        g, u, d = self.names
        return [ParamSource(g, (self.intermediate_size, self.hidden_size)),
                ParamSource(u, (self.intermediate_size, self.hidden_size)),
                ParamSource(d, (self.hidden_size, self.intermediate_size))]

    def load(self, tensors, dtype, device) -> None:
        g, u, d = self.names
        self.gate_up = place(torch.cat([tensors[g], tensors[u]], dim=0), "matrix", dtype, device)
        self.down = place(tensors[d], "matrix", dtype, device)

    def make_decode_copies(self) -> int:
        self.gate_up_blocked, self.down_blocked = decode_copy(self.gate_up), decode_copy(self.down)
        return sum(t.numel() * t.element_size() for t in (self.gate_up_blocked, self.down_blocked)
                   if t is not None)

    def forward(self, x):
        x = as_tensor(x)
        a = ops.gated_act(linear(x, self.gate_up, blocked=self.gate_up_blocked), self.act, self.limit)
        return linear(a, self.down, blocked=self.down_blocked)


@register_part("feed_forward", "mlp")
class PlainMLP(Part):
    """down(act(up(x))), two matrices without bias and no gate; ``activation`` "relu2": the square
    of relu."""
    kernel_libraries = ("moe",) + LINEAR_LIBRARIES

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "relu2",
                 up_name: str = "up", down_name: str = "down"):
        if activation != "relu2":
            raise ValueError(f"unknown activation {activation!r} (known: 'relu2')")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.act = ops.ACT_RELU2
        self.names = (up_name, down_name)
        self.up = self.down = self.up_blocked = self.down_blocked = None

    def param_sources(self) -> List[ParamSource]:
        u, d = self.names
        return [ParamSource(u, (self.intermediate_size, self.hidden_size)),
                ParamSource(d, (self.hidden_size, self.intermediate_size))]

    def load(self, tensors, dtype, device) -> None:
        u, d = self.names
        self.up = place(tensors[u], "matrix", dtype, device)
        self.down = place(tensors[d], "matrix", dtype, device)

    def make_decode_copies(self) -> int:
        self.up_blocked, self.down_blocked = decode_copy(self.up), decode_copy(self.down)
        return sum(t.numel() * t.element_size() for t in (self.up_blocked, self.down_blocked) if t is not None)

    def forward(self, x):
        x = as_tensor(x)
        a = ops.unary_act(linear(x, self.up, blocked=self.up_blocked), self.act)
        return linear(a, self.down, blocked=self.down_blocked)


@register_part("feed_forward", "routed_experts")
class RoutedExperts(Part):
    """A mixture of feed-forward experts: router logits z = W_r x in float32 (from the rounded x
    and W_r of the engine's dtype, summed in float32), scores sigmoid(z) or, with ``score``
    "softmax", the softmax of z over all router outputs; the ``top`` outputs with the largest
    scores are taken (with ``correction_name``: the largest score + a per-output vector of the
    checkpoint; the weights stay the scores without it); their scores are the weights
    (``renormalize``: divided by their sum + renorm_eps; then times route_scale).
    ``weight_on_input``: the weight multiplies what the expert reads, y = sum_k expert_k(s_k x),
    instead of what it returns. Experts are gated, down(act(gate(x), up(x))) with ``activation``
    "silu" or "clamped", or, with "relu2", down(relu(up(x))^2) without a gate. ``identity``: that
    many router outputs behind the experts' have no tensors; their expert returns its input.
    ``groups`` = (count, keep): the router outputs form ``count`` equal groups of neighbours; a
    group's score is the sum of its two largest choice scores (score + correction), and only
    outputs of the ``keep`` best groups can be chosen (the others count as minus infinity).
    ``shared``: a dense feed-forward that every token runs, added times sigmoid(w_sg . x) when
    ``shared_gate``. The result is float32 (the sum over a token's experts is made there).
    Nothing comes back to the host: routing, the grouping of tokens by expert and the experts'
    products are kernels of csrc/moe.hip.

    Checkpoint tensors: ``router`` [E + identity, hidden], ``e<i>.gate|up|down`` (no gate for
    "relu2"), and for the shared expert ``shared.*`` and ``shared.sg`` [1, hidden] (names are
    parameters)."""
    kernel_libraries = ("moe",) + LINEAR_LIBRARIES

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, top: int,
                 activation: str = "clamped", limit: float = 0.0, weight_on_input: bool = True,
                 renormalize: bool = False, shared: Optional[Part] = None, shared_gate: bool = True,
                 score: str = "sigmoid", correction_name: Optional[str] = None, identity: int = 0,
                 renorm_eps: float = 0.0, route_scale: float = 1.0, groups=None,
                 router_name: str = "router", expert_prefix: str = "e", shared_prefix: str = "shared.",
                 shared_gate_name: str = "shared.sg", gate_name: str = "gate", up_name: str = "up",
                 down_name: str = "down"):
        if identity < 0 or not 0 < top <= num_experts + identity:
            raise ValueError(f"{top} of {num_experts} + {identity} experts")
        if activation not in ("silu", "clamped", "relu2"):
            raise ValueError(f"unknown expert activation {activation!r}")
        if score not in ("sigmoid", "softmax"):
            raise ValueError(f"unknown router score {score!r} (known: 'sigmoid', 'softmax')")
        if identity and weight_on_input:
            raise ValueError("experts that return their input take their weight on the output")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.num_experts, self.top, self.identity = int(num_experts), int(top), int(identity)
        self.act = {"silu": ops.ACT_SILU, "clamped": ops.ACT_CLAMPED, "relu2": ops.ACT_RELU2}[activation]
        self.gated = activation != "relu2"
        self.limit = float(limit)
        self.weight_on_input, self.renormalize = bool(weight_on_input), bool(renormalize)
        self.score = ops.SCORE_SOFTMAX if score == "softmax" else ops.SCORE_SIGMOID
        self.renorm_eps, self.route_scale = float(renorm_eps), float(route_scale)
        self.groups, self.keep_groups = (int(groups[0]), int(groups[1])) if groups else (1, 1)
        outputs = self.num_experts + self.identity
        if self.groups < 1 or outputs % self.groups or not 1 <= self.keep_groups <= self.groups \
                or self.keep_groups * (outputs // self.groups) < self.top or self.groups > 64:
            raise ValueError(f"{self.groups} groups of which {self.keep_groups} are kept do not fit {outputs} "
                             f"router outputs with {self.top} chosen (at most 64 equal groups)")
        self.correction_name = correction_name
        self.shared = shared
        self.shared_gate = bool(shared_gate) and shared is not None
        self.router_name, self.expert_prefix = router_name, expert_prefix
        self.shared_prefix, self.shared_gate_name = shared_prefix, shared_gate_name
        self.names = (gate_name, up_name, down_name)
        self.router = self.gate_up = self.down = self.correction = None
        if shared is not None:
            self.kernel_libraries = tuple(dict.fromkeys(self.kernel_libraries + tuple(shared.kernel_libraries)))

    def param_sources(self) -> List[ParamSource]:
        g, u, d = self.names
        I, W = self.intermediate_size, self.hidden_size
        out = [ParamSource(self.router_name, (self.num_experts + self.identity, W))]
        if self.correction_name:
            out.append(ParamSource(self.correction_name, (self.num_experts + self.identity,), "vector",
                                   init=("normal", 0.0, 0.02)))
        for e in range(self.num_experts):
            p = f"{self.expert_prefix}{e}."
            if self.gated:
                out.append(ParamSource(p + g, (I, W)))
            out += [ParamSource(p + u, (I, W)), ParamSource(p + d, (W, I))]
        if self.shared is not None:
            for src in self.shared.param_sources():
                out.append(ParamSource(self.shared_prefix + src.name, src.shape, src.kind, src.init))
            if self.shared_gate:
                out.append(ParamSource(self.shared_gate_name, (1, W)))
        return out

    def load(self, tensors, dtype, device) -> None:
        g, u, d = self.names
        router = [tensors[self.router_name]]
        if self.shared_gate:
            router.append(tensors[self.shared_gate_name])
        self.router = place(torch.cat(router, dim=0), "matrix", dtype, device)
        if self.correction_name:
            self.correction = place(tensors[self.correction_name], "vector", dtype, device)
        names = [f"{self.expert_prefix}{e}." for e in range(self.num_experts)]
        first = (lambda p: torch.cat([tensors[p + g], tensors[p + u]], dim=0)) if self.gated \
            else (lambda p: tensors[p + u])
        self.gate_up = place(torch.stack([first(p) for p in names]), "matrix", dtype, device)
        self.down = place(torch.stack([tensors[p + d] for p in names]), "matrix", dtype, device)
        if self.shared is not None:
            n = len(self.shared_prefix)
            self.shared.load({k[n:]: t for k, t in tensors.items()
                              if k.startswith(self.shared_prefix) and k != self.shared_gate_name}, dtype, device)

    def make_decode_copies(self) -> int:
        return self.shared.make_decode_copies() if self.shared is not None else 0

    def forward(self, x):
        x = as_tensor(x)
        logits = linear(x, self.router, out_dtype=torch.float32)
        r = ops.moe_route(logits, self.num_experts, self.top, 1 if self.shared_gate else 0, self.renormalize,
                          self.score, self.correction, self.identity, self.renorm_eps, self.route_scale,
                          self.groups, self.keep_groups)
        shared = self.shared.forward(x) if self.shared is not None else None
        return ops.moe_experts(x, r, self.gate_up, self.down, self.act, self.limit, self.weight_on_input,
                               shared, r.extra)
