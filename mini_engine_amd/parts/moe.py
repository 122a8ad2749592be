"""A feed-forward of many small gated experts of which every token uses a few, chosen by a router."""
from __future__ import annotations

from ..kernels import ops
from .base import FeedForward, ParamSpec, register_part


@register_part("feed_forward", "moe")
class RoutedExperts(FeedForward):
    """out = sum over the token's chosen experts e of weight_e * W_down[e] (silu(W_gate[e] x) * (W_up[e] x)), plus,
    if there is one, a gated feed-forward that every token passes (`shared`, any `FeedForward`).

    The router is float32: scores = softmax(W_router x) over all experts. `group_count` > 1: the experts form that
    many equal groups of neighbours, a group scores as its best expert, and only the experts of the `group_keep`
    best groups can be chosen. The `top` largest scores are chosen; their weights are the scores divided by their
    sum. The experts' weights are stored per expert and packed here: `gate_up` [experts * 2 ff, hidden] (an expert's
    gate rows, then its up rows), `down` [experts * hidden, ff]. The routed part comes back as float32 partial sums
    [top, T, hidden], one per choice, and the shared part beside it: whoever adds the layer's output to the stream
    adds them all (`FeedForward.forward` may return a tuple)."""

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, top: int, group_count: int = 1,
                 group_keep: int = 1, shared: FeedForward | None = None):
        super().__init__()
        if not 1 <= top <= num_experts:
            raise ValueError(f"top {top} of {num_experts} experts")
        if group_count < 1 or num_experts % group_count or not 1 <= group_keep <= group_count:
            raise ValueError(f"{num_experts} experts do not form {group_count} equal groups of which {group_keep} are kept")
        if group_keep * (num_experts // group_count) < top:
            raise ValueError("the kept groups hold fewer experts than a token uses")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.num_experts, self.top, self.group_count, self.group_keep = num_experts, top, group_count, group_keep
        self.add_param("router", ParamSpec((num_experts, hidden_size), init="matrix", dtype="float32"))
        self.add_param("gate_up", ParamSpec((num_experts * 2 * intermediate_size, hidden_size), init="matrix", dtype="compute"))
        self.add_param("down", ParamSpec((num_experts * hidden_size, intermediate_size), init="matrix", dtype="compute"))
        if shared is not None:
            self.add_child("shared", shared)
        else:
            self.shared = None

    def forward(self, x):
        E, F, h = self.num_experts, self.intermediate_size, self.hidden_size
        routed = ops.route_and_run_experts(x, self.router, self.top, self.group_count, self.group_keep,
                                           self.gate_up.view(E, 2 * F, h), self.down.view(E, h, F))
        if self.shared is None:
            return routed
        return routed, self.shared.forward(x)
