"""A feed-forward of many small experts of which every token uses a few, chosen by a router."""
from __future__ import annotations

from ..kernels import ops
from .base import FeedForward, ParamSpec, few_tokens, register_part, side_branch


@register_part("feed_forward", "moe")
class RoutedExperts(FeedForward):
    """out = sum over the token's chosen experts e of weight_e * expert_e(x), plus, if there is one, a feed-forward that
    every token passes (`shared`, any `FeedForward`). An expert is W_down[e] (silu(W_gate[e] x) * (W_up[e] x)), or with
    `gated=False` W_down[e] relu(W_up[e] x)^2.

    The router is float32. `scoring` "softmax": scores = softmax(W_router x) over all experts; "sigmoid": a sigmoid
    each. `correction`: a stored number per expert joins the scores for the choice only (the weights use the scores
    without it). `group_count` > 1: the experts form that many equal groups of neighbours, a group scores as the sum of
    its `group_top` largest choice scores (1: as its best expert), and only the experts of the `group_keep` best groups
    can be chosen. The `top` largest choice scores are chosen; their weights are the scores, divided by their sum
    (`normalise`) or not, times `route_scale`. The experts' weights are stored per expert and packed here: `gate_up`
    [experts * 2 ff, hidden] (an expert's gate rows, then its up rows; up rows only without a gate), `down` [experts *
    hidden, ff]. The routed part comes back as float32 partial sums [top, T, hidden], one per choice, and the shared
    part beside it: whoever adds the layer's output to the stream adds them all (`FeedForward.forward` may return a
    tuple). With `sum_outputs` the parts are added here, in one kernel, into one float32 tensor [T, hidden]; a shared
    part that is gated per token (`ActivatedMLP(token_gate=True)`) gets its gate in the same pass. With `side_stream` the
    shared part then runs, in steps of few tokens, on a second stream beside the routed one (`base.side_branch`); it is off:
    the shared part is three short launches, and parting and meeting cost more than they save (a decode step of 8 requests at
    1,024 wide, 28 layers: 2.84 ms without, 3.19 ms with)."""

    side_stream = False

    def __init__(self, hidden_size: int, intermediate_size: int, num_experts: int, top: int, group_count: int = 1,
                 group_keep: int = 1, shared: FeedForward | None = None, gated: bool = True, scoring: str = "softmax",
                 correction: bool = False, group_top: int = 1, normalise: bool = True, route_scale: float = 1.0,
                 sum_outputs: bool = False):
        super().__init__()
        if not 1 <= top <= num_experts:
            raise ValueError(f"top {top} of {num_experts} experts")
        if group_count < 1 or num_experts % group_count or not 1 <= group_keep <= group_count:
            raise ValueError(f"{num_experts} experts do not form {group_count} equal groups of which {group_keep} are kept")
        if group_keep * (num_experts // group_count) < top:
            raise ValueError("the kept groups hold fewer experts than a token uses")
        if scoring not in ("softmax", "sigmoid") or group_top < 1:
            raise ValueError("scoring is 'softmax' or 'sigmoid', group_top positive")
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.num_experts, self.top, self.group_count, self.group_keep = num_experts, top, group_count, group_keep
        self.gated, self.scoring, self.group_top = bool(gated), scoring, int(group_top)
        self.normalise, self.route_scale, self.sum_outputs = bool(normalise), float(route_scale), bool(sum_outputs)
        rows = (2 if self.gated else 1) * intermediate_size
        self.add_param("router", ParamSpec((num_experts, hidden_size), init="matrix", dtype="float32"))
        self.add_param("gate_up", ParamSpec((num_experts * rows, hidden_size), init="matrix", dtype="compute"))
        self.add_param("down", ParamSpec((num_experts * hidden_size, intermediate_size), init="matrix", dtype="compute"))
        if correction:
            self.add_param("correction", ParamSpec((num_experts,), init="matrix", dtype="float32"))
        else:
            self.correction = None
        if shared is not None:
            self.add_child("shared", shared)
        else:
            self.shared = None
        self._rule = None

    def set_param(self, local, tensor):
        super().set_param(local, tensor)
        self._rule = None

    def rule(self) -> "ops.RouteRule":
        if self._rule is None:
            self._rule = ops.RouteRule(self.scoring, self.correction, self.group_top, self.normalise, self.route_scale)
        return self._rule

    def forward(self, x):
        E, F, h = self.num_experts, self.intermediate_size, self.hidden_size
        run = lambda: ops.route_and_run_experts(x, self.router, self.top, self.group_count, self.group_keep,
                                                self.gate_up.view(E, (2 if self.gated else 1) * F, h), self.down.view(E, h, F),
                                                rule=self.rule(), gated=self.gated)
        if not self.sum_outputs:
            routed = run()
            return routed if self.shared is None else (routed, self.shared.forward(x))
        if self.shared is None:
            return ops.weighted_sum([(run(), 1.0, None)])
        gated = getattr(self.shared, "token_gate", False)
        pass_shared = lambda: self.shared.forward(x, defer_gate=True) if gated else self.shared.forward(x)
        if self.side_stream and few_tokens(x):
            with side_branch(x.device, 1) as branch:
                s = pass_shared()
            routed = run()
            branch.join()
        else:
            routed, s = run(), pass_shared()
        return ops.weighted_sum([(routed, 1.0, None), (s.rows, 1.0, None, s.gate) if gated else (s, 1.0, None)])
