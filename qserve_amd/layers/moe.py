"""Mixture of small feed-forward experts behind a grouped top-k router.

score = softmax(router . h) over all experts (float).  The experts form `groups` equal groups of neighbours; a group's score
is its largest expert score and only experts of the `keep` best groups are eligible (groups = keep = 1: a plain top-k
router).  The `top_k` eligible experts with the largest scores are used, weighted by those scores as they are (no
renormalisation).  Expert: down . act(up . h), act = relu(.)^2, no biases.
"""
import torch


class GroupedTopKMoE:
    def __init__(self, ops, *, router, up, down, top_k, groups=1, keep=1):
        """router [E, D]; up: list of E [ff, D]; down: list of E [D, ff] (stacked here into [E, ff, D] / [E, D, ff])."""
        self.ops = ops
        self.router = router.contiguous()
        self.up, self.down = torch.stack(list(up)).contiguous(), torch.stack(list(down)).contiguous()
        E, ff, D = self.up.shape
        self.top_k, self.groups, self.keep = int(top_k), int(groups), int(keep)
        if self.router.shape != (E, D) or self.down.shape != (E, D, ff):
            raise ValueError("mixture of experts: router / expert shapes do not fit each other")
        if E % self.groups or not 0 < self.keep <= self.groups or not 0 < self.top_k <= self.keep * (E // self.groups):
            raise ValueError(f"router: {E} experts, {self.groups} groups, keep {self.keep}, top {self.top_k}")

    def __call__(self, h):
        idx, wt = self.ops.moe_route(h, self.router, self.top_k, self.groups, self.keep)
        return self.ops.moe_experts(h, self.up, self.down, idx, wt)


def _interleave(gate, up):
    """[..., ff, D] gate and up rows -> [..., 2 ff, D] with row 2f = gate f and row 2f + 1 = up f, so that one product gives a
    gated unit's two halves as neighbours (qserve_amd.layers.ops `glu`)."""
    return torch.stack([gate, up], dim=-2).reshape(*gate.shape[:-2], 2 * gate.size(-2), gate.size(-1)).contiguous()


class GatedFeedForward:
    """Dense gated feed-forward: down . (act(gate . h) * (up . h)), no biases; act: "silu" or "gelu_tanh"."""

    def __init__(self, ops, *, gate, up, down, act="silu"):
        if gate.shape != up.shape or down.shape != (gate.size(1), gate.size(0)):
            raise ValueError("gated feed-forward: gate / up / down shapes do not fit each other")
        if act not in ("silu", "gelu_tanh"):
            raise ValueError(f"gated feed-forward: unknown activation {act!r}")
        self.ops, self.w_in, self.w_down, self.act = ops, _interleave(gate, up), down.contiguous(), act

    def __call__(self, h):
        from .ops import linear
        a = linear(h, self.w_in)
        return linear(self.ops.glu(a) if self.act == "silu" else self.ops.glu(a, self.act), self.w_down)


class TopKGatedMoE:
    """Mixture of gated experts behind a plain top-k router with a bias: logits z = router . h + bias (float); the `top_k`
    largest are chosen and weighted by the softmax over the chosen logits only.  Expert: down . (silu(gate . h) * (up . h))."""

    def __init__(self, ops, *, router, bias, gate, up, down, top_k):
        """router [E, D], bias [E]; gate / up: lists of E [ff, D]; down: list of E [D, ff]."""
        self.ops = ops
        self.router, self.bias = router.contiguous(), bias.contiguous()
        self.up = _interleave(torch.stack(list(gate)), torch.stack(list(up)))          # [E, 2 ff, D]
        self.down = torch.stack(list(down)).contiguous()
        E, ff2, D = self.up.shape
        self.top_k = int(top_k)
        if self.router.shape != (E, D) or self.bias.shape != (E,) or self.down.shape != (E, D, ff2 // 2):
            raise ValueError("mixture of experts: router / expert shapes do not fit each other")
        if not 0 < self.top_k <= E:
            raise ValueError(f"router: {E} experts, top {self.top_k}")

    def __call__(self, h):
        idx, wt = self.ops.moe_route(h, self.router, self.top_k, 1, 1, bias=self.bias, renorm=True)
        return self.ops.moe_experts(h, self.up, self.down, idx, wt, act="swiglu")


class CorrectedSigmoidMoE:
    """Mixture of gated experts behind a sigmoid router with a choice correction: scores s = sigmoid(router . h) (float); experts
    are CHOSEN by s + correction, inside the `keep` groups (of `groups` equal groups of neighbours) whose two largest corrected
    scores sum highest; the chosen experts are WEIGHTED by their plain s times `scale` (no division by the chosen scores' sum).  Expert: down .
    (silu(gate . h) * (up . h)).  An optional shared expert of the same form runs for every token.
    Returns the list of outputs to be summed ([routed] or [routed, shared]): the caller's residual kernel adds them in one pass."""

    def __init__(self, ops, *, router, correction, gate, up, down, top_k, groups=1, keep=1, scale=1.0, shared=None):
        """router [E, D], correction [E]; gate / up: lists of E [ff, D]; down: list of E [D, ff]; shared: a GatedFeedForward or None."""
        self.ops = ops
        self.router, self.correction = router.contiguous(), correction.float().contiguous()
        self.up = _interleave(torch.stack(list(gate)), torch.stack(list(up)))          # [E, 2 ff, D]
        self.down = torch.stack(list(down)).contiguous()
        E, ff2, D = self.up.shape
        self.top_k, self.groups, self.keep, self.scale, self.shared = int(top_k), int(groups), int(keep), float(scale), shared
        if self.router.shape != (E, D) or self.correction.shape != (E,) or self.down.shape != (E, D, ff2 // 2):
            raise ValueError("mixture of experts: router / expert shapes do not fit each other")
        if E % self.groups or not 0 < self.keep <= self.groups or not 0 < self.top_k <= self.keep * (E // self.groups):
            raise ValueError(f"router: {E} experts, {self.groups} groups, keep {self.keep}, top {self.top_k}")

    def __call__(self, h):
        idx, wt = self.ops.moe_route(h, self.router, self.top_k, self.groups, self.keep, score="sigmoid", correction=self.correction,
                                     group_top=2, scale=self.scale)
        y = [self.ops.moe_experts(h, self.up, self.down, idx, wt, act="swiglu")]
        if self.shared is not None:
            y.append(self.shared(h))
        return y


class ReluSquaredFeedForward:
    """Dense feed-forward without a gate: down . relu(up . h)^2, no biases."""

    def __init__(self, ops, *, up, down):
        if down.shape != (up.size(1), up.size(0)):
            raise ValueError("feed-forward: up / down shapes do not fit each other")
        self.ops, self.w_up, self.w_down = ops, up.contiguous(), down.contiguous()

    def __call__(self, h):
        from .ops import linear
        return linear(self.ops.relu_sq(linear(h, self.w_up)), self.w_down)


class IdentityExpertMoE:
    """Mixture of clamped gated experts and identity experts behind a softmax router with a choice correction.  Scores s =
    softmax(router . h) over ALL router outputs (float); the `top_k` outputs with the largest s + correction are chosen and
    weighted by their plain s (no renormalisation).  The last `identity` router outputs have no tensors: their expert returns its
    input.  The others: g = min(gate . h, limit), u = clamp(up . h, -limit, limit), down . (g sigmoid(1.702 g) (u + 1))."""

    def __init__(self, ops, *, router, correction, gate, up, down, top_k, identity=0, limit):
        """router [E + identity, D], correction [E + identity]; gate / up: lists of E [ff, D]; down: list of E [D, ff]."""
        self.ops = ops
        self.router, self.correction = router.contiguous(), correction.float().contiguous()
        self.up = _interleave(torch.stack(list(gate)), torch.stack(list(up)))          # [E, 2 ff, D]
        self.down = torch.stack(list(down)).contiguous()
        E, ff2, D = self.up.shape
        self.top_k, self.identity, self.limit = int(top_k), int(identity), float(limit)
        n = E + self.identity
        if self.router.shape != (n, D) or self.correction.shape != (n,) or self.down.shape != (E, D, ff2 // 2) or self.identity < 0:
            raise ValueError("mixture of experts: router / expert shapes do not fit each other")
        if not 0 < self.top_k <= n:
            raise ValueError(f"router: {n} outputs, top {self.top_k}")

    def __call__(self, h):
        idx, wt = self.ops.moe_route(h, self.router, self.top_k, 1, 1, correction=self.correction)
        return self.ops.moe_experts(h, self.up, self.down, idx, wt, act="clamped_glu", limit=self.limit)
