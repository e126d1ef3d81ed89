"""Feed-forward parts."""

import torch

from ..ops import kernels
from ..weights.loader import MATRIX, VECTOR, ParamSpec
from .base import FeedForward, site_memo
from .registry import register_feed_forward

ACTIVATIONS = ("gelu_tanh", "gelu_erf", "relu2")


@register_feed_forward("dense")
class DenseFeedForward(FeedForward):
    """``residual += act(x W_up + b_up) W_down + b_down``
    (src/model/paged_decoder.py:178-179,224-228; activations ``:273-280``)."""

    graph_safe = True

    accepts_pending_norm = True

    def __init__(self, width: int, dtype, inner: int, activation: str, bias: bool = True):
        if activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {activation!r}; known: {', '.join(ACTIVATIONS)}")
        self.width = width
        self.dtype = dtype
        self.inner = inner
        self.activation = activation
        self.bias = bias
        self._memo_up, self._memo_down = {}, {}

    def parameters(self):
        params = {
            "up.weight": ParamSpec((self.inner, self.width), MATRIX),
            "down.weight": ParamSpec((self.width, self.inner), MATRIX),
        }
        if self.bias:
            params["up.bias"] = ParamSpec((self.inner,), VECTOR)
            params["down.bias"] = ParamSpec((self.width,), VECTOR)
        return params

    def bind(self, tensors):
        self.up_weight = tensors["up.weight"]
        self.down_weight = tensors["down.weight"]
        self.up_bias = tensors.get("up.bias")
        self.down_bias = tensors.get("down.bias")
        # copies in the layout that the products of few rows (decode steps) read fastest
        self.up_packed = kernels.pack_decode_weight(self.up_weight)
        self.down_packed = kernels.pack_decode_weight(self.down_weight)
        self._memo_up.clear()
        self._memo_down.clear()

    def forward(self, x, residual, ctx):
        hidden = ctx.workspace.first_rows("ffn", self.inner, self.dtype, ctx.tokens)
        # (the hidden rows belong to these two calls alone: at 17 to 64 rows the first may leave
        # them in the order in which the second reads them)
        _, hidden_packed = kernels.linear(x, self.up_weight, self.up_bias, hidden,
                                          epilogue=self.activation, packed=self.up_packed,
                                          packed_out=True, memo=site_memo(self._memo_up, ctx.workspace),
                                          shared=ctx.shared_calls)
        kernels.linear(hidden, self.down_weight, self.down_bias, residual, epilogue="residual",
                       packed=self.down_packed, a_packed=hidden_packed, memo=site_memo(self._memo_down, ctx.workspace),
                       shared=ctx.shared_calls)


@register_feed_forward("gated")
class GatedFeedForward(FeedForward):
    """``residual += W_down (act(W_gate x) * (W_up x))``, no biases; ``activation``: ``silu`` or
    ``gelu_tanh``.  One packed product gives ``[gate | up]`` in float; the activation and the
    product of the halves are 32-bit."""

    graph_safe = True

    accepts_pending_norm = True

    def __init__(self, width: int, dtype, inner: int, activation: str = "silu"):
        if activation not in kernels.GATE_ACTIVATIONS:
            raise ValueError(f"unknown gate activation {activation!r}; known: "
                             f"{', '.join(kernels.GATE_ACTIVATIONS)}")
        self.width = width
        self.dtype = dtype
        self.inner = inner
        self.activation = activation
        self._memo_up, self._memo_down = {}, {}

    def parameters(self):
        return {
            "gate_up.weight": ParamSpec((2 * self.inner, self.width), MATRIX),
            "down.weight": ParamSpec((self.width, self.inner), MATRIX),
        }

    def bind(self, tensors):
        self.gate_up_weight = tensors["gate_up.weight"]
        self.down_weight = tensors["down.weight"]
        self.gate_up_packed = kernels.pack_decode_weight(self.gate_up_weight)
        self.down_packed = kernels.pack_decode_weight(self.down_weight)
        self._memo_up.clear()
        self._memo_down.clear()

    def forward(self, x, residual, ctx):
        tokens = ctx.tokens
        both = ctx.workspace.first_rows("ffn_gate_up", 2 * self.inner, torch.float32, tokens)
        kernels.linear(x, self.gate_up_weight, None, both, packed=self.gate_up_packed,
                       memo=site_memo(self._memo_up, ctx.workspace), shared=ctx.shared_calls)
        hidden = ctx.workspace.first_rows("ffn", self.inner, self.dtype, tokens)
        kernels.silu_gate(both, hidden, self.activation)
        kernels.linear(hidden, self.down_weight, None, residual, epilogue="residual",
                       packed=self.down_packed, memo=site_memo(self._memo_down, ctx.workspace),
                       shared=ctx.shared_calls)


@register_feed_forward("moe")
class MixtureOfExperts(FeedForward):
    """``experts`` small feed-forwards (no biases) of which each token uses ``top``:

        s = softmax(W_router x) over all experts, the logits in 32-bit
        experts form ``groups`` equal groups of neighbours; a group's score is its largest s and
        only experts of the ``keep`` best groups may be chosen; the ``top`` largest s among them are
        residual += sum over the chosen e of (s_e * scale) * W_down,e (silu(W_gate,e x) * (W_up,e x))

    The weights are not renormalised.  The experts' matrices are stacked, ``[experts, gate rows
    | up rows, width]`` and ``[experts, width, inner]``; the choice stays on the device
    (``csrc/moe.hip``).

    Options: ``score="sigmoid"``: ``s = sigmoid(z)``; ``correction``: a number per expert
    (``router.correction``) is added to ``s`` for the choice only, the weights use ``s`` without it;
    ``group_top``: a group's score is the sum of that many of its largest choice scores;
    ``normalise``: the chosen scores are divided by their sum (+ 1e-20) before ``scale``;
    ``form="relu2"``: an expert is ``W_down,e relu(W_up,e x)^2`` (``up.weight [experts * inner,
    width]``); ``shared_inner > 0``: one more expert of the same form and that inner width
    (``shared.*``) runs for every token with weight one.  Steps of few tokens run a shared
    expert of the plain form whose inner width is a multiple of the others' inside the experts'
    own two launches, cut into experts of their width that every token uses (squaring is element
    by element, so the cut is exact); steps of many tokens run it as two dense products."""

    graph_safe = True

    accepts_pending_norm = False

    SCORES = ("softmax", "sigmoid")
    FORMS = ("gated_silu", "relu2")

    def __init__(self, width: int, dtype, inner: int, experts: int, top: int, groups: int = 1,
                 keep: int = 1, scale: float = 1.0, score: str = "softmax", correction: bool = False,
                 group_top: int = 1, normalise: bool = False, form: str = "gated_silu",
                 shared_inner: int = 0):
        if groups < 1 or experts % groups:
            raise ValueError(f"{groups} groups do not divide {experts} experts")
        if not 1 <= keep <= groups:
            raise ValueError(f"keep ({keep}) must lie in 1..groups ({groups})")
        if not 1 <= top <= (experts // groups) * keep:
            raise ValueError(f"top ({top}) exceeds the experts that may be chosen")
        if score not in self.SCORES:
            raise ValueError(f"unknown router score {score!r}; known: {', '.join(self.SCORES)}")
        if form not in self.FORMS:
            raise ValueError(f"unknown expert form {form!r}; known: {', '.join(self.FORMS)}")
        if not 1 <= group_top <= 8:
            raise ValueError(f"group_top ({group_top}) must lie in 1..8")
        self.width = width
        self.dtype = dtype
        self.inner = inner
        self.experts = experts
        self.top = top
        self.groups = groups
        self.keep = keep
        self.scale = float(scale)
        self.sigmoid = score == "sigmoid"
        self.has_correction = bool(correction)
        self.group_top = int(group_top)
        self.normalise = bool(normalise)
        self.gated = form == "gated_silu"
        self.first_rows = (2 if self.gated else 1) * inner     # rows of an expert's first matrix
        self.first_name = "gate_up.weight" if self.gated else "up.weight"
        self.shared = None
        self.shared_pieces = 0      # the shared expert as that many experts of the others' width
        if shared_inner:
            if self.gated:
                self.shared = GatedFeedForward(width, dtype, shared_inner)
            else:
                self.shared = DenseFeedForward(width, dtype, shared_inner, "relu2", bias=False)
                pieces = shared_inner // inner
                # (the row kernels keep a token's hidden rows of all its experts in LDS)
                if shared_inner == pieces * inner and pieces <= 64 and (top + pieces) * inner * 4 <= 64 * 1024:
                    self.shared_pieces = pieces

    def parameters(self):
        params = {
            "router.weight": ParamSpec((self.experts, self.width), VECTOR),
            self.first_name: ParamSpec((self.experts * self.first_rows, self.width), MATRIX),
            "down.weight": ParamSpec((self.experts * self.width, self.inner), MATRIX),
        }
        if self.has_correction:
            params["router.correction"] = ParamSpec((self.experts,), VECTOR)
        if self.shared is not None:
            for name, spec in self.shared.parameters().items():
                params["shared." + name] = spec
        return params

    def bind(self, tensors):
        self.router_weight = tensors["router.weight"]
        self.correction = tensors["router.correction"] if self.has_correction else None
        self.first_weight = tensors[self.first_name].view(self.experts, self.first_rows, self.width)
        if self.gated:
            self.gate_up_weight = self.first_weight
        self.down_weight = tensors["down.weight"].view(self.experts, self.width, self.inner)
        if self.shared is not None:
            self.shared.bind({name: tensors["shared." + name] for name in self.shared.parameters()})
        if self.shared_pieces:
            pieces = self.shared_pieces
            self.shared_extra = (
                self.shared.up_weight.view(pieces, self.inner, self.width),
                self.shared.down_weight.view(self.width, pieces, self.inner).transpose(0, 1).contiguous())

    def forward(self, x, residual, ctx):
        tokens = ctx.tokens
        workspace = ctx.workspace
        sorted_path = (tokens * self.top >= kernels.MOE_GROUPED_FROM
                       and kernels.moe_grouped_supported(self.dtype, self.width, self.inner))
        # few tokens: the shared expert's pieces ride along as experts that every token uses
        fixed = 0 if sorted_path else self.shared_pieces
        chosen = self.top + fixed
        ids = workspace.first_rows("moe_ids", chosen, torch.int32, tokens)
        weights = workspace.first_rows("moe_weights", chosen, torch.float32, tokens)
        kernels.moe_route(x, self.router_weight, self.groups, self.keep, self.top, self.scale, ids,
                          weights, sigmoid=self.sigmoid, correction=self.correction,
                          group_top=self.group_top, normalise=self.normalise, fixed=fixed)
        most = workspace.max_rows * (self.top + self.shared_pieces)
        hidden = workspace.rows("moe_hidden", self.inner, self.dtype, max_rows=most)
        if sorted_path:
            # many rows: sorted by expert, tiles on the matrix cores
            tiles = kernels.moe_grouped_tiles(most, self.experts)
            kernels.moe_experts_grouped(
                x, self.first_weight, self.down_weight, ids, weights, hidden,
                workspace.rows("moe_out", self.width, torch.float32, max_rows=most),
                workspace.flat("moe_order", tiles * kernels.MOE_TILE, torch.int32),
                workspace.flat("moe_tiles", tiles, torch.int32), residual, gated=self.gated)
        else:
            kernels.moe_experts(x, self.first_weight, self.down_weight, ids, weights, hidden, residual,
                                gated=self.gated, extra=self.shared_extra if fixed else None)
        if self.shared is not None and not fixed:
            self.shared.forward(x, residual, ctx)
