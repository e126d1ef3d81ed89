"""Recurrent mixers whose state is a vector per channel."""

import torch

from ..ops import kernels
from ..weights.loader import MATRIX, VECTOR, ParamSpec
from .base import Mixer, SlotStateSpec, site_memo
from .registry import register_mixer


@register_mixer("selective_scan")
class SelectiveScan(Mixer):
    """A selective state-space mixer (Mamba).  With ``h`` the layer's input:

        [u | z] = W_in h                                               (inner channels each)
        x_t = silu(conv(u)_t)       a causal convolution per channel over ``taps`` inputs, with bias
        [low | B | C] = W_x x_t                                        (dt_rank, states, states)
        dt = softplus(W_dt low + b_dt),   A = -exp(A_log)              (per channel / channel x state)
        S_t[c, n] = exp(dt_c A[c, n]) S_(t-1)[c, n] + dt_c x_c B_n
        y_c = (sum_n S_t[c, n] C_n + D_c x_c) * silu(z_c),   out = W_o y

    Per request the slot keeps the recurrence's numbers and, behind them, each channel's last
    ``taps - 1`` raw inputs, so that a prompt may be cut anywhere.  Both start at zero.  The
    projections' results are written in float; step sizes, decays, state and sums are 32-bit in
    both engine dtypes (``csrc/selective_scan.hip``)."""

    graph_safe = True

    accepts_pending_norm = True

    # tokens beyond one per item from which a step's items are cut into pieces that run side by side
    PIECES_FROM = 96

    def __init__(self, width: int, dtype, inner: int, states: int, dt_rank: int, taps: int):
        if not 0 < states <= 256:
            raise ValueError(f"states {states} must lie in 1..256")
        if not 1 <= taps <= 64:
            raise ValueError(f"taps {taps} must lie in 1..64")
        self.width = width
        self.dtype = dtype
        self.inner = inner
        self.states = states
        self.dt_rank = dt_rank
        self.taps = taps
        self._memo_in, self._memo_x, self._memo_out = {}, {}, {}

    def parameters(self):
        return {
            "in.weight": ParamSpec((2 * self.inner, self.width), MATRIX),
            "conv.weight": ParamSpec((self.inner, self.taps), VECTOR),
            "conv.bias": ParamSpec((self.inner,), VECTOR),
            "x.weight": ParamSpec((self.dt_rank + 2 * self.states, self.inner), MATRIX),
            "dt.weight": ParamSpec((self.inner, self.dt_rank), MATRIX),
            "dt.bias": ParamSpec((self.inner,), VECTOR),
            "a_log": ParamSpec((self.inner, self.states), VECTOR),
            "skip": ParamSpec((self.inner,), VECTOR),
            "out.weight": ParamSpec((self.width, self.inner), MATRIX),
        }

    def bind(self, tensors):
        for name in self.parameters():
            setattr(self, name.replace(".", "_"), tensors[name])
        self.in_packed = kernels.pack_decode_weight(self.in_weight)
        self.x_packed = kernels.pack_decode_weight(self.x_weight)
        self.out_packed = kernels.pack_decode_weight(self.out_weight)
        for memo in (self._memo_in, self._memo_x, self._memo_out):
            memo.clear()

    def cache_spec(self):
        return SlotStateSpec((self.inner, self.states + self.taps - 1), torch.float32)

    def forward(self, x, residual, ctx, cache):
        tokens = ctx.tokens
        workspace = ctx.workspace
        inner, rank, states = self.inner, self.dt_rank, self.states
        proj = workspace.first_rows("scan_proj", 2 * inner, torch.float32, tokens)
        kernels.linear(x, self.in_weight, None, proj, packed=self.in_packed,
                       memo=site_memo(self._memo_in, workspace), shared=ctx.shared_calls)
        activated = workspace.first_rows("scan_x", inner, self.dtype, tokens)
        kernels.conv_silu(proj, 0, self.conv_weight, self.conv_bias, cache.state, states, activated,
                          ctx.tok_item, ctx.cu_tokens, ctx.slots)
        low = workspace.first_rows("scan_low", rank + 2 * states, torch.float32, tokens)
        kernels.linear(activated, self.x_weight, None, low, packed=self.x_packed,
                       memo=site_memo(self._memo_x, workspace), shared=ctx.shared_calls)
        y = workspace.first_rows("scan_y", inner, self.dtype, tokens)
        scratch = None
        items = ctx.slots.numel()
        pieces = tokens - items >= self.PIECES_FROM
        dt = step_weights = None
        if pieces or rank > kernels.SCAN_FUSED_RANK:
            dt = workspace.first_rows("scan_dt", inner, torch.float32, tokens)
            kernels.step_size(low[:, :rank], self.dt_weight, self.dt_bias, dt)
        else:
            # decoded tokens and short portions: the recurrence works its step sizes out itself
            step_weights = (0, self.dt_weight, self.dt_bias)
        if pieces:
            # some item brings a long portion: pieces of it run side by side.  The scratch is
            # asked for at its largest, so that it never moves under recorded launches.
            most = kernels.selective_scan_records(workspace.max_rows, cache.state.shape[0], inner, states)
            scratch = (workspace.flat("scan_records", most[0], torch.float32),
                       workspace.flat("scan_sums", most[1], torch.float32))
        kernels.selective_scan(activated, dt, low, rank, rank + states, proj, 0, inner, self.a_log,
                               self.skip, cache.state, y, ctx.cu_tokens, ctx.slots, self.taps,
                               scratch=scratch, step_weights=step_weights)
        kernels.linear(y, self.out_weight, None, residual, epilogue="residual",
                       packed=self.out_packed, memo=site_memo(self._memo_out, workspace),
                       shared=ctx.shared_calls)


@register_mixer("gated_linear_recurrence")
class GatedLinearRecurrence(Mixer):
    """The recurrent block of Griffin with its real-gated linear recurrent unit.  With ``h`` the
    layer's input, two branches of ``inner`` channels:

        y = gelu_tanh(W_y h + b_y)
        u = conv(W_x h + b_x)           a causal convolution per channel over ``taps`` inputs, with bias
        r = sigmoid(A_b u_b + a_b),  i = sigmoid(I_b u_b + i_b)     block by block: the channels in
                                                                   ``blocks`` runs, a square matrix each
        a = exp(-decay_scale * r * softplus(lam)),   S_t = a S_(t-1) + sqrt(1 - a^2) * i * u
        out = W_o (S * y)

    One packed product gives ``[y | x]`` in float, one block-diagonal product the gates of a run
    ``[r | i]``.  Per request the slot keeps S and, behind it, each channel's last ``taps - 1``
    inputs of the convolution; both start at zero.  Gates, decays and the state are 32-bit in
    both engine dtypes (``csrc/linear_recurrence.hip``)."""

    graph_safe = True

    accepts_pending_norm = True

    def __init__(self, width: int, dtype, inner: int, blocks: int, taps: int, decay_scale: float = 8.0):
        if inner % blocks:
            raise ValueError(f"{inner} channels do not split into {blocks} equal runs")
        if not 1 <= taps <= 64:
            raise ValueError(f"taps {taps} must lie in 1..64")
        self.width = width
        self.dtype = dtype
        self.inner = inner
        self.blocks = blocks
        self.block = inner // blocks
        self.taps = taps
        self.decay_scale = float(decay_scale)
        self._memo_in, self._memo_out = {}, {}

    def parameters(self):
        return {
            "in.weight": ParamSpec((2 * self.inner, self.width), MATRIX),
            "in.bias": ParamSpec((2 * self.inner,), VECTOR),
            "conv.weight": ParamSpec((self.inner, self.taps), VECTOR),
            "conv.bias": ParamSpec((self.inner,), VECTOR),
            "gates.weight": ParamSpec((self.blocks, 2 * self.block, self.block), MATRIX),
            "gates.bias": ParamSpec((self.blocks, 2 * self.block), VECTOR),
            "lam": ParamSpec((self.inner,), VECTOR),
            "out.weight": ParamSpec((self.width, self.inner), MATRIX),
        }

    def bind(self, tensors):
        for name in self.parameters():
            setattr(self, name.replace(".", "_"), tensors[name])
        self.gates_bias = self.gates_bias.reshape(-1)
        self.in_packed = kernels.pack_decode_weight(self.in_weight)
        self.out_packed = kernels.pack_decode_weight(self.out_weight)
        for memo in (self._memo_in, self._memo_out):
            memo.clear()

    def cache_spec(self):
        return SlotStateSpec((self.inner, self.taps), torch.float32)

    def forward(self, x, residual, ctx, cache):
        tokens = ctx.tokens
        workspace = ctx.workspace
        inner = self.inner
        proj = workspace.first_rows("lru_proj", 2 * inner, torch.float32, tokens)
        kernels.linear(x, self.in_weight, self.in_bias, proj, packed=self.in_packed,
                       memo=site_memo(self._memo_in, workspace), shared=ctx.shared_calls)
        u = workspace.first_rows("lru_u", inner, torch.float32, tokens)
        kernels.conv_silu(proj, inner, self.conv_weight, self.conv_bias, cache.state, 1, u,
                          ctx.tok_item, ctx.cu_tokens, ctx.slots, activation=False)
        gates = workspace.first_rows("lru_gates", 2 * inner, torch.float32, tokens)
        kernels.block_linear(u, self.block, self.gates_weight, self.gates_bias, gates, 2 * self.block)
        y = workspace.first_rows("lru_y", inner, self.dtype, tokens)
        kernels.lru_scan(proj, 0, inner, u, gates, self.block, self.lam, self.decay_scale, cache.state,
                         y, ctx.cu_tokens, ctx.slots, self.taps)
        kernels.linear(y, self.out_weight, None, residual, epilogue="residual",
                       packed=self.out_packed, memo=site_memo(self._memo_out, workspace),
                       shared=ctx.shared_calls)
