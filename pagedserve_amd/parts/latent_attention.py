"""Attention over a cached latent instead of cached keys and values."""

import torch

from ..ops import kernels
from ..weights.loader import MATRIX, VECTOR, ParamSpec
from .attention import Attention
from .base import PagedKVSpec, site_memo
from .position import rotary_frequencies
from .registry import register_mixer


@register_mixer("latent_attention")
class LatentAttention(Attention):
    """Multi-head attention whose keys and values are projections of one small latent per token
    (multi-head latent attention; DeepSeek-AI, "DeepSeek-V2: A Strong, Economical, and Efficient
    Mixture-of-Experts Language Model").  With ``h`` the layer's input:

        q = W_q h                     per head [dim unrotated | rot_dim rotated]
        [c' | r] = W_dkv h            c = rms_norm(c') * gamma (``rank`` numbers), r: one rotated
                                      key part (``rot_dim``) that all heads share
        k_h = [W_uk_h c | rot(r)],    v_h = W_uv_h c
        score = (q_h . k_h) * scale,  causal softmax,  o_h = sum p v
        out = W_o (concat(o_h) * sigmoid(W_g h))

    Only ``c`` and the rotated ``r`` are cached, as ONE row per token that all heads read:
    ``[c | rot(r) | zeros]``.  The head's key matrix moves to the query side, ``(W_uk_h c) . q =
    c . (W_uk_h^T q)``, and the value matrix behind the softmax, ``sum p (W_uv_h c) = W_uv_h (sum p
    c)``: the attention kernels see one key/value head of ``rank + rot_dim`` (rounded up to 16)
    whose values are its own key rows (``PagedKVSpec.values_in_keys``: one pool, no second copy),
    and two block-diagonal products (``kernels.block_linear``) carry the heads' matrices.  The
    dispatch between the attention kernels is the parent's.

    Rotation: the ``rot_dim`` part whole, pairs laid out as halves by default, frequencies
    optionally stretched (``parts/position.py: rotary_frequencies``).  ``score_cap`` as in the
    parent.  Norm, angles, scores, softmax and the gate's sigmoid are 32-bit.

    ``query_rank > 0``: the queries come through a latent of their own, ``q = W_uq (rms_norm(W_dq
    h) * gamma_q)`` (``query_down.weight``, ``query_norm.gamma``, ``query_up.weight``); the norm
    runs inside the second product where that kernel takes it.  ``out_gate=False``: no gate."""

    def __init__(self, width: int, dtype, heads: int, dim: int, rot_dim: int, value_dim: int,
                 rank: int, scale: float, norm_eps: float = 1e-6, rotary_base: float = 10000.0,
                 rotary_scaling=None, rotary_layout: str = "halves", score_cap: float = 0.0,
                 out_gate: bool = True, query_rank: int = 0):
        if rot_dim < 0 or rot_dim % 2:
            raise ValueError(f"rot_dim {rot_dim} must be even")
        cache_dim = -(-(rank + rot_dim) // 16) * 16
        if cache_dim > 256:
            raise ValueError(f"a latent of {rank} with a rotated part of {rot_dim} is cached {cache_dim} "
                             "wide: at most 256")
        if rotary_layout not in ("neighbours", "halves"):
            raise ValueError(f"rotary_layout {rotary_layout!r}; known: neighbours, halves")
        self.width = width
        self.dtype = dtype
        self.heads = heads
        self.kv_heads = 1
        self.dim = dim
        self.rot_dim = rot_dim
        self.value_dim = value_dim
        self.rank = rank
        self.scale = float(scale)
        self.window = 0
        self.norm_eps = float(norm_eps)
        self.rotary_base = float(rotary_base)
        self.rotary_scaling = None if rotary_scaling is None else tuple(float(v) for v in rotary_scaling)
        self.rotary_halves = rotary_layout == "halves"
        self.score_cap = float(score_cap or 0.0)
        if self.score_cap < 0:
            raise ValueError("a score cap must be positive (0: none)")
        self.out_gate = bool(out_gate)
        self.query_rank = int(query_rank)
        if self.query_rank < 0:
            raise ValueError("query_rank must not be negative (0: queries straight from the input)")
        # what the cache and the attention kernels see
        self.head_dim = cache_dim
        self.q_cols = heads * cache_dim
        self.sink = None
        self.position = None
        # (the parent's path that merges key ranges inside the output projection is not taken:
        # the heads' value matrices and the gate lie between the attention and that projection)
        self.out_packed = None
        self._memo_in, self._memo_out, self._memo_attention = {}, {}, {}
        self._memo_query_down, self._memo_query_up = {}, {}

    def _columns(self):
        """First column of the queries, of [latent | rotated key part] and of the gates in the
        packed product, and its width.  Queries that come through a latent of their own are not
        in that product."""
        q_col = 0
        kv_col = q_col + (0 if self.query_rank else self.heads * (self.dim + self.rot_dim))
        gate_col = kv_col + self.rank + self.rot_dim
        return q_col, kv_col, gate_col, gate_col + (self.heads * self.value_dim if self.out_gate else 0)

    def parameters(self):
        params = self._own_parameters()
        if self.query_rank:
            params["query_down.weight"] = ParamSpec((self.query_rank, self.width), MATRIX)
            params["query_norm.gamma"] = ParamSpec((self.query_rank,), VECTOR)
            params["query_up.weight"] = ParamSpec((self.heads * (self.dim + self.rot_dim), self.query_rank), MATRIX)
        return params

    def _own_parameters(self):
        return {
            "in.weight": ParamSpec((self._columns()[3], self.width), MATRIX),
            "latent_norm.gamma": ParamSpec((self.rank,), VECTOR),
            "key_up.weight": ParamSpec((self.heads * self.dim, self.rank), MATRIX),
            "value_up.weight": ParamSpec((self.heads * self.value_dim, self.rank), MATRIX),
            "out.weight": ParamSpec((self.width, self.heads * self.value_dim), MATRIX),
        }

    def bind(self, tensors):
        self.in_weight = tensors["in.weight"]
        self.latent_gamma = tensors["latent_norm.gamma"]
        # a head's key matrix [dim, rank] turned: it takes the head's unrotated query to the latent's space
        self.query_to_latent = (tensors["key_up.weight"].view(self.heads, self.dim, self.rank)
                                .transpose(1, 2).contiguous())
        self.latent_to_value = tensors["value_up.weight"].view(self.heads, self.value_dim, self.rank).contiguous()
        self.out_weight = tensors["out.weight"]
        self.out_bias = None
        self.freqs = None
        self.rotary_magnitude = 1.0
        if self.rot_dim:
            freqs, self.rotary_magnitude = rotary_frequencies(self.rot_dim, self.rotary_base, self.rotary_scaling)
            self.freqs = freqs.to(torch.float32).to(self.out_weight.device)
        self.in_packed = kernels.pack_decode_weight(self.in_weight)
        self.out_projection_packed = kernels.pack_decode_weight(self.out_weight)
        if self.query_rank:
            self.query_down_weight = tensors["query_down.weight"]
            self.query_gamma = tensors["query_norm.gamma"]
            self.query_up_weight = tensors["query_up.weight"]
            self.query_down_packed = kernels.pack_decode_weight(self.query_down_weight)
            self.query_up_packed = kernels.pack_decode_weight(self.query_up_weight)
        for memo in (self._memo_in, self._memo_out, self._memo_attention, self._memo_query_down,
                     self._memo_query_up):
            memo.clear()

    def cache_spec(self):
        return PagedKVSpec(1, self.head_dim, 0, values_in_keys=True)

    def forward(self, x, residual, ctx, cache):
        if not cache.writes:
            raise NotImplementedError("a latent attention layer writes its own cache entry")
        tokens = ctx.tokens
        workspace = ctx.workspace
        tables = ctx.tables[cache.group]
        q_col, kv_col, gate_col, total = self._columns()
        proj, queries, _, gates = workspace.column_views(
            "latent_proj", total, torch.float32, tokens, (kv_col, gate_col - kv_col, total - gate_col))
        if self.query_rank:
            # the queries' own latent: its product in float, the norm inside the next product
            # where the kernel takes it (x may be a norm that has not run: run it once for both)
            if isinstance(x, kernels.PendingNorm):
                x = x.materialize()
            low = workspace.first_rows("latent_query_low", self.query_rank, torch.float32, tokens)
            kernels.linear(x, self.query_down_weight, None, low, packed=self.query_down_packed,
                           memo=site_memo(self._memo_query_down, workspace), shared=ctx.shared_calls)
            normed = kernels.PendingNorm(low, self.query_gamma, None, self.norm_eps, True,
                                         workspace.first_rows("latent_query_normed", self.query_rank,
                                                              self.dtype, tokens))
            queries = workspace.first_rows("latent_queries", self.heads * (self.dim + self.rot_dim),
                                           torch.float32, tokens)
            kernels.linear(normed, self.query_up_weight, None, queries, packed=self.query_up_packed,
                           memo=site_memo(self._memo_query_up, workspace), shared=ctx.shared_calls)
        kernels.linear(x, self.in_weight, None, proj, packed=self.in_packed,
                       memo=site_memo(self._memo_in, workspace), shared=ctx.shared_calls)
        q = workspace.first_rows("latent_q", self.q_cols, self.dtype, tokens)
        # every head's unrotated query part through its turned key matrix: the first `rank` places
        kernels.block_linear(queries, self.dim + self.rot_dim, self.query_to_latent, None, q, self.head_dim)
        kernels.latent_prepare(proj, q_col, kv_col, q, cache.k_pool, self.latent_gamma, self.norm_eps,
                               ctx.tok_item, ctx.positions, tables, self.heads, self.dim, self.rank,
                               freqs=self.freqs, rot_dims=self.rot_dim, halves=self.rotary_halves,
                               magnitude=self.rotary_magnitude,
                               queries=queries if self.query_rank else None)
        self._gates = gates if self.out_gate else None
        context = workspace.first_rows("latent_context", self.q_cols, self.dtype, tokens)
        return self._attend(q, context, None, residual, ctx, cache, tables)

    def _project_out(self, context, residual, ctx):
        # the weighted latents (the first `rank` places of a head's row) through the head's value
        # matrix, times the gate
        values = ctx.workspace.first_rows("latent_values", self.heads * self.value_dim, self.dtype, ctx.tokens)
        kernels.block_linear(context, self.head_dim, self.latent_to_value, None, values, self.value_dim,
                             gate=self._gates)
        kernels.linear(values, self.out_weight, None, residual, epilogue="residual",
                       packed=self.out_projection_packed, memo=site_memo(self._memo_out, ctx.workspace),
                       shared=ctx.shared_calls)
