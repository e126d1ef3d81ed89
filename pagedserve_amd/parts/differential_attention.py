"""Differential attention: two softmax maps per head over the same values, the second taken off
the first."""

import torch

from ..ops import kernels
from ..weights.loader import MATRIX, VECTOR, ParamSpec
from .attention import Attention
from .base import PagedKVSpec, site_memo
from .registry import register_mixer


@register_mixer("differential_attention")
class DifferentialAttention(Attention):
    """Attention whose heads each run two maps of queries and keys over one set of values
    (Ye et al., "Differential Transformer").  With ``h`` the layer's input, H heads, G key/value
    heads (head j reads key/value head ``j // (H / G)``):

        q = W_q h   [H, 2, dim]      k = W_k h   [G, 2, dim]      v = W_v h   [G, vdim]
        a_m = softmax_window((q_m . k_m) * scale) v             m = 0, 1, the same v for both
        o = a_0 - lambda a_1,   lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff
        o <- o / sqrt(mean(o^2) + eps) * (1 - diff)             per head, no weight
        out = W_o (concat(o) * sigmoid(W_g h))                  (``out_gate``)

    No positions enter the scores.  ``window``: a query sees itself and the ``window - 1`` tokens
    before it (0: all).  The attention kernels see ``2 H`` query heads, one per map.  Where the two
    maps' keys fit one cached head (``2 dim <= 256``) a key/value head is cached once: its two
    maps' keys side by side, ``[k_0 | k_1]``, and its values, both ``max(2 dim, vdim)`` rounded
    up to 16 wide; the query of map m stands at the places of ``k_m`` with zeros elsewhere, so its
    product with the cached row is its own map's score, and the ``2 H / G`` query heads of a
    key/value head read the same rows (head j's map m is the kernels' head ``2 j + m``).  Wider
    maps are cached apart, ``2 G`` key/value heads of ``max(dim, vdim)``, map-major (map m of head
    j is the kernels' head ``m H + j``, of key head g their ``m G + g``, so that grouped heads
    still find their key head by one division), the values of head g under both of its maps.
    One launch behind the attention kernels takes the difference, norms, scales and gates
    (``kernels.differential_combine``); scores, softmax, the difference, the norm and the sigmoid
    are 32-bit.

    ``reads_cache``: the layer has no key and value projections and reads the cache entry that
    another layer of the same geometry writes (``LayerCall.writes_cache = False``), with its own
    queries, window and constants.  ``cache_window``: the window of the cache entry where that is
    not the layer's own (an entry that layers with different windows read keeps the widest)."""

    graph_safe = True
    accepts_pending_norm = True

    def __init__(self, width: int, dtype, heads: int, kv_heads: int, head_dim: int, value_dim: int,
                 scale: float, diff: float, window: int = 0, norm_eps: float = 1e-6,
                 out_gate: bool = True, reads_cache: bool = False, cache_window=None):
        if heads % kv_heads != 0:
            raise ValueError(f"heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        if not 0 < head_dim <= 256 or not 0 < value_dim <= 256:
            raise ValueError(f"head sizes {head_dim} and {value_dim} must lie in 1..256")
        self.width = width
        self.dtype = dtype
        self.maps = 2
        self.true_heads = heads
        self.true_kv_heads = kv_heads
        # what the attention kernels see
        self.map_dim = head_dim
        self.value_dim = value_dim
        self.heads = self.maps * heads
        self.packed = self.maps * head_dim <= 256
        if self.packed:
            self.kv_heads = kv_heads
            self.key_dim = self.maps * head_dim
        else:
            self.kv_heads = self.maps * kv_heads
            self.key_dim = head_dim
        self.head_dim = -(-max(self.key_dim, value_dim) // 16) * 16
        self.scale = float(scale)
        self.diff = float(diff)
        self.window = int(window)
        self.cache_window = self.window if cache_window is None else int(cache_window)
        if self.cache_window and (self.window == 0 or self.window > self.cache_window):
            raise ValueError(f"a window of {self.window or 'all'} keys does not fit a cache entry that keeps "
                             f"{self.cache_window}")
        self.norm_eps = float(norm_eps)
        self.out_gate = bool(out_gate)
        self.reads_cache = bool(reads_cache)
        self.q_cols = self.heads * self.head_dim
        self.kv_cols = self.kv_heads * self.head_dim
        self.score_cap = 0.0
        self.sink = None
        self.position = None
        # (key ranges are never merged inside the output projection: the difference of the maps
        # lies between the attention and that projection)
        self.out_packed = None
        self._memo_qkv, self._memo_out, self._memo_attention = {}, {}, {}

    def _projection_columns(self):
        """First column of the queries, keys, values and gates in the packed product, and its width."""
        q_col = 0
        k_col = q_col + self.heads * self.map_dim
        v_col = k_col + (0 if self.reads_cache else self.maps * self.true_kv_heads * self.map_dim)
        gate_col = v_col + (0 if self.reads_cache else self.true_kv_heads * self.value_dim)
        return q_col, k_col, v_col, gate_col, gate_col + (self.true_heads * self.value_dim if self.out_gate else 0)

    def parameters(self):
        params = {
            "qkv.weight": ParamSpec((self._projection_columns()[4], self.width), MATRIX),
            "out.weight": ParamSpec((self.width, self.true_heads * self.value_dim), MATRIX),
        }
        for name in ("lambda_q1", "lambda_k1", "lambda_q2", "lambda_k2"):
            params[name] = ParamSpec((self.map_dim,), VECTOR)
        return params

    def _map_major(self, rows, heads):
        """Rows laid out head by head as [map 0 | map 1] into all heads' map 0, then their map 1."""
        return (rows.view(heads, self.maps, self.map_dim, -1).transpose(0, 1)
                .reshape(heads * self.maps * self.map_dim, -1))

    def bind(self, tensors):
        stored = tensors["qkv.weight"]
        q_col, k_col, v_col, _, _ = self._projection_columns()
        weight = stored
        if not self.packed:
            weight = stored.clone()
            weight[q_col:k_col] = self._map_major(stored[q_col:k_col], self.true_heads)
            if not self.reads_cache:
                weight[k_col:v_col] = self._map_major(stored[k_col:v_col], self.true_kv_heads)
        self.qkv_weight = weight
        self.out_weight = tensors["out.weight"]
        # one number for the layer, worked out once in 32-bit
        first = (tensors["lambda_q1"].float() * tensors["lambda_k1"].float()).sum()
        second = (tensors["lambda_q2"].float() * tensors["lambda_k2"].float()).sum()
        self.lam = (torch.exp(first) - torch.exp(second) + self.diff).reshape(1).to(torch.float32).contiguous()
        self.qkv_packed = kernels.pack_decode_weight(self.qkv_weight)
        self.out_projection_packed = kernels.pack_decode_weight(self.out_weight)
        for memo in (self._memo_qkv, self._memo_out, self._memo_attention):
            memo.clear()

    def cache_spec(self):
        return PagedKVSpec(self.kv_heads, self.head_dim, self.cache_window)

    def forward(self, x, residual, ctx, cache):
        if cache.writes == self.reads_cache:
            raise ValueError("a differential layer with key and value projections writes its cache entry, "
                             "one without reads another layer's")
        tokens = ctx.tokens
        workspace = ctx.workspace
        tables = ctx.tables[cache.group]
        q_col, k_col, v_col, gate_col, total = self._projection_columns()
        proj, _, gates = workspace.column_views("diff_proj", total, torch.float32, tokens,
                                                (gate_col, total - gate_col))
        kernels.linear(x, self.qkv_weight, None, proj, packed=self.qkv_packed,
                       memo=site_memo(self._memo_qkv, workspace), shared=ctx.shared_calls)
        q = workspace.first_rows("attn_q", self.q_cols, self.dtype, tokens)
        kernels.attention_prepare(proj, (q_col, k_col, v_col), q, cache.k_pool, cache.v_pool, ctx.tok_item,
                                  ctx.positions, tables, self.heads, self.key_dim, self.value_dim,
                                  value_heads=self.true_kv_heads, store=not self.reads_cache,
                                  query_maps=self.maps if self.packed else 1)
        self._gates = gates if self.out_gate else None
        context = workspace.first_rows("attn", self.q_cols, self.dtype, tokens)
        return self._attend(q, context, None, residual, ctx, cache, tables)

    def _attend(self, q, context, gates, residual, ctx, cache, tables):
        """Steps of decoded tokens only: the split-KV kernels leave their records per key range and
        one launch merges the ranges of both maps, takes the difference, norms and gates
        (``kernels.differential_merge``).  Other steps take the parent's dispatch and the launch
        that works on the attention's output rows."""
        tokens = ctx.tokens
        singles = ctx.single_tokens.numel() if ctx.single_tokens is not None else 0
        if singles != tokens or not kernels.decode_supported(self.head_dim):
            return super()._attend(q, context, gates, residual, ctx, cache, tables)
        records = self._range_records(ctx)
        if kernels.shared_decode_supported(self.dtype, self.heads, self.kv_heads, self.head_dim, None):
            # many query heads (two maps of every head) to a key/value head: a tile of keys is
            # loaded once for all of them
            splits = self._shared_splits(singles, ctx.max_kv_len)
            kernels.attention_decode_shared(q, cache.k_pool, cache.v_pool, None, None, ctx.positions, tables,
                                            self.heads, self.scale, splits, records, window=self.window)
        else:
            splits, waves = self._splits(singles, ctx.max_kv_len)
            kernels.attention_decode_partial(q, cache.k_pool, cache.v_pool, records, None, ctx.positions,
                                             tables, self.heads, self.scale, splits, window=self.window,
                                             waves=waves)
        values = ctx.workspace.first_rows("diff_values", self.true_heads * self.value_dim, self.dtype, tokens)
        kernels.differential_merge(records, tokens, splits, self.lam, 1.0 - self.diff, self.norm_eps,
                                   self._gates, values, self.true_heads, self.value_dim, self.head_dim,
                                   map_major=not self.packed)
        self._project_values(values, residual, ctx)

    def _project_out(self, context, residual, ctx):
        values = ctx.workspace.first_rows("diff_values", self.true_heads * self.value_dim, self.dtype, ctx.tokens)
        kernels.differential_combine(context, self.lam, 1.0 - self.diff, self.norm_eps, self._gates, values,
                                     self.true_heads, self.value_dim, self.head_dim, map_major=not self.packed)
        self._project_values(values, residual, ctx)

    def _project_values(self, values, residual, ctx):
        kernels.linear(values, self.out_weight, None, residual, epilogue="residual",
                       packed=self.out_projection_packed, memo=site_memo(self._memo_out, ctx.workspace),
                       shared=ctx.shared_calls)
