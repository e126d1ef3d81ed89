"""Multi-head attention over the paged cache."""

import torch

from ..ops import kernels
from ..weights.loader import MATRIX, VECTOR, ParamSpec
from .base import Mixer, PagedKVSpec, site_memo
from .position import rotary_frequencies
from .registry import register_mixer


@register_mixer("attention")
class Attention(Mixer):
    """Packed QKV projection, cache write, attention over the request's cached keys,
    output projection added to the residual stream.

    One product gives ``[q | k | v]`` (src/model/paged_decoder.py:47-53); head ``j`` owns
    columns ``j*head_dim`` onward of each part (``:63-69``).  Keys and values of the
    step's tokens are stored before attention runs, so a token attends to itself and a
    prompt portion, a whole prompt and a decoded token are one case: every query at
    position p reads keys ``0..p`` (the last ``window`` of them) from the pages.
    ``scale`` multiplies the scores (``head_dim**-0.5`` in src/model/paged_attention.py:27).

    Options, all off by default; any of them puts one launch between the projection (then
    written in float) and the attention kernels (``kernels.attention_prepare``):

    * ``value_dim``: the values' head size where it is not the keys'.  Heads are then cached
      ``cache_dim`` wide (the larger size rounded up to 16, zeros behind), the one head size that
      the attention kernels see; the output projection gets zero columns to match.
    * ``qk_norm``: queries and keys are RMS-normed over the whole projection (all heads at
      once) with a weight per column (``q_norm.gamma``, ``k_norm.gamma``) and ``norm_eps``,
      before the rotation.
    * ``rotary_dims`` / ``rotary_base``: the first ``rotary_dims`` dimensions of every query
      and key head are rotated by the position, dimension 2i with 2i+1, angle ``p base^(-2i/dims)``.
    * ``sink``: a learned number per head (``sink``) whose exponential joins the softmax's
      denominator; it has no key and no value.
    * ``value_mix``: ``"source"`` leaves the step's values for later layers; ``"mix"`` caches
      ``(1 - l) v + l v_source`` with the learned ``value_mix.weight`` ``l`` and the source's
      values of the same token.
    * ``head_gate``: each head's output is multiplied by ``sigmoid`` of a projection of the
      layer's input (one more row per head in the packed product, ``[q | k | v | gate]``); the
      attention kernels do it where they store the output.
    * ``out_bias``: whether the output projection has a bias, where that differs from ``bias``
      (which then speaks for the packed projection alone).
    * ``rotary_layout``: ``"neighbours"`` (dimension 2i with 2i+1) or ``"halves"`` (dimension i
      with i + rotary_dims / 2); ``rotary_scaling = (factor, original, fast, slow)`` stretches
      the frequencies and scales cosine and sine (``parts/position.py: rotary_frequencies``).
    * ``head_norm``: after the rotation every query and key head is divided by its own root
      mean square (no weight, ``norm_eps``).
    * ``values_from_keys``: there is no value projection; the values are the keys as projected,
      before rotation and norm (the packed product is ``[q | k]``).
    * ``score_cap``: ``c > 0``: a scaled score ``s`` enters the softmax as ``c tanh(s / c)``.
    * ``pad_heads``: heads are cached with their size rounded up to a multiple of this (zeros
      behind), so that a head size which the tiled kernels do not take still runs on them.

    ``rotary_layout="halves"``, ``rotary_scaling``, ``head_norm`` and ``values_from_keys`` go
    through the launch that treats every head on its own (``kernels.attention_prepare_heads``);
    that one does not norm over the whole projection or mix values.
    """

    graph_safe = True

    accepts_pending_norm = True

    # decoded tokens and prompt portions of one step in one attention launch where the kernel
    # takes the shape (``kernels.attention_mixed``)
    fuse_mixed = True

    # the step's index arrays list the queries of a prompt portion in tiles of these sizes (the
    # tiled kernel's three; ``kernels.attention_prefill`` checks them against the library's)
    query_tile = (kernels.PREFILL_TILE, kernels.PREFILL_SMALL_TILE, kernels.PREFILL_LARGE_TILE)

    VALUE_MIXES = ("none", "source", "mix")

    def __init__(self, width: int, dtype, heads: int, kv_heads: int, head_dim: int, scale: float,
                 window: int = 0, bias: bool = True, value_dim: int = 0, qk_norm: bool = False,
                 norm_eps: float = 1e-6, rotary_dims: int = 0, rotary_base: float = 10000.0,
                 sink: bool = False, value_mix: str = "none", head_gate: bool = False,
                 out_bias=None, rotary_layout: str = "neighbours", rotary_scaling=None,
                 head_norm: bool = False, values_from_keys: bool = False, score_cap: float = 0.0,
                 pad_heads: int = 0):
        if heads % kv_heads != 0:
            raise ValueError(f"heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        if not 0 < head_dim <= 256:
            raise ValueError(f"head_dim {head_dim} must lie in 1..256")
        if not 0 <= value_dim <= 256:
            raise ValueError(f"value_dim {value_dim} must lie in 1..256")
        if value_mix not in self.VALUE_MIXES:
            raise ValueError(f"value_mix {value_mix!r}; known: {', '.join(self.VALUE_MIXES)}")
        if rotary_dims < 0 or rotary_dims % 2 or rotary_dims > head_dim:
            raise ValueError(f"rotary_dims {rotary_dims} must be even and at most head_dim {head_dim}")
        self.width = width
        self.dtype = dtype
        self.heads = heads
        self.kv_heads = kv_heads
        self.key_dim = head_dim
        self.value_dim = value_dim or head_dim
        self.scale = float(scale)
        self.window = int(window)
        self.bias = bias
        # (the output projection's bias goes with the packed projection's unless named apart)
        self.out_has_bias = bool(bias) if out_bias is None else bool(out_bias)
        self.qk_norm = bool(qk_norm)
        self.norm_eps = float(norm_eps)
        self.rotary_dims = int(rotary_dims)
        self.rotary_base = float(rotary_base)
        self.has_sink = bool(sink)
        self.value_mix = value_mix
        self.head_gate = bool(head_gate)
        if rotary_layout not in ("neighbours", "halves"):
            raise ValueError(f"rotary_layout {rotary_layout!r}; known: neighbours, halves")
        self.rotary_halves = rotary_layout == "halves"
        self.rotary_scaling = None if rotary_scaling is None else tuple(float(v) for v in rotary_scaling)
        self.head_norm = bool(head_norm)
        self.values_from_keys = bool(values_from_keys)
        self.score_cap = float(score_cap or 0.0)
        if self.score_cap < 0:
            raise ValueError("a score cap must be positive (0: none)")
        if self.values_from_keys and self.value_dim != self.key_dim:
            raise ValueError("values that are the keys have the keys' head size")
        # the launch that treats every head on its own
        self.head_wise = (self.head_norm or self.values_from_keys or self.rotary_scaling is not None
                          or (self.rotary_halves and self.rotary_dims > 0))
        if self.head_wise and (self.qk_norm or value_mix != "none"):
            raise ValueError("a norm over the whole projection and mixed values do not go with "
                             "rotary halves, scaled frequencies, head norms or values from keys")
        self.prepared = (self.value_dim != self.key_dim or self.qk_norm or self.rotary_dims > 0
                         or value_mix != "none" or self.head_gate or self.head_wise
                         or (pad_heads > 1 and head_dim % pad_heads != 0))
        # the head size that the cache and the attention kernels see
        self.head_dim = head_dim
        if self.value_dim != self.key_dim:
            self.head_dim = -(-max(self.key_dim, self.value_dim) // 16) * 16
        elif self.prepared and head_dim % 2:
            self.head_dim = head_dim + 1
        if pad_heads > 1:
            self.head_dim = -(-self.head_dim // pad_heads) * pad_heads
        if self.head_dim > 256:
            raise ValueError(f"heads of {head_dim} cached {self.head_dim} wide: at most 256")
        self.q_cols = heads * self.head_dim         # columns of the queries and of the context
        self.kv_cols = kv_heads * self.head_dim
        self.sink = None
        self.position = None
        # what ``kernels.linear`` keeps per call site and step shape (its ``memo``), per workspace
        self._memo_qkv, self._memo_out, self._memo_attention = {}, {}, {}

    def _projection_columns(self):
        """First column of the queries, keys, values and gates in the packed product, and its width."""
        q_col = 0
        k_col = q_col + self.heads * self.key_dim
        v_col = k_col + self.kv_heads * self.key_dim
        if self.values_from_keys:
            # (no value columns: the key columns are read twice)
            gate_col = v_col
            return q_col, k_col, k_col, gate_col, gate_col + (self.heads if self.head_gate else 0)
        gate_col = v_col + self.kv_heads * self.value_dim
        return q_col, k_col, v_col, gate_col, gate_col + (self.heads if self.head_gate else 0)

    def parameters(self):
        total = self._projection_columns()[4]
        params = {
            "qkv.weight": ParamSpec((total, self.width), MATRIX),
            "out.weight": ParamSpec((self.width, self.heads * self.value_dim), MATRIX),
        }
        if self.bias:
            params["qkv.bias"] = ParamSpec((total,), VECTOR)
        if self.out_has_bias:
            params["out.bias"] = ParamSpec((self.width,), VECTOR)
        if self.qk_norm:
            params["q_norm.gamma"] = ParamSpec((self.heads * self.key_dim,), VECTOR)
            params["k_norm.gamma"] = ParamSpec((self.kv_heads * self.key_dim,), VECTOR)
        if self.has_sink:
            params["sink"] = ParamSpec((self.heads,), VECTOR)
        if self.value_mix == "mix":
            params["value_mix.weight"] = ParamSpec((), VECTOR)
        return params

    def bind(self, tensors):
        self.qkv_weight = tensors["qkv.weight"]
        self.out_weight = tensors["out.weight"]
        self.qkv_bias = tensors.get("qkv.bias")
        self.out_bias = tensors.get("out.bias")
        self.q_gamma = tensors.get("q_norm.gamma")
        self.k_gamma = tensors.get("k_norm.gamma")
        self.sink = tensors.get("sink")
        self.mix_weight = tensors["value_mix.weight"].reshape(1) if self.value_mix == "mix" else None
        if self.head_dim != self.value_dim:
            # heads are cached wider than the values: the context has zero columns there, and
            # the output projection gets zero columns to match
            padded = self.out_weight.new_zeros((self.width, self.heads, self.head_dim))
            padded[:, :, :self.value_dim] = self.out_weight.view(self.width, self.heads, self.value_dim)
            self.out_weight = padded.view(self.width, self.q_cols)
        self.freqs = None
        self.rotary_magnitude = 1.0
        if self.rotary_dims:
            # base^(-2i/dims), worked out in 64-bit and rounded once; the angle is float(p) * f
            freqs, self.rotary_magnitude = rotary_frequencies(self.rotary_dims, self.rotary_base,
                                                              self.rotary_scaling)
            self.freqs = freqs.to(torch.float32).to(self.out_weight.device)
        # copies in the layout that the products of few rows (decode steps) read fastest
        self.qkv_packed = kernels.pack_decode_weight(self.qkv_weight)
        self.out_packed = kernels.pack_decode_weight(self.out_weight)
        self._memo_qkv.clear()
        self._memo_out.clear()
        self._memo_attention.clear()

    def cache_spec(self):
        return PagedKVSpec(self.kv_heads, self.head_dim, self.window)

    def _project_prepared(self, x, ctx, cache, tables):
        """Projection in float, then norm, rotation, value mixing and cache write in one launch;
        returns the queries (engine dtype, heads ``head_dim`` wide) and the gates' columns."""
        if not cache.writes:
            raise NotImplementedError("an attention layer with prepared queries and keys writes its own cache entry")
        tokens = ctx.tokens
        q_col, k_col, v_col, gate_col, total = self._projection_columns()
        proj = ctx.workspace.first_rows("attn_proj", total, torch.float32, tokens)
        kernels.linear(x, self.qkv_weight, self.qkv_bias, proj, packed=self.qkv_packed,
                       memo=site_memo(self._memo_qkv, ctx.workspace), shared=ctx.shared_calls)
        q = ctx.workspace.first_rows("attn_q", self.q_cols, self.dtype, tokens)
        v_first = None
        if self.value_mix != "none":
            v_first = ctx.workspace.first_rows("values_source", self.kv_heads * self.value_dim,
                                               self.dtype, tokens)
        if self.head_wise:
            kernels.attention_prepare_heads(
                proj, (q_col, k_col, v_col), q, cache.k_pool, cache.v_pool, ctx.tok_item, ctx.positions,
                tables, self.heads, self.key_dim, self.value_dim, freqs=self.freqs,
                rot_dims=self.rotary_dims, halves=self.rotary_halves, magnitude=self.rotary_magnitude,
                head_norm=self.head_norm, eps=self.norm_eps)
            return q, (proj[:, gate_col:gate_col + self.heads] if self.head_gate else None)
        kernels.attention_prepare(
            proj, (q_col, k_col, v_col), q, cache.k_pool, cache.v_pool, ctx.tok_item, ctx.positions,
            tables, self.heads, self.key_dim, self.value_dim, q_gamma=self.q_gamma,
            k_gamma=self.k_gamma, eps=self.norm_eps, freqs=self.freqs, rot_dims=self.rotary_dims,
            v_first=v_first, v_lambda=self.mix_weight,
            v_mode=self.VALUE_MIXES.index(self.value_mix))
        return q, (proj[:, gate_col:gate_col + self.heads] if self.head_gate else None)

    def _project_out(self, context, residual, ctx):
        kernels.linear(context, self.out_weight, self.out_bias, residual, epilogue="residual",
                       packed=self.out_packed, memo=site_memo(self._memo_out, ctx.workspace),
                       shared=ctx.shared_calls)

    def forward(self, x, residual, ctx, cache):
        tokens = ctx.tokens
        tables = ctx.tables[cache.group]
        gates = None
        if self.prepared:
            q, gates = self._project_prepared(x, ctx, cache, tables)
        else:
            q = self._project_plain(x, ctx, cache, tables)
        context = ctx.workspace.first_rows("attn", self.q_cols, self.dtype, tokens)
        return self._attend(q, context, gates, residual, ctx, cache, tables)

    def _project_plain(self, x, ctx, cache, tables):
        tokens = ctx.tokens
        total = self.q_cols + 2 * self.kv_cols
        # (the step's rows and their three column views, made once per row count for all layers)
        qkv, q, k, v = ctx.workspace.column_views("qkv", total, self.dtype, tokens,
                                                  (self.q_cols, self.kv_cols, self.kv_cols))
        rotates = self.position is not None and self.position.transforms_qk
        if cache.writes and not rotates:
            # keys and values go to their pages from the product's own epilogue
            kernels.linear(x, self.qkv_weight, self.qkv_bias, qkv,
                           scatter=(cache.k_pool, cache.v_pool, ctx.tok_item, ctx.positions, tables,
                                    self.q_cols, self.kv_cols), packed=self.qkv_packed,
                           scatter_only=True, memo=site_memo(self._memo_qkv, ctx.workspace),
                           shared=ctx.shared_calls)
        else:
            kernels.linear(x, self.qkv_weight, self.qkv_bias, qkv, packed=self.qkv_packed,
                           memo=site_memo(self._memo_qkv, ctx.workspace),
                           shared=ctx.shared_calls)
            if rotates:
                self.position.apply_to_qk(q, k, ctx)
            if cache.writes:
                kernels.kv_write(k, v, cache.k_pool, cache.v_pool, ctx.tok_item, ctx.positions,
                                 tables)
        return q

    def _attend(self, q, context, gates, residual, ctx, cache, tables):
        tokens = ctx.tokens
        sink = self.sink
        singles = ctx.single_tokens.numel() if ctx.single_tokens is not None else 0
        if not kernels.decode_supported(self.head_dim):
            # a head size that the split-KV kernel does not take: every token, decoded ones
            # too, goes to the kernel that takes all sizes
            singles = 0
        merged_splits = 0
        if gates is None and singles == tokens and kernels.merge_linear_supported(
                self.dtype, tokens, self.head_dim, self.out_packed):
            merged_splits = self._merged_splits(singles, ctx.max_kv_len)
        if merged_splits:
            # a decode step of few tokens over long contexts: the key ranges are merged inside
            # the output projection, which is split over the heads: no launch for the merge
            splits = merged_splits
            partial = self._range_records(ctx)
            kernels.attention_decode_partial(q, cache.k_pool, cache.v_pool, partial, ctx.tok_item,
                                             ctx.positions, tables, self.heads, self.scale, splits,
                                             window=self.window, waves=4, sink=sink, softcap=self.score_cap)
            kernels.attention_merge_linear(partial, singles, self.heads, self.head_dim, splits,
                                           self.out_weight, self.out_packed, self.out_bias, residual)
            return
        tiled = singles < tokens and kernels.prefill_supported(self.dtype, self.head_dim, tables.shape[1])
        if singles and tiled and self._one_launch(singles, ctx, tables):
            # decoded tokens beside prompt portions: one launch whose blocks are of both kinds
            tile_item, tile_q0 = ctx.query_tiles[kernels.PREFILL_TILE]
            kernels.attention_mixed(q, cache.k_pool, cache.v_pool, context, ctx.single_tokens,
                                    ctx.tok_item, ctx.positions, tile_item, tile_q0, ctx.cu_tokens,
                                    ctx.kv_lens, tables, self.heads, self.scale, self.window,
                                    memo=site_memo(self._memo_attention, ctx.workspace),
                                    shared=ctx.shared_calls, sink=sink, gate=gates, softcap=self.score_cap)
            return self._project_out(context, residual, ctx)
        if singles and kernels.shared_decode_supported(self.dtype, self.heads, self.kv_heads, self.head_dim, sink):
            # many heads to a key/value head: blocks that load a tile of keys once for all of them
            kernels.attention_decode_shared(q, cache.k_pool, cache.v_pool, context,
                                            None if singles == tokens else ctx.tok_item, ctx.positions,
                                            tables, self.heads, self.scale,
                                            self._shared_splits(singles, ctx.max_kv_len),
                                            self._range_records(ctx), window=self.window,
                                            tok_list=None if singles == tokens else ctx.single_tokens,
                                            gate=gates, softcap=self.score_cap)
        elif singles:
            # one-token items: keys of a request are cut into ranges so that few requests
            # still fill the chip
            splits, waves = self._splits(singles, ctx.max_kv_len)
            partial = None
            if splits > 1:
                partial = self._range_records(ctx)
            # in a step of single tokens only, token t is item t: without the index the kernel
            # asks for its block table a trip to memory earlier (64 requests of 12 heads: 1.6 %
            # of the step).  The path above, of few blocks with one or two pages each, measured
            # 0.6 % slower with it, and so did a grid of more than four blocks per compute unit,
            # which waits for bytes and not for a trip (64 requests of 25 heads: 1 us a launch):
            # both keep the index.
            direct = (singles == tokens
                      and singles * self.heads * splits <= 4 * kernels.compute_units())
            kernels.attention_decode(q, cache.k_pool, cache.v_pool, context,
                                     None if direct else ctx.tok_item,
                                     ctx.positions, tables, self.heads, self.scale, splits,
                                     partial=partial, window=self.window, waves=waves,
                                     tok_list=None if singles == tokens else ctx.single_tokens,
                                     sink=sink, gate=gates, softcap=self.score_cap)
        whole = singles == 0
        if tiled:
            size = kernels.PREFILL_TILE
            tile_item, tile_q0 = ctx.query_tiles[size]
            if kernels.prefill_small_tile_pays(self.heads, self.head_dim, tile_item.numel()):
                size = kernels.PREFILL_SMALL_TILE
                tile_item, tile_q0 = ctx.query_tiles[size]
            elif kernels.prefill_large_tile_pays(self.heads, self.head_dim,
                                                 ctx.query_tiles[kernels.PREFILL_LARGE_TILE][0].numel(),
                                                 ctx.max_kv_len):
                size = kernels.PREFILL_LARGE_TILE
                tile_item, tile_q0 = ctx.query_tiles[size]
            kernels.attention_prefill(q, cache.k_pool, cache.v_pool, context, tile_item,
                                      tile_q0, ctx.cu_tokens, ctx.kv_lens, tables,
                                      self.heads, self.scale, self.window,
                                      max_kv_len=ctx.max_kv_len, query_tile=size,
                                      memo=site_memo(self._memo_attention, ctx.workspace),
                                      shared=ctx.shared_calls, sink=sink, gate=gates, softcap=self.score_cap)
        elif singles < tokens and kernels.tiled_f32_supported(self.dtype, self.head_dim):
            # 32-bit: tiles of queries too, on plain float arithmetic.  The tiles hold the items
            # of several tokens; one-token items that the split-KV kernel did not take (a head
            # size that it refuses) go to the kernel that takes all sizes
            tile_item, tile_q0 = ctx.query_tiles[kernels.PREFILL_TILE]
            if tile_item.numel():
                kernels.attention_tiled_f32(q, cache.k_pool, cache.v_pool, context, tile_item, tile_q0,
                                            ctx.cu_tokens, ctx.kv_lens, tables, self.heads, self.scale,
                                            self.window, sink=sink, gate=gates, softcap=self.score_cap)
            if not singles and ctx.single_tokens is not None and ctx.single_tokens.numel():
                kernels.attention_rowwise(q, cache.k_pool, cache.v_pool, context, ctx.tok_item,
                                          ctx.positions, tables, self.heads, self.scale, self.window,
                                          tok_list=None if ctx.single_tokens.numel() == tokens
                                          else ctx.single_tokens, sink=sink, gate=gates, softcap=self.score_cap)
        elif singles < tokens:
            kernels.attention_rowwise(q, cache.k_pool, cache.v_pool, context, ctx.tok_item,
                                      ctx.positions, tables, self.heads, self.scale, self.window,
                                      tok_list=None if whole else ctx.portion_tokens, sink=sink, gate=gates, softcap=self.score_cap)
        self._project_out(context, residual, ctx)

    def _one_launch(self, singles: int, ctx, tables) -> bool:
        """Whether a step's one-token items and its items of several tokens go to the kernel
        that runs both kinds of block in one grid: where it takes the shape, where the prompts
        are not so long that tiles of 128 queries are the better cut, and not where a handful
        of tokens is decoded over long contexts.  Its decode blocks are of four waves over all
        keys of a request, also where the decode kernel alone would run ranges or blocks of
        sixteen waves: beside the tiles' blocks they are not what the launch waits for (a
        portion of 512 beside 8 tokens over 900 keys: the step 0.978 against 1.005 ms at GPT-2
        small shape, 16 over 300 keys 0.90 against 0.99, 24 over 600 keys 0.97 against 1.08; at
        medium shape 16 over 900 keys 2.24 against 2.34), unless they are so few that their
        eight rounds of loads are (2 and 4 tokens over 900 keys: 0.956 against 0.946 and 0.974
        against 0.958 ms)."""
        if not (self.fuse_mixed and kernels.mixed_supported(self.dtype, self.head_dim, tables.shape[1])):
            return False
        visible = ctx.max_kv_len if self.window <= 0 else min(ctx.max_kv_len, self.window)
        if 4 * singles * self.heads < kernels.compute_units() and visible > 512:
            return False
        large_tiles = ctx.query_tiles[kernels.PREFILL_LARGE_TILE][0].numel()
        return not kernels.prefill_large_tile_pays(self.heads, self.head_dim, large_tiles, ctx.max_kv_len)

    def _range_records(self, ctx):
        """Scratch for one record per (token, head, key range): always asked for at its largest
        (both rules below keep tokens x heads x ranges under six blocks per compute unit beside
        one per pair), so that it never moves under the launches that recorded steps hold.
        Layers of equal heads and head size share one buffer; a layer of other sizes has its
        own, so that no layer makes another's grow."""
        worst = ((6 * kernels.compute_units() + ctx.workspace.max_rows * self.heads)
                 * (self.head_dim + 2))
        return ctx.workspace.flat(f"attn_partial_{self.heads}x{self.head_dim}", worst, torch.float32)

    def _merged_splits(self, count: int, max_kv_len: int) -> int:
        """Ranges per request for the path that merges them inside the output projection, or 0
        where the other path is as fast or faster: more (token, head) pairs than three quarters
        of the compute units (16 requests of 12 heads still gain 2 %), and, from half a pair
        per unit on, contexts that feed fewer than three ranges (16 requests over 100 keys:
        3 % slower).  Fewer pairs take this path at every length, also with a single range:
        the other path would cut 130 to 250 keys into two ranges and merge them with a launch
        of its own (1 to 4 requests over 20 to 250 keys: 5 % of the step, 8 requests 2 %).
        About three blocks of four waves per compute unit, never more ranges than the keys of
        the longest request can feed; and not where the projection's blocks would read more
        than 12 MB of records between them (wide models)."""
        visible = max_kv_len if self.window <= 0 else min(max_kv_len, self.window)
        pairs = count * self.heads
        units = kernels.compute_units()
        most = max(1, -(-visible // kernels.decode_keys_per_block(self.head_dim, 4)))
        if pairs > units * 3 // 4 or (most < 3 and 2 * pairs > units):
            return 0
        wanted = max(1, -(-3 * units // pairs))
        splits = min(most, wanted, 64)
        # Every block of 16 output columns merges the records of its head again: together they
        # read the records as often as the projection has column tiles, which grows with the
        # square of the heads.  Beyond some 12 MB of that the other path is ahead (decode steps
        # over 1,024 keys, merged against not: 8 requests of 16 heads, 12.3 MB, 0.837 against
        # 0.821 ms; 4 of 25 heads, 21 MB, 2.089 against 1.995; under it 4 requests of 16 heads
        # 0.724 against 0.771, 2 of 25 heads 1.903 against 1.951, 16 of 12 heads 2 % ahead).
        tiles = -(-self.width // 16)
        if tiles * pairs * splits * (self.head_dim + 2) * 4 > 12_000_000:
            return 0
        return splits

    def _shared_splits(self, count: int, max_kv_len: int) -> int:
        """Ranges per request of the decode kernel whose blocks serve a group's heads together:
        about two blocks per compute unit, no range shorter than a tile of keys, and never more
        records than the scratch holds (six per unit beside one per token and head)."""
        visible = max_kv_len if self.window <= 0 else min(max_kv_len, self.window)
        units = kernels.compute_units()
        group = self.heads // self.kv_heads
        blocks = count * self.kv_heads * -(-group // kernels.SHARED_DECODE_HEADS)
        wanted = -(-2 * units // blocks)
        most = -(-visible // kernels.SHARED_DECODE_KEYS)
        room = 1 + 6 * units // (count * self.heads)
        return max(1, min(wanted, most, room, 64))

    def _splits(self, count: int, max_kv_len: int):
        """(ranges per request, waves per block) of the decode kernel, by the number of (token,
        head) pairs per compute unit and the keys that a query sees:

        * from three and a half pairs per unit: one block of 4 waves per pair fills the chip;
        * from one and a half: the same at short contexts; from 2,048 keys on a handful of long
          blocks per unit would leave units idle towards the end, so the keys are cut into
          ranges until six blocks come to a unit;
        * between one and one and a half: blocks of 16 waves would come two to some units and
          one to the others, and the kernel would last as long as the units with two (24
          requests of 12 heads at 1,000 keys: 22.3 us): ranges of 4-wave blocks, four blocks to a
          unit (19.0 us with the launch that merges them), six over thousands of keys;
        * up to one pair per unit: one block of 16 waves takes a whole request's keys and no
          second launch is needed (two or three such blocks per request while each still has
          a unit of its own); just under a pair per unit and from 4,096 keys on, ranges of
          4-wave blocks are ahead again;
        * few pairs: ranges of 4-wave blocks until four blocks come to a unit.

        Never more ranges than the keys of the longest request can feed, and never more than
        six blocks per unit beside one per pair (the scratch for the records is sized for
        that)."""
        visible = max_kv_len if self.window <= 0 else min(max_kv_len, self.window)
        pairs = count * self.heads
        units = kernels.compute_units()
        if 2 * pairs >= 7 * units:
            return 1, 4
        if pairs >= units + units // 2:
            # One block of 4 waves per pair fills the chip at short contexts.  At long ones a
            # handful of blocks per unit, each walking thousands of keys, leaves units idle
            # towards the end: ranges until six blocks come to a unit (32 requests of 12 heads
            # at 8,192 keys: 126 instead of 172 us), none under 2,048 keys.
            return max(1, min(-(-6 * units // pairs), visible // 1024)), 4
        if pairs > units:
            # (four blocks to a unit, six over thousands of keys)
            blocks = (6 if visible >= 4096 else 4) * units
            return max(1, min(-(-blocks // pairs), visible // 256)), 4
        if 4 * pairs >= 3 * units and visible >= 4096:
            # nearly a pair per unit over thousands of keys: six blocks of 4 waves to a unit are
            # ahead of one block of 16 waves per pair (17 requests of 12 heads at 4,096 keys:
            # 41.4 against 44.2 us, at 16,384 keys 141 against 155)
            return min(-(-6 * units // pairs), 64), 4
        if pairs >= units // 4 and visible > kernels.decode_keys_per_block(self.head_dim, 4):
            # contexts of several thousand keys: two or three such blocks per request, as
            # long as every block still has a compute unit of its own
            return max(1, min(units // pairs, visible // 1024)), 16
        most = max(1, -(-visible // kernels.decode_keys_per_block(self.head_dim, 4)))
        wanted = max(1, -(-4 * units // pairs))
        return min(most, wanted, 64), 4
