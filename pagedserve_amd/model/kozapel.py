"""Kozapel as data: a decoder whose layers are listed one by one in its configuration.

The scaled token embedding fills a residual stream that is kept in several copies; every
sublayer reads a weighted sum of the copies through an RMS norm (plain scale) and its result is
mixed back into all of them.  The mixer of a layer is one of

* ``attention``: differential attention (two softmax maps per head over the same values, the
  second taken off the first, a norm per head, a sigmoid gate on the heads' outputs) with
  grouped heads under a sliding window and no positions; a layer may read the keys and values
  that an earlier layer cached instead of projecting its own;
* ``latent_attention``: attention over a cached latent with a shared rotated key part, the
  queries through a latent of their own.

The feed-forward is gated with the tanh form of gelu, or a mixture of experts (sigmoid scores,
a correction per expert for the choice, groups scored by their two best, normalised weights,
squared-ReLU experts, one shared expert).  The final norm is followed by a head matrix of its own.
"""

import math

import torch

from ..config.kozapel import KozapelConfig
from ..config.registry import Architecture, register_architecture
from ..config.spec import BlockSpec, LayerCall, ModelSpec, PartSpec
from ..weights.loader import WeightSource

# a group of experts is scored by the sum of this many of its largest choice scores
GROUP_TOP = 2


def _mixer_spec(config, index, layer):
    mixer = layer.mixer
    if layer.type == "attention":
        source = index if mixer.kv_from is None else mixer.kv_from
        return PartSpec.make(
            "differential_attention", heads=mixer.heads, kv_heads=mixer.kv_heads, head_dim=mixer.dim,
            value_dim=mixer.vdim, scale=mixer.scale, diff=mixer.diff, window=mixer.window,
            norm_eps=config.norm_eps, out_gate=True, reads_cache=mixer.kv_from is not None,
            cache_window=config.cache_window(source))
    return PartSpec.make(
        "latent_attention", heads=mixer.heads, dim=mixer.dim, rot_dim=mixer.rot_dim,
        value_dim=mixer.vdim, rank=mixer.kv_rank, scale=mixer.scale, norm_eps=config.norm_eps,
        rotary_base=mixer.rot_base, rotary_layout="neighbours", out_gate=False,
        query_rank=mixer.q_rank)


def _feed_forward_spec(mlp):
    if mlp.kind == "dense":
        return PartSpec.make("gated", inner=mlp.ff, activation="gelu_tanh")
    return PartSpec.make("moe", inner=mlp.ff, experts=mlp.experts, top=mlp.top, groups=mlp.groups,
                         keep=mlp.keep, scale=mlp.scale, score="sigmoid", correction=True,
                         group_top=GROUP_TOP, normalise=True, form="relu2", shared_inner=mlp.shared_ff)


def build_spec(config: KozapelConfig) -> ModelSpec:
    norm = PartSpec.make("rmsnorm", eps=config.norm_eps)
    connection = PartSpec.make("hyper", streams=config.streams) if config.streams else None
    blocks = []
    for index, layer in enumerate(config.layers):
        parts = {"norm1": norm, "mixer": _mixer_spec(config, index, layer)}
        if connection is not None:
            parts["connect1"] = connection
        if layer.mlp is not None:
            parts["norm2"] = norm
            parts["feed_forward"] = _feed_forward_spec(layer.mlp)
            if connection is not None:
                parts["connect2"] = connection
        arrangement = "hyper_connected" if connection is not None else "pre_norm"
        if layer.mlp is None:
            arrangement += "_mixer"
        blocks.append(BlockSpec.make(arrangement, **parts))
    # cache entries are numbered in the order of the layers that write one; a layer that reads
    # another layer's keys and values names that layer's entry
    entry_of, schedule = {}, []
    for index, layer in enumerate(config.layers):
        source = getattr(layer.mixer, "kv_from", None)
        if source is None:
            entry_of[index] = len(entry_of)
            schedule.append(LayerCall(block=index, cache=entry_of[index]))
        else:
            schedule.append(LayerCall(block=index, cache=entry_of[source], writes_cache=False))
    return ModelSpec(
        architecture=config.architecture,
        vocab_size=config.vocab,
        width=config.width,
        max_positions=config.max_positions,
        position=PartSpec.make("none"),
        blocks=tuple(blocks),
        schedule=tuple(schedule),
        final_norm=norm,
        tie_head=False,
        eos_token_id=None,
        embedding=PartSpec.make("lookup", scale=config.embedding_scale),
        head=PartSpec.make("linear", bias=False),
        streams=config.streams,
    )


def _expert_names(prefix, experts, name):
    return tuple(f"{prefix}e{e}.{name}" for e in range(experts))


def weight_sources(config: KozapelConfig, spec: ModelSpec):
    """Parameter path -> checkpoint tensor(s).  Matrices are stored ``[out, in]``; projections
    that read the same input are joined into one packed product, the experts' matrices are
    stacked one behind the other."""
    sources = {
        "embedding.table": WeightSource("embed"),
        "final_norm.gamma": WeightSource("final.norm"),
        "head.weight": WeightSource("head"),
    }
    for i, layer in enumerate(config.layers):
        b, l = f"blocks.{i}.", f"l{i}."
        m = l + "mix."
        sources[b + "norm1.gamma"] = WeightSource(l + "norm1")
        if layer.type == "attention":
            packed = (m + "q", m + "g") if layer.mixer.kv_from is not None else (m + "q", m + "k", m + "v", m + "g")
            sources[b + "mixer.qkv.weight"] = WeightSource(packed)
            for ours, theirs in (("lambda_q1", "lq1"), ("lambda_k1", "lk1"), ("lambda_q2", "lq2"),
                                 ("lambda_k2", "lk2")):
                sources[b + "mixer." + ours] = WeightSource(m + theirs)
            sources[b + "mixer.out.weight"] = WeightSource(m + "o")
        else:
            sources[b + "mixer.query_down.weight"] = WeightSource(m + "dq")
            sources[b + "mixer.query_norm.gamma"] = WeightSource(m + "dq.norm")
            sources[b + "mixer.query_up.weight"] = WeightSource(m + "uq")
            sources[b + "mixer.in.weight"] = WeightSource(m + "dkv")
            sources[b + "mixer.latent_norm.gamma"] = WeightSource(m + "dkv.norm")
            sources[b + "mixer.key_up.weight"] = WeightSource(m + "uk")
            sources[b + "mixer.value_up.weight"] = WeightSource(m + "uv")
            sources[b + "mixer.out.weight"] = WeightSource(m + "o")
        if layer.mlp is not None:
            f = l + "mlp."
            sources[b + "norm2.gamma"] = WeightSource(l + "norm2")
            if layer.mlp.kind == "dense":
                sources[b + "feed_forward.gate_up.weight"] = WeightSource((f + "gate", f + "up"))
                sources[b + "feed_forward.down.weight"] = WeightSource(f + "down")
            else:
                sources[b + "feed_forward.router.weight"] = WeightSource(f + "router")
                sources[b + "feed_forward.router.correction"] = WeightSource(f + "correction")
                sources[b + "feed_forward.up.weight"] = WeightSource(_expert_names(f, layer.mlp.experts, "up"))
                sources[b + "feed_forward.down.weight"] = WeightSource(_expert_names(f, layer.mlp.experts, "down"))
                if layer.mlp.shared_ff:
                    sources[b + "feed_forward.shared.up.weight"] = WeightSource(f + "shared.up")
                    sources[b + "feed_forward.shared.down.weight"] = WeightSource(f + "shared.down")
        if config.streams:
            for q in (1, 2) if layer.mlp is not None else (1,):
                for name in ("in", "out", "mix"):
                    sources[b + f"connect{q}.{name}"] = WeightSource(l + f"hc{q}.{name}")
    return sources


def complete_raw(raw: dict, shape_of) -> dict:
    """The raw configuration with the sizes that it leaves out filled in from the shapes of the
    stored tensors (``shape_of(name)``: the shape, or None where the file has no such tensor).  A
    size that the file names is never touched; one that no tensor gives stays out, and the typed
    reader then reports it."""
    import copy

    raw = copy.deepcopy(raw)

    def rows(name, axis=0):
        shape = shape_of(name)
        return None if shape is None or len(shape) <= axis else int(shape[axis])

    def fill(target, key, value):
        if isinstance(target, dict) and key not in target and value is not None and value > 0:
            target[key] = int(value)

    def ratio(a, b):
        return a // b if a is not None and b and a % b == 0 else None

    fill(raw, "vocab", rows("embed"))
    fill(raw, "width", rows("embed", 1))
    fill(raw, "streams", rows("l0.hc1.in"))
    listed = raw.get("layers")
    if not isinstance(listed, list):
        return raw
    for index, layer in enumerate(listed):
        if not isinstance(layer, dict) or not isinstance(layer.get("mixer"), dict):
            continue
        m, p = layer["mixer"], f"l{index}.mix."
        if layer.get("type") == "attention":
            fill(m, "dim", rows(p + "lq1"))
            dim = m.get("dim")
            fill(m, "heads", ratio(rows(p + "q"), 2 * dim if dim else 0))
            source = m.get("kv_from")
            if source is None:
                fill(m, "kv_heads", ratio(rows(p + "k"), 2 * dim if dim else 0))
                fill(m, "vdim", ratio(rows(p + "v"), m.get("kv_heads")))
            else:
                fill(m, "vdim", ratio(rows(p + "o", 1), m.get("heads")))
                if isinstance(source, int) and 0 <= source < index and isinstance(listed[source].get("mixer"), dict):
                    fill(m, "kv_heads", listed[source]["mixer"].get("kv_heads"))
        elif layer.get("type") == "latent_attention":
            fill(m, "q_rank", rows(p + "dq"))
            fill(m, "kv_rank", rows(p + "dkv.norm"))
            if m.get("kv_rank") and rows(p + "dkv") is not None and "rot_dim" not in m:
                m["rot_dim"] = rows(p + "dkv") - m["kv_rank"]
            if "heads" not in m and m.get("rot_dim") and rows(p + "uq") is not None and rows(p + "uk") is not None:
                fill(m, "heads", ratio(rows(p + "uq") - rows(p + "uk"), m["rot_dim"]))
            fill(m, "dim", ratio(rows(p + "uk"), m.get("heads")))
            fill(m, "vdim", ratio(rows(p + "uv"), m.get("heads")))
        mlp, f = layer.get("mlp"), f"l{index}.mlp."
        if isinstance(mlp, dict):
            if mlp.get("kind", "dense") == "dense":
                fill(mlp, "ff", rows(f + "gate"))
            else:
                if rows(f + "e0.up") is not None:
                    fill(mlp.setdefault("expert", {}), "ff", rows(f + "e0.up"))
                if isinstance(mlp.get("router"), dict):
                    fill(mlp["router"], "experts", rows(f + "router"))
                if rows(f + "shared.up") is not None:
                    fill(mlp.setdefault("shared", {}), "ff", rows(f + "shared.up"))
    return raw


def random_tensors(config: KozapelConfig, seed: int, device="cpu"):
    """Checkpoint tensors of a random model, drawn from one seeded generator in a fixed order.
    Matrices N(0, 1/sqrt(in)); scales, corrections and the stream weights such that every part
    matters in the output."""
    generator = torch.Generator(device=device).manual_seed(int(seed))

    def normal(shape, std=1.0):
        return torch.randn(shape, generator=generator, dtype=torch.float32, device=device) * std

    def matrix(rows, columns, gain=1.0):
        return normal((rows, columns), gain / math.sqrt(columns))

    d = config.width
    streams = config.streams
    tensors = {"embed": normal((config.vocab, d), 1.0 / max(config.embedding_scale, 1e-6))}
    for i, layer in enumerate(config.layers):
        l, m = f"l{i}.", f"l{i}.mix."
        mixer = layer.mixer
        tensors[l + "norm1"] = 1.0 + normal((d,), 0.1)
        if layer.type == "attention":
            tensors[m + "q"] = matrix(mixer.heads * 2 * mixer.dim, d)
            if mixer.kv_from is None:
                tensors[m + "k"] = matrix(mixer.kv_heads * 2 * mixer.dim, d)
                tensors[m + "v"] = matrix(mixer.kv_heads * mixer.vdim, d)
            for name in ("lq1", "lk1", "lq2", "lk2"):
                tensors[m + name] = normal((mixer.dim,), 0.1)
            tensors[m + "g"] = matrix(mixer.heads * mixer.vdim, d)
            tensors[m + "o"] = matrix(d, mixer.heads * mixer.vdim)
        else:
            tensors[m + "dq"] = matrix(mixer.q_rank, d)
            tensors[m + "dq.norm"] = 1.0 + normal((mixer.q_rank,), 0.1)
            tensors[m + "uq"] = matrix(mixer.heads * (mixer.dim + mixer.rot_dim), mixer.q_rank)
            tensors[m + "dkv"] = matrix(mixer.kv_rank + mixer.rot_dim, d)
            tensors[m + "dkv.norm"] = 1.0 + normal((mixer.kv_rank,), 0.1)
            tensors[m + "uk"] = matrix(mixer.heads * mixer.dim, mixer.kv_rank)
            tensors[m + "uv"] = matrix(mixer.heads * mixer.vdim, mixer.kv_rank)
            tensors[m + "o"] = matrix(d, mixer.heads * mixer.vdim)
        mlp = layer.mlp
        if mlp is not None:
            f = l + "mlp."
            tensors[l + "norm2"] = 1.0 + normal((d,), 0.1)
            if mlp.kind == "dense":
                tensors[f + "gate"] = matrix(mlp.ff, d)
                tensors[f + "up"] = matrix(mlp.ff, d)
                tensors[f + "down"] = matrix(d, mlp.ff)
            else:
                for e in range(mlp.experts):
                    tensors[f + f"e{e}.up"] = matrix(mlp.ff, d)
                    tensors[f + f"e{e}.down"] = matrix(d, mlp.ff)
                tensors[f + "router"] = matrix(mlp.experts, d)
                tensors[f + "correction"] = normal((mlp.experts,), 0.1)
                if mlp.shared_ff:
                    tensors[f + "shared.up"] = matrix(mlp.shared_ff, d)
                    tensors[f + "shared.down"] = matrix(d, mlp.shared_ff)
        if streams:
            for q in (1, 2) if mlp is not None else (1,):
                tensors[l + f"hc{q}.in"] = 1.0 / streams + normal((streams,), 0.1)
                tensors[l + f"hc{q}.out"] = 1.0 + normal((streams,), 0.2)
                tensors[l + f"hc{q}.mix"] = (torch.eye(streams, device=device)
                                             + normal((streams, streams), 0.1))
    tensors["final.norm"] = 1.0 + normal((d,), 0.1)
    tensors["head"] = matrix(config.vocab, d)
    return tensors


KOZAPEL = register_architecture(Architecture(
    name="Kozapel",
    config_class=KozapelConfig,
    build_spec=build_spec,
    weight_sources=weight_sources,
    random_tensors=random_tensors,
    complete_raw=complete_raw,
    model_type="kozapel",
))
