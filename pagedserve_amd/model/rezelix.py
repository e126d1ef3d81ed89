"""Rezelix as data: a decoder whose layers are listed one by one in its configuration.

The embedded rows are RMS-normed; that is the residual stream.  Each layer is a pre-norm block
(RMS norms with a plain scale) of a mixer and an optional gated feed-forward, and what a sublayer
adds to the stream is multiplied by a learned factor per column.  The mixer is one of

* ``rglru``: Griffin's recurrent block (a gelu branch times a real-gated linear recurrent unit
  behind a short causal convolution, gates computed block by block);
* ``attention``: causal attention with grouped heads whose values are the keys as projected,
  rotary positions in halves with stretched frequencies, queries and keys divided by their own
  root mean square per head, and a tanh cap on the scores;
* ``latent_attention``: attention over a cached latent with a shared rotated key part and a
  sigmoid gate on the heads' outputs.

The final norm is followed by a head matrix of its own.
"""

import math

import torch

from ..config.registry import Architecture, register_architecture
from ..config.rezelix import RezelixConfig
from ..config.spec import BlockSpec, LayerCall, ModelSpec, PartSpec
from ..weights.loader import WeightSource

# the factor in the decay's exponent, log a = -8 r softplus(lam)
DECAY_SCALE = 8.0


def _scaling(rot):
    if rot is None or rot.scaling is None:
        return None
    s = rot.scaling
    return (s.factor, s.original, s.fast, s.slow)


def _mixer_spec(config, layer):
    mixer = layer.mixer
    if layer.type == "rglru":
        return PartSpec.make("gated_linear_recurrence", inner=mixer.width, blocks=mixer.blocks,
                             taps=mixer.conv, decay_scale=DECAY_SCALE)
    rot = mixer.rot
    if layer.type == "attention":
        return PartSpec.make(
            "attention", heads=mixer.heads, kv_heads=mixer.kv_heads, head_dim=mixer.dim,
            scale=mixer.scale, bias=False, norm_eps=config.norm_eps,
            rotary_dims=rot.dims if rot else 0, rotary_base=rot.base if rot else 10000.0,
            rotary_layout="halves", rotary_scaling=_scaling(rot), head_norm=True,
            values_from_keys=True, score_cap=mixer.softcap, pad_heads=16)
    return PartSpec.make(
        "latent_attention", heads=mixer.heads, dim=mixer.dim, rot_dim=mixer.rot_dim,
        value_dim=mixer.vdim, rank=mixer.kv_rank, scale=mixer.scale, norm_eps=config.norm_eps,
        rotary_base=rot.base if rot else 10000.0, rotary_scaling=_scaling(rot),
        rotary_layout="halves", score_cap=mixer.softcap)


def build_spec(config: RezelixConfig) -> ModelSpec:
    norm = PartSpec.make("rmsnorm", eps=config.norm_eps)
    scale = PartSpec.make("column_scale")
    blocks = []
    for layer in config.layers:
        parts = {"norm1": norm, "mixer": _mixer_spec(config, layer), "scale1": scale}
        arrangement = "pre_norm_scaled_mixer"
        if layer.mlp is not None:
            parts.update(norm2=norm, feed_forward=PartSpec.make("gated", inner=layer.mlp.ff), scale2=scale)
            arrangement = "pre_norm_scaled"
        blocks.append(BlockSpec.make(arrangement, **parts))
    return ModelSpec(
        architecture=config.architecture,
        vocab_size=config.vocab,
        width=config.width,
        max_positions=config.max_positions,
        position=PartSpec.make("none"),
        blocks=tuple(blocks),
        schedule=tuple(LayerCall(block=index, cache=index) for index in range(len(blocks))),
        final_norm=norm,
        tie_head=False,
        eos_token_id=None,
        embedding=PartSpec.make("lookup"),
        head=PartSpec.make("linear", bias=False),
        embedding_norm=norm,
    )


def weight_sources(config: RezelixConfig, spec: ModelSpec):
    """Parameter path -> checkpoint tensor(s).  Matrices are stored ``[out, in]``; projections
    that read the same input are joined into one packed product, the two gates' matrices of a
    recurrent layer block by block."""
    sources = {
        "embedding.table": WeightSource("embed"),
        "embedding_norm.gamma": WeightSource("embed.norm"),
        "final_norm.gamma": WeightSource("final.norm"),
        "head.weight": WeightSource("head"),
    }
    for i, layer in enumerate(config.layers):
        b, l = f"blocks.{i}.", f"l{i}."
        m = l + "mix."
        sources[b + "norm1.gamma"] = WeightSource(l + "norm1")
        sources[b + "scale1.weight"] = WeightSource(l + "ls1")
        if layer.type == "rglru":
            sources[b + "mixer.in.weight"] = WeightSource((m + "y", m + "x"))
            sources[b + "mixer.in.bias"] = WeightSource((m + "y.b", m + "x.b"))
            sources[b + "mixer.conv.weight"] = WeightSource(m + "conv")
            sources[b + "mixer.conv.bias"] = WeightSource(m + "conv.b")
            sources[b + "mixer.gates.weight"] = WeightSource((m + "ra", m + "ri"), axis=1)
            sources[b + "mixer.gates.bias"] = WeightSource((m + "ra.b", m + "ri.b"), axis=1)
            sources[b + "mixer.lam"] = WeightSource(m + "lam")
            sources[b + "mixer.out.weight"] = WeightSource(m + "o")
        elif layer.type == "attention":
            sources[b + "mixer.qkv.weight"] = WeightSource((m + "q", m + "k"))
            sources[b + "mixer.out.weight"] = WeightSource(m + "o")
        else:
            sources[b + "mixer.in.weight"] = WeightSource((m + "q", m + "dkv", m + "g"))
            sources[b + "mixer.latent_norm.gamma"] = WeightSource(m + "dkv.norm")
            sources[b + "mixer.key_up.weight"] = WeightSource(m + "uk")
            sources[b + "mixer.value_up.weight"] = WeightSource(m + "uv")
            sources[b + "mixer.out.weight"] = WeightSource(m + "o")
        if layer.mlp is not None:
            f = l + "mlp."
            sources[b + "norm2.gamma"] = WeightSource(l + "norm2")
            sources[b + "scale2.weight"] = WeightSource(l + "ls2")
            sources[b + "feed_forward.gate_up.weight"] = WeightSource((f + "gate", f + "up"))
            sources[b + "feed_forward.down.weight"] = WeightSource(f + "down")
    return sources


def random_tensors(config: RezelixConfig, seed: int, device="cpu"):
    """Checkpoint tensors of a random model, drawn from one seeded generator in a fixed order.
    Matrices N(0, 1/sqrt(in)); scales, biases and decays such that every part matters in the
    output and the recurrences neither die nor forget at once."""
    generator = torch.Generator(device=device).manual_seed(int(seed))

    def normal(shape, std=1.0):
        return torch.randn(shape, generator=generator, dtype=torch.float32, device=device) * std

    def uniform(shape, low, high):
        return torch.rand(shape, generator=generator, dtype=torch.float32, device=device) * (high - low) + low

    def matrix(rows, columns, gain=1.0):
        return normal((rows, columns), gain / math.sqrt(columns))

    d = config.width
    tensors = {"embed": normal((config.vocab, d)), "embed.norm": 1.0 + normal((d,), 0.1)}
    for i, layer in enumerate(config.layers):
        l, m = f"l{i}.", f"l{i}.mix."
        mixer = layer.mixer
        tensors[l + "norm1"] = 1.0 + normal((d,), 0.1)
        tensors[l + "ls1"] = 0.5 + normal((d,), 0.1)
        if layer.type == "rglru":
            w, blocks = mixer.width, mixer.blocks
            size = w // blocks
            tensors[m + "y"] = matrix(w, d)
            tensors[m + "y.b"] = normal((w,), 0.1)
            tensors[m + "x"] = matrix(w, d)
            tensors[m + "x.b"] = normal((w,), 0.1)
            tensors[m + "conv"] = normal((w, mixer.conv), 1.0 / math.sqrt(mixer.conv))
            tensors[m + "conv.b"] = normal((w,), 0.1)
            tensors[m + "ra"] = normal((blocks, size, size), 1.0 / math.sqrt(size))
            tensors[m + "ra.b"] = normal((blocks, size), 0.1)
            tensors[m + "ri"] = normal((blocks, size, size), 1.0 / math.sqrt(size))
            tensors[m + "ri.b"] = normal((blocks, size), 0.1)
            # a^(1 / r) between 0.9 and 0.999 at r = 1: softplus(lam) = -ln(a) / 8
            decay = uniform((w,), 0.9, 0.999)
            rate = -torch.log(decay) / DECAY_SCALE
            tensors[m + "lam"] = torch.log(torch.expm1(rate))
            tensors[m + "o"] = matrix(d, w)
        elif layer.type == "attention":
            tensors[m + "q"] = matrix(mixer.heads * mixer.dim, d)
            tensors[m + "k"] = matrix(mixer.kv_heads * mixer.dim, d)
            tensors[m + "o"] = matrix(d, mixer.heads * mixer.vdim)
        else:
            tensors[m + "q"] = matrix(mixer.heads * (mixer.dim + mixer.rot_dim), d)
            tensors[m + "dkv"] = matrix(mixer.kv_rank + mixer.rot_dim, d)
            tensors[m + "dkv.norm"] = 1.0 + normal((mixer.kv_rank,), 0.1)
            tensors[m + "uk"] = matrix(mixer.heads * mixer.dim, mixer.kv_rank)
            tensors[m + "uv"] = matrix(mixer.heads * mixer.vdim, mixer.kv_rank)
            tensors[m + "g"] = matrix(mixer.heads * mixer.vdim, d)
            tensors[m + "o"] = matrix(d, mixer.heads * mixer.vdim)
        if layer.mlp is not None:
            f = l + "mlp."
            tensors[l + "norm2"] = 1.0 + normal((d,), 0.1)
            tensors[l + "ls2"] = 0.5 + normal((d,), 0.1)
            tensors[f + "gate"] = matrix(layer.mlp.ff, d)
            tensors[f + "up"] = matrix(layer.mlp.ff, d)
            tensors[f + "down"] = matrix(d, layer.mlp.ff)
    tensors["final.norm"] = 1.0 + normal((d,), 0.1)
    tensors["head"] = matrix(config.vocab, d)
    return tensors


REZELIX = register_architecture(Architecture(
    name="Rezelix",
    config_class=RezelixConfig,
    build_spec=build_spec,
    weight_sources=weight_sources,
    random_tensors=random_tensors,
    model_type="rezelix",
))
