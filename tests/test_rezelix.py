"""Rezelix without a GPU: the configuration reader, the model's description as parts, the map
from checkpoint tensors to parameters, what the cache holds, the rotation's stretched
frequencies, and the plain implementation's own consistency (a sequence in pieces equals the
sequence in one go; latent attention through the cached latent equals the direct form)."""

import copy

import pytest
import torch

import plain_rezelix as plain
import rezelix_models
from pagedserve_amd.config.base import ConfigError
from pagedserve_amd.config.registry import resolve_architecture
from pagedserve_amd.config.rezelix import RezelixConfig
from pagedserve_amd.model.decoder import DecoderModel
from pagedserve_amd.parts.position import rotary_frequencies

F64 = torch.float64


def test_the_architecture_is_found_by_its_name():
    entry = resolve_architecture({"architecture": "Rezelix"})
    assert entry.name == "Rezelix" and entry.config_class is RezelixConfig


@pytest.mark.parametrize("which", sorted(rezelix_models.MODELS))
def test_configuration_round_trip_and_spec(which):
    raw = rezelix_models.MODELS[which][0]
    config = RezelixConfig.from_dict(raw)
    assert RezelixConfig.from_dict(config.to_dict()) == config
    spec = resolve_architecture(raw).build_spec(config)
    assert spec.vocab_size == raw["vocab"] and not spec.tie_head and spec.streams == 0
    assert spec.embedding_norm is not None and spec.embedding_norm.kind == "rmsnorm"
    for layer, block in zip(raw["layers"], spec.blocks):
        names = [name for name, _ in block.parts]
        assert ("feed_forward" in names) == (layer["mlp"] is not None) == ("scale2" in names)
        assert block.arrangement == ("pre_norm_scaled" if layer["mlp"] is not None else "pre_norm_scaled_mixer")
        assert block.scale1.kind == "column_scale"
        mixer, wanted = dict(block.mixer.params), layer["mixer"]
        rot = wanted.get("rot")
        scaling = None
        if rot and rot.get("scaling"):
            s = rot["scaling"]
            scaling = (s["factor"], s["original"], s["fast"], s["slow"])
        if layer["type"] == "rglru":
            assert block.mixer.kind == "gated_linear_recurrence"
            assert (mixer["inner"], mixer["blocks"], mixer["taps"], mixer["decay_scale"]) == (
                wanted["width"], wanted["blocks"], wanted["conv"], 8.0)
        elif layer["type"] == "attention":
            assert block.mixer.kind == "attention"
            assert (mixer["heads"], mixer["kv_heads"], mixer["head_dim"], mixer["scale"]) == (
                wanted["heads"], wanted["kv_heads"], wanted["dim"], wanted["scale"])
            assert mixer["values_from_keys"] and mixer["head_norm"] and mixer["rotary_layout"] == "halves"
            assert mixer["score_cap"] == (wanted.get("softcap") or 0.0)
            assert mixer["rotary_dims"] == (rot["dims"] if rot else 0) and mixer["rotary_scaling"] == scaling
            assert not mixer["bias"] and mixer["norm_eps"] == raw["norm"]["eps"]
        else:
            assert block.mixer.kind == "latent_attention"
            assert (mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["value_dim"], mixer["rank"],
                    mixer["scale"]) == (wanted["heads"], wanted["dim"], wanted["rot_dim"], wanted["vdim"],
                                        wanted["kv_rank"], wanted["scale"])
            assert mixer["rotary_scaling"] == scaling and mixer["rotary_base"] == rot["base"]
        if layer["mlp"] is not None:
            assert block.feed_forward.kind == "gated" and dict(block.feed_forward.params)["inner"] == layer["mlp"]["ff"]


def test_configuration_errors_name_the_layer_and_key():
    raw = rezelix_models.MODELS["A"][0]
    cases = [
        (lambda c: c["layers"][0].__setitem__("type", "mamba"), "layers[0]"),
        (lambda c: c["layers"][0]["mixer"].__setitem__("blocks", 5), "blocks"),
        (lambda c: c["layers"][1]["mixer"].__setitem__("kv_heads", 3), "kv_heads"),
        (lambda c: c["layers"][1]["mixer"].__setitem__("vdim", 8), "vdim"),
        (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 7), "rot.dims"),
        (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].pop("fast"), "fast"),
        (lambda c: c["layers"][2]["mixer"]["rot"].__setitem__("dims", 2), "rot_dim"),
        (lambda c: c["layers"][2]["mixer"].pop("kv_rank"), "kv_rank"),
        (lambda c: c["layers"][3]["mlp"].__setitem__("kind", "moe"), "mlp.kind"),
        (lambda c: c["norm"].pop("eps"), "eps"),
        (lambda c: c.pop("layers"), "layers"),
    ]
    for change, word in cases:
        broken = copy.deepcopy(raw)
        change(broken)
        with pytest.raises(ConfigError) as caught:
            RezelixConfig.from_dict(broken)
        assert word in str(caught.value), (word, str(caught.value))


@pytest.mark.parametrize("which", sorted(rezelix_models.MODELS))
def test_every_parameter_has_its_checkpoint_tensor_and_the_cache_what_it_needs(which):
    raw = rezelix_models.MODELS[which][0]
    entry = resolve_architecture(raw)
    config = RezelixConfig.from_dict(raw)
    spec = entry.build_spec(config)
    model = DecoderModel(spec, torch.float32, "cpu")
    stored = plain.random_checkpoint(raw, 0)
    sources = entry.weight_sources(config, spec)
    used = set()
    for path, param in model.parameters().items():
        source = sources[path]
        assert source.result_shape([tuple(stored[name].shape) for name in source.names]) == tuple(param.shape), path
        used.update(source.names)
    assert used == set(stored)
    drawn = entry.random_tensors(config, 3)
    assert {name: tuple(t.shape) for name, t in drawn.items()} == {name: tuple(t.shape) for name, t in stored.items()}
    groups, states = model.cache_requirements()
    layers = raw["layers"]
    assert sorted(state.entry for state in states) == [i for i, l in enumerate(layers) if l["type"] == "rglru"]
    for state in states:
        mixer = layers[state.entry]["mixer"]
        assert state.shape == (mixer["width"], mixer["conv"]) and state.dtype == torch.float32
    for group in groups:
        (index,) = group.entries
        mixer = layers[index]["mixer"]
        if layers[index]["type"] == "latent_attention":
            # one row per token that is key and value at once
            assert group.kv_heads == 1 and group.values_in_keys and group.window == 0
            assert group.head_dim >= mixer["kv_rank"] + mixer["rot_dim"] and group.head_dim % 16 == 0
        else:
            assert group.kv_heads == mixer["kv_heads"] and not group.values_in_keys
            assert group.head_dim >= mixer["dim"] and group.head_dim % 16 == 0


def test_one_pool_serves_keys_and_values_of_a_latent_and_counts_once():
    from pagedserve_amd.cache.manager import CacheGroupSpec, CacheManager

    shared = CacheGroupSpec((0,), 1, 32, values_in_keys=True)
    apart = CacheGroupSpec((1,), 1, 32)
    cache = CacheManager([shared, apart], 4, 8, 2, torch.float32, "cpu")
    keys, values = cache.entry_pools(0)
    assert keys.data_ptr() == values.data_ptr() and keys.shape == (4, 1, 8, 32)
    keys, values = cache.entry_pools(1)
    assert keys.data_ptr() != values.data_ptr()
    assert 2 * cache.bytes_per_page(0) == cache.bytes_per_page(1)
    assert shared.geometry() != CacheGroupSpec((0,), 1, 32).geometry()


@pytest.mark.parametrize("dims,base,scaling", [
    (8, 500.0, (4.0, 16, 8.0, 1.0)), (64, 10000.0, (6.0, 64, 24.0, 1.0)), (32, 150000.0, (3.0, 32, 16.0, 2.0)),
    (48, 1000.0, (16.0, 32, 4.0, 1.0)), (12, 10000.0, None), (2, 50.0, (3.0, 100, 2.0, 1.0))])
def test_stretched_frequencies(dims, base, scaling):
    rot = {"dims": dims, "base": base}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    want, want_magnitude = plain.stretched_frequencies(rot)
    got, magnitude = rotary_frequencies(dims, base, scaling)
    assert torch.allclose(got, want, rtol=1e-12, atol=0) and abs(magnitude - want_magnitude) < 1e-12
    if scaling:
        plain_ones = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
        # every pair lies between its own frequency and that divided by the factor; the slowest is divided
        assert bool(((got <= plain_ones * (1 + 1e-12)) & (got >= plain_ones / scaling[0] * (1 - 1e-12))).all())


# ------------------------------------------------------------------ the plain implementation against itself
def test_the_recurrence_in_pieces_equals_the_recurrence_in_one_go():
    g = torch.Generator().manual_seed(0)
    tokens, channels = 23, 6
    u = torch.randn((tokens, channels), generator=g, dtype=F64)
    r = torch.rand((tokens, channels), generator=g, dtype=F64)
    i = torch.rand((tokens, channels), generator=g, dtype=F64)
    lam = torch.randn(channels, generator=g, dtype=F64)
    whole, last = plain.gated_recurrence(u, r, i, lam)
    state, pieces = None, []
    for begin, end in ((0, 1), (1, 8), (8, 10), (10, 23)):
        out, state = plain.gated_recurrence(u[begin:end], r[begin:end], i[begin:end], lam, state=state)
        pieces.append(out)
    assert torch.allclose(torch.cat(pieces), whole, atol=1e-13) and torch.allclose(state, last, atol=1e-13)
    # a gate of one and a constant input: the state approaches u / sqrt(1 - a^2) * (1 - a) ... from zero
    ones = torch.ones((400, 1), dtype=F64)
    out, _ = plain.gated_recurrence(ones, ones, ones, torch.tensor([0.0], dtype=F64))
    a = torch.exp(-8.0 * torch.log(torch.tensor(2.0, dtype=F64)))
    assert abs(float(out[-1]) - float(torch.sqrt(1 - a * a) / (1 - a))) < 1e-9


def test_the_convolution_in_pieces_needs_the_last_inputs():
    g = torch.Generator().manual_seed(1)
    x = torch.randn((11, 5), generator=g, dtype=F64)
    weight = torch.randn((5, 4), generator=g, dtype=F64)
    bias = torch.randn(5, generator=g, dtype=F64)
    whole = plain.causal_convolution(x, weight, bias)
    assert torch.allclose(whole[0], bias + weight[:, 3] * x[0])       # the last column is the current token's
    later = plain.causal_convolution(x[6:], weight, bias, before=x[3:6])
    assert torch.allclose(later, whole[6:], atol=1e-13)


def test_latent_attention_through_the_cached_latent_equals_the_direct_form():
    """The scores and outputs when only the latent and the shared rotated key part are kept:
    the head's key matrix on the query's side, the value matrix behind the weighted sum."""
    raw = rezelix_models.MODELS["A"][0]
    mixer = raw["layers"][2]["mixer"]
    w = {name: t.to(F64) for name, t in plain.random_checkpoint(raw, 5).items()}
    g = torch.Generator().manual_seed(2)
    tokens = 9
    u = torch.randn((tokens, raw["width"]), generator=g, dtype=F64)
    prefix, eps = "l2.mix.", raw["norm"]["eps"]
    positions = list(range(tokens))
    direct = plain.latent_attention(u, w, prefix, mixer, eps, positions)
    heads, dim, rot_dim, vdim, rank = (mixer[k] for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
    q = (u @ w[prefix + "q"].T).view(tokens, heads, dim + rot_dim)
    down = u @ w[prefix + "dkv"].T
    latent = plain.rms_norm(down[:, :rank], w[prefix + "dkv.norm"], eps)
    row = torch.cat([latent, plain.rotate_halves(down[:, rank:].view(tokens, 1, rot_dim), positions, mixer["rot"])[:, 0]], 1)
    key_up = w[prefix + "uk"].view(heads, dim, rank)
    value_up = w[prefix + "uv"].view(heads, vdim, rank)
    q_latent = torch.einsum("thd,hdr->thr", q[:, :, :dim], key_up)
    q_row = torch.cat([q_latent, plain.rotate_halves(q[:, :, dim:], positions, mixer["rot"])], 2)
    context = plain.causal_attention(q_row, row.view(tokens, 1, -1), row.view(tokens, 1, -1), mixer["scale"])
    out = torch.einsum("thr,hvr->thv", context[:, :, :rank], value_up).reshape(tokens, heads * vdim)
    out = (out * torch.sigmoid(u @ w[prefix + "g"].T)) @ w[prefix + "o"].T
    assert torch.allclose(out, direct, atol=1e-10)


def test_a_prompt_in_one_go_equals_its_tokens_one_after_the_other():
    raw = rezelix_models.MODELS["B"][0]
    w = plain.random_checkpoint(raw, 9)
    tokens = [5, 17, 3, 99, 0, 42, 7]
    logits, after = plain.forward(raw, w, tokens)
    assert len(after) == len(raw["layers"])
    for cut in (1, 4):
        shorter, _ = plain.forward(raw, w, tokens[:cut])
        assert torch.allclose(shorter, logits[:cut], atol=1e-10)     # causal: later tokens change nothing
