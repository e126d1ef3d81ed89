"""Kozapel without a GPU: the configuration reader, the model's description as parts (cache
entries that several layers read, their windows), the map from checkpoint tensors to parameters,
what the cache holds, and the plain implementation's own consistency (a prompt against its
prefixes, a window as wide as the prompt against none, latent attention through the cached
latent against the direct form, the router's choice)."""

import copy
import math

import pytest
import torch

import kozapel_models
import plain_kozapel as plain
from pagedserve_amd.config.base import ConfigError
from pagedserve_amd.config.kozapel import KozapelConfig
from pagedserve_amd.config.registry import resolve_architecture
from pagedserve_amd.model import load_model

F64 = torch.float64


def test_the_architecture_is_found_by_its_name():
    entry = resolve_architecture({"architecture": "Kozapel"})
    assert entry.name == "Kozapel" and entry.config_class is KozapelConfig


@pytest.mark.parametrize("which", sorted(kozapel_models.MODELS))
def test_configuration_round_trip_and_spec(which):
    raw = kozapel_models.MODELS[which][0]
    config = KozapelConfig.from_dict(raw)
    assert KozapelConfig.from_dict(config.to_dict()) == config
    spec = resolve_architecture(raw).build_spec(config)
    streams = raw.get("streams", 0)
    assert spec.vocab_size == raw["vocab"] and not spec.tie_head and spec.streams == streams
    assert dict(spec.embedding.params)["scale"] == raw["embedding"]["scale"]
    writers = {}
    for index, (layer, block, call) in enumerate(zip(raw["layers"], spec.blocks, spec.schedule)):
        names = [name for name, _ in block.parts]
        assert ("feed_forward" in names) == (layer["mlp"] is not None)
        assert ("connect1" in names) == bool(streams)
        assert block.arrangement == ("hyper_connected" if streams else "pre_norm") + (
            "" if layer["mlp"] is not None else "_mixer")
        mixer, wanted = dict(block.mixer.params), layer["mixer"]
        source = wanted.get("kv_from")
        if source is None:
            writers[index] = call.cache
            assert call.writes_cache and call.cache == len(writers) - 1
        else:
            assert not call.writes_cache and call.cache == writers[source]
        if layer["type"] == "attention":
            assert block.mixer.kind == "differential_attention"
            assert (mixer["heads"], mixer["kv_heads"], mixer["head_dim"], mixer["value_dim"], mixer["scale"],
                    mixer["diff"]) == (wanted["heads"], wanted["kv_heads"], wanted["dim"], wanted["vdim"],
                                       wanted["scale"], wanted["diff"])
            assert mixer["window"] == (wanted.get("mask") or {}).get("size", 0)
            assert mixer["reads_cache"] == (source is not None)
            # the entry keeps the widest window of all layers that read it
            entry = index if source is None else source
            windows = [(l["mixer"].get("mask") or {}).get("size", 0) for i, l in enumerate(raw["layers"])
                       if i == entry or l["mixer"].get("kv_from") == entry]
            assert mixer["cache_window"] == (0 if 0 in windows else max(windows))
        else:
            assert block.mixer.kind == "latent_attention"
            assert (mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["value_dim"], mixer["rank"],
                    mixer["query_rank"], mixer["scale"]) == (
                wanted["heads"], wanted["dim"], wanted["rot_dim"], wanted["vdim"], wanted["kv_rank"],
                wanted["q_rank"], wanted["scale"])
            assert mixer["rotary_layout"] == "neighbours" and not mixer["out_gate"]
        mlp = layer["mlp"]
        if mlp is not None and mlp["kind"] == "dense":
            assert block.feed_forward.kind == "gated"
            assert dict(block.feed_forward.params) == {"inner": mlp["ff"], "activation": "gelu_tanh"}
        elif mlp is not None:
            ff = dict(block.feed_forward.params)
            assert block.feed_forward.kind == "moe" and ff["score"] == "sigmoid" and ff["form"] == "relu2"
            assert ff["correction"] and ff["normalise"] and ff["group_top"] == 2
            assert (ff["inner"], ff["experts"], ff["top"], ff["groups"], ff["keep"], ff["scale"]) == (
                mlp["expert"]["ff"], mlp["router"]["experts"], mlp["router"]["top"],
                mlp["router"]["groups"]["count"], mlp["router"]["groups"]["keep"], mlp["router"]["scale"])
            assert ff["shared_inner"] == (mlp.get("shared") or {}).get("ff", 0)


def test_configuration_errors_name_the_layer_and_key():
    raw = kozapel_models.MODELS["A"][0]
    cases = [
        (lambda c: c["layers"][0].__setitem__("type", "mamba"), "layers[0]"),
        (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3), "kv_heads"),
        (lambda c: c["layers"][0]["mixer"].pop("diff"), "diff"),
        (lambda c: c["layers"][0]["mixer"]["mask"].__setitem__("size", 0), "size"),
        (lambda c: c["layers"][1]["mixer"].pop("q_rank"), "q_rank"),
        (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 2), "rot_dim"),
        (lambda c: c["layers"][1]["mlp"]["router"]["groups"].__setitem__("count", 4), "groups"),
        (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 5), "top"),
        (lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 2), "kv_from"),
        (lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 1), "kv_from"),
        (lambda c: c["layers"][2]["mixer"].__setitem__("vdim", 8), "layer 0"),
        (lambda c: c["layers"][3]["mlp"] if False else c["layers"][0]["mlp"].__setitem__("kind", "glu"), "mlp.kind"),
        (lambda c: c["norm"].pop("eps"), "eps"),
    ]
    for change, word in cases:
        broken = copy.deepcopy(raw)
        change(broken)
        with pytest.raises(ConfigError) as caught:
            KozapelConfig.from_dict(broken)
        assert word in str(caught.value), (word, str(caught.value))


@pytest.mark.parametrize("which", sorted(kozapel_models.MODELS))
def test_every_stored_tensor_feeds_a_parameter_and_the_cache_is_what_the_layers_need(tmp_path, which):
    folder, raw, tensors, _ = kozapel_models.folder_of(tmp_path, which)
    model, _ = load_model(folder, dtype="float32", device="cpu")
    stored = sum(t.numel() for t in tensors.values())
    assert model.parameter_count == stored
    groups, states = model.cache_requirements()
    assert not states
    writers = [l for l in raw["layers"] if l["mixer"].get("kv_from") is None]
    assert sum(len(group.entries) for group in groups) == len(writers)
    for group in groups:
        if group.values_in_keys:
            assert group.kv_heads == 1      # one latent row per token, read as keys and as values
        elif raw["layers"][0]["mixer"].get("dim", 0) * 2 > 256:
            assert group.kv_heads % 2 == 0  # maps too wide for one cached head: a head per map
    # experts stacked one behind the other, in their order
    for index, layer in enumerate(raw["layers"]):
        mlp = layer["mlp"]
        if mlp is not None and mlp["kind"] == "moe":
            part = model.blocks[index].parts()["feed_forward"]
            ff = mlp["expert"]["ff"]
            assert torch.equal(part.first_weight[1].double(), tensors[f"l{index}.mlp.e1.up"])
            assert torch.equal(part.down_weight[-1].double(),
                               tensors[f"l{index}.mlp.e{mlp['router']['experts'] - 1}.down"])
            assert part.first_weight.shape[1] == ff
        if layer["type"] == "attention":
            part = model.blocks[index].mixer
            m = layer["mixer"]
            q = tensors[f"l{index}.mix.q"].view(m["heads"], 2, m["dim"], -1)
            rows = part.qkv_weight[:2 * m["heads"] * m["dim"]].double()
            if part.packed:
                # the two maps' keys lie side by side in one cached head, as they are stored
                assert part.kv_heads == m["kv_heads"] and part.head_dim >= max(2 * m["dim"], m["vdim"])
                assert torch.equal(rows.view(m["heads"], 2, m["dim"], -1), q)
            else:
                # a cached head per map: the maps of all heads lie map by map in the packed product
                assert part.kv_heads == 2 * m["kv_heads"] and part.head_dim >= max(m["dim"], m["vdim"])
                assert torch.equal(rows.view(2, m["heads"], m["dim"], -1)[1, m["heads"] - 1], q[m["heads"] - 1, 1])
            assert math.isclose(float(part.lam), plain.differential_lambda(tensors, f"l{index}.mix.", m["diff"]),
                                rel_tol=1e-5)


def test_a_missing_tensor_is_named(tmp_path):
    from safetensors.torch import load_file, save_file

    folder, raw, _, _ = kozapel_models.folder_of(tmp_path, "A")
    path = folder + "/model.safetensors"
    stored = load_file(path)
    del stored["l1.mlp.correction"]
    save_file(stored, path)
    with pytest.raises(Exception) as caught:
        load_model(folder, dtype="float32", device="cpu")
    assert "l1.mlp.correction" in str(caught.value)


# ------------------------------------------------------------ the plain implementation itself
@pytest.mark.parametrize("which", ["A", "B", "D"])
def test_a_prompt_gives_its_prefixes_logits(which):
    raw, _, seed = kozapel_models.MODELS[which]
    w = plain.as_f64(plain.random_checkpoint(raw, seed))
    tokens = torch.randint(0, raw["vocab"], (21,), generator=torch.Generator().manual_seed(3)).tolist()
    whole = plain.forward(raw, w, tokens)
    for cut in (1, 8, 20):
        assert torch.allclose(plain.forward(raw, w, tokens[:cut]), whole[:cut], atol=1e-9)


def test_a_window_as_wide_as_the_prompt_is_no_window_and_a_narrower_one_is():
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(12, 6, generator=g, dtype=F64) for _ in range(3))
    full = plain.masked_attention(q, k, v, 0.4)
    assert torch.allclose(plain.masked_attention(q, k, v, 0.4, window=12), full)
    narrow = plain.masked_attention(q, k, v, 0.4, window=3)
    assert torch.allclose(narrow[:3], full[:3]) and not torch.allclose(narrow[3:], full[3:])
    # a window of one: every query sees itself only
    assert torch.allclose(plain.masked_attention(q, k, v, 0.4, window=1), v)


def test_latent_attention_through_the_cached_latent_equals_the_direct_form():
    mixer = {"heads": 3, "dim": 8, "rot_dim": 4, "vdim": 6, "kv_rank": 10, "q_rank": 7, "scale": 0.3,
             "rot": {"dims": 4, "base": 50.0}}
    raw = {"vocab": 11, "width": 16, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
           "layers": [{"type": "latent_attention", "mixer": mixer, "mlp": None}]}
    w = plain.as_f64(plain.random_checkpoint(raw, 4))
    p = "l0.mix."
    h = torch.randn(9, 16, generator=torch.Generator().manual_seed(1), dtype=F64)
    positions = torch.arange(9)
    direct = plain.latent_attention(h, w, p, mixer, 1e-5, positions)
    # one cached row per token, [normed latent | rotated part]; the key matrix on the query's
    # side, the value matrix behind the weighted sum of the latents
    down = h @ w[p + "dkv"].T
    rows = torch.cat([plain.rms_norm(down[:, :10], w[p + "dkv.norm"], 1e-5),
                      plain.rotate_neighbours(down[:, None, 10:], positions, 4, 50.0)[:, 0]], dim=1)
    q = (plain.rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], 1e-5) @ w[p + "uq"].T).view(9, 3, 12)
    out = torch.zeros(9, 3, 6, dtype=F64)
    for head in range(3):
        uk = w[p + "uk"].view(3, 8, 10)[head]
        uv = w[p + "uv"].view(3, 6, 10)[head]
        folded = torch.cat([q[:, head, :8] @ uk,
                            plain.rotate_neighbours(q[:, head:head + 1, 8:], positions, 4, 50.0)[:, 0]], dim=1)
        out[:, head] = plain.masked_attention(folded, rows, rows[:, :10], 0.3) @ uv.T
    assert torch.allclose(out.reshape(9, 18) @ w[p + "o"].T, direct, atol=1e-10)


def test_the_router_keeps_the_best_groups_and_norms_the_weights():
    router = {"experts": 6, "top": 2, "scale": 1.5, "groups": {"count": 3, "keep": 1}}
    w = {"r.router": torch.zeros(6, 4, dtype=F64), "r.correction": torch.zeros(6, dtype=F64)}
    # scores by hand: expert 4 is the best alone, but group 0 holds the best pair
    logits = torch.tensor([1.0, 0.9, -3.0, -3.0, 2.0, -4.0], dtype=F64)
    w["r.router"][:, 0] = logits
    h = torch.tensor([[1.0, 0.0, 0.0, 0.0]], dtype=F64)
    chosen, weights = plain.route(h, w, "r.", router)
    assert chosen[0] == [0, 1]
    s = torch.sigmoid(logits[:2])
    assert torch.allclose(weights[0], s / s.sum() * 1.5)
    # a correction moves the choice but not the weights' values
    w["r.correction"][2:4] = 5.0
    chosen, weights = plain.route(h, w, "r.", router)
    assert chosen[0] == [2, 3] and math.isclose(float(weights[0].sum()), 1.5)
    s = torch.sigmoid(logits[2:4])
    assert torch.allclose(weights[0], s / s.sum() * 1.5)
    # negative choice scores everywhere: the closed groups still lose (minus infinity, not zero)
    w["r.correction"][:] = -9.0
    w["r.correction"][4:] = -9.5
    chosen, _ = plain.route(h, w, "r.", router)
    assert chosen[0] == [0, 1]


@pytest.mark.parametrize("which", sorted(kozapel_models.MODELS))
def test_sizes_that_the_file_leaves_out_come_from_the_tensors(tmp_path, which):
    """Every size that a tensor's shape gives may be missing from ``config.json``: the loader
    fills it in before the typed configuration is read, and names what still lacks."""
    import json

    folder, raw, tensors, _ = kozapel_models.folder_of(tmp_path, which)
    full, _ = load_model(folder, dtype="float32", device="cpu")
    stripped = copy.deepcopy(raw)
    for key in ("vocab", "width", "streams"):
        stripped.pop(key, None)
    for layer in stripped["layers"]:
        for key in ("dim", "vdim", "kv_heads", "q_rank", "kv_rank", "rot_dim"):
            layer["mixer"].pop(key, None)
        if layer["type"] == "attention" or layer["mixer"].get("rot"):
            layer["mixer"].pop("heads", None)
        mlp = layer["mlp"]
        if mlp is not None and mlp["kind"] == "dense":
            mlp.pop("ff")
        elif mlp is not None:
            mlp.pop("expert")
            mlp["router"].pop("experts")
            mlp.pop("shared", None)
    with open(folder + "/config.json", "w") as handle:
        json.dump(stripped, handle)
    again, config = load_model(folder, dtype="float32", device="cpu")
    assert config == KozapelConfig.from_dict(raw)
    assert again.parameter_count == full.parameter_count
    # a size that no tensor gives is still reported by its name
    del stripped["layers"][0]["mixer"]["scale"]
    with open(folder + "/config.json", "w") as handle:
        json.dump(stripped, handle)
    with pytest.raises(ConfigError) as caught:
        load_model(folder, dtype="float32", device="cpu")
    assert "scale" in str(caught.value)
