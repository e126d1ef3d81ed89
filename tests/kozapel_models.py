"""Small Kozapel configurations for the tests: sizes, head counts, layer orders, windows and
constants that differ from each other in every respect, and folders with random weights."""

import json
import os

import torch

import plain_kozapel


def _attention(heads, kv_heads, dim, vdim, scale, diff, window=None, kv_from=None, mlp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if window is not None:
        mixer["mask"] = {"size": window}
    if kv_from is not None:
        mixer["kv_from"] = kv_from
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base, mlp=None):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
             "q_rank": q_rank, "scale": scale}
    if rot_dim:
        mixer["rot"] = {"dims": rot_dim, "base": base}
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _moe(ff, experts, top, count, keep, scale, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff},
           "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


# grouped heads (two to a key/value head), values wider than keys, a reader whose window is
# narrower than its source's, three copies of the stream, a latent narrower than its heads
# together, experts in three groups of two
MODEL_A = {
    "architecture": "Kozapel", "vocab": 97, "width": 64, "streams": 3, "norm": {"eps": 1e-5},
    "embedding": {"scale": 0.7},
    "layers": [_attention(4, 2, 16, 24, 0.3, 0.3, window=9, mlp=_dense(96)),
               _latent(3, 8, 4, 12, 20, 10, 0.3, 100.0, mlp=_moe(24, 6, 2, 3, 2, 1.7, shared=16)),
               _attention(4, 2, 16, 24, 0.25, 0.6, window=5, kv_from=0, mlp=_moe(16, 6, 3, 2, 1, 0.9, shared=40)),
               _attention(2, 1, 8, 8, 0.4, 0.2, window=33)],
}
# sizes that are multiples of nothing: heads of 12 with values of 20, a window of one token (a
# query sees itself only), one copy of the stream, one latent head with an odd unrotated part,
# every expert chosen, groups of one expert, no shared expert
MODEL_B = {
    "architecture": "Kozapel", "vocab": 131, "width": 40, "streams": 1, "norm": {"eps": 1e-6},
    "embedding": {"scale": 1.0},
    "layers": [_latent(1, 5, 2, 7, 9, 6, 0.5, 50.0, mlp=_moe(10, 4, 4, 1, 1, 1.0)),
               _attention(3, 3, 12, 20, 0.25, 0.8, window=1, mlp=None),
               _attention(3, 3, 12, 20, 0.2, 0.1, window=12, mlp=_moe(12, 4, 2, 4, 2, 2.0, shared=8)),
               _attention(3, 3, 12, 20, 0.3, 0.5, window=7, kv_from=2, mlp=_dense(50))],
}
# sizes that the matrix-core kernels take as they are: keys wider than values, four heads on one
# key/value head, a window of whole pages, more experts than a wave has lanes, two readers of
# one layer's keys of which one sees further than the layer itself
MODEL_C = {
    "architecture": "Kozapel", "vocab": 256, "width": 128, "streams": 4, "norm": {"eps": 1e-6},
    "embedding": {"scale": 0.25},
    "layers": [_attention(4, 1, 64, 32, 0.125, 0.5, window=32, mlp=_moe(32, 72, 5, 8, 3, 2.5, shared=64)),
               _attention(4, 1, 64, 32, 0.11, 0.4, window=48, kv_from=0, mlp=_dense(256)),
               _latent(4, 32, 32, 64, 96, 64, 0.125, 150000.0, mlp=_dense(128)),
               _attention(4, 1, 64, 32, 0.1, 0.7, window=17, kv_from=0, mlp=_moe(64, 8, 1, 1, 1, 1.0, shared=32))],
}
# one plain stream (no copies), attention without a window, heads of 128, a latent cached 256
# wide without a feed-forward, no rotated part in the other latent layer
MODEL_D = {
    "architecture": "Kozapel", "vocab": 77, "width": 64, "norm": {"eps": 1e-5},
    "embedding": {"scale": 2.0},
    "layers": [_latent(2, 24, 48, 16, 208, 32, 0.1, 1000.0),
               _attention(2, 2, 128, 128, 0.06, 0.5, mlp=_dense(40)),
               _latent(5, 6, 0, 8, 12, 7, 0.3, 0.0, mlp=_moe(8, 3, 1, 3, 1, 3.0, shared=24)),
               _attention(2, 2, 128, 128, 0.05, 0.3, window=200, kv_from=1)],
}

# maps too wide to lie side by side in one cached head (two key/value heads per head's pair of
# maps instead), two heads on one key/value head, a reader of such a layer, two copies of the stream
MODEL_E = {
    "architecture": "Kozapel", "vocab": 53, "width": 48, "streams": 2, "norm": {"eps": 1e-5},
    "embedding": {"scale": 1.5},
    "layers": [_attention(2, 1, 136, 40, 0.08, 0.4, window=10, mlp=_dense(64)),
               _attention(2, 1, 136, 40, 0.07, 0.6, window=6, kv_from=0, mlp=_moe(8, 2, 1, 2, 2, 1.0, shared=8))],
}

# name -> (configuration, page size, seed)
MODELS = {"A": (MODEL_A, 8, 0), "B": (MODEL_B, 16, 1), "C": (MODEL_C, 16, 2), "D": (MODEL_D, 4, 3),
          "E": (MODEL_E, 8, 4)}


def write_folder(folder, raw, tensors):
    """Store a checkpoint as this design's are stored (bfloat16) and return the values as stored."""
    from safetensors.torch import save_file

    stored = {name: tensor.to(torch.bfloat16).contiguous() for name, tensor in tensors.items()}
    os.makedirs(folder, exist_ok=True)
    save_file(stored, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    return plain_kozapel.as_f64({name: tensor.float() for name, tensor in stored.items()})


def folder_of(tmp_path, which):
    """(folder, raw configuration, checkpoint tensors as stored in float64, page size)."""
    raw, page_size, seed = MODELS[which]
    folder = os.path.join(str(tmp_path), f"kozapel_{which}")
    return folder, raw, write_folder(folder, raw, plain_kozapel.random_checkpoint(raw, seed)), page_size


LOUD, ASK = 1, 2      # tokens of the models below


def loud_key_model(tmp_path, kind, window=24):
    """A model of two layers in which one pair of tokens stands out: the key of LOUD and the
    query of ASK point the same way and are long, so that an ASK gives nearly all its weight to a
    LOUD that it sees.  ``kind="attention"``: in the first map of a differential layer under a
    window (a key just inside the window is heard, one just outside is not), read once more by a
    second layer that uses the first one's keys; ``kind="latent_attention"``: through the latent,
    however many hundred keys lie between.  Returns (folder, raw, tensors)."""
    width = 64
    if kind == "attention":
        layers = [_attention(2, 1, 16, 16, 0.05, 0.5, window=window, mlp=_dense(32)),
                  _attention(2, 1, 16, 16, 0.05, 0.5, window=window - 3, kv_from=0)]
    else:
        layers = [_latent(2, 16, 4, 16, 16, 12, 1.0, 100.0, mlp=_dense(32)),
                  _attention(2, 2, 8, 8, 0.3, 0.5, window=6)]
    raw = {"architecture": "Kozapel", "vocab": 50, "width": width, "streams": 2, "norm": {"eps": 1e-5},
           "embedding": {"scale": 1.0}, "layers": layers}
    w = plain_kozapel.random_checkpoint(raw, 17)
    # the two tokens' embeddings: long along directions 0 and 1, where no other token has anything
    w["embed"][:, :2] = 0
    w["embed"][LOUD] = 0
    w["embed"][LOUD, 0] = 8.0
    w["embed"][ASK] = 0
    w["embed"][ASK, 1] = 8.0
    w["l0.norm1"][:2] = 1.0
    w["l0.hc1.in"] = torch.tensor([0.5, 0.5])
    if kind == "attention":
        q, k = w["l0.mix.q"], w["l0.mix.k"]
        q[:, :2] = 0
        k[:, :2] = 0
        # first map of every head: [heads, map, dim, width]
        k.view(1, 2, 16, width)[:, 0, :4, 0] = 3.0
        q.view(2, 2, 16, width)[:, 0, :4, 1] = 3.0
        # the second layer reads the same keys with queries of its own
        q2 = w["l1.mix.q"]
        q2[:, :2] = 0
        q2.view(2, 2, 16, width)[:, 0, :4, 1] = 2.0
        w["l1.norm1"][:2] = 1.0
    else:
        # the latent of LOUD lies along its first four numbers; every head's key matrix passes
        # them on to the head's first four key dimensions, where the queries of ASK are long
        down = w["l0.mix.dkv"]
        down[:, :2] = 0
        down[:4, 0] = 3.0
        w["l0.mix.dkv.norm"][:4] = 1.0
        up = w["l0.mix.uk"].view(2, 16, 16)
        up[:, :4, :4] = torch.eye(4) * 2.0
        dq = w["l0.mix.dq"]
        dq[:, :2] = 0
        dq[:4, 1] = 3.0
        w["l0.mix.dq.norm"][:4] = 1.0
        uq = w["l0.mix.uq"].view(2, 20, 12)
        uq[:, :4, :4] = torch.eye(4) * 1.5
    folder = os.path.join(str(tmp_path), f"kozapel_loud_{kind}")
    return folder, raw, write_folder(folder, raw, w)
