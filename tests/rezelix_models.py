"""Small Rezelix configurations for the tests: sizes, head counts, layer orders, rotations and
constants that differ from each other in every respect, and folders with random weights."""

import json
import math
import os

import torch

import plain_rezelix


def _rot(dims, base, scaling=None):
    out = {"dims": dims, "base": base}
    if scaling is not None:
        factor, original, fast, slow = scaling
        out["scaling"] = {"factor": factor, "original": original, "fast": fast, "slow": slow}
    return out


def _recurrent(width, blocks, conv, mlp=None):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}, "mlp": mlp}


def _attention(heads, kv_heads, dim, scale, rot, softcap=None, mlp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if rot is not None:
        mixer["rot"] = rot
    if softcap is not None:
        mixer["softcap"] = softcap
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def _latent(heads, dim, rot_dim, vdim, rank, scale, rot, mlp=None):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if rot is not None:
        mixer["rot"] = rot
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


# a recurrent layer first and last, part of every attention head rotated with stretched
# frequencies, a cap that bites, a latent narrower than the heads together, three gate blocks
MODEL_A = {
    "architecture": "Rezelix", "vocab": 97, "width": 64, "norm": {"eps": 1e-5},
    "layers": [_recurrent(48, 3, 4),
               _attention(4, 2, 16, 0.4, _rot(8, 500.0, (4.0, 16, 8.0, 1.0)), softcap=3.0, mlp=_dense(96)),
               _latent(3, 8, 4, 12, 20, 0.3, _rot(4, 100.0, (2.0, 8, 4.0, 0.5)), mlp=_dense(80)),
               _recurrent(48, 3, 4, mlp=_dense(72))],
}
# sizes that are multiples of nothing: heads of 12 (cached 16 wide), as many key/value heads as
# heads, every dimension rotated, plain frequencies, no cap; one latent head with an odd unrotated
# part; a recurrent layer of one block whose convolution has a single tap (no inputs to keep)
MODEL_B = {
    "architecture": "Rezelix", "vocab": 131, "width": 40, "norm": {"eps": 1e-6},
    "layers": [_attention(3, 3, 12, 0.25, _rot(12, 10000.0), mlp=None),
               _recurrent(30, 1, 1, mlp=_dense(50)),
               _latent(1, 5, 2, 7, 9, 0.5, _rot(2, 50.0), mlp=None),
               _recurrent(20, 5, 2)],
}
# sizes that the matrix-core kernels take as they are; one key/value head under four heads; a
# latent cached 128 wide; attention layers only after the first
MODEL_C = {
    "architecture": "Rezelix", "vocab": 256, "width": 128, "norm": {"eps": 1e-6},
    "layers": [_recurrent(128, 2, 4, mlp=_dense(256)),
               _attention(4, 1, 64, 0.125, _rot(64, 10000.0, (6.0, 64, 24.0, 1.0)), softcap=15.0, mlp=_dense(256)),
               _latent(4, 32, 32, 64, 96, 0.125, _rot(32, 150000.0, (3.0, 32, 16.0, 2.0)), mlp=_dense(128))],
}
# wide heads: attention heads of 128 (the decode path that merges key ranges inside the output
# projection), a latent cached 256 wide (beyond what the 32-bit tiled kernel takes), no rotation
# in the attention layer at all, five gate blocks, two taps
MODEL_D = {
    "architecture": "Rezelix", "vocab": 77, "width": 64, "norm": {"eps": 1e-5},
    "layers": [_latent(2, 24, 48, 16, 200, 0.1, _rot(48, 1000.0, (16.0, 32, 4.0, 1.0)), mlp=_dense(40)),
               _attention(2, 2, 128, 0.09, None, softcap=8.0, mlp=None),
               _recurrent(200, 5, 2, mlp=_dense(64))],
}
# layers of one kind only, and sizes at their ends: a gate block per channel and one block for
# all, one tap and five, no feed-forward anywhere; one latent head and a latent layer without a
# rotated part; a latent cached at the widest row the attention kernels take (192 + 64) under
# eight heads; heads of 8 under one key/value head
EDGE_MODELS = {
    "only_recurrent": [_recurrent(24, 24, 1), _recurrent(24, 1, 5, mlp=_dense(16)), _recurrent(64, 2, 3)],
    "only_latent": [_latent(1, 4, 2, 3, 5, 0.7, _rot(2, 10.0)), _latent(5, 6, 0, 8, 12, 0.3, None, mlp=_dense(24))],
    "widest_latent": [_latent(8, 64, 64, 32, 192, 0.09, _rot(64, 40000.0, (3.0, 256, 20.0, 1.0)), mlp=_dense(64)),
                      _recurrent(32, 4, 3)],
    "only_attention": [_attention(8, 1, 8, 0.35, _rot(2, 7.0)),
                       _attention(2, 2, 40, 0.2, _rot(40, 30000.0, (6.0, 512, 24.0, 1.5)), softcap=12.0, mlp=_dense(48)),
                       _attention(16, 2, 32, 0.18, _rot(16, 100.0), softcap=2.0)],
}


def edge_folder(tmp_path, which, width=48, vocab=61):
    """(folder, raw configuration, checkpoint tensors as stored) of one of the models above."""
    raw = {"architecture": "Rezelix", "vocab": vocab, "width": width, "norm": {"eps": 1e-5},
           "layers": EDGE_MODELS[which]}
    folder = os.path.join(str(tmp_path), f"rezelix_edge_{which}")
    return folder, raw, write_folder(folder, raw, plain_rezelix.random_checkpoint(raw, 5))


# name -> (configuration, page size, seed)
MODELS = {"A": (MODEL_A, 8, 0), "B": (MODEL_B, 16, 1), "C": (MODEL_C, 16, 2), "D": (MODEL_D, 4, 3)}


def write_folder(folder, raw, tensors):
    """Store a checkpoint as this design's are stored (bfloat16) and return the values as stored."""
    from safetensors.torch import save_file

    stored = {name: tensor.to(torch.bfloat16).contiguous() for name, tensor in tensors.items()}
    os.makedirs(folder, exist_ok=True)
    save_file(stored, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    return {name: tensor.float() for name, tensor in stored.items()}


def folder_of(tmp_path, which):
    """(folder, raw configuration, checkpoint tensors as stored, page size)."""
    raw, page_size, seed = MODELS[which]
    folder = os.path.join(str(tmp_path), f"rezelix_{which}")
    return folder, raw, write_folder(folder, raw, plain_rezelix.random_checkpoint(raw, seed)), page_size


LOUD, ASK = 1, 2      # tokens of the model below


def loud_key_model(tmp_path, kind, decay=0.9995):
    """A model of one attention layer (``kind``: ``attention`` or ``latent_attention``) and one
    recurrent layer in which one pair of tokens stands out: the key of LOUD and the query of ASK
    point the same way and are long, so that an ASK gives nearly all its weight to a LOUD however
    many hundred keys lie between them (a key that is lost, or a page that is read for another,
    shows in the logits), and the recurrent layer keeps what LOUD wrote into its state for as
    long.  Returns (folder, raw, tensors)."""
    width = 64
    if kind == "attention":
        layer = _attention(2, 1, 16, 1.0, None, softcap=50.0)
    else:
        layer = _latent(2, 16, 4, 16, 16, 1.0, _rot(4, 100.0))
    raw = {"architecture": "Rezelix", "vocab": 50, "width": width, "norm": {"eps": 1e-5},
           "layers": [layer, _recurrent(32, 2, 3)]}
    w = plain_rezelix.random_checkpoint(raw, 17)
    # the two tokens' embeddings: long along directions 0 and 1, where no other token has anything
    w["embed"][:, :2] = 0
    w["embed"][LOUD] = 0
    w["embed"][LOUD, 0] = 8.0
    w["embed"][ASK] = 0
    w["embed"][ASK, 1] = 8.0
    w["embed.norm"][:2] = 1.0
    w["l0.norm1"][:2] = 1.0
    q = w["l0.mix.q"]
    q[:, 0] = 0
    q[:, 1] = 0
    if kind == "attention":
        # queries and keys are divided by their root mean square per head: the direction counts,
        # and the scale of 1.0 on heads of 16 makes a matching pair score 16
        k = w["l0.mix.k"]
        k[:, 0] = 0
        k[:, 1] = 0
        k.view(1, 16, width)[:, :4, 0] = 3.0
        q.view(2, 16, width)[:, :4, 1] = 3.0
    else:
        # the latent of LOUD lies along its first four numbers; every head's key matrix passes
        # them on to the head's first four key dimensions, where the queries of ASK are long
        down = w["l0.mix.dkv"]
        down[:, 0] = 0
        down[:, 1] = 0
        down[:4, 0] = 3.0
        w["l0.mix.dkv.norm"][:4] = 1.0
        up = w["l0.mix.uk"].view(2, 16, 16)
        up[:, :4, :4] = torch.eye(4) * 2.0
        q.view(2, 20, width)[:, :4, 1] = 1.5
    # the recurrent layer: slow decays, so that what LOUD wrote is still there hundreds of tokens on
    w["l1.mix.lam"] = torch.full((32,), math.log(math.expm1(-math.log(decay) / 8.0)))
    folder = os.path.join(str(tmp_path), f"rezelix_loud_{kind}")
    return folder, raw, write_folder(folder, raw, w)
