"""A plain, slow Rezelix in float64 on the CPU, written from the design's equations: one function
per mechanism, loops over tokens where the design has a recurrence or a causal sum.  It shares no
code with the engine; the tests hold the engine's kernels and whole models against it.

Notation: ``x`` the stream ``[T, d]``, ``u = rms_norm(x) * w`` a sublayer's input.  Matrices are
stored ``[out, in]`` and applied as ``W u``.  ``w`` maps checkpoint names to float64 tensors.
"""

import math

import torch

F64 = torch.float64


def rms_norm(x, weight, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------------------ rotation
def stretched_frequencies(rot):
    """(frequency of each of the ``dims / 2`` pairs, factor on cosine and sine) of a ``rot`` entry."""
    dims, base = rot["dims"], float(rot["base"])
    freqs = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    scaling = rot.get("scaling")
    if not scaling:
        return torch.tensor(freqs, dtype=F64), 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def index_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    low = max(math.floor(index_of(float(scaling["fast"]))), 0)
    high = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
    out = []
    for i, f in enumerate(freqs):
        ramp = min(max((i - low) / max(high - low, 0.001), 0.0), 1.0)
        out.append(f / factor * ramp + f * (1.0 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate_halves(x, positions, rot):
    """``x [T, heads, n]``: the first ``rot.dims`` dimensions of every head turned by the token's
    position, dimension i paired with i + dims / 2; the rest passes."""
    if not rot or not rot.get("dims"):
        return x
    dims = rot["dims"]
    half = dims // 2
    freqs, magnitude = stretched_frequencies(rot)
    out = x.clone()
    for t, p in enumerate(positions):
        for i in range(half):
            angle = float(p) * float(freqs[i])
            c, s = math.cos(angle) * magnitude, math.sin(angle) * magnitude
            a, b = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = a * c - b * s
            out[t, :, i + half] = b * c + a * s
    return out


# ------------------------------------------------------------------ attention
def capped(scores, cap):
    return scores if not cap else cap * torch.tanh(scores / cap)


def causal_attention(q, k, v, scale, cap=0.0):
    """Position i over all j <= i; query head h reads key/value head ``h // (H / G)``."""
    tokens, heads, _ = q.shape
    groups = k.shape[1]
    out = torch.zeros((tokens, heads, v.shape[2]), dtype=F64)
    for i in range(tokens):
        for h in range(heads):
            g = h // (heads // groups)
            scores = capped((k[:i + 1, g] @ q[i, h]) * scale, cap)
            out[i, h] = torch.softmax(scores, 0) @ v[:i + 1, g]
    return out


def attention(u, w, prefix, mixer, eps, positions):
    """Values are the keys as projected; queries and keys are rotated, then divided by their own
    root mean square per head."""
    tokens = u.shape[0]
    heads, groups, dim = mixer["heads"], mixer["kv_heads"], mixer["dim"]
    q = (u @ w[prefix + "q"].T).view(tokens, heads, dim)
    k = (u @ w[prefix + "k"].T).view(tokens, groups, dim)
    v = k.clone()
    q = rms_norm(rotate_halves(q, positions, mixer.get("rot")), None, eps)
    k = rms_norm(rotate_halves(k, positions, mixer.get("rot")), None, eps)
    o = causal_attention(q, k, v, mixer["scale"], mixer.get("softcap") or 0.0)
    return o.reshape(tokens, heads * dim) @ w[prefix + "o"].T


def latent_attention(u, w, prefix, mixer, eps, positions):
    tokens = u.shape[0]
    heads, dim, rot_dim = mixer["heads"], mixer["dim"], mixer["rot_dim"]
    vdim, rank = mixer["vdim"], mixer["kv_rank"]
    q = (u @ w[prefix + "q"].T).view(tokens, heads, dim + rot_dim)
    down = u @ w[prefix + "dkv"].T
    latent = rms_norm(down[:, :rank], w[prefix + "dkv.norm"], eps)
    shared = down[:, rank:].view(tokens, 1, rot_dim)
    rot = mixer.get("rot")
    q_turned = rotate_halves(q[:, :, dim:], positions, rot)
    k_turned = rotate_halves(shared, positions, rot)
    keys = (latent @ w[prefix + "uk"].T).view(tokens, heads, dim)
    values = (latent @ w[prefix + "uv"].T).view(tokens, heads, vdim)
    full_q = torch.cat([q[:, :, :dim], q_turned], dim=2)
    full_k = torch.cat([keys, k_turned.expand(tokens, heads, rot_dim)], dim=2)
    o = causal_attention(full_q, full_k, values, mixer["scale"], mixer.get("softcap") or 0.0)
    o = o.reshape(tokens, heads * vdim) * torch.sigmoid(u @ w[prefix + "g"].T)
    return o @ w[prefix + "o"].T


# ------------------------------------------------------------------ recurrent block
def causal_convolution(x, weight, bias, before=None):
    """``y_t[c] = bias[c] + sum_j weight[c, j] x_(t - taps + 1 + j)[c]``; ``before``: the ``taps - 1``
    inputs ahead of the first (zeros when None)."""
    tokens, channels = x.shape
    taps = weight.shape[1]
    before = torch.zeros((taps - 1, channels), dtype=F64) if before is None else before
    padded = torch.cat([before, x])
    out = torch.zeros((tokens, channels), dtype=F64)
    for t in range(tokens):
        out[t] = bias + (padded[t:t + taps].T * weight).sum(1)
    return out


def block_gate(u, matrices, bias):
    """``sigmoid(M_b u_b + b_b)`` run by run: ``matrices [blocks, n, n]``, ``bias [blocks, n]``."""
    tokens = u.shape[0]
    blocks, size, _ = matrices.shape
    out = torch.zeros((tokens, blocks * size), dtype=F64)
    for b in range(blocks):
        out[:, b * size:(b + 1) * size] = u[:, b * size:(b + 1) * size] @ matrices[b].T + bias[b]
    return torch.sigmoid(out)


def gated_recurrence(u, r, i, lam, decay_scale=8.0, state=None):
    """``a = exp(-decay_scale r softplus(lam))``, ``S_t = a S_(t-1) + sqrt(1 - a^2) i u``;
    returns (S of every token, the last S)."""
    tokens, channels = u.shape
    state = torch.zeros(channels, dtype=F64) if state is None else state.clone()
    out = torch.zeros((tokens, channels), dtype=F64)
    rate = softplus(lam)
    for t in range(tokens):
        a = torch.exp(-decay_scale * r[t] * rate)
        state = a * state + torch.sqrt(1.0 - a * a) * i[t] * u[t]
        out[t] = state
    return out, state


def recurrent_block(h, w, prefix, mixer):
    y = gelu_tanh(h @ w[prefix + "y"].T + w[prefix + "y.b"])
    u = causal_convolution(h @ w[prefix + "x"].T + w[prefix + "x.b"], w[prefix + "conv"], w[prefix + "conv.b"])
    r = block_gate(u, w[prefix + "ra"], w[prefix + "ra.b"])
    i = block_gate(u, w[prefix + "ri"], w[prefix + "ri.b"])
    states, _ = gated_recurrence(u, r, i, w[prefix + "lam"])
    return (states * y) @ w[prefix + "o"].T


# ------------------------------------------------------------------ feed-forward, model
def gated_feed_forward(u, w, prefix):
    return (silu(u @ w[prefix + "gate"].T) * (u @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def forward(raw, w, token_ids):
    """(logits ``[T, vocab]``, the stream after every layer) of one request from position 0."""
    eps = raw["norm"]["eps"]
    w = {name: tensor.to(F64) for name, tensor in w.items()}
    positions = list(range(len(token_ids)))
    x = rms_norm(w["embed"][torch.tensor(token_ids)], w["embed.norm"], eps)
    after = []
    for index, layer in enumerate(raw["layers"]):
        name = f"l{index}."
        u = rms_norm(x, w[name + "norm1"], eps)
        if layer["type"] == "rglru":
            mixed = recurrent_block(u, w, name + "mix.", layer["mixer"])
        elif layer["type"] == "attention":
            mixed = attention(u, w, name + "mix.", layer["mixer"], eps, positions)
        else:
            mixed = latent_attention(u, w, name + "mix.", layer["mixer"], eps, positions)
        x = x + mixed * w[name + "ls1"]
        if layer.get("mlp") is not None:
            u = rms_norm(x, w[name + "norm2"], eps)
            x = x + gated_feed_forward(u, w, name + "mlp.") * w[name + "ls2"]
        after.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T, after


def random_checkpoint(raw, seed):
    """Random weights of the configuration ``raw`` (a dict of config.json keys), such that every
    part matters in the output."""
    g = torch.Generator().manual_seed(seed)

    def normal(*shape, std=1.0):
        return torch.randn(shape, generator=g, dtype=torch.float32) * std

    def matrix(rows, columns, gain=1.0):
        return normal(rows, columns, std=gain / math.sqrt(columns))

    d = raw["width"]
    w = {"embed": normal(raw["vocab"], d), "embed.norm": 1 + normal(d, std=0.2),
         "final.norm": 1 + normal(d, std=0.2), "head": matrix(raw["vocab"], d)}
    for index, layer in enumerate(raw["layers"]):
        name, m, mixer = f"l{index}.", f"l{index}.mix.", layer["mixer"]
        w[name + "norm1"] = 1 + normal(d, std=0.2)
        w[name + "ls1"] = 0.6 + normal(d, std=0.2)
        if layer["type"] == "rglru":
            width, blocks = mixer["width"], mixer["blocks"]
            size = width // blocks
            w[m + "y"], w[m + "y.b"] = matrix(width, d), normal(width, std=0.2)
            w[m + "x"], w[m + "x.b"] = matrix(width, d), normal(width, std=0.2)
            w[m + "conv"] = normal(width, mixer["conv"], std=1 / math.sqrt(mixer["conv"]))
            w[m + "conv.b"] = normal(width, std=0.2)
            w[m + "ra"], w[m + "ra.b"] = normal(blocks, size, size, std=1 / math.sqrt(size)), normal(blocks, size, std=0.3)
            w[m + "ri"], w[m + "ri.b"] = normal(blocks, size, size, std=1 / math.sqrt(size)), normal(blocks, size, std=0.3)
            # decays between 0.5 and 0.999 at r = 1
            decay = torch.rand(width, generator=g) * 0.499 + 0.5
            w[m + "lam"] = torch.log(torch.expm1(-torch.log(decay) / 8.0))
            w[m + "o"] = matrix(d, width)
        elif layer["type"] == "attention":
            w[m + "q"] = matrix(mixer["heads"] * mixer["dim"], d, 2.0)
            w[m + "k"] = matrix(mixer["kv_heads"] * mixer["dim"], d, 2.0)
            w[m + "o"] = matrix(d, mixer["heads"] * mixer["dim"])
        else:
            heads, rank = mixer["heads"], mixer["kv_rank"]
            w[m + "q"] = matrix(heads * (mixer["dim"] + mixer["rot_dim"]), d, 2.0)
            w[m + "dkv"] = matrix(rank + mixer["rot_dim"], d, 2.0)
            w[m + "dkv.norm"] = 1 + normal(rank, std=0.2)
            w[m + "uk"] = matrix(heads * mixer["dim"], rank)
            w[m + "uv"] = matrix(heads * mixer["vdim"], rank)
            w[m + "g"] = matrix(heads * mixer["vdim"], d, 2.0)
            w[m + "o"] = matrix(d, heads * mixer["vdim"])
        if layer.get("mlp") is not None:
            f, ff = name + "mlp.", layer["mlp"]["ff"]
            w[name + "norm2"] = 1 + normal(d, std=0.2)
            w[name + "ls2"] = 0.6 + normal(d, std=0.2)
            w[f + "gate"], w[f + "up"], w[f + "down"] = matrix(ff, d), matrix(ff, d), matrix(d, ff)
    return w


def greedy_generate(raw, w, prompt, count):
    """``count`` tokens after ``prompt``, each the most likely one (the lowest id on ties)."""
    tokens = list(prompt)
    for _ in range(count):
        logits, _ = forward(raw, w, tokens)
        tokens.append(int(torch.argmax(logits[-1])))
    return tokens[len(prompt):]
