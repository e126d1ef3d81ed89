"""A plain, slow Kozapel in float64 on the CPU, written from the design's equations: one function
per mechanism, loops over tokens and heads where the design has a causal sum or a choice.  It
shares no code with the engine; the tests hold the engine's kernels and whole models against it.

Notation: the stream is kept in ``s`` copies ``X [s, T, d]``; a sublayer reads ``u = sum_s
in[s] X_s`` through its norm and writes ``X'_t = sum_s mix[s, t] X_s + out[t] y``.  Matrices are
stored ``[out, in]`` and applied as ``W u``.  ``w`` maps checkpoint names to float64 tensors.
"""

import math

import torch

F64 = torch.float64


def rms_norm(x, weight, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def relu2(z):
    return torch.clamp(z, min=0.0) ** 2


# ------------------------------------------------------------------ rotation
def rotate_neighbours(x, positions, dims, base):
    """``x [T, heads, n]``: the first ``dims`` dimensions of every head turned by the token's
    position, dimension 2i paired with 2i + 1, angle ``p * base^(-2i / dims)``; the rest passes."""
    if not dims:
        return x
    out = x.clone()
    for i in range(dims // 2):
        angle = positions.to(F64) * base ** (-2.0 * i / dims)
        c, s = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


# ------------------------------------------------------------------ softmax attention
def masked_attention(q, k, v, scale, window=0):
    """One head: ``q [T, n]``, ``k [T, n]``, ``v [T, m]``; query i sees keys j <= i, and with a
    window only those with ``i - j < window``."""
    tokens = q.shape[0]
    out = torch.zeros(tokens, v.shape[1], dtype=F64)
    for i in range(tokens):
        first = 0 if window <= 0 else max(0, i - window + 1)
        scores = (k[first:i + 1] @ q[i]) * scale
        weights = torch.softmax(scores, dim=0)
        out[i] = weights @ v[first:i + 1]
    return out


def differential_lambda(w, prefix, diff):
    return (math.exp(float((w[prefix + "lq1"] * w[prefix + "lk1"]).sum()))
            - math.exp(float((w[prefix + "lq2"] * w[prefix + "lk2"]).sum())) + diff)


def differential_attention(h, w, prefix, mixer, eps, keys_values=None):
    """Two softmax maps per head over the same values, the second taken off the first.  Returns
    (the mixer's output, (keys, values)); ``keys_values`` are another layer's, used instead of
    projections of this layer's own."""
    tokens = h.shape[0]
    heads, kv_heads, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
    diff = float(mixer["diff"])
    window = int((mixer.get("mask") or {}).get("size", 0))
    q = (h @ w[prefix + "q"].T).view(tokens, heads, 2, dim)
    if keys_values is None:
        k = (h @ w[prefix + "k"].T).view(tokens, kv_heads, 2, dim)
        v = (h @ w[prefix + "v"].T).view(tokens, kv_heads, vdim)
    else:
        k, v = keys_values
    lam = differential_lambda(w, prefix, diff)
    group = heads // kv_heads
    out = torch.zeros(tokens, heads, vdim, dtype=F64)
    for head in range(heads):
        g = head // group
        a1 = masked_attention(q[:, head, 0], k[:, g, 0], v[:, g], mixer["scale"], window)
        a2 = masked_attention(q[:, head, 1], k[:, g, 1], v[:, g], mixer["scale"], window)
        out[:, head] = rms_norm(a1 - lam * a2, None, eps) * (1.0 - diff)
    gate = torch.sigmoid(h @ w[prefix + "g"].T)
    return (out.reshape(tokens, heads * vdim) * gate) @ w[prefix + "o"].T, (k, v)


# ------------------------------------------------------------------ latent attention
def latent_attention(h, w, prefix, mixer, eps, positions):
    """Queries through a normed latent; keys and values from one normed latent per token, with a
    rotated key part that all heads share.  Written in its direct form (keys and values per head)."""
    tokens = h.shape[0]
    heads, dim, rot_dim, vdim, rank = (mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"],
                                       mixer["kv_rank"])
    base = float((mixer.get("rot") or {}).get("base", 10000.0))
    cq = rms_norm(h @ w[prefix + "dq"].T, w[prefix + "dq.norm"], eps)
    q = (cq @ w[prefix + "uq"].T).view(tokens, heads, dim + rot_dim)
    q_plain, q_rot = q[..., :dim], rotate_neighbours(q[..., dim:], positions, rot_dim, base)
    down = h @ w[prefix + "dkv"].T
    c = rms_norm(down[:, :rank], w[prefix + "dkv.norm"], eps)
    k_rot = rotate_neighbours(down[:, None, rank:], positions, rot_dim, base)[:, 0]
    k_plain = (c @ w[prefix + "uk"].T).view(tokens, heads, dim)
    v = (c @ w[prefix + "uv"].T).view(tokens, heads, vdim)
    out = torch.zeros(tokens, heads, vdim, dtype=F64)
    for head in range(heads):
        qh = torch.cat([q_plain[:, head], q_rot[:, head]], dim=1)
        kh = torch.cat([k_plain[:, head], k_rot], dim=1)
        out[:, head] = masked_attention(qh, kh, v[:, head], mixer["scale"])
    return out.reshape(tokens, heads * vdim) @ w[prefix + "o"].T


# ------------------------------------------------------------------ feed-forwards
def gated_feed_forward(h, w, prefix):
    return (gelu_tanh(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def plain_expert(h, w, prefix):
    return relu2(h @ w[prefix + "up"].T) @ w[prefix + "down"].T


def route(h, w, prefix, router):
    """Per token: (chosen experts, their weights).  Sigmoid scores; the choice adds a correction
    per expert and is limited to the best groups (a group's score: its two largest choice scores
    summed); the weights are the chosen scores without the correction, normalised, times a factor."""
    experts, top = router["experts"], router["top"]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    count, keep = groups["count"], groups["keep"]
    size = experts // count
    scores = torch.sigmoid(h @ w[prefix + "router"].T)
    choice = scores + w[prefix + "correction"]
    chosen, weights = [], []
    for t in range(h.shape[0]):
        group_scores = [float(torch.topk(choice[t, g * size:(g + 1) * size], min(2, size)).values.sum())
                        for g in range(count)]
        kept = sorted(range(count), key=lambda g: (-group_scores[g], g))[:keep]
        offered = torch.full((experts,), -math.inf, dtype=F64)
        for g in kept:
            offered[g * size:(g + 1) * size] = choice[t, g * size:(g + 1) * size]
        ids = sorted(range(experts), key=lambda e: (-float(offered[e]), e))[:top]
        s = scores[t, ids]
        chosen.append(ids)
        weights.append(s / (s.sum() + 1e-20) * float(router["scale"]))
    return chosen, weights


def mixture_of_experts(h, w, prefix, mlp):
    chosen, weights = route(h, w, prefix, mlp["router"])
    out = torch.zeros(h.shape[0], w[prefix + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for e, weight in zip(chosen[t], weights[t]):
            out[t] += weight * plain_expert(h[t:t + 1], w, f"{prefix}e{e}.")[0]
    if mlp.get("shared"):
        out = out + plain_expert(h, w, prefix + "shared.")
    return out


def feed_forward(h, w, prefix, mlp):
    if mlp["kind"] == "dense":
        return gated_feed_forward(h, w, prefix)
    return mixture_of_experts(h, w, prefix, mlp)


# ------------------------------------------------------------------ the stream in copies
def read_copies(X, w, prefix):
    return torch.einsum("s,std->td", w[prefix + "in"], X)


def write_copies(X, y, w, prefix):
    return torch.einsum("sr,std->rtd", w[prefix + "mix"], X) + w[prefix + "out"][:, None, None] * y[None]


# ------------------------------------------------------------------ the model
def forward(config, w, tokens, return_layers=False):
    """Logits ``[T, vocab]`` of one sequence (positions from 0); with ``return_layers`` also the
    sum of the copies after every layer ``[layers, T, d]``."""
    eps = float(config["norm"]["eps"])
    streams = int(config.get("streams") or 0)
    ids = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(ids))
    x = w["embed"][ids] * float(config["embedding"]["scale"])
    X = x[None].repeat(max(streams, 1), 1, 1)
    kept = {}
    after = []
    for index, layer in enumerate(config["layers"]):
        l = f"l{index}."
        mixer = layer["mixer"]
        u = read_copies(X, w, l + "hc1.") if streams else X[0]
        h = rms_norm(u, w[l + "norm1"], eps)
        if layer["type"] == "attention":
            source = mixer.get("kv_from")
            y, kept[index] = differential_attention(h, w, l + "mix.", mixer, eps,
                                                    None if source is None else kept[source])
        else:
            y = latent_attention(h, w, l + "mix.", mixer, eps, positions)
        X = write_copies(X, y, w, l + "hc1.") if streams else X + y[None]
        if layer.get("mlp") is not None:
            u = read_copies(X, w, l + "hc2.") if streams else X[0]
            y = feed_forward(rms_norm(u, w[l + "norm2"], eps), w, l + "mlp.", layer["mlp"])
            X = write_copies(X, y, w, l + "hc2.") if streams else X + y[None]
        after.append(X.sum(0))
    logits = rms_norm(X.sum(0), w["final.norm"], eps) @ w["head"].T
    if return_layers:
        return logits, torch.stack(after)
    return logits


# ------------------------------------------------------------------ random weights
def random_checkpoint(config, seed):
    """Checkpoint tensors (float32 values that bfloat16 holds exactly) for ``config``."""
    generator = torch.Generator().manual_seed(seed)

    def normal(shape, std=1.0):
        return torch.randn(shape, generator=generator) * std

    def matrix(rows, columns, gain=1.0):
        return normal((rows, columns), gain / math.sqrt(columns))

    d = config["width"]
    streams = int(config.get("streams") or 0)
    t = {"embed": normal((config["vocab"], d), 1.0 / float(config["embedding"]["scale"]))}
    for index, layer in enumerate(config["layers"]):
        l, m = f"l{index}.", f"l{index}.mix."
        mixer = layer["mixer"]
        t[l + "norm1"] = 1.0 + normal((d,), 0.1)
        if layer["type"] == "attention":
            heads, kv_heads, dim, vdim = mixer["heads"], mixer["kv_heads"], mixer["dim"], mixer["vdim"]
            t[m + "q"] = matrix(heads * 2 * dim, d, 2.0)
            if mixer.get("kv_from") is None:
                t[m + "k"] = matrix(kv_heads * 2 * dim, d, 2.0)
                t[m + "v"] = matrix(kv_heads * vdim, d)
            for name in ("lq1", "lk1", "lq2", "lk2"):
                t[m + name] = normal((dim,), 0.3)
            t[m + "g"] = matrix(heads * vdim, d)
            t[m + "o"] = matrix(d, heads * vdim)
        else:
            heads, dim, rot_dim, vdim = mixer["heads"], mixer["dim"], mixer["rot_dim"], mixer["vdim"]
            t[m + "dq"] = matrix(mixer["q_rank"], d)
            t[m + "dq.norm"] = 1.0 + normal((mixer["q_rank"],), 0.1)
            t[m + "uq"] = matrix(heads * (dim + rot_dim), mixer["q_rank"], 2.0)
            t[m + "dkv"] = matrix(mixer["kv_rank"] + rot_dim, d)
            t[m + "dkv.norm"] = 1.0 + normal((mixer["kv_rank"],), 0.1)
            t[m + "uk"] = matrix(heads * dim, mixer["kv_rank"], 2.0)
            t[m + "uv"] = matrix(heads * vdim, mixer["kv_rank"])
            t[m + "o"] = matrix(d, heads * vdim)
        mlp = layer.get("mlp")
        if mlp is not None:
            f = l + "mlp."
            t[l + "norm2"] = 1.0 + normal((d,), 0.1)
            if mlp["kind"] == "dense":
                t[f + "gate"] = matrix(mlp["ff"], d)
                t[f + "up"] = matrix(mlp["ff"], d)
                t[f + "down"] = matrix(d, mlp["ff"])
            else:
                experts = mlp["router"]["experts"]
                for e in range(experts):
                    t[f + f"e{e}.up"] = matrix(mlp["expert"]["ff"], d)
                    t[f + f"e{e}.down"] = matrix(d, mlp["expert"]["ff"])
                t[f + "router"] = matrix(experts, d, 2.0)
                t[f + "correction"] = normal((experts,), 0.3)
                if mlp.get("shared"):
                    t[f + "shared.up"] = matrix(mlp["shared"]["ff"], d)
                    t[f + "shared.down"] = matrix(d, mlp["shared"]["ff"])
        for q in ((1, 2) if mlp is not None else (1,)) if streams else ():
            t[l + f"hc{q}.in"] = 1.0 / streams + normal((streams,), 0.1)
            t[l + f"hc{q}.out"] = 1.0 + normal((streams,), 0.2)
            t[l + f"hc{q}.mix"] = torch.eye(streams) + normal((streams, streams), 0.1)
    t["final.norm"] = 1.0 + normal((d,), 0.1)
    t["head"] = matrix(config["vocab"], d)
    return {name: value.to(torch.bfloat16).to(torch.float32) for name, value in t.items()}


def as_f64(tensors):
    return {name: value.to(F64) for name, value in tensors.items()}


def greedy_generate(config, w, prompt, count):
    """``count`` tokens after ``prompt``, each the most likely one (the whole sequence is run
    again for every token: no cache to get wrong)."""
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(torch.argmax(forward(config, w, tokens)[-1])))
    return tokens[len(prompt):]
