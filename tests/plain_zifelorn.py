"""The Zifelorn decoder written out plainly: whole sequence, no cache, float64, one function per mechanism.

It shares no code with the package.  ``forward(config, weights, ids)`` takes the config.json dictionary, a
name -> tensor dictionary and one request's token ids and returns the logits of every position; with
``streams`` (a list) it also appends the residual stream after every layer.

Notation: n tokens, stream s [n, width]; a layer is  s += norm1(mixer(s)),  s += norm2(ff(s)):  the norm sits
on the branch's output, the branch reads the stream itself.
"""
from __future__ import annotations

import math

import torch


def rms_norm(x, weight, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_interleaved(x, positions, base, dims):
    """x [n, heads, d]: the first ``dims`` elements turn in adjacent pairs (2i, 2i + 1) by position * base^(-2i / dims)."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    angle = positions.double()[:, None] * freq[None, :]
    cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def latent_kv(w, p, m, h, eps, positions):
    """What a latent-attention layer keeps per token: the normed latent [n, kv_rank] and the one rotated key part
    [n, rot_dim] all heads share."""
    r = m["kv_rank"]
    down = h @ w[p + "dkv"].T
    c = rms_norm(down[:, :r], w[p + "dkv.norm"], eps)
    k_rot = rotate_interleaved(down[:, None, r:], positions, m["rot"]["base"], m["rot"]["dims"])[:, 0]
    return c, k_rot


def latent_attention(w, p, m, h, eps, positions, kv):
    """kv = (c, k_rot) of this layer or of the layer it borrows from."""
    n = h.shape[0]
    H, d, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, k_rot = kv
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).view(n, H, d + dr)
    q_plain = q[..., :d]
    q_rot = rotate_interleaved(q[..., d:], positions, m["rot"]["base"], m["rot"]["dims"])
    k_plain = (c @ w[p + "uk"].T).view(n, H, d)
    v = (c @ w[p + "uv"].T).view(n, H, dv)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    visible = torch.tril(torch.ones(n, n, dtype=torch.bool))
    scores = scores.masked_fill(~visible, float("-inf"))
    heads = torch.einsum("hij,jhd->ihd", torch.softmax(scores, -1), v).reshape(n, H * dv)
    return (heads * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def causal_conv(x, taps, bias):
    """x [n, channels]; taps [channels, K], the last column multiplies the current token; zeros before the start."""
    n, K = x.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, x.shape[1], dtype=x.dtype), x])
    return sum(padded[k:k + n] * taps[:, k] for k in range(K)) + bias


def rglru(w, p, m, h):
    n, width, B = h.shape[0], m["width"], m["blocks"]
    y = gelu_tanh(h @ w[p + "y"].T + w[p + "y.b"])
    u = causal_conv(h @ w[p + "x"].T + w[p + "x.b"], w[p + "conv"], w[p + "conv.b"])
    ub = u.view(n, B, width // B)
    r = torch.sigmoid(torch.einsum("nbi,boi->nbo", ub, w[p + "ra"]) + w[p + "ra.b"]).reshape(n, width)
    i = torch.sigmoid(torch.einsum("nbi,boi->nbo", ub, w[p + "ri"]) + w[p + "ri.b"]).reshape(n, width)
    log_a = -8.0 * r * torch.nn.functional.softplus(w[p + "lam"])
    a = log_a.exp()
    drive = torch.sqrt(1.0 - a * a) * i * u
    state, out = torch.zeros(width, dtype=h.dtype), []
    for t in range(n):
        state = a[t] * state + drive[t]
        out.append(state)
    return (torch.stack(out) * y) @ w[p + "o"].T


def dense_ff(w, p, h):
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def moe_ff(w, p, f, h, chosen=None):
    E, top = f["router"]["experts"], f["router"]["top"]
    z = h @ w[p + "router"].T + w[p + "router.b"]
    best = z.topk(top, -1)
    share = torch.softmax(best.values, -1)
    if chosen is not None:
        srt = z.sort(-1, descending=True).values
        chosen.append(float((srt[:, top - 1] - srt[:, top]).min()) if top < E else float("inf"))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(best.indices[t, j])
            out[t] += share[t, j] * (torch.relu(h[t] @ w[f"{p}e{e}.up"].T) ** 2 @ w[f"{p}e{e}.down"].T)
    return out


def forward(config, weights, ids, streams=None, margins=None):
    w = {k: (v.double() if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    n = len(ids)
    positions = torch.arange(n)
    s = w["embed"][torch.tensor(ids)] * config["embedding"]["scale"]
    kept = {}
    for i, layer in enumerate(config["layers"]):
        m, p = layer["mixer"], f"l{i}.mix."
        if layer["type"] == "latent_attention":
            if m.get("kv_from") is None:
                kept[i] = latent_kv(w, p, m, s, eps, positions)
            branch = latent_attention(w, p, m, s, eps, positions, kept[i if m.get("kv_from") is None else m["kv_from"]])
        elif layer["type"] == "rglru":
            branch = rglru(w, p, m, s)
        else:
            raise ValueError(layer["type"])
        s = s + rms_norm(branch, w[f"l{i}.norm1"], eps)
        f = layer.get("mlp")
        if f is not None:
            branch = dense_ff(w, f"l{i}.mlp.", s) if f["kind"] == "dense" else moe_ff(w, f"l{i}.mlp.", f, s, margins)
            s = s + rms_norm(branch, w[f"l{i}.norm2"], eps)
        if streams is not None:
            streams.append(s.clone())
    return rms_norm(s, w["final.norm"], eps) @ w["embed"].T * config["logit_scale"]
