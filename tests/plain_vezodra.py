"""The Vezodra decoder written out plainly: whole sequence, no cache, float64, one function per mechanism.

It shares no code with the package.  ``forward(config, weights, ids)`` takes the config.json dictionary, a
name -> tensor dictionary and one request's token ids and returns the logits of every position; with
``streams`` (a list) it also appends the residual stream after every layer run (a looped layer counts every time).

Notation: n tokens, stream s [n, width].  A layer is  s += mixer(c(N1 s)) + ff(N2 s)  with both norms of the
same s, and c(h) = h + conv(h), a short causal convolution per channel on what the mixer reads.
"""
from __future__ import annotations

import math

import torch


def rms_norm(x, weight, eps):
    y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def input_conv(h, taps):
    """h [n, channels] -> h + conv(h); taps [channels, K], the last column multiplies the current token, zeros
    stand before the sequence's start."""
    n, K = h.shape[0], taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, h.shape[1], dtype=h.dtype), h])
    return h + sum(padded[j:j + n] * taps[:, j] for j in range(K))


def frequencies(rot):
    dims = rot["dims"]
    f = torch.tensor([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    factor = (rot.get("scaling") or {}).get("factor")
    return f / factor if factor else f


def rotate(x, positions, rot, layout):
    """x [n, heads, d].  The first rot.dims elements of every head turn: in the 'interleaved' layout element 2i
    with 2i + 1, in the 'half' layout element i with i + dims / 2; pair i by the angle position * f_i."""
    dims = rot["dims"]
    angle = positions.double()[:, None] * frequencies(rot)[None, :]
    cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
    if layout == "interleaved":
        first, second = slice(0, dims, 2), slice(1, dims, 2)
    else:
        first, second = slice(0, dims // 2), slice(dims // 2, dims)
    u, v = x[..., first], x[..., second]
    out = x.clone()
    out[..., first] = u * cos - v * sin
    out[..., second] = v * cos + u * sin
    return out


def softmax_attention(q, k, v, scale, window=None, sink=None):
    """q [n, H, d], k [n, G, d], v [n, G, dv], scale a number or one per query head.  Query i sees keys j <= i
    (with a window: i - j < window).  ``sink``: a score that joins every softmax's denominator and has no value."""
    n, H, _ = q.shape
    G = k.shape[1]
    rep = H // G
    scores = torch.einsum("ihd,jhd->hij", q, k.repeat_interleave(rep, 1))
    scores = scores * (scale.view(H, 1, 1) if torch.is_tensor(scale) else scale)
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    visible = j <= i
    if window is not None:
        visible = visible & (i - j < window)
    scores = scores.masked_fill(~visible, float("-inf"))
    top = scores.max(-1, keepdim=True).values
    if sink is not None:
        top = top.clamp(min=sink)
    e = torch.exp(scores - top)
    denom = e.sum(-1, keepdim=True)
    if sink is not None:
        denom = denom + torch.exp(sink - top)
    return torch.einsum("hij,jhd->ihd", e / denom, v.repeat_interleave(rep, 1))


def sink_attention(w, p, m, h, positions, sink=0.0):
    """Mixer 'attention': values are the keys as projected (before they turn), a per-head temperature on the
    scores, a sink of score 0, a sigmoid gate per head on the output."""
    n, H, G, d = h.shape[0], m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[p + "q"].T).view(n, H, d)
    k = (h @ w[p + "k"].T).view(n, G, d)
    v = k
    q, k = rotate(q, positions, m["rot"], "interleaved"), rotate(k, positions, m["rot"], "interleaved")
    o = softmax_attention(q, k, v, m["scale"] * w[p + "temp"], sink=sink)
    o = o * torch.sigmoid(h @ w[p + "g"].T)[:, :, None]
    return o.reshape(n, H * d) @ w[p + "o"].T


def window_attention(w, p, m, h, positions, eps):
    """Left half of the mixer 'parallel': q and k normed over their whole projection, half-layout rotation with
    scaled frequencies, a sliding window, ordinary softmax."""
    n, H, G, d, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm(h @ w[p + "q"].T, w[p + "q.norm"], eps).view(n, H, d)
    k = rms_norm(h @ w[p + "k"].T, w[p + "k.norm"], eps).view(n, G, d)
    v = (h @ w[p + "v"].T).view(n, G, dv)
    q, k = rotate(q, positions, m["rot"], "half"), rotate(k, positions, m["rot"], "half")
    o = softmax_attention(q, k, v, m["scale"], window=m["mask"]["size"])
    return o.reshape(n, H * dv) @ w[p + "o"].T


def delta_rule(w, p, m, h, eps, state=None):
    """Right half of the mixer 'parallel': per head a state S [key channel, value channel] with
    S <- diag(decay) S - (a * u)(u^T S) + k v^T  (both terms of the old S), read out as S^T r."""
    n, H, d = h.shape[0], m["heads"], m["dim"]
    r = (h @ w[p + "r"].T).view(n, H, d)
    k = (h @ w[p + "k"].T).view(n, H, d)
    v = (h @ w[p + "v"].T).view(n, H, d)
    decay = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ w[p + "w1"].T) @ w[p + "w2"].T + w[p + "w0"])).view(n, H, d)
    a = torch.sigmoid(h @ w[p + "a"].T + w[p + "a.b"]).view(n, H, d)
    u = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
    S = torch.zeros(H, d, d, dtype=h.dtype) if state is None else state
    out = []
    for t in range(n):
        seen = torch.einsum("hi,hij->hj", u[t], S)                      # u^T S of the old state
        S = decay[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * seen[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        out.append(torch.einsum("hij,hi->hj", S, r[t]))
    o = rms_norm(torch.stack(out), None, eps).reshape(n, H * d) * w[p + "norm"]
    return (o * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def parallel_mixer(w, p, m, h, positions, eps):
    left = window_attention(w, p + "left.", m["left"], h, positions, eps)
    right = delta_rule(w, p + "right.", m["right"], h, eps)
    return 0.5 * (rms_norm(left, w[p + "left.out"], eps) + rms_norm(right, w[p + "right.out"], eps))


def dense_ff(w, p, h):
    z = h @ w[p + "gate"].T
    return (z * torch.sigmoid(z) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def run_order(config):
    """Layer indices in the order they run: layers start .. stop - 1 of 'loop' run 'times' times in a row."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(config, weights, ids, streams=None, sink=0.0):
    """``sink``: the score of the 'attention' mixer's sink (the design fixes 0; None leaves it out, for tests that
    show that it matters)."""
    w = {k: (v.double() if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    positions = torch.arange(len(ids))
    s = w["embed"][torch.tensor(ids)]
    for i in run_order(config):
        layer, p = config["layers"][i], f"l{i}."
        h = rms_norm(s, w[p + "norm1"], eps)
        if config.get("canon") is not None:
            h = input_conv(h, w[p + "canon1"])
        if layer["type"] == "attention":
            branch = sink_attention(w, p + "mix.", layer["mixer"], h, positions, sink)
        elif layer["type"] == "parallel":
            branch = parallel_mixer(w, p + "mix.", layer["mixer"], h, positions, eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            branch = branch + dense_ff(w, p + "mlp.", rms_norm(s, w[p + "norm2"], eps))
        s = s + branch
        if streams is not None:
            streams.append(s.clone())
    return rms_norm(s, w["final.norm"], eps) @ w["embed"].T
