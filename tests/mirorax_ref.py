"""Plain, slow restatement of the Mirorax design (test infrastructure only).

One function per mechanism, float64 numpy, whole sequences at once (no cache, no
state object): position t of every function sees exactly the positions its mask
allows. Nothing here is shared with the product path; the tests compare the HIP
engine against these functions on small random models.

A model is (cfg, w): cfg the parsed config.json dict, w a dict name -> float64
array under the checkpoint's tensor names.

The design in short. Every layer is a parallel block: h = rms(x) w1, x += ls1 * mix(h) +
ls2 * ff(h) (the feed-forward may be absent). A run of layers may be looped: it is walked
`times` times with the same weights, pass t adding the vector step[t] to the stream before
its first layer. Mixers: grouped-query softmax attention without positions, with biased
projections and an elementwise sigmoid output gate; latent attention with a low-rank
key/value latent, one rotated key part shared by all heads, a sliding window and a learned
per-head sink in the softmax's denominator. Feed-forwards: a clamped gated pair, or routed
silu-gated experts (top-k of the biased router logits, softmax over the chosen) plus a
shared expert.
"""

from __future__ import annotations

import numpy as np

F = np.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z**3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def rotate(x, dims, base, positions):
    """x [T, ..., n]: the first `dims` entries of the last axis turn in interleaved pairs
    (2i, 2i + 1) by the angle position * base^(-2i / dims); the rest pass."""
    half = dims // 2
    f = np.array([base ** (-2.0 * i / dims) for i in range(half)], F)
    ang = np.asarray(positions, F)[:, None] * f[None, :]
    shape = (len(positions),) + (1,) * (x.ndim - 2) + (half,)
    c, s = np.cos(ang).reshape(shape), np.sin(ang).reshape(shape)
    out = x.copy()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def visible(size, T):
    """mask[i, j]: position i sees position j; size None: every j <= i, else 0 <= i - j < size."""
    i = np.arange(T)[:, None]
    j = np.arange(T)[None, :]
    m = j <= i
    if size is not None:
        m = m & (i - j < size)
    return m


def softmax_rows(s, mask, sink=None):
    """s [H, T, T]. Softmax over the visible keys of every row. sink [H]: the denominator of
    head h also holds exp(sink[h]), which belongs to no key and carries no value."""
    s = np.where(mask, s, -np.inf)
    m = np.max(s, axis=-1, keepdims=True)
    if sink is not None:
        m = np.maximum(m, sink[:, None, None])
    e = np.where(mask, np.exp(s - m), 0.0)
    den = e.sum(axis=-1, keepdims=True)
    if sink is not None:
        den = den + np.exp(sink[:, None, None] - m)
    return e / den


def mixer_attention(cfg, w, pre, h, m, weights_out=None):
    """Grouped-query attention: biased q / k / v / o projections, no positions, causal,
    plain softmax, heads times sigmoid(W_g h) elementwise before the output projection."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rep = H // G
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).reshape(T, H, D)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).reshape(T, G, D)
    v = (h @ w[pre + "v"].T + w[pre + "v.b"]).reshape(T, G, V)
    s = np.stack([q[:, i] @ k[:, i // rep].T for i in range(H)]) * m["scale"]
    p = softmax_rows(s, visible(None, T)[None])
    if weights_out is not None:
        weights_out.append(p)
    o = np.stack([p[i] @ v[:, i // rep] for i in range(H)], axis=1).reshape(T, H * V)
    o = o * sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T + w[pre + "o.b"]


def mixer_latent(cfg, w, pre, h, m, weights_out=None):
    """Latent attention: every head's query is [dim plain | rot_dim rotated]; W_dkv h gives the
    latent (first kv_rank rows, rms-normed) and one rotated key part shared by all heads (last
    rot_dim rows, not normed); per head the plain key is W_uk c and the value W_uv c. Sliding
    window, softmax with a learned per-head sink."""
    T = h.shape[0]
    eps = cfg["norm"]["eps"]
    H, D, R, V, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = np.arange(T)
    q = (h @ w[pre + "q"].T).reshape(T, H, D + R)
    dkv = h @ w[pre + "dkv"].T
    c = rms_norm(dkv[:, :rank], w[pre + "dkv.norm"], eps)
    dims, base = m["rot"]["dims"], m["rot"]["base"]
    k_rot = rotate(dkv[:, rank:], dims, base, pos)              # [T, R]
    q_rot = rotate(q[:, :, D:], dims, base, pos)                # [T, H, R]
    k_plain = (c @ w[pre + "uk"].T).reshape(T, H, D)
    v = (c @ w[pre + "uv"].T).reshape(T, H, V)
    s = np.stack([q[:, i, :D] @ k_plain[:, i].T + q_rot[:, i] @ k_rot.T for i in range(H)]) * m["scale"]
    p = softmax_rows(s, visible(m["mask"]["size"], T)[None], sink=w[pre + "sink"])
    if weights_out is not None:
        weights_out.append(p)
    o = np.stack([p[i] @ v[:, i] for i in range(H)], axis=1).reshape(T, H * V)
    return o @ w[pre + "o"].T


MIXERS = {"attention": mixer_attention, "latent_attention": mixer_latent}


def ff_clamped(w, pre, h, limit):
    """W_down (g sigmoid(1.702 g) (u + 1)), g = min(W_gate h, limit), u = clamp(W_up h, +-limit)."""
    g = np.minimum(h @ w[pre + "gate"].T, limit)
    u = np.clip(h @ w[pre + "up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def ff_silu(w, pre, h):
    """W_down (silu(W_gate h) * W_up h)."""
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def route(w, pre, h, top):
    """(chosen experts [T, top], weights [T, top]): the `top` largest biased router logits
    (ties: the lower index), weights = softmax over the chosen logits only."""
    z = h @ w[pre + "router"].T + w[pre + "router.b"]
    idx = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zc = np.take_along_axis(z, idx, axis=-1)
    e = np.exp(zc - zc.max(axis=-1, keepdims=True))
    return idx, e / e.sum(axis=-1, keepdims=True)


def ff_moe(w, pre, h, mlp, choice_out=None):
    idx, wt = route(w, pre, h, mlp["router"]["top"])
    if choice_out is not None:
        choice_out.append((idx, wt))
    out = np.zeros((h.shape[0], w[pre + "e0.down"].shape[0]), F)
    for t in range(h.shape[0]):
        for k in range(idx.shape[1]):
            out[t] += wt[t, k] * ff_silu(w, f"{pre}e{idx[t, k]}.", h[t:t + 1])[0]
    if mlp.get("shared"):
        out = out + ff_silu(w, pre + "shared.", h)
    return out


def feed_forward(w, pre, h, mlp, choice_out=None):
    if mlp["kind"] == "dense":
        return ff_clamped(w, pre, h, mlp["limit"])
    return ff_moe(w, pre, h, mlp, choice_out)


def layer(cfg, w, i, x, weights_out=None, choice_out=None):
    """The parallel block: both sublayers read the same normed input, each result is scaled
    elementwise by its own vector, and their sum joins the stream."""
    e = cfg["layers"][i]
    p = f"l{i}."
    h = rms_norm(x, w[p + "norm1"], cfg["norm"]["eps"])
    y = MIXERS[e["type"]](cfg, w, p + "mix.", h, e["mixer"], weights_out) * w[p + "ls1"]
    if e.get("mlp"):
        y = y + feed_forward(w, p + "mlp.", h, e["mlp"], choice_out) * w[p + "ls2"]
    return x + y


def layer_runs(cfg):
    """[(layer index, step row or None)]: the order the layers run in, the looped run unrolled;
    the step row is given for the first layer of every pass."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t if i == a else None) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, n)]


def forward(cfg, w, tokens, layers_out=None, weights_out=None, choice_out=None):
    """Logits [T, vocab] of a whole sequence; layers_out (a list) receives the residual
    stream after every layer run."""
    x = w["embed"][np.asarray(tokens)].astype(F)
    for i, step in layer_runs(cfg):
        if step is not None:
            x = x + w["loop.step"][step]
        x = layer(cfg, w, i, x, weights_out, choice_out)
        if layers_out is not None:
            layers_out.append(x.copy())
    return rms_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T
