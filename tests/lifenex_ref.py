"""Plain, slow restatement of the Lifenex design (test infrastructure only).

One function per mechanism, float64 numpy, whole sequences at once (no cache, no state
object): recurrences are walked token by token from a zero state, attention rows see the
positions their mask allows. Nothing here is shared with the product path; the tests
compare the HIP engine against these functions on small random models.

A model is (cfg, w): cfg the parsed config.json dict, w a dict name -> float64 array under
the checkpoint's tensor names.

The design in short. x = rms(E[token]) w_e. Every layer is a parallel block with two norms of
the same stream: x += mix(rms(x) w1) + ff(rms(x) w2) (the feed-forward may be absent). Mixers:
"mamba2", a selective state-space layer (one input projection into gate | x | B | C | step,
a biased causal convolution with silu over x | B | C, per head S <- exp(-exp(A) dt) S + dt B x^T,
y = S^T C + D x, the gated result rms-normed in equal parts); "parallel", two mixers reading the
same input whose rms-normed results are averaged: softmax attention without rotation (per-head
weighted rms norm of queries and keys, a query temperature that grows with the logarithm of the
position's block number, a learned bias per head and bucketed distance, a learned sink in the
denominator) beside a gated delta rule with one decay per head and key channel (low-rank decay
and gate projections, sigmoid output gate). Feed-forwards: W_d relu(W_u h)^2, or routed silu-gated
experts (sigmoid scores, a correction added for the choice only, groups ranked by the sum of
their two best, weights not renormalised) plus a shared expert scaled by a sigmoid gate.
Logits: the embedding table on the final norm, times logit_scale.
"""

from __future__ import annotations

import numpy as np

F = np.float64


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def causal_conv(x, taps_w, bias=None):
    """x [T, C], taps_w [C, taps] (last column = the current token), zeros before the start."""
    T, C = x.shape
    taps = taps_w.shape[1]
    pad = np.concatenate([np.zeros((taps - 1, C), F), x], axis=0)
    out = np.zeros((T, C), F)
    for j in range(taps):
        out += pad[j:j + T] * taps_w[:, j][None, :]
    return out if bias is None else out + bias[None, :]


# ------------------------------------------------------------------ state-space mixer
def ssm_scan(x, B, C, dt, a_log, d_skip, groups):
    """x [T, H, P], B / C [T, G, N], dt [T, H] (already softplus'd). Per head h with group
    g = h // (H / G): S <- exp(-exp(a_log[h]) dt) S + dt B x^T (S is N x P), y = S^T C + D x."""
    T, H, P = x.shape
    N = B.shape[2]
    rep = H // groups
    y = np.zeros((T, H, P), F)
    for h in range(H):
        g = h // rep
        S = np.zeros((N, P), F)
        for t in range(T):
            S = np.exp(-np.exp(a_log[h]) * dt[t, h]) * S + dt[t, h] * np.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + d_skip[h] * x[t, h]
    return y


def grouped_rms(x, parts, w, eps):
    """x [T, n] rms-normed in `parts` equal parts, each by its own root mean square; times w [n]."""
    T, n = x.shape
    xs = x.reshape(T, parts, n // parts)
    xs = xs / np.sqrt(np.mean(xs * xs, axis=-1, keepdims=True) + eps)
    return xs.reshape(T, n) * w


def mixer_mamba2(cfg, w, pre, h, m):
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner, eps = H * P, cfg["norm"]["eps"]
    zz = h @ w[pre + "in"].T
    z, xbc, dt = zz[:, :inner], zz[:, inner:2 * inner + 2 * G * N], zz[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[pre + "conv"], w[pre + "conv.b"]))
    T = len(h)
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[pre + "dt_bias"][None, :])
    y = ssm_scan(x, B, C, dt, w[pre + "A_log"], w[pre + "D"], G).reshape(T, inner)
    y = grouped_rms(y * silu(z), m["norm_groups"], w[pre + "norm"], eps)
    return y @ w[pre + "o"].T


# ------------------------------------------------------------------ attention
def distance_bucket(n, rows, far):
    """Bucket of the distances n >= 0 (an integer array) in a table of `rows` rows: exact below
    half = rows // 2, then logarithmic up to `far`, everything beyond in the last row."""
    n = np.asarray(n)
    half = rows // 2
    big = np.maximum(n, half).astype(F)
    log = half + np.floor(np.log(big / half) / np.log(far / half) * (rows - half)).astype(np.int64)
    return np.where(n < half, n, np.minimum(rows - 1, log))


def query_temperature(p, coef, every):
    return 1.0 + coef * np.log(np.floor((p + 1) / every) + 1.0)


def softmax_sink(s, sink):
    """s [T, T] with -inf where masked; the denominator also holds exp(sink)."""
    m = np.maximum(np.max(s, axis=-1, keepdims=True), sink)
    e = np.exp(s - m)
    return e / (np.sum(e, axis=-1, keepdims=True) + np.exp(sink - m))


def mixer_attention(cfg, w, pre, h, m, weights_out=None):
    H, G, D, V, eps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], cfg["norm"]["eps"]
    T = len(h)
    q = rms_norm((h @ w[pre + "q"].T).reshape(T, H, D), w[pre + "q.norm"], eps)
    k = rms_norm((h @ w[pre + "k"].T).reshape(T, G, D), w[pre + "k.norm"], eps)
    v = (h @ w[pre + "v"].T).reshape(T, G, V)
    temp = query_temperature(np.arange(T), m["q_temp"]["coef"], m["q_temp"]["every"])
    q = q * temp[:, None, None]
    rel = w[pre + "rel"]
    dist = np.arange(T)[:, None] - np.arange(T)[None, :]
    bucket = distance_bucket(np.maximum(dist, 0), rel.shape[0], m["bias_max"])
    mask = dist >= 0
    out = np.zeros((T, H, V), F)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"] + rel[bucket, hd]
        s = np.where(mask, s, -np.inf)
        p = softmax_sink(s, w[pre + "sink"][hd])
        if weights_out is not None:
            weights_out.append(p)
        out[:, hd] = p @ v[:, g]
    return out.reshape(T, H * V) @ w[pre + "o"].T


# ------------------------------------------------------------------ gated delta rule
def unit(x):
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + 1e-6)


def delta_scan(q, k, v, beta, g):
    """q, k [T, KH, D], v [T, H, V], beta [T, H], g [T, H, D] (a decay per key channel). Per head:
    S <- g * S (rows); u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, H, V = v.shape
    KH, D = q.shape[1], q.shape[2]
    rep = H // KH
    o = np.zeros((T, H, V), F)
    for h in range(H):
        kh = h // rep
        S = np.zeros((D, V), F)
        for t in range(T):
            S = g[t, h][:, None] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, kh])
            S = S + np.outer(k[t, kh], u)
            o[t, h] = S.T @ q[t, kh]
    return o


def mixer_delta(cfg, w, pre, h, m):
    H, KH, D, V, eps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], cfg["norm"]["eps"]
    T = len(h)
    q = silu(causal_conv(h @ w[pre + "q"].T, w[pre + "q.conv"])).reshape(T, KH, D)
    k = silu(causal_conv(h @ w[pre + "k"].T, w[pre + "k.conv"])).reshape(T, KH, D)
    v = silu(causal_conv(h @ w[pre + "v"].T, w[pre + "v.conv"])).reshape(T, H, V)
    q = unit(q) * D ** -0.5
    k = unit(k)
    beta = sigmoid(h @ w[pre + "b"].T)
    a = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"][None, :]
    g = np.exp(-np.exp(w[pre + "A_log"])[None, :, None] * softplus(a).reshape(T, H, D))
    o = delta_scan(q, k, v, beta, g)
    o = rms_norm(o, w[pre + "norm"], eps)
    gate = sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T).reshape(T, H, V)
    return (o * gate).reshape(T, H * V) @ w[pre + "o"].T


def mixer_pair(cfg, w, pre, h, m, weights_out=None):
    eps = cfg["norm"]["eps"]
    a = mixer_attention(cfg, w, pre + "left.", h, m["left"], weights_out)
    b = mixer_delta(cfg, w, pre + "right.", h, m["right"])
    return 0.5 * (rms_norm(a, w[pre + "left.out"], eps) + rms_norm(b, w[pre + "right.out"], eps))


# ------------------------------------------------------------------ feed-forwards
def ff_relu2(w, pre, h):
    return np.maximum(h @ w[pre + "up"].T, 0.0) ** 2 @ w[pre + "down"].T


def ff_silu(w, pre, h):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def route(z, correction, top, count, keep):
    """Router logits z [E] -> (chosen experts, their weights). Scores sigmoid(z); the choice
    uses score + correction: a group's rank is the sum of its two largest choice scores, only
    the `keep` best groups can be chosen from, the `top` largest choice scores there win
    (ties: the lower index). Weights: the chosen scores, without the correction."""
    s = sigmoid(z)
    c = s + correction
    E = len(z)
    gs = E // count
    grp = np.array([np.sort(c[g * gs:(g + 1) * gs])[::-1][:2].sum() for g in range(count)], F)
    allowed = np.zeros(E, bool)
    for g in np.argsort(-grp, kind="stable")[:keep]:
        allowed[g * gs:(g + 1) * gs] = True
    c = np.where(allowed, c, -np.inf)
    idx = np.argsort(-c, kind="stable")[:top]
    return idx, s[idx]


def ff_moe(w, pre, h, mlp, choice_out=None):
    r = mlp["router"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    out = np.zeros((len(h), w[pre + "e0.down"].shape[0]), F)
    zs = h @ w[pre + "router"].T
    for t in range(len(h)):
        idx, wt = route(zs[t], w[pre + "correction"], r["top"], g["count"], g["keep"])
        if choice_out is not None:
            choice_out.append((idx, wt))
        for e, a in zip(idx, wt):
            out[t] += a * ff_silu(w, f"{pre}e{e}.", h[t:t + 1])[0]
    if mlp.get("shared"):
        out += sigmoid(h @ w[pre + "shared.sg"].T) * ff_silu(w, pre + "shared.", h)
    return out


def feed_forward(w, pre, h, mlp, choice_out=None):
    if mlp["kind"] == "dense":
        return ff_relu2(w, pre, h)
    return ff_moe(w, pre, h, mlp, choice_out)


# ------------------------------------------------------------------ the model
def layer(cfg, w, i, x, weights_out=None, choice_out=None):
    e, p, eps = cfg["layers"][i], f"l{i}.", cfg["norm"]["eps"]
    h1 = rms_norm(x, w[p + "norm1"], eps)
    if e["type"] == "mamba2":
        y = mixer_mamba2(cfg, w, p + "mix.", h1, e["mixer"])
    elif e["type"] == "parallel":
        y = mixer_pair(cfg, w, p + "mix.", h1, e["mixer"], weights_out)
    else:
        raise ValueError(e["type"])
    if e.get("mlp"):
        y = y + feed_forward(w, p + "mlp.", rms_norm(x, w[p + "norm2"], eps), e["mlp"], choice_out)
    return x + y


def forward(cfg, w, tokens, layers_out=None, weights_out=None, choice_out=None):
    """Logits [T, vocab] of a whole sequence from position 0."""
    eps = cfg["norm"]["eps"]
    x = rms_norm(w["embed"][np.asarray(tokens)], w["embed.norm"], eps)
    for i in range(len(cfg["layers"])):
        x = layer(cfg, w, i, x, weights_out, choice_out)
        if layers_out is not None:
            layers_out.append(x.copy())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T * cfg.get("logit_scale", 1.0)
