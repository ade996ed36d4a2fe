"""The Ralepel decoder, plainly: float64, numpy, whole sequences, no cache, one function per mechanism.

Imports nothing from the package.  ``cfg`` is config.json as a dict, ``w`` maps tensor names to float64 arrays.

    layer:        x <- x + N1(mixer(x));  x <- x + N2(ff(x))          N(y) = y / sqrt(mean(y^2) + eps) * weight
    attention:    q = Wq x + bq, k = Wk x + bk, v = k (as projected); q, k <- q / rms(q), k / rms(k) per head (no weight);
                  s_ij = scale * q_i.k_j - slope_h (i - j) for 0 <= i - j < window, slope_h = 2^(-8 (h + 1) / H);
                  p_ij = exp(s_ij) / (exp(sink_h) + sum_j' exp(s_ij'));  out = Wo concat_h(sum_j p_ij v_j) + bo
    latent:       q = Wq x, per head [plain part, turned part]; (c, r) = Wdkv x; c <- N(c) with its own weight;
                  the turned parts of q and the one shared r are rotated by the position;
                  k_h = [Wuk_h c, r], v_h = Wuv_h c; causal softmax of scale * q.k; out = Wo concat_h(...)
                  a layer with ``kv_from`` takes (c, r) as layer kv_from made them
    feed-forward: down(silu(gate x) * (up x)); or a mixture: z = R x + b, the ``top`` largest z chosen, weights =
                  softmax over the chosen z, out = sum w_e expert_e(x) + sigmoid(sg . x) * shared(x)
"""
import numpy as np


def rms_unit(y, eps):
    return y / np.sqrt(np.mean(y * y, axis=-1, keepdims=True) + eps)


def silu(z):
    return z / (1.0 + np.exp(-z))


def gated(x, gate, up, down):
    return (silu(x @ gate.T) * (x @ up.T)) @ down.T


def slopes(heads):
    return np.array([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)])


def sink_attention(x, m, w, pre, eps):
    """``x [n, width]`` of one sequence from its position 0; ``m``: the mixer's entry of the configuration."""
    n = x.shape[0]
    H, G, dh = m["heads"], m["kv_heads"], m["dim"]
    window = (m.get("mask") or {}).get("size", 0) or n + 1
    q = (x @ w[pre + "q"].T + w[pre + "q.b"]).reshape(n, H, dh)
    k = (x @ w[pre + "k"].T + w[pre + "k.b"]).reshape(n, G, dh)
    v = k.copy()
    q, k = rms_unit(q, eps), rms_unit(k, eps)
    sl = slopes(H)
    sink = w[pre + "sink"]
    i, j = np.arange(n)[:, None], np.arange(n)[None, :]
    seen = (j <= i) & (i - j < window)
    out = np.zeros((n, H, dh))
    for h in range(H):
        g = h // (H // G)
        s = m["scale"] * (q[:, h] @ k[:, g].T) - sl[h] * (i - j)
        s = np.where(seen, s, -np.inf)
        top = np.maximum(s.max(axis=1, keepdims=True), sink[h])
        e = np.exp(s - top)
        p = e / (e.sum(axis=1, keepdims=True) + np.exp(sink[h] - top))
        out[:, h] = p @ v[:, g]
    return out.reshape(n, H * dh) @ w[pre + "o"].T + w[pre + "o.b"]


def turn(t, positions, base):
    """Rotate ``t [n, ..., dims]``: dim i pairs with dim i + dims/2, angle = position * base^(-2i/dims)."""
    dims = t.shape[-1]
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims)
    a = positions[:, None] * f[None, :]
    while a.ndim < t.ndim:
        a = a[:, None]
    u, v = t[..., :half], t[..., half:]
    return np.concatenate([u * np.cos(a) - v * np.sin(a), v * np.cos(a) + u * np.sin(a)], axis=-1)


def latent_pair(x, m, w, pre, eps):
    """What a latent layer caches: the normed latent ``c [n, rank]`` and the rotated shared key part ``r [n, rot]``."""
    n = x.shape[0]
    rank = m["kv_rank"]
    both = x @ w[pre + "dkv"].T
    c = rms_unit(both[:, :rank], eps) * w[pre + "dkv.norm"]
    r = turn(both[:, rank:], np.arange(n, dtype=np.float64), m["rot"]["base"])
    return c, r


def latent_attention(x, m, w, pre, pair):
    n = x.shape[0]
    H, dn, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c, r = pair
    q = (x @ w[pre + "q"].T).reshape(n, H, dn + dr)
    qn, qr = q[..., :dn], turn(q[..., dn:], np.arange(n, dtype=np.float64), m["rot"]["base"])
    kn = (c @ w[pre + "uk"].T).reshape(n, H, dn)
    v = (c @ w[pre + "uv"].T).reshape(n, H, dv)
    seen = np.arange(n)[None, :] <= np.arange(n)[:, None]
    out = np.zeros((n, H, dv))
    for h in range(H):
        s = m["scale"] * (qn[:, h] @ kn[:, h].T + qr[:, h] @ r.T)
        s = np.where(seen, s, -np.inf)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (e / e.sum(axis=1, keepdims=True)) @ v[:, h]
    return out.reshape(n, H * dv) @ w[pre + "o"].T


def route(x, f, w, pre):
    """``(ids [n, top], weights [n, top])``: the largest logits first; ties go to the lower index."""
    z = x @ w[pre + "router"].T + w[pre + "router.b"]
    ids = np.argsort(-z, axis=1, kind="stable")[:, :f["router"]["top"]]
    zc = np.take_along_axis(z, ids, axis=1)
    e = np.exp(zc - zc.max(axis=1, keepdims=True))
    return ids, e / e.sum(axis=1, keepdims=True)


def mixture(x, f, w, pre):
    ids, wts = route(x, f, w, pre)
    out = np.zeros_like(x)
    for t in range(x.shape[0]):
        for e, p in zip(ids[t], wts[t]):
            ex = f"{pre}e{e}."
            out[t] += p * gated(x[t:t + 1], w[ex + "gate"], w[ex + "up"], w[ex + "down"])[0]
    if f.get("shared") is not None:
        s = pre + "shared."
        g = 1.0 / (1.0 + np.exp(-(x @ w[s + "sg"].T)))
        out += g * gated(x, w[s + "gate"], w[s + "up"], w[s + "down"])
    return out


def feed_forward(x, f, w, pre):
    if f["kind"] == "dense":
        return gated(x, w[pre + "gate"], w[pre + "up"], w[pre + "down"])
    return mixture(x, f, w, pre)


def forward(cfg, w, tokens, streams=None):
    """Logits ``[n, vocab]`` of one sequence.  ``streams``: a list that takes the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)]
    pairs = {}
    for i, layer in enumerate(cfg["layers"]):
        m, pre = layer["mixer"], f"l{i}.mix."
        if layer["type"] == "attention":
            a = sink_attention(x, m, w, pre, eps)
        else:
            src = m.get("kv_from")
            if src is None:
                pairs[i] = latent_pair(x, m, w, pre, eps)
                src = i
            a = latent_attention(x, m, w, pre, pairs[src])
        x = x + rms_unit(a, eps) * w[f"l{i}.norm1"]
        if layer.get("mlp") is not None:
            x = x + rms_unit(feed_forward(x, layer["mlp"], w, f"l{i}.mlp."), eps) * w[f"l{i}.norm2"]
        if streams is not None:
            streams.append(x.copy())
    return (rms_unit(x, eps) * w["final.norm"]) @ w["head"].T
