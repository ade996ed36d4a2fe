"""A plain, slow implementation of the Mufotar decoder: float64, numpy, whole sequences, no cache, one function per
mechanism.  It imports nothing from the package; the tests compare the engine with it.

A model is ``(cfg, W)``: ``cfg`` the dictionary of config.json, ``W`` a dictionary from tensor names to arrays.

The design in this file's notation.  ``x`` is the residual stream ``[T, width]`` of one sequence, positions ``0 .. T-1``.

  layer:     n = LN(x);  x <- x + mixer(n) + ff(n)          one layer norm (weight, bias), both sublayers read ``n``
  delta:     q, k (kv_heads x dim), v (heads x vdim) = silu(conv(W h)) each; q, k made unit vectors per head,
             q times dim^-1/2; beta = sigmoid(W_b h); g = exp(-exp(A_log) softplus(W_a h + dt_bias));
             S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;
             out = W_o (o / rms(o) * w_norm * silu(W_g h))
  parallel:  left_scale * attention(h) + right_scale * mamba(h)
  attention: grouped queries, RMS norm per head on q and k with a weight over the head's dims, a rotation of the
             first ``rot.dims`` dims in half-split pairs, causal softmax of ``scale * q . k``
  mamba:     [x | z] = W_in h;  x = silu(conv(x) + b);  [dt | B | C] = W_x x;  dt = softplus(W_dt dt + b_dt);
             S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;  y_c = sum_n S[c, n] C_n + D_c x_c;
             out = W_o (y * silu(z))
  ff dense:  W_down (gelu_tanh(W_gate h) * (W_up h))
  ff moe:    s = softmax(W_router h);  the ``top`` largest of s + correction are chosen;  weights = s_chosen / sum;
             experts are gated with silu;  the last ``identity`` router outputs stand for experts that return h;
             a shared expert of the same form is added for every token
  output:    LN_final(x) @ embed^T, then cap * tanh(. / cap)
"""
import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (z + 0.044715 * z ** 3)))


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * w + b


def rms_div(x, eps):
    return x / np.sqrt((x ** 2).mean(-1, keepdims=True) + eps)


def rotate_half_split(x, positions, base, dims):
    """x [T, heads, dim]: dim i of the first ``dims`` is paired with dim i + dims/2."""
    half = dims // 2
    freq = base ** (-2.0 * np.arange(half) / dims)
    ang = positions[:, None] * freq[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    out = x.copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def causal_conv(x, w, bias=None):
    """x [T, C], w [C, taps]: out[t] = sum_j w[:, j] x[t - taps + 1 + j], zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C)), x], 0)
    out = np.zeros((T, C))
    for j in range(taps):
        out += padded[j:j + T] * w[:, j]
    return out if bias is None else out + bias


def softmax_attention(h, W, pre, m, eps):
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[pre + "q"].T).reshape(T, H, dim)
    k = (h @ W[pre + "k"].T).reshape(T, G, dim)
    v = (h @ W[pre + "v"].T).reshape(T, G, vdim)
    q = rms_div(q, eps) * W[pre + "q.norm"]
    k = rms_div(k, eps) * W[pre + "k.norm"]
    pos = np.arange(T, dtype=np.float64)
    if m.get("rot"):
        q = rotate_half_split(q, pos, m["rot"]["base"], m["rot"]["dims"])
        k = rotate_half_split(k, pos, m["rot"]["base"], m["rot"]["dims"])
    out = np.zeros((T, H, vdim))
    mask = np.tril(np.ones((T, T), dtype=bool))
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        s = np.where(mask, s, -np.inf)
        s = s - s.max(-1, keepdims=True)
        p = np.exp(s)
        p /= p.sum(-1, keepdims=True)
        out[:, hd] = p @ v[:, g]
    return out.reshape(T, H * vdim) @ W[pre + "o"].T


def selective_scan(h, W, pre, m):
    T = h.shape[0]
    inner, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = h @ W[pre + "in"].T
    x, z = xz[:, :inner], xz[:, inner:]
    x = silu(causal_conv(x, W[pre + "conv"], W[pre + "conv.b"]))
    low = x @ W[pre + "x"].T
    dt = softplus(low[:, :R] @ W[pre + "dt"].T + W[pre + "dt.b"])
    B, C = low[:, R:R + N], low[:, R + N:R + 2 * N]
    A = -np.exp(W[pre + "A_log"])
    S = np.zeros((inner, N))
    y = np.zeros((T, inner))
    for t in range(T):
        S = np.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + W[pre + "D"] * x[t]
    return (y * silu(z)) @ W[pre + "o"].T


def gated_delta(h, W, pre, m, eps):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ W[pre + "q"].T, W[pre + "q.conv"])).reshape(T, G, dk)
    k = silu(causal_conv(h @ W[pre + "k"].T, W[pre + "k.conv"])).reshape(T, G, dk)
    v = silu(causal_conv(h @ W[pre + "v"].T, W[pre + "v.conv"])).reshape(T, H, dv)
    q = q / np.sqrt((q ** 2).sum(-1, keepdims=True) + 1e-6) * dk ** -0.5
    k = k / np.sqrt((k ** 2).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ W[pre + "b"].T)
    g = np.exp(-np.exp(W[pre + "A_log"]) * softplus(h @ W[pre + "a"].T + W[pre + "dt_bias"]))
    gate = silu(h @ W[pre + "g"].T).reshape(T, H, dv)
    o = np.zeros((T, H, dv))
    for hd in range(H):
        kv = hd // (H // G)
        S = np.zeros((dk, dv))
        for t in range(T):
            S = g[t, hd] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kv])
            S = S + np.outer(k[t, kv], u)
            o[t, hd] = S.T @ q[t, kv]
    o = rms_div(o, eps) * W[pre + "norm"] * gate
    return o.reshape(T, H * dv) @ W[pre + "o"].T


def side_by_side(h, W, pre, m, eps):
    return m["left_scale"] * softmax_attention(h, W, pre + "left.", m["left"], eps) \
        + m["right_scale"] * selective_scan(h, W, pre + "right.", m["right"])


def gated_ff(h, W, pre, act):
    return (act(h @ W[pre + "gate"].T) * (h @ W[pre + "up"].T)) @ W[pre + "down"].T


def route(h, W, pre, f):
    """(chosen [T, top], weights [T, top]) of the mixture's router."""
    z = h @ W[pre + "router"].T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z)
    s /= s.sum(-1, keepdims=True)
    choice = s + W[pre + "correction"]
    top = f["router"]["top"]
    chosen = np.argsort(-choice, axis=-1, kind="stable")[:, :top]
    picked = np.take_along_axis(s, chosen, -1)
    return chosen, picked / (picked.sum(-1, keepdims=True) + 1e-20)


def mixture_ff(h, W, pre, f):
    T = h.shape[0]
    real = f["router"]["experts"]
    chosen, wts = route(h, W, pre, f)
    out = np.zeros_like(h)
    for t in range(T):
        for e, w in zip(chosen[t], wts[t]):
            if e >= real:
                out[t] += w * h[t]
            else:
                out[t] += w * gated_ff(h[t:t + 1], W, f"{pre}e{e}.", silu)[0]
    if f.get("shared") is not None:
        out += gated_ff(h, W, pre + "shared.", silu)
    return out


def feed_forward(h, W, pre, f):
    if f is None:
        return np.zeros_like(h)
    if f["kind"] == "dense":
        return gated_ff(h, W, pre, gelu_tanh)
    return mixture_ff(h, W, pre, f)


def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out``: a list that takes the residual stream after every layer run."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in W.items() if np.asarray(v).dtype.kind == "f"}
    eps = cfg["norm"]["eps"]
    x = W["embed"][np.asarray(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of", i)
        p = f"l{src}."
        h = layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps)
        if layer["type"] == "delta":
            a = gated_delta(h, W, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "parallel":
            a = side_by_side(h, W, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        x = x + (a + feed_forward(h, W, p + "mlp.", layer.get("mlp")))
        if layers_out is not None:
            layers_out.append(x.copy())
    y = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    logits = y @ W["embed"].T
    cap = cfg.get("logit_softcap")
    return cap * np.tanh(logits / cap) if cap else logits
