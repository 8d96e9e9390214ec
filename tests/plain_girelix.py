"""Plain implementation of the Girelix design in numpy float64: one function per mechanism, whole sequences
only (no cache, no state carried between calls), written from the design's equations and sharing no code with
the package.  `weights` maps checkpoint names to arrays; `cfg` is the config.json dictionary."""
import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rms_norm(x, w, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def rotate_pairs(x, positions, dims, base):
    """x [T, heads, dim]: lanes 2i and 2i + 1 (i < dims / 2) of each head turned by position * base^(-2i/dims)."""
    out = x.copy()
    for i in range(dims // 2):
        a = positions.astype(np.float64) * base ** (-2.0 * i / dims)
        c, s = np.cos(a)[:, None], np.sin(a)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def softmax_attention(W, p, m, h):
    """Causal grouped-query attention whose values are the unrotated keys and whose denominator holds a sink."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = np.arange(T)
    q = (h @ W[p + "q"].T).reshape(T, H, dk)
    k = (h @ W[p + "k"].T).reshape(T, G, dk)
    v = k.copy()
    assert dv == dk
    rot = m.get("rot")
    if rot:
        q, k = rotate_pairs(q, pos, rot["dims"], rot["base"]), rotate_pairs(k, pos, rot["dims"], rot["base"])
    out = np.zeros((T, H, dv))
    for hd in range(H):
        c = hd // (H // G)
        for i in range(T):
            s = (k[: i + 1, c] @ q[i, hd]) * m["scale"]
            sink = W[p + "sink"][hd]
            top = max(s.max(), sink)
            e = np.exp(s - top)
            out[i, hd] = (e @ v[: i + 1, c]) / (e.sum() + math.exp(sink - top))
    return out.reshape(T, H * dv) @ W[p + "o"].T


def lightning_attention(W, p, m, h, eps, state=None):
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with SiLU on q, k and v; norm over all heads together, a
    sigmoid gate, the output projection.  Returns (result, last states)."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W[p + "q"].T).reshape(T, H, dk)
    k = silu(h @ W[p + "k"].T).reshape(T, H, dk)
    v = silu(h @ W[p + "v"].T).reshape(T, H, dv)
    S = np.zeros((H, dk, dv)) if state is None else state.copy()
    o = np.zeros((T, H, dv))
    for t in range(T):
        for hd in range(H):
            S[hd] = m["decay"][hd] * S[hd] + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S[hd].T @ q[t, hd]
    o = rms_norm(o.reshape(T, H * dv), W[p + "norm"], eps) * sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T, S


def two_mixers(W, p, m, h, eps):
    left = softmax_attention(W, p + "left.", m["left"], h)
    right, _ = lightning_attention(W, p + "right.", m["right"], h, eps)
    return m["left_scale"] * left + m["right_scale"] * right


def route(W, p, f, h):
    """-> (chosen [T, top] indices into experts + identity experts, weights [T, top])."""
    r = f["router"]
    n_id = int(r.get("identity", 0))
    n = r["experts"] + n_id
    z = h @ W[p + "router"].T
    z = z - z.max(axis=-1, keepdims=True)
    s = np.exp(z) / np.exp(z).sum(axis=-1, keepdims=True)
    choice = s + W[p + "correction"] if p + "correction" in W else s.copy()
    groups = r.get("groups")
    if groups:
        size = n // groups["count"]
        best = choice.reshape(-1, groups["count"], size).max(axis=-1)                 # [T, groups]
        order = np.argsort(-best, axis=-1, kind="stable")[:, : groups["keep"]]
        allowed = np.zeros_like(best, dtype=bool)
        np.put_along_axis(allowed, order, True, axis=-1)
        choice = np.where(np.repeat(allowed, size, axis=-1), choice, -np.inf)
    chosen = np.argsort(-choice, axis=-1, kind="stable")[:, : r["top"]]
    w = np.take_along_axis(s, chosen, axis=-1)
    return chosen, w / (w.sum(axis=-1, keepdims=True) + 1e-20)


def experts(W, p, f, h):
    r = f["router"]
    E = r["experts"]
    chosen, w = route(W, p, f, h)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t], w[t]):
            if e >= E:
                out[t] += a * h[t]
            else:
                g, u = h[t] @ W[f"{p}e{e}.gate"].T, h[t] @ W[f"{p}e{e}.up"].T
                out[t] += a * ((silu(g) * u) @ W[f"{p}e{e}.down"].T)
    return out


def layer(W, cfg, i, x):
    L, l = cfg["layers"][i], f"l{i}."
    eps = cfg["norm"]["eps"]
    h = rms_norm(x, W[l + "norm1"], eps)
    y = two_mixers(W, l + "mix.", L["mixer"], h, eps) * W[l + "ls1"]
    if L.get("mlp") is not None:
        y = y + experts(W, l + "mlp.", L["mlp"], h) * W[l + "ls2"]
    return x + cfg["residual_mult"] * y


def forward(W, cfg, tokens, residuals=None):
    """Logits [T, vocab] of one whole sequence; residuals (a list) receives the stream after every layer."""
    x = W["embed"][np.asarray(tokens)].astype(np.float64)
    for i in range(len(cfg["layers"])):
        x = layer(W, cfg, i, x)
        if residuals is not None:
            residuals.append(x.copy())
    return rms_norm(x, W["final.norm"], cfg["norm"]["eps"]) @ W["head"].T
