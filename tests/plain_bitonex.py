"""Plain implementation of the Bitonex design in numpy float64: one function per mechanism, whole sequences only
(no cache; the only thing carried is the lightning state a caller may pass on), written from the design's equations
and sharing no code with the package.  `W` maps checkpoint names to arrays; `cfg` is the config.json dictionary."""
import math

import numpy as np


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_norm(x, w, eps):
    """w: a vector over the lanes, or one number for all of them."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def turn(x, positions, dims, base, layout):
    """x [T, heads, lanes]: the first `dims` lanes of each head turned by position * base^(-2i/dims); pair i is lanes
    (i, i + dims/2) for layout "half" and (2i, 2i + 1) for "interleaved"."""
    out = x.copy()
    for i in range(dims // 2):
        a = positions.astype(np.float64) * float(base) ** (-2.0 * i / dims)
        c, s = np.cos(a)[:, None], np.sin(a)[:, None]
        lo, hi = (i, i + dims // 2) if layout == "half" else (2 * i, 2 * i + 1)
        u, v = x[..., lo], x[..., hi]
        out[..., lo] = u * c - v * s
        out[..., hi] = v * c + u * s
    return out


def causal_softmax_heads(q, k, v, scale_of_head, group):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; head h reads key-value head h // group; -> [T, H, dv]."""
    T, H = q.shape[:2]
    out = np.zeros((T, H, v.shape[-1]))
    for h in range(H):
        c = h // group
        for i in range(T):
            s = (k[: i + 1, c] @ q[i, h]) * scale_of_head[h]
            e = np.exp(s - s.max())
            out[i, h] = (e @ v[: i + 1, c]) / e.sum()
    return out


def attention(W, p, m, h):
    """Grouped-query softmax attention: partial rotation of pairs half the turning lanes apart, a temperature per
    head on the scores, a sigmoid gate on the concatenated heads."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = np.arange(T)
    q = (h @ W[p + "q"].T).reshape(T, H, dk)
    k = (h @ W[p + "k"].T).reshape(T, G, dk)
    v = (h @ W[p + "v"].T).reshape(T, G, dv)
    rot = m.get("rot")
    if rot and rot["dims"]:
        q, k = turn(q, pos, rot["dims"], rot["base"], "half"), turn(k, pos, rot["dims"], rot["base"], "half")
    scales = m["scale"] * W[p + "temp"].astype(np.float64)
    o = causal_softmax_heads(q, k, v, scales, H // G).reshape(T, H * dv)
    return (o * sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def lightning(W, p, m, h, eps, state=None):
    """S_t = a_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with SiLU on q, k, v; one RMS norm over all heads' lanes, a
    sigmoid gate, the output projection.  -> (result, last states [H, dk, dv])."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ W[p + "q"].T).reshape(T, H, dk)
    k = silu(h @ W[p + "k"].T).reshape(T, H, dk)
    v = silu(h @ W[p + "v"].T).reshape(T, H, dv)
    decay = m["decay"] if isinstance(m["decay"], (list, tuple)) else [m["decay"]] * H      # one number: every head's
    S = np.zeros((H, dk, dv)) if state is None else state.copy()
    o = np.zeros((T, H, dv))
    for t in range(T):
        for hd in range(H):
            S[hd] = decay[hd] * S[hd] + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S[hd].T @ q[t, hd]
    o = rms_norm(o.reshape(T, H * dv), W[p + "norm"], eps) * sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T, S


def latent_rows(W, p, m, h, eps):
    """What a latent-attention layer with a down-projection keeps per token: (latent [T, kv_rank], turned shared key
    part [T, rot_dim])."""
    T = h.shape[0]
    R, dr = m["kv_rank"], m["rot_dim"]
    down = h @ W[p + "dkv"].T
    c = rms_norm(down[:, :R], W[p + "dkv.norm"], eps)
    kr = turn(down[:, None, R:], np.arange(T), m["rot"]["dims"], m["rot"]["base"], "interleaved")[:, 0]
    return c, kr


def latent_attention(W, p, m, h, eps, rows):
    """Queries through a normed latent; keys and values expanded per head from the latent in `rows` (this layer's own
    or an earlier layer's), one turned key part shared by the heads."""
    T = h.shape[0]
    H, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = rows
    cq = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).reshape(T, H, dn + dr)
    qn = q[..., :dn]
    qr = turn(q[..., dn:], np.arange(T), m["rot"]["dims"], m["rot"]["base"], "interleaved")
    kn = (c @ W[p + "uk"].T).reshape(T, H, dn)
    v = (c @ W[p + "uv"].T).reshape(T, H, dv)
    qq = np.concatenate([qn, qr], axis=-1)
    kk = np.concatenate([kn, np.broadcast_to(kr[:, None, :], (T, H, dr))], axis=-1)
    o = causal_softmax_heads(qq, kk, v, [m["scale"]] * H, 1)
    return o.reshape(T, H * dv) @ W[p + "o"].T


def dense(W, p, h):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def residual_gate(W, name, h):
    return sigmoid(h @ W[name].T + W[name + ".b"])


def forward(W, cfg, tokens, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the residual after every layer)."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = W["embed"][np.asarray(tokens)].astype(np.float64)
    kept, after = {}, []
    for i, layer in enumerate(cfg["layers"]):
        l, m, kind = f"l{i}.", layer["mixer"], layer["type"]
        h = rms_norm(x, W[l + "norm1"], eps)
        if kind == "attention":
            y = attention(W, l + "mix.", m, h)
        elif kind == "lightning":
            y, _ = lightning(W, l + "mix.", m, h, eps)
        elif kind == "latent_attention":
            if m.get("kv_from") is None:
                kept[i] = latent_rows(W, l + "mix.", m, h, eps)
                rows = kept[i]
            else:
                rows = kept[m["kv_from"]]
            y = latent_attention(W, l + "mix.", m, h, eps, rows)
        else:
            raise ValueError(kind)
        x = x + mult * y * residual_gate(W, l + "rg1", h)
        if layer.get("mlp") is not None:
            h = rms_norm(x, W[l + "norm2"], eps)
            x = x + mult * dense(W, l + "mlp.", h) * residual_gate(W, l + "rg2", h)
        after.append(x.copy())
    z = rms_norm(x, W["final.norm"], eps) @ W["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * np.tanh(z / cap)
    return (z, np.stack(after)) if return_layers else z
