"""Plain implementation of the Digasun design in numpy float64: one function per mechanism, whole sequences
only (no cache, no state carried between calls), written from the design's equations and sharing no code with
the package.  `weights` maps checkpoint names to arrays; `cfg` is the config.json dictionary."""
import math

import numpy as np


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rms_unit(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(axis=-1, keepdims=True)
    var = ((x - mu) ** 2).mean(axis=-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * w + b


def causal_conv(h, w):
    """h [T, D], w [D, taps]: out_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros before the start."""
    T, D = h.shape
    taps = w.shape[1]
    out = np.zeros_like(h)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotate(x, positions, dims, base):
    """x [T, heads, dim]: the first `dims` lanes of each head turned by position, lane i paired with i + dims/2."""
    out = x.copy()
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims)
    a = positions[:, None].astype(np.float64) * f[None, :]          # [T, half]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


def attention_keys_values(W, p, m, h, positions):
    """The rotated keys [T, G, dim] and the values [T, G, vdim] of a layer that has projections of its own."""
    T = h.shape[0]
    G = m["kv_heads"]
    k = (h @ W[p + "k"].T + W[p + "k.b"]).reshape(T, G, m["dim"])
    v = (h @ W[p + "v"].T + W[p + "v.b"]).reshape(T, G, m["vdim"])
    return rotate(k, positions, m["rot"]["dims"], m["rot"]["base"]), v


def attention(W, p, m, h, k, v):
    """h [T, D] the mixer's input; k [T, G, dim] rotated keys and v [T, G, vdim] values (own or borrowed)."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = np.arange(T)
    q = rotate((h @ W[p + "q"].T + W[p + "q.b"]).reshape(T, H, dk), positions, m["rot"]["dims"], m["rot"]["base"])
    window = m["mask"]["size"] if m.get("mask") else 0
    sink, talk = W[p + "sink"], W[p + "talk"]
    weights = np.zeros((H, T, T))
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]
        for i in range(T):
            lo = max(0, i - window + 1) if window else 0
            row = s[i, lo:i + 1]
            mx = max(row.max(), sink[hd])
            e = np.exp(row - mx)
            weights[hd, i, lo:i + 1] = e / (e.sum() + math.exp(sink[hd] - mx))
    mixed = np.einsum("hg,gij->hij", talk, weights)
    out = np.zeros((T, H, dv))
    for hd in range(H):
        out[:, hd] = mixed[hd] @ v[:, hd // (H // G)]
    return out.reshape(T, H * dv) @ W[p + "o"].T + W[p + "o.b"]


def gla(W, p, m, h, eps):
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).reshape(T, H, dk) * dk ** -0.5
    k = (h @ W[p + "k"].T).reshape(T, H, dk)
    v = (h @ W[p + "v"].T).reshape(T, H, dv)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / m["tau"])).reshape(T, H, dk)
    S = np.zeros((H, dk, dv))
    o = np.zeros((T, H, dv))
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hkv,hk->hv", S, q[t])
    o = rms_unit(o, eps) * W[p + "norm"]
    return (o.reshape(T, H * dv) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def dense_ff(W, p, mlp, h):
    lim = mlp["limit"]
    g = np.minimum(h @ W[p + "gate"].T, lim)
    u = np.clip(h @ W[p + "up"].T, -lim, lim)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def expert(W, p, h):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def moe_ff(W, p, mlp, h):
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = h @ W[p + "router"].T + W[p + "router.b"]
    out = np.zeros((h.shape[0], W[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        chosen = np.argsort(-z[t], kind="stable")[:top]
        w = np.exp(z[t, chosen] - z[t, chosen].max())
        w /= w.sum()
        for e, we in zip(chosen, w):
            out[t] += we * expert(W, f"{p}e{e}.", h[t:t + 1])[0]
    if mlp.get("shared"):
        out += expert(W, p + "shared.", h) * sigmoid(h @ W[p + "shared.sg"].T)
    return out


def feed_forward(W, p, mlp, h):
    return dense_ff(W, p, mlp, h) if mlp["kind"] == "dense" else moe_ff(W, p, mlp, h)


def token_side(W, cfg, i, x, tokens):
    d, eps = cfg["token_side"]["dim"], cfg["norm"]["eps"]
    e = W["side.embed"][tokens][:, i * d:(i + 1) * d]
    g = gelu_tanh(x @ W[f"l{i}.side.gate"].T) * e
    y = g @ W[f"l{i}.side.proj"].T
    return rms_unit(y, eps) * W[f"l{i}.side.norm"]


def forward(cfg, weights, tokens, return_layers=False):
    """Logits [T, vocab] of one sequence from its first token; with return_layers also the residual after each layer."""
    W = {k: np.asarray(v, dtype=np.float64) for k, v in weights.items()}
    tokens = np.asarray(tokens)
    T = len(tokens)
    eps = cfg["norm"]["eps"]
    positions = np.arange(T)
    x = W["embed"][tokens] * cfg["embedding"]["scale"]
    kept = {}
    layers = []
    for i, layer in enumerate(cfg["layers"]):
        l, m = f"l{i}.", layer["mixer"]
        h = layer_norm(x, W[l + "norm1"], W[l + "norm1.b"], eps)
        hm = h + causal_conv(h, W[l + "canon1"]) if cfg.get("canon") else h
        if layer["type"] == "attention":
            if m.get("kv_from") is not None:
                k, v = kept[m["kv_from"]]
            else:
                k, v = kept[i] = attention_keys_values(W, l + "mix.", m, hm, positions)
            delta = attention(W, l + "mix.", m, hm, k, v)
        else:
            delta = gla(W, l + "mix.", m, hm, eps)
        if layer.get("mlp"):
            hf = h + causal_conv(h, W[l + "canon2"]) if cfg.get("canon") else h
            delta = delta + feed_forward(W, l + "mlp.", layer["mlp"], hf)
        x = x + delta
        if cfg.get("token_side"):
            x = x + token_side(W, cfg, i, x, tokens)
        layers.append(x.copy())
    logits = layer_norm(x, W["final.norm"], W["final.norm.b"], eps) @ W["head"].T
    return (logits, np.stack(layers)) if return_layers else logits
