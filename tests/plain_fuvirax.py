"""Plain, slow implementation of the Fuvirax design in numpy, one function per mechanism.

Everything runs on whole sequences in float64 (or whatever dtype the inputs bring), token after
token where a mechanism is recurrent.  It shares no code with the package: the tests compare the
engine's kernels, cache and scheduler against these functions.  ``w`` maps tensor names to arrays,
``cfg`` is the dictionary of a config.json.
"""
import math

import numpy as np


# ---- small functions ------------------------------------------------------------------------
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.log1p(np.exp(-np.abs(z))) + np.maximum(z, 0.0)


def layer_norm(x, weight, bias, eps):
    mu = x.mean(-1, keepdims=True)
    var = ((x - mu) ** 2).mean(-1, keepdims=True)
    return (x - mu) / np.sqrt(var + eps) * weight + bias


def rms_norm(x, weight, eps):
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * weight


def xielu(z, p, q):
    """Positive side: softplus(p) z^2 + z/2; other side: (1/2 + softplus(q)) (e^z - 1 - z) + z/2."""
    a_pos, a_neg = softplus(p), 0.5 + softplus(q)
    zn = np.minimum(z, 0.0)
    return np.where(z > 0, a_pos * z * z + 0.5 * z, a_neg * (np.expm1(zn) - zn) + 0.5 * z)


def dense_feed_forward(x, up, down, act):
    return xielu(x @ up.T, act[0], act[1]) @ down.T


def token_shift(x, mu, before=None):
    """x[t] + (x[t-1] - x[t]) * mu; the token before the first one is `before` (zeros if None).
    Returns the shifted rows and the last unshifted row (what the next token would need)."""
    prev = np.concatenate([(np.zeros_like(x[:1]) if before is None else before[None]), x[:-1]], axis=0)
    return x + (prev - x) * mu, x[-1]


def rotate_half(x, positions, base, dims):
    """Turns the first `dims` lanes of the last axis: lane i pairs with lane i + dims/2."""
    half = dims // 2
    f = base ** (-2.0 * np.arange(half) / dims)
    a = positions[:, None] * f[None, :]
    shape = (len(positions),) + (1,) * (x.ndim - 2) + (half,)
    c, s = np.cos(a).reshape(shape), np.sin(a).reshape(shape)
    u, v = x[..., :half], x[..., half:dims]
    return np.concatenate([u * c - v * s, v * c + u * s, x[..., dims:]], axis=-1)


def short_conv(x, taps_w, history=None):
    """Causal convolution per channel.  x [T, C], taps_w [C, taps] (last column: the current token).
    history: the taps-1 inputs before x (zeros if None).  Returns (y, the new history)."""
    taps = taps_w.shape[1]
    hist = np.zeros((taps - 1, x.shape[1]), dtype=x.dtype) if history is None else history
    full = np.concatenate([hist, x], axis=0)
    y = np.zeros_like(x)
    for j in range(taps):
        y += full[j:j + x.shape[0]] * taps_w[:, j][None, :]
    return y, full[full.shape[0] - (taps - 1):]


# ---- mixers ---------------------------------------------------------------------------------
def latent_attention(x, w, p, m, eps, start=0):
    """Attention whose keys and values are expanded from a shared low-rank latent.  x [T, width]."""
    T = x.shape[0]
    H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = np.arange(start, start + T, dtype=np.float64)
    q = (x @ w[p + "q"].T).reshape(T, H, dn + dr)
    down = x @ w[p + "dkv"].T
    latent = rms_norm(down[:, :R], w[p + "dkv.norm"], eps)
    k_rot = rotate_half(down[:, R:], pos, m["rot"]["base"], m["rot"]["dims"])
    q_rot = rotate_half(q[:, :, dn:], pos, m["rot"]["base"], m["rot"]["dims"])
    k_plain = (latent @ w[p + "uk"].T).reshape(T, H, dn)
    val = (latent @ w[p + "uv"].T).reshape(T, H, dv)
    out = np.zeros((T, H, dv), dtype=x.dtype)
    for h in range(H):
        s = (q[:, h, :dn] @ k_plain[:, h].T + q_rot[:, h] @ k_rot.T) * m["scale"]
        s = np.where(np.tril(np.ones((T, T), dtype=bool)), s, -np.inf)
        s = np.exp(s - s.max(-1, keepdims=True))
        out[:, h] = (s / s.sum(-1, keepdims=True)) @ val[:, h]
    return out.reshape(T, H * dv) @ w[p + "o"].T


def hgrn2(x, w, p, m, eps, state=None):
    """Linear recurrence with one gate f per channel: f of the old state, 1 - f of the new value.  Returns (y, state)."""
    T = x.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(x @ w[p + "q"].T).reshape(T, H, dk)
    v = (x @ w[p + "v"].T).reshape(T, H, dv)
    low = w[p + "lower"]
    f = (low + (1.0 - low) * sigmoid(x @ w[p + "f"].T + w[p + "f.b"])).reshape(T, H, dk)
    S = np.zeros((H, dk, dv), dtype=x.dtype) if state is None else state.copy()
    out = np.zeros((T, H, dv), dtype=x.dtype)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = np.einsum("hkv,hk->hv", S, q[t])
    out = rms_norm(out, w[p + "norm"], eps)
    return out.reshape(T, H * dv) @ w[p + "o"].T, S


def channel_delta(x, w, p, m, eps, state=None):
    """Delta rule with one decay per key channel.  state: (S, history of q, of k, of v) or None."""
    T = x.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    S, hq, hk, hv = (None, None, None, None) if state is None else state
    q, hq = short_conv(x @ w[p + "q"].T, w[p + "q.conv"], hq)
    k, hk = short_conv(x @ w[p + "k"].T, w[p + "k.conv"], hk)
    v, hv = short_conv(x @ w[p + "v"].T, w[p + "v.conv"], hv)
    q, k, v = silu(q).reshape(T, G, dk), silu(k).reshape(T, G, dk), silu(v).reshape(T, H, dv)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * dk ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(x @ w[p + "b"].T)
    rate = np.exp(w[p + "A_log"])[None, :, None]
    decay = np.exp(-rate * softplus((x @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).reshape(T, H, dk))
    gate = sigmoid((x @ w[p + "g1"].T) @ w[p + "g2"].T).reshape(T, H, dv)
    S = np.zeros((H, dk, dv), dtype=x.dtype) if S is None else S.copy()
    out = np.zeros((T, H, dv), dtype=x.dtype)
    rep = H // G
    for t in range(T):
        for h in range(H):
            kk, qq = k[t, h // rep], q[t, h // rep]
            S[h] = decay[t, h][:, None] * S[h]
            u = beta[t, h] * (v[t, h] - S[h].T @ kk)
            S[h] = S[h] + np.outer(kk, u)
            out[t, h] = S[h].T @ qq
    out = out / np.sqrt((out * out).mean(-1, keepdims=True) + eps) * w[p + "norm"] * gate
    return out.reshape(T, H * dv) @ w[p + "o"].T, (S, hq, hk, hv)


MIXERS = {"latent_attention": lambda x, w, p, m, eps: latent_attention(x, w, p, m, eps),
          "hgrn2": lambda x, w, p, m, eps: hgrn2(x, w, p, m, eps)[0],
          "channel_delta": lambda x, w, p, m, eps: channel_delta(x, w, p, m, eps)[0]}


# ---- the layer and the model ------------------------------------------------------------------
def hyper_read(streams, read_w):
    return np.tensordot(read_w, streams, axes=(0, 0))


def hyper_write(streams, mix, out_w, y):
    """streams [S, T, width]; new stream t = sum_s mix[s, t] streams[s] + out_w[t] y."""
    return np.einsum("st,snd->tnd", mix, streams) + out_w[:, None, None] * y[None]


def layer(streams, w, i, spec, eps):
    p = f"l{i}."
    x = layer_norm(hyper_read(streams, w[p + "hc1.in"]), w[p + "norm1"], w[p + "norm1.b"], eps)
    x, _ = token_shift(x, w[p + "shift"])
    y = MIXERS[spec["type"]](x, w, p + "mix.", spec["mixer"], eps) * w[p + "ls1"]
    streams = hyper_write(streams, w[p + "hc1.mix"], w[p + "hc1.out"], y)
    if spec.get("mlp") is not None:
        x = layer_norm(hyper_read(streams, w[p + "hc2.in"]), w[p + "norm2"], w[p + "norm2.b"], eps)
        y = dense_feed_forward(x, w[p + "mlp.up"], w[p + "mlp.down"], w[p + "mlp.act"]) * w[p + "ls2"]
        streams = hyper_write(streams, w[p + "hc2.mix"], w[p + "hc2.out"], y)
    return streams


def layer_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    body = list(range(loop["start"], loop["stop"]))
    return list(range(loop["start"])) + body * loop["times"] + list(range(loop["stop"], n))


def forward(tokens, w, cfg, trace=None):
    """Logits [T, vocab] of one whole sequence.  trace: a list that receives the summed streams after
    every layer run."""
    eps = cfg["norm"]["eps"]
    e = w["embed"][np.asarray(tokens)]
    streams = np.repeat(e[None], cfg["streams"], axis=0)
    for i in layer_order(cfg):
        streams = layer(streams, w, i, cfg["layers"][i], eps)
        if trace is not None:
            trace.append(streams.sum(0))
    x = layer_norm(streams.sum(0), w["final.norm"], w["final.norm.b"], eps)
    return x @ w["embed"].T * cfg["logit_scale"]
