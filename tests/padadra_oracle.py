"""Plain float64 implementation of the Padadra equations: one function per mechanism, a loop per
token, no cache, no batching, no state carried between calls.  It shares no code with the
package; the tests compare the engine with it.

Notation: ``sd`` maps checkpoint names to float64 arrays, ``cfg`` is the config.json dictionary,
``h`` is a mixer's input [T, W] for ONE sequence that starts at position 0.
"""
import math

import numpy as np


def to_f64(sd):
    import torch
    return {k: (v.double().numpy() if v.dtype != torch.int32 else v.numpy()) for k, v in sd.items()}


def unit_rms(x, eps):
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def embed(sd, cfg, tokens):
    e = cfg.get("embedding") or {}
    x = sd["embed"][np.asarray(tokens)] * float(e.get("scale", 1.0))
    bg = e.get("bigram")
    if bg:
        n = int(bg["buckets"])
        for t, tok in enumerate(tokens):
            row = n if t == 0 else (int(tokens[t - 1]) * int(bg["mul_prev"]) + int(tok) * int(bg["mul_cur"])) % n
            x[t] = x[t] + sd["bigram"][row]
    return x


def short_conv(u, w):
    """y_t = sum_j w[:, j] u_(t - taps + 1 + j); u [T, C], w [C, taps]; zeros before the start."""
    T, taps = u.shape[0], w.shape[1]
    y = np.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def scaled_freqs(dims, base, scaling):
    f = np.array([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)])
    if not scaling:
        return f
    factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = f.copy()
    for i, fi in enumerate(f):
        wl = 2.0 * math.pi / fi
        if wl < orig / high:
            continue
        if wl > orig / low:
            out[i] = fi / factor
        else:
            s = (orig / wl - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate_pairs(x, angle):
    """x [..., 2 n]: pair (2i, 2i + 1) turned by angle[i]."""
    y = x.copy()
    a, b = x[..., 0::2], x[..., 1::2]
    c, s = np.cos(angle), np.sin(angle)
    y[..., 0::2] = a * c - b * s
    y[..., 1::2] = b * c + a * s
    return y


def windowed_sink_attention(q, k, v, sink, scale, window):
    """q [T, H, d], k [T, G, d], v [T, G, e]; position i sees 0 <= i - j < window (all when
    window is None); the denominator also holds exp(sink[h])."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        lo = 0 if window is None else max(0, i - window + 1)
        for h in range(H):
            g = h // (H // G)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            m = max(s.max(), sink[h])
            p = np.exp(s - m)
            out[i, h] = (p @ v[lo:i + 1, g]) / (p.sum() + math.exp(sink[h] - m))
    return out


def left_mixer(sd, p, m, h, eps):
    T = h.shape[0]
    H, G, d, e = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = h @ sd[p + "q"].T + sd[p + "q.b"]
    k = h @ sd[p + "k"].T + sd[p + "k.b"]
    v = h @ sd[p + "v"].T + sd[p + "v.b"]
    if m.get("conv"):
        q, k, v = (short_conv(u, sd[p + n + ".conv"]) for u, n in ((q, "q"), (k, "k"), (v, "v")))
    q = unit_rms(q, eps) * sd[p + "q.norm"]
    k = unit_rms(k, eps) * sd[p + "k.norm"]
    q, k, v = q.reshape(T, H, d), k.reshape(T, G, d), v.reshape(T, G, e)
    pos = np.arange(T, dtype=np.float64)
    rot = m.get("rot")
    if rot and int(rot["dims"]):
        r = int(rot["dims"])
        f = scaled_freqs(r, rot["base"], rot.get("scaling"))
        ang = pos[:, None, None] * f[None, None, :]
        q[..., :r] = rotate_pairs(q[..., :r], ang)
        k[..., :r] = rotate_pairs(k[..., :r], ang)
    base = float(rot["base"]) if rot else 10000.0
    fv = np.array([base ** (-2.0 * i / e) for i in range(e // 2)])
    angv = pos[:, None, None] * fv[None, None, :]
    v = rotate_pairs(v, angv)
    mask = m.get("mask")
    o = windowed_sink_attention(q, k, v, sd[p + "sink"], float(m["scale"]), int(mask["size"]) if mask else None)
    o = rotate_pairs(o, -angv)
    return o.reshape(T, H * e) @ sd[p + "o"].T


def hgrn2_mixer(sd, p, m, h, eps):
    T = h.shape[0]
    H, d, e = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(h @ sd[p + "q"].T).reshape(T, H, d)
    v = (h @ sd[p + "v"].T).reshape(T, H, e)
    low = sd[p + "lower"]
    f = (low + (1.0 - low) * sigmoid(h @ sd[p + "f"].T + sd[p + "f.b"])).reshape(T, H, d)
    S = np.zeros((H, d, e))
    out = np.zeros((T, H, e))
    for t in range(T):
        for a in range(H):
            S[a] = f[t, a][:, None] * S[a] + np.outer(1.0 - f[t, a], v[t, a])
            out[t, a] = S[a].T @ q[t, a]
    out = unit_rms(out, eps) * sd[p + "norm"]
    return out.reshape(T, H * e) @ sd[p + "o"].T


def parallel_mixer(sd, p, m, h, eps):
    a = unit_rms(left_mixer(sd, p + "left.", m["left"], h, eps), eps) * sd[p + "left.out"]
    b = unit_rms(hgrn2_mixer(sd, p + "right.", m["right"], h, eps), eps) * sd[p + "right.out"]
    return 0.5 * (a + b)


def channel_delta_mixer(sd, p, m, h, eps):
    T = h.shape[0]
    H, G, d, e = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q, k, v = h @ sd[p + "q"].T, h @ sd[p + "k"].T, h @ sd[p + "v"].T
    if m.get("conv"):
        q, k, v = (short_conv(u, sd[p + n + ".conv"]) for u, n in ((q, "q"), (k, "k"), (v, "v")))
    q, k, v = silu(q).reshape(T, G, d), silu(k).reshape(T, G, d), silu(v).reshape(T, H, e)
    q = q / np.sqrt((q * q).sum(-1, keepdims=True) + 1e-6) * d ** -0.5
    k = k / np.sqrt((k * k).sum(-1, keepdims=True) + 1e-6)
    beta = sigmoid(h @ sd[p + "b"].T)
    a = ((h @ sd[p + "a1"].T) @ sd[p + "a2"].T + sd[p + "dt_bias"]).reshape(T, H, d)
    decay = np.exp(-np.exp(sd[p + "A_log"])[None, :, None] * softplus(a))
    gate = sigmoid((h @ sd[p + "g1"].T) @ sd[p + "g2"].T).reshape(T, H, e)
    S = np.zeros((H, d, e))
    out = np.zeros((T, H, e))
    for t in range(T):
        for a_ in range(H):
            g = a_ // (H // G)
            S[a_] = decay[t, a_][:, None] * S[a_]
            u = beta[t, a_] * (v[t, a_] - S[a_].T @ k[t, g])
            S[a_] = S[a_] + np.outer(k[t, g], u)
            out[t, a_] = S[a_].T @ q[t, g]
    out = unit_rms(out, eps) * sd[p + "norm"] * gate
    return out.reshape(T, H * e) @ sd[p + "o"].T


def feed_forward(sd, p, f, h):
    if f["kind"] != "dense":
        raise ValueError(f["kind"])
    return np.square(np.maximum(h @ sd[p + "up"].T, 0.0)) @ sd[p + "down"].T


MIXERS = {"parallel": parallel_mixer, "channel_delta": channel_delta_mixer}


def forward(sd, cfg, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out`` receives the stream after every layer."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    x = embed(sd, cfg, tokens)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = MIXERS[layer["type"]](sd, p + "mix.", layer["mixer"], unit_rms(x, eps) * sd[p + "norm1"], eps)
        if layer.get("mlp"):
            y = y + feed_forward(sd, p + "mlp.", layer["mlp"], unit_rms(x, eps) * sd[p + "norm2"])
        x = x + mult * y
        if layers_out is not None:
            layers_out.append(x.copy())
    return (unit_rms(x, eps) * sd["final.norm"]) @ sd["head"].T
