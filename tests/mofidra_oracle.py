"""Plain, slow float64 implementation of the Mofidra equations: the oracle of the tests.

One function per mechanism, whole sequences only (no cache, no batching, no paging); it
shares no code with the package.  ``cfg`` is the config.json dictionary, ``sd`` the checkpoint
tensors by name.
"""
import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return unit_rms(x, eps) * (1.0 + w.to(F64))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def relu_squared(z):
    return torch.clamp(z, min=0.0) ** 2


def rotate(x, positions, dims, base):
    """x [T, heads, dim]: feature i < dims/2 pairs with i + dims/2; the rest pass through."""
    if dims == 0:
        return x
    half = dims // 2
    out = x.clone()
    for i in range(half):
        ang = positions.to(F64) * float(base) ** (-2.0 * i / dims)
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * c - v * s
        out[..., i + half] = v * c + u * s
    return out


def differential_lambda(sd, prefix, diff):
    lq1, lk1, lq2, lk2 = (sd[prefix + n].to(F64) for n in ("lq1", "lk1", "lq2", "lk2"))
    return float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) + diff)


def differential_attention(h, sd, prefix, m, eps):
    """h [T, width] -> [T, width].  Two softmax maps per head over the same values."""
    T = h.shape[0]
    H, G, d, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ sd[prefix + "q"].to(F64).T).view(T, H, 2, d)
    k = (h @ sd[prefix + "k"].to(F64).T).view(T, G, 2, d)
    v = (h @ sd[prefix + "v"].to(F64).T).view(T, G, vd)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = torch.stack([rotate(q[:, :, j], pos, rot["dims"], rot["base"]) for j in range(2)], 2)
    k = torch.stack([rotate(k[:, :, j], pos, rot["dims"], rot["base"]) for j in range(2)], 2)
    lam = differential_lambda(sd, prefix, m["diff"])
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        maps = []
        for j in range(2):
            out = torch.zeros(T, vd, dtype=F64)
            for t in range(T):
                sc = (k[:t + 1, g, j] @ q[t, hh, j]) * m["scale"]
                out[t] = torch.softmax(sc, 0) @ v[:t + 1, g]
            maps.append(out)
        o = maps[0] - lam * maps[1]
        heads.append(unit_rms(o, eps) * (1.0 - m["diff"]))
    return torch.cat(heads, -1) @ sd[prefix + "o"].to(F64).T


def expert(h, sd, prefix, act):
    return act(h @ sd[prefix + "up"].to(F64).T) @ sd[prefix + "down"].to(F64).T


def routed_experts(h, sd, prefix, f):
    E, top = f["router"]["experts"], f["router"]["top"]
    z = h @ sd[prefix + "router"].to(F64).T + sd[prefix + "router.b"].to(F64)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        w = torch.softmax(z[t, order], 0)
        for wj, e in zip(w, order):
            out[t] += wj * expert(h[t:t + 1], sd, prefix + f"e{e}.", relu_squared)[0]
    if f.get("shared"):
        gate = torch.sigmoid(h @ sd[prefix + "shared.sg"].to(F64).T)
        out = out + gate * expert(h, sd, prefix + "shared.", relu_squared)
    return out


def feed_forward(h, sd, prefix, f):
    if f is None:
        return torch.zeros_like(h)
    if f["kind"] == "dense":
        return expert(h, sd, prefix, gelu_tanh)
    return routed_experts(h, sd, prefix, f)


def layer_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    span = list(range(loop["start"], loop["stop"]))
    return list(range(loop["start"])) + span * loop["times"] + list(range(loop["stop"], n))


def router_margins(cfg, sd, tokens):
    """Per position, the smallest gap between a chosen and a not-chosen router logit over all
    layer runs (a position whose margin is tiny has two equally valid routings)."""
    gaps = [torch.full((len(tokens),), math.inf, dtype=F64)]

    def hook(h, prefix, f):
        if f is not None and f["kind"] == "moe" and f["router"]["top"] < f["router"]["experts"]:
            z = h @ sd[prefix + "router"].to(F64).T + sd[prefix + "router.b"].to(F64)
            s = torch.sort(z, -1, descending=True).values
            gaps.append(s[:, f["router"]["top"] - 1] - s[:, f["router"]["top"]])
    forward(cfg, sd, tokens, hook)
    return torch.stack(gaps).min(0).values


def router_margin(cfg, sd, tokens):
    return float(router_margins(cfg, sd, tokens).min())


def forward(cfg, sd, tokens, hook=None, stream=None):
    """Logits [T, vocab] (float64) of one whole sequence; ``stream`` collects x after every layer run."""
    eps = cfg["norm"]["eps"]
    x = sd["embed"].to(F64)[torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for i in layer_order(cfg):
        spec = cfg["layers"][i]
        h = layer_norm(x, sd[f"l{i}.norm1"], eps)
        if hook is not None:
            hook(h, f"l{i}.mlp.", spec["mlp"])
        x = x + (differential_attention(h, sd, f"l{i}.mix.", spec["mixer"], eps) + feed_forward(h, sd, f"l{i}.mlp.", spec["mlp"]))
        if stream is not None:
            stream.append(x.clone())
    return layer_norm(x, sd["final.norm"], eps) @ sd["head"].to(F64).T
