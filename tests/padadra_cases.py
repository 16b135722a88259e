"""Small Padadra configurations, random checkpoints on disk and engines for the tests."""
import json
import os

import torch

from byzantine_consensus_llm_agents_amd.models.config import PadadraConfig
from byzantine_consensus_llm_agents_amd.models.padadra import PadadraModel


def left(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, window=20, rot_dims=8, base=5000.0, scaling=(3.0, 1.0, 3.0, 48), scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if conv:
        m["conv"] = conv
    if window:
        m["mask"] = {"size": window}
    m["rot"] = {"dims": rot_dims, "base": base}
    if scaling:
        m["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return m


def parallel(l, heads=2, dim=12, vdim=20, ff=40):
    return {"type": "parallel", "mixer": {"left": l, "right": {"heads": heads, "dim": dim, "vdim": vdim}},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def delta(heads=4, kv_heads=2, dim=16, vdim=12, conv=4, ff=40, ranks=(6, 5)):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "decay_rank": ranks[0], "gate_rank": ranks[1]}
    if conv:
        m["conv"] = conv
    return {"type": "channel_delta", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=48, vocab=53, bigram=(31, 5, 3), scale=2.0, eps=1e-5, mult=0.8):
    emb = {"scale": scale}
    if bigram:
        emb["bigram"] = dict(zip(("buckets", "mul_prev", "mul_cur"), bigram))
    return {"architecture": "Padadra", "width": width, "vocab": vocab, "embedding": emb, "norm": {"eps": eps},
            "residual_mult": mult, "layers": layers}


# every branch: with / without convolution, window, rotary, frequency scaling, bigram, feed-forward;
# GQA and MHA on both mixers; key and value widths that differ; taps 2 .. 5; sizes off the 16-wide
# MFMA grid and past 64 state columns / 64 state rows; windows shorter than a page and across pages
CASES = {
    "mixed": config([parallel(left()), delta(ff=0), parallel(left(2, 1, 24, 16, 2, 7, 24, 900.0, None), 3, 8, 8),
                     delta(3, 3, 20, 18, 2, 24, (4, 7))]),
    "plain": config([delta(2, 1, 8, 8, 0, 24), parallel(left(2, 2, 16, 16, 0, 0, 0, 10000.0, None), 1, 16, 16, 0)],
                    width=32, vocab=37, bigram=None, scale=1.0, mult=1.0),
    "wide": config([parallel(left(6, 2, 72, 40, 5, 33, 36, 20000.0, (4.0, 1.0, 4.0, 64)), 2, 96, 72, 56),
                    delta(2, 1, 80, 72, 3, 0, (9, 3))], width=64, vocab=45, bigram=(17, 1009, 7), eps=1e-6, mult=0.5),
}


def checkpoint(cfg_dict, path, seed=0):
    """Write config.json + model.safetensors (bf16) under `path`; returns the tensors."""
    from safetensors.torch import save_file
    cfg = PadadraConfig.from_dict(cfg_dict, "test")
    sd = PadadraModel(cfg, None, "cpu").random_state_dict(seed, std=0.12)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(cfg_dict, fh)
    save_file({k: v.contiguous() for k, v in sd.items()}, os.path.join(path, "model.safetensors"))
    return sd


def engine(path, backend="torch", dtype=torch.float32, pool_tokens=512, rows=4, max_len=512, **kw):
    from byzantine_consensus_llm_agents_amd.engine.engine import EngineArgs, InferenceEngine
    args = EngineArgs.from_configs(path, backend=backend, weights=path, seed=0, dtype=dtype, kv_block_size=16,
                                   max_batch_seqs=rows, max_model_len=max_len, kv_pool_tokens=pool_tokens,
                                   use_hip_graphs=kw.pop("use_hip_graphs", False), prefix_caching=kw.pop("prefix_caching", False),
                                   **kw)
    return InferenceEngine(args)


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def segments(parts, rows, device="cpu"):
    """AttnMeta of a packed step over segments ``parts`` = [(first position, count)] that continue
    the state rows ``rows`` (no KV fields: for ops that only read the segment tables)."""
    from byzantine_consensus_llm_agents_amd.models.transformer import AttnMeta
    pos, seg, qs = [], [], [0]
    for i, (a, n) in enumerate(parts):
        pos += list(range(a, a + n))
        seg += [i] * n
        qs.append(qs[-1] + n)
    i32 = dict(dtype=torch.int32, device=device)
    return AttnMeta(positions=torch.tensor(pos, **i32), slots=None, block_tables=None, seq_lens=None,
                    q_start=torch.tensor(qs, **i32), state_rows=torch.tensor(rows, **i32), token_seq=torch.tensor(seg, **i32))


def random_config(seed):
    """A configuration drawn from a seed: sizes, head counts, layer order, windows, taps, constants."""
    import random
    r = random.Random(seed)
    even = lambda lo, hi: 2 * r.randint(lo // 2, hi // 2)  # noqa: E731
    layers = []
    for _ in range(r.randint(2, 5)):
        ff = r.choice([0, 24, 40, 72])
        if r.random() < 0.55:
            kv = r.choice([1, 2, 3])
            heads = kv * r.choice([1, 2, 4])
            dim, vdim = even(6, 80), even(6, 80)
            rot = r.choice([0, even(2, dim), dim])
            scaling = r.choice([None, (r.choice([2.0, 4.0, 8.0]), 1.0, r.choice([2.0, 4.0]), r.choice([16, 64, 256]))])
            l = left(heads, kv, dim, vdim, r.choice([0, 2, 3, 4, 5]), r.choice([0, 1, 5, 16, 23, 64]), rot,
                     r.choice([100.0, 10000.0, 500000.0]), scaling if rot else None, r.choice([None, 0.2, 0.05]))
            layers.append(parallel(l, r.randint(1, 4), even(4, 72), r.randint(3, 72), ff))
        else:
            kv = r.choice([1, 2, 3])
            layers.append(delta(kv * r.choice([1, 2]), kv, even(4, 100), r.randint(3, 72), r.choice([0, 2, 4]), ff,
                                (r.randint(2, 9), r.randint(2, 9))))
    return config(layers, width=even(24, 96), vocab=r.randint(20, 90),
                  bigram=r.choice([None, (r.randint(5, 40), r.randint(1, 2000), r.randint(1, 50))]),
                  scale=r.choice([1.0, 3.0]), eps=r.choice([1e-5, 1e-6]), mult=r.choice([1.0, 0.7, 0.4]))
