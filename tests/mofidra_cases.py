"""Small Mofidra configurations, random checkpoints on disk and engines for the tests."""
import json
import os

import torch

from byzantine_consensus_llm_agents_amd.models.config import MofidraConfig
from byzantine_consensus_llm_agents_amd.models.mofidra import MofidraModel


def mixer(heads=4, kv_heads=2, dim=16, vdim=24, rot_dims=8, base=5000.0, diff=0.3, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
            "scale": scale if scale is not None else dim ** -0.5, "rot": {"dims": rot_dims, "base": base}}


def dense(ff=48):
    return {"kind": "dense", "ff": ff}


def moe(experts=4, top=2, ff=20, shared=28):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def config(layers, width=64, vocab=61, loop=None, scale=3.0, eps=1e-5):
    cfg = {"architecture": "Mofidra", "width": width, "vocab": vocab, "embedding": {"scale": scale},
           "norm": {"eps": eps}, "layers": [{"type": "attention", "mixer": m, "mlp": f} for m, f in layers]}
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


# every branch: GQA and MHA, partial / full / no rotary, dense / routed / no feed-forward, with and
# without the always-on expert, top 1 .. all experts, a loop in the middle, sizes off the MFMA grid
CASES = {
    "mixed": config([(mixer(), moe()), (mixer(4, 4, 16, 16, 16), dense()), (mixer(2, 1, 24, 40, 12), moe(3, 1, 16, 0)),
                     (mixer(4, 2, 16, 24, 0), None), (mixer(3, 3, 20, 18, 20, diff=0.7), moe(5, 5, 12, 8))],
                    loop=(1, 3, 3)),
    "plain": config([(mixer(2, 2, 32, 32, 32, scale=0.11), dense(40)), (mixer(2, 1, 32, 64, 16), moe(8, 2, 16, 32))],
                    width=48, vocab=37, scale=1.0),
    "wide": config([(mixer(2, 1, 72, 136, 36), moe(6, 3, 24, 16)), (mixer(2, 2, 72, 136, 72), dense(32))],
                   width=96, vocab=45, loop=(0, 2, 2), scale=8.0, eps=1e-6),
}


def checkpoint(cfg_dict, path, seed=0):
    """Write config.json + model.safetensors (bf16) under `path`; returns the tensors."""
    from safetensors.torch import save_file
    cfg = MofidraConfig.from_dict(cfg_dict, "test")
    sd = MofidraModel(cfg, None, "cpu").random_state_dict(seed, std=0.12)
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
