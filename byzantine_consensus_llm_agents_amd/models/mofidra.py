"""Mofidra: parallel-sublayer decoder with differential attention and dense / MoE feed-forwards.

Per layer run (the loop span of the config repeats with shared weights, every run with a
KV cache of its own):

    h = norm(x) * (1 + w)                      one norm feeds both sublayers (fp32 stream x)
    x = x + (mixer(h) + ff(h))

mixer: q / k carry two ``dim``-wide maps per head; each map is a causal softmax attention over
the same values; ``o = a_0 - lam a_1`` with one ``lam`` per layer, then a weightless unit norm
per head times ``1 - diff``.  ff: dense gelu(tanh) layer, or top-k routed relu^2 experts
(weights = softmax over the chosen logits) plus a sigmoid-gated always-on expert.

Kernel plan of one layer run (HIP backend; the torch backend runs the same ops from
``ops/reference.py``):

    fused projection GEMM  [q | k | v | up | shared.up]  (one pass over h)
    rope_multi_kv_write    partial rotary per map + paged K / V^T write
    multimap_attention     prefill tiles (MFMA) and single-token rows (split-KV decode)
    o GEMM; act + down GEMM; moe_route -> grouped expert GEMMs (MFMA, device-side routing)
    residual_add_rmsnorm32 x += o + ff, fused with the NEXT run's norm (fp32 stream)

No host synchronisation anywhere: a decode step is capturable in a HIP graph.
"""

import math
from typing import Dict, List, Optional

import torch

from .config import MofidraConfig
from .transformer import AttnMeta, TPGroup


class MofidraModel:
    # the engine lists one-token segments of a packed step apart from the prefill tiles
    # (AttnMeta.single): they run the split-KV decode kernel
    split_single_rows = True
    logits_dtype = torch.float32
    supports_cascade = False

    def __init__(self, cfg: MofidraConfig, ops, device, dtype=torch.bfloat16, tp: Optional[TPGroup] = None,
                 quant: Optional[str] = None):
        if quant is not None:
            raise ValueError("Mofidra: quantised weights are not supported")
        self.tp = tp or TPGroup()
        if self.tp.size != 1:
            raise ValueError("Mofidra: tensor parallelism is not supported")
        self.cfg, self.ops, self.device, self.dtype, self.quant = cfg, ops, torch.device(device), dtype, None
        self.layers: List[Dict[str, torch.Tensor]] = []
        self.embed = self.lm_head = self.final_norm = None
        # engine-facing sizes (activation reserve estimates)
        self.n_q = max(l.mixer.heads for l in cfg.layers)
        self.n_kv = max(l.mixer.kv_heads for l in cfg.layers)
        self.hd = max(max(l.mixer.maps * l.mixer.dim, l.mixer.vdim) for l in cfg.layers)
        self.inter = max([l.mlp.ff * max(1, l.mlp.top) + l.mlp.shared_ff for l in cfg.layers if l.mlp] or [0])
        self.vocab_local = cfg.vocab_size
        # query rows per prefill attention tile: what the backend's kernel takes for the largest heads
        rows_fn = getattr(ops, "multimap_tile_rows", None)
        self.prefill_tile_rows = min([rows_fn(l.mixer.dim, l.mixer.vdim) for l in cfg.layers]) if rows_fn else 64

    # ------------------------------------------------------------- KV cache
    def kv_block_bytes(self, block_size: int, dtype) -> int:
        item = torch.tensor([], dtype=dtype).element_size()
        return sum((self.cfg.layers[i].mixer.k_width + self.cfg.layers[i].mixer.v_width) * block_size * item
                   for i in self.cfg.layer_runs)

    def alloc_kv(self, num_blocks: int, block_size: int, dtype, device=None):
        """Per layer run: K [NB, G, BS, maps * dim], V [NB, G, vdim, BS] (block ids are shared
        by all runs: one block table per sequence)."""
        dev = device or self.device
        ks, vs = [], []
        for i in self.cfg.layer_runs:
            m = self.cfg.layers[i].mixer
            ks.append(torch.zeros(num_blocks, m.kv_heads, block_size, m.maps * m.dim, dtype=dtype, device=dev))
            vs.append(torch.zeros(num_blocks, m.kv_heads, m.vdim, block_size, dtype=dtype, device=dev))
        return ks, vs

    # ------------------------------------------------------------- weights
    def tensor_shapes(self) -> Dict[str, tuple]:
        """Checkpoint tensor names -> shapes."""
        c, W = self.cfg, self.cfg.hidden_size
        out = {"embed": (c.vocab_size, W), "final.norm": (W,), "head": (c.vocab_size, W)}
        for i, l in enumerate(c.layers):
            m, p = l.mixer, f"l{i}."
            out.update({p + "norm1": (W,), p + "mix.q": (m.q_width, W), p + "mix.k": (m.k_width, W),
                        p + "mix.v": (m.v_width, W), p + "mix.o": (W, m.heads * m.vdim)})
            out.update({p + f"mix.{n}": (m.dim,) for n in ("lq1", "lk1", "lq2", "lk2")})
            f = l.mlp
            if f is not None and f.kind == "dense":
                out.update({p + "mlp.up": (f.ff, W), p + "mlp.down": (W, f.ff)})
            elif f is not None:
                for e in range(f.experts):
                    out.update({p + f"mlp.e{e}.up": (f.ff, W), p + f"mlp.e{e}.down": (W, f.ff)})
                out.update({p + "mlp.router": (f.experts, W), p + "mlp.router.b": (f.experts,)})
                if f.shared_ff:
                    out.update({p + "mlp.shared.up": (f.shared_ff, W), p + "mlp.shared.down": (W, f.shared_ff),
                                p + "mlp.shared.sg": (1, W)})
        return out

    def random_state_dict(self, seed: int = 0, std: float = 0.05) -> Dict[str, torch.Tensor]:
        """bf16-representable random weights under the checkpoint names (tests, benchmarks)."""
        gen = torch.Generator().manual_seed(seed)
        sd = {}
        for name, shape in self.tensor_shapes().items():
            if name.endswith("norm1") or name == "final.norm":
                t = torch.randn(shape, generator=gen) * 0.1
            elif ".mix.l" in name:
                t = torch.randn(shape, generator=gen) * 0.3
            elif name.endswith("router.b"):
                t = torch.randn(shape, generator=gen) * 0.5
            elif name == "embed":
                t = torch.randn(shape, generator=gen)
            else:
                t = torch.randn(shape, generator=gen) * (std if name != "head" else 1.0 / math.sqrt(shape[1]))
            sd[name] = t.to(torch.bfloat16)
        return sd

    def init_random(self, seed: int = 0, std: float = 0.05):
        self.load_hf_state_dict(self.random_state_dict(seed, std))

    def load_hf_state_dict(self, sd):
        """Load the checkpoint tensors (names of `tensor_shapes`); projections that read the same
        input are stacked into one GEMM weight, experts into [E, ...] tensors."""
        c, dev, dt = self.cfg, self.device, self.dtype

        def get(name, dtype=None):
            return sd[name].to(device=dev, dtype=dtype or dt).contiguous()

        from ..ops.reference import rope_inv_freq
        self.layers = []
        for i, l in enumerate(c.layers):
            m, f, p = l.mixer, l.mlp, f"l{i}."
            fused = [get(p + "mix.q"), get(p + "mix.k"), get(p + "mix.v")]
            L = {"norm": get(p + "norm1", torch.float32), "o": get(p + "mix.o"),
                 "inv_freq": rope_inv_freq(m.rot_dims, m.rot_base, dev)}
            lq1, lk1, lq2, lk2 = (sd[p + f"mix.{n}"].float() for n in ("lq1", "lk1", "lq2", "lk2"))
            # one number per layer, fp32: exp(<lq1, lk1>) - exp(<lq2, lk2>) + diff
            L["lam"] = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) + m.diff)
            if f is not None and f.kind == "dense":
                fused.append(get(p + "mlp.up"))
                L["down"] = get(p + "mlp.down")
            elif f is not None:
                L["e_up"] = torch.stack([get(p + f"mlp.e{e}.up") for e in range(f.experts)]).contiguous()
                L["e_down"] = torch.stack([get(p + f"mlp.e{e}.down") for e in range(f.experts)]).contiguous()
                L["router"] = get(p + "mlp.router", torch.float32)
                L["router_b"] = get(p + "mlp.router.b", torch.float32)
                if f.shared_ff:
                    fused.append(get(p + "mlp.shared.up"))
                    L["s_down"] = get(p + "mlp.shared.down")
                    L["s_gate"] = get(p + "mlp.shared.sg", torch.float32).reshape(-1)
            L["fused"] = torch.cat(fused).contiguous()
            self.layers.append(L)
        self.embed = get("embed")
        self.lm_head = get("head")
        self.final_norm = get("final.norm", torch.float32)

    def weight_bytes(self) -> int:
        n = sum(t.numel() * t.element_size() for L in self.layers for t in L.values() if torch.is_tensor(t))
        return n + self.embed.numel() * self.embed.element_size() + self.lm_head.numel() * self.lm_head.element_size()

    # ------------------------------------------------------------- forward
    def forward(self, tokens: torch.Tensor, meta: AttnMeta, k_cache, v_cache, trace: Optional[list] = None):
        """Logits (fp32) of the rows ``meta.logits_idx`` (all rows when None).  ``trace``: a list
        that receives a copy of the residual stream after every layer run (debugging)."""
        ops, c = self.ops, self.cfg
        eps, dt = c.rms_eps, self.dtype
        runs = c.layer_runs
        h, x = ops.embed_scale_rmsnorm(tokens, self.embed, c.embed_scale, self.layers[runs[0]]["norm"], eps, 1.0, dt)
        for r, li in enumerate(runs):
            spec, L = c.layers[li], self.layers[li]
            m, f = spec.mixer, spec.mlp
            y = ops.linear(h, L["fused"])
            q = ops.rope_multi_kv_write(y, meta.positions, meta.slots, m.heads, m.kv_heads, m.maps, m.dim, m.vdim,
                                        L["inv_freq"], k_cache[r], v_cache[r])
            attn = ops.multimap_attention(q, k_cache[r], v_cache[r], meta, m.scale, m.maps, L["lam"], eps,
                                          1.0 - m.diff, m.vdim)
            last = r == len(runs) - 1
            if last and meta.logits_idx is not None:
                # past the last attention only the rows whose logits are asked for matter
                idx = meta.logits_idx
                attn, x, h, y = (t.index_select(0, idx) for t in (attn, x, h, y))
            parts = [ops.linear(attn, L["o"])]
            gate = gated = None
            off = m.q_width + m.k_width + m.v_width
            if f is not None and f.kind == "dense":
                parts.append(ops.linear(ops.act_fn(y[:, off:off + f.ff], "gelu_tanh"), L["down"]))
            elif f is not None:
                idx_e, w_e, gate = ops.moe_route(h, L["router"], L["router_b"], f.top, L.get("s_gate"))
                parts.append(ops.moe_experts(h, L["e_up"], L["e_down"], idx_e, w_e, "relu2"))
                if f.shared_ff:
                    gated = ops.linear(ops.act_fn(y[:, off:off + f.shared_ff], "relu2"), L["s_down"])
            w_next = self.final_norm if last else self.layers[runs[r + 1]]["norm"]
            h = ops.residual_add_rmsnorm32(x, parts, w_next, eps, 1.0, dt, gate, gated)
            if trace is not None:
                trace.append(x.clone())
        return ops.linear(h, self.lm_head).float()
