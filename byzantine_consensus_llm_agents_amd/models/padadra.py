"""Padadra: parallel-sublayer decoder whose mixers carry per-sequence state.

Every layer is ``x <- x + m (mixer(g1 x^) + ff(g2 x^))`` with ``x^ = x / rms(x)`` and scalar gains
g1, g2 (fp32 residual stream x).  The embedding adds a hashed bigram row (previous and current
token).  Two layer types:

* ``parallel``: half the sum of two mixers over the same input, each RMS-normed over the width:
  a sliding-window softmax attention with a per-head sink (short convolution on q / k / v, one
  norm over the whole q and k projections, interleaved-pair rotary with wavelength-dependent
  frequency scaling, values rotated by their own position and the head output turned back by the
  query's), and an HGRN2 recurrence (the forget gate also weights the write);
* ``channel_delta``: a gated delta rule with one decay per head and key channel, short
  convolutions + silu on q / k / v, unit-vector q / k, a low-rank sigmoid output gate.

Feed-forward: ``down(relu(up h)^2)``.

State per sequence, besides the paged K / V of the attention layers: the previous token, the last
``taps - 1`` inputs of every convolution, and one fp32 ``dim x vdim`` matrix per recurrent head.
It lives in tables indexed by the engine's state row (``alloc_state``); a segment that starts at
position 0 starts from empty state, so rows are reused without a reset.

Kernel plan of one layer (HIP backend; the torch backend runs the same ops from
``ops/reference.py``):

    fused projection GEMM over g1 x^ (+ bias)   [q | k | v | right.q | right.f | right.v]  or
                                                [q | k | v | beta | a1 | g1]
    short_conv                 causal taps over the packed rows + the state row's tail
    rope_pairs_kv_write        q / k norm, rotary, value rotation, paged K / V^T write
    multimap_attention         one map, window + sink: prefill tiles (MFMA) / split-KV decode
    hgrn2_prepare / delta_prepare   fp32 read / write / decay vectors
    gated_state_scan           the recurrence, state columns in registers
    head_norm_gate             per-head RMS norm (x sigmoid gate)
    o GEMMs; up GEMM over g2 x^ -> relu^2 -> down GEMM
    residual_mix_norm          x += m (...) fused with the out-norms of both mixers and the NEXT
                               layer's two scalar norms

Large prefill steps run the recurrent branch (prepare, scan, head norm) on a second stream
beside the attention branch and the feed-forward.

No host synchronisation anywhere: a decode step is capturable in a HIP graph.
"""

import math
from typing import Dict, List, Optional

import torch

from .config import PadadraConfig
from .transformer import AttnMeta, TPGroup


class PadadraModel:
    split_single_rows = True
    logits_dtype = torch.float32
    supports_cascade = False
    has_seq_state = True      # recurrent state: a cached prompt prefix cannot stand in for its tokens
    # Packed steps of at least this many rows run a layer's recurrence on a second stream beside the
    # attention branch and the feed-forward (the token-sequential scan leaves most of the chip idle);
    # None = never.  Decode steps (captured into graphs) and small steps stay on one stream.
    overlap_min_rows = 2048

    def __init__(self, cfg: PadadraConfig, ops, device, dtype=torch.bfloat16, tp: Optional[TPGroup] = None,
                 quant: Optional[str] = None):
        if quant is not None:
            raise ValueError("Padadra: quantised weights are not supported")
        self.tp = tp or TPGroup()
        if self.tp.size != 1:
            raise ValueError("Padadra: tensor parallelism is not supported")
        self.cfg, self.ops, self.device, self.dtype, self.quant = cfg, ops, torch.device(device), dtype, None
        self.layers: List[Dict[str, torch.Tensor]] = []
        self.embed = self.bigram = self.lm_head = None
        self.final_gain = 1.0
        self._side_stream = None
        attn = [l.attn for l in cfg.layers if l.attn is not None]
        self.n_q = max([a.heads for a in attn] + [l.state.heads for l in cfg.layers])
        self.n_kv = max([a.kv_heads for a in attn] or [1])
        self.hd = max([max(a.dim, a.vdim) for a in attn] + [max(l.state.dim, l.state.vdim) for l in cfg.layers])
        self.inter = max([l.mlp.ff for l in cfg.layers if l.mlp] or [0])
        self.vocab_local = cfg.vocab_size
        rows_fn = getattr(ops, "multimap_tile_rows", None)
        self.prefill_tile_rows = min([rows_fn(a.dim, a.vdim) for a in attn] or [64]) if rows_fn else 64

    # ------------------------------------------------------------- KV cache and state
    def kv_block_bytes(self, block_size: int, dtype) -> int:
        item = torch.tensor([], dtype=dtype).element_size()
        return sum((l.attn.k_width + l.attn.v_width) * block_size * item for l in self.cfg.layers if l.attn is not None)

    def alloc_kv(self, num_blocks: int, block_size: int, dtype, device=None):
        """Per layer K [NB, G, BS, dim] / V [NB, G, vdim, BS] for the attention layers, None for
        the others (block ids are shared by all layers: one block table per sequence)."""
        dev = device or self.device
        ks, vs = [], []
        for l in self.cfg.layers:
            a = l.attn
            ks.append(None if a is None else torch.zeros(num_blocks, a.kv_heads, block_size, a.dim, dtype=dtype, device=dev))
            vs.append(None if a is None else torch.zeros(num_blocks, a.kv_heads, a.vdim, block_size, dtype=dtype, device=dev))
        return ks, vs

    def _conv_channels(self, l) -> int:
        if l.attn is not None:
            return l.attn.q_width + l.attn.k_width + l.attn.v_width if l.attn.conv > 1 else 0
        s = l.state
        return 2 * s.kv_heads * s.dim + s.heads * s.vdim if s.conv > 1 else 0

    def alloc_state(self, rows: int, device=None) -> dict:
        """State tables with ``rows`` rows: ``prev`` int32 [rows] (previous token), per layer
        ``conv`` [rows, taps - 1, channels] (activation dtype; None without a convolution) and
        ``S`` fp32 [rows, heads, dim, vdim]."""
        dev = device or self.device
        layers = []
        for l in self.cfg.layers:
            s = l.state
            taps = l.attn.conv if l.attn is not None else s.conv
            ch = self._conv_channels(l)
            layers.append({"conv": torch.zeros(rows, taps - 1, ch, dtype=self.dtype, device=dev) if ch else None,
                           "S": torch.zeros(rows, s.heads, s.dim, s.vdim, dtype=torch.float32, device=dev)})
        return {"prev": torch.zeros(rows, dtype=torch.int32, device=dev), "layers": layers}

    @staticmethod
    def state_tensors(state: dict) -> List[torch.Tensor]:
        """Every table of `alloc_state` (row-indexed in dimension 0): what the engine moves when
        it moves a row."""
        out = [state["prev"]]
        for L in state["layers"]:
            out.extend(t for t in (L["conv"], L["S"]) if t is not None)
        return out

    def state_row_bytes(self) -> int:
        item = torch.tensor([], dtype=self.dtype).element_size()
        n = 4
        for l in self.cfg.layers:
            s = l.state
            taps = l.attn.conv if l.attn is not None else s.conv
            n += max(0, taps - 1) * self._conv_channels(l) * item + 4 * s.heads * s.dim * s.vdim
        return n

    # ------------------------------------------------------------- weights
    def tensor_shapes(self) -> Dict[str, tuple]:
        """Checkpoint tensor names -> shapes."""
        c, W = self.cfg, self.cfg.hidden_size
        out = {"embed": (c.vocab_size, W), "final.norm": (), "head": (c.vocab_size, W)}
        if c.bigram:
            out["bigram"] = (c.bigram[0] + 1, W)
        for i, l in enumerate(c.layers):
            p, s = f"l{i}.", l.state
            out[p + "norm1"] = ()
            if l.mlp is not None:
                out.update({p + "norm2": (), p + "mlp.up": (l.mlp.ff, W), p + "mlp.down": (W, l.mlp.ff)})
            if l.attn is not None:
                a, q = l.attn, p + "mix.left."
                for n, width in (("q", a.q_width), ("k", a.k_width), ("v", a.v_width)):
                    out.update({q + n: (width, W), q + n + ".b": (width,)})
                    if a.conv:
                        out[q + n + ".conv"] = (width, a.conv)
                out.update({q + "q.norm": (a.q_width,), q + "k.norm": (a.k_width,), q + "sink": (a.heads,),
                            q + "o": (W, a.heads * a.vdim), p + "mix.left.out": (W,), p + "mix.right.out": (W,)})
                r = p + "mix.right."
                out.update({r + "q": (s.heads * s.dim, W), r + "f": (s.heads * s.dim, W), r + "f.b": (s.heads * s.dim,),
                            r + "lower": (s.heads * s.dim,), r + "v": (s.heads * s.vdim, W), r + "norm": (s.vdim,),
                            r + "o": (W, s.heads * s.vdim)})
            else:
                q = p + "mix."
                ra, rg = s.decay_rank or max(4, W // 16), s.gate_rank or max(4, W // 16)
                for n, width in (("q", s.kv_heads * s.dim), ("k", s.kv_heads * s.dim), ("v", s.heads * s.vdim)):
                    out[q + n] = (width, W)
                    if s.conv:
                        out[q + n + ".conv"] = (width, s.conv)
                out.update({q + "b": (s.heads, W), q + "A_log": (s.heads,), q + "norm": (s.vdim,), q + "a1": (ra, W),
                            q + "a2": (s.heads * s.dim, ra), q + "dt_bias": (s.heads * s.dim,), q + "g1": (rg, W),
                            q + "g2": (s.heads * s.vdim, rg), q + "o": (W, s.heads * s.vdim)})
        return out

    def random_state_dict(self, seed: int = 0, std: float = 0.05) -> Dict[str, torch.Tensor]:
        """bf16-representable random weights under the checkpoint names (tests, benchmarks)."""
        gen = torch.Generator().manual_seed(seed)
        sd = {}
        for name, shape in self.tensor_shapes().items():
            r = torch.randn(shape, generator=gen)
            if name.endswith(("norm1", "norm2")) or name == "final.norm" or name.endswith((".norm", ".out")):
                t = 1.0 + 0.2 * r
            elif name.endswith(".conv"):
                t = r * 0.4
            elif name.endswith(".lower"):
                t = torch.sigmoid(r)              # a bound inside (0, 1)
            elif name.endswith(("sink", ".b", "dt_bias")):
                t = r * 0.5
            elif name.endswith("A_log"):
                t = r * 0.5 - 1.0
            elif name in ("embed", "bigram"):
                t = r * 0.7
            elif name.endswith(("a2", "g2")):
                t = r * (1.0 / math.sqrt(shape[1]))
            else:
                t = r * (std if name != "head" else 1.0 / math.sqrt(shape[1]))
            sd[name] = t.to(torch.bfloat16)
        return sd

    def init_random(self, seed: int = 0, std: float = 0.05):
        self.load_hf_state_dict(self.random_state_dict(seed, std))

    def load_hf_state_dict(self, sd):
        """Load the checkpoint tensors (names of `tensor_shapes`).  Projections that read the same
        input are stacked into one GEMM weight (sizes the config does not give, the low ranks,
        come from the tensors); convolution weights of q / k / v are stacked likewise."""
        c, dev, dt = self.cfg, self.device, self.dtype
        from ..ops.reference import rope_inv_freq, scaled_inv_freq

        def get(name, dtype=None):
            return sd[name].to(device=dev, dtype=dtype or dt).contiguous()

        def f32(name):
            return get(name, torch.float32)

        def zeros(n):
            return torch.zeros(n, dtype=dt, device=dev)

        self.layers = []
        for i, l in enumerate(c.layers):
            p, s = f"l{i}.", l.state
            L = {"gain1": float(sd[p + "norm1"].float()), "gain2": float(sd[p + "norm2"].float()) if l.mlp is not None else None}
            if l.mlp is not None:
                L["up"], L["down"] = get(p + "mlp.up"), get(p + "mlp.down")
            if l.attn is not None:
                a, q, r = l.attn, p + "mix.left.", p + "mix.right."
                names = (q + "q", q + "k", q + "v")
                L["fused"] = torch.cat([get(n) for n in names] + [get(r + "q"), get(r + "f"), get(r + "v")]).contiguous()
                n_right = 2 * s.heads * s.dim + s.heads * s.vdim
                L["bias"] = torch.cat([get(n + ".b") for n in names] + [zeros(n_right)]).contiguous()
                if a.conv:
                    L["conv_w"] = torch.cat([f32(n + ".conv") for n in names]).contiguous()
                L["q_norm"], L["k_norm"], L["sink"] = f32(q + "q.norm"), f32(q + "k.norm"), f32(q + "sink")
                L["inv_freq"] = scaled_inv_freq(a.rot_dims, a.rot_base, a.rot_scaling, dev)
                L["v_inv_freq"] = rope_inv_freq(a.vdim, a.rot_base, dev)
                L["o_left"], L["o_right"] = get(q + "o"), get(r + "o")
                L["out_left"], L["out_right"] = f32(p + "mix.left.out"), f32(p + "mix.right.out")
                L["f_bias"], L["lower"], L["head_norm"] = f32(r + "f.b"), f32(r + "lower"), f32(r + "norm")
            else:
                q = p + "mix."
                names = (q + "q", q + "k", q + "v")
                L["fused"] = torch.cat([get(n) for n in names] + [get(q + "b"), get(q + "a1"), get(q + "g1")]).contiguous()
                L["bias"] = None
                if s.conv:
                    L["conv_w"] = torch.cat([f32(n + ".conv") for n in names]).contiguous()
                L["rank_a"], L["rank_g"] = sd[q + "a1"].shape[0], sd[q + "g1"].shape[0]
                L["a2"], L["g2"], L["o"] = get(q + "a2"), get(q + "g2"), get(q + "o")
                L["a_log"], L["dt_bias"], L["head_norm"] = f32(q + "A_log"), f32(q + "dt_bias"), f32(q + "norm")
            self.layers.append(L)
        self.embed = get("embed")
        self.bigram = get("bigram") if c.bigram else None
        self.lm_head = get("head")
        self.final_gain = float(sd["final.norm"].float())

    def weight_bytes(self) -> int:
        n = sum(t.numel() * t.element_size() for L in self.layers for t in L.values() if torch.is_tensor(t))
        n += self.bigram.numel() * self.bigram.element_size() if self.bigram is not None else 0
        return n + self.embed.numel() * self.embed.element_size() + self.lm_head.numel() * self.lm_head.element_size()

    # ------------------------------------------------------------- forward
    def _gains(self, i: int):
        """Scalar norm gains that follow layer i - 1: layer i's norm1 (and norm2), or the final norm."""
        if i == len(self.layers):
            return (self.final_gain,)
        L = self.layers[i]
        return (L["gain1"],) if L["gain2"] is None else (L["gain1"], L["gain2"])

    def _fork(self, enabled: bool, fn):
        """Queue ``fn()`` behind everything queued so far: on the side stream when ``enabled`` (the
        caller goes on with independent work and calls the returned ``join`` before it reads the
        result), else at once.  Returns ``join``: ``join()`` gives ``fn``'s result."""
        if not enabled:
            out = fn()
            return lambda: out
        main = torch.cuda.current_stream()
        if self._side_stream is None:
            self._side_stream = torch.cuda.Stream(self.device)
        side = self._side_stream
        side.wait_stream(main)
        with torch.cuda.stream(side):
            out = fn()

        def join():
            main.wait_stream(side)
            out.record_stream(main)   # allocated on the side stream, read on this one
            return out
        return join

    def forward(self, tokens: torch.Tensor, meta: AttnMeta, k_cache, v_cache, trace: Optional[list] = None):
        """Logits (fp32) of the rows ``meta.logits_idx`` (all rows when None).  ``meta.state`` holds
        the tables of `alloc_state`, ``meta.state_rows`` every segment's row in them.  ``trace``: a
        list that receives a copy of the residual stream after every layer (debugging)."""
        ops, c = self.ops, self.cfg
        eps, dt, mult = c.rms_eps, self.dtype, c.residual_mult
        st = meta.state
        if st is None or meta.state_rows is None or meta.q_start is None or meta.token_seq is None:
            raise ValueError("Padadra: the step carries no sequence state (state, state_rows, q_start, token_seq)")
        x, hs = ops.embed_hashed_bigram_norm(tokens, meta, st["prev"], self.embed, c.embed_scale, self.bigram,
                                             c.bigram[1:] if c.bigram else None, eps, self._gains(0), dt)
        n_layers = len(c.layers)
        pos = meta.positions
        overlap = (self.overlap_min_rows is not None and not meta.decode and tokens.numel() >= self.overlap_min_rows
                   and self.device.type == "cuda" and not torch.cuda.is_current_stream_capturing())
        for i, (spec, L) in enumerate(zip(c.layers, self.layers)):
            s, S = spec.state, st["layers"][i]
            last = i == n_layers - 1
            sel = meta.logits_idx if last else None
            y = ops.linear(hs[0], L["fused"], L["bias"])
            normed, plain = [], []

            def feed_forward():
                """The layer's feed-forward (of the rows still needed); independent of the mixer."""
                nonlocal x, hs
                if sel is not None:
                    x = x.index_select(0, sel)
                    hs = tuple(h.index_select(0, sel) for h in hs)
                if spec.mlp is not None:
                    plain.append(ops.linear(ops.act_fn(ops.linear(hs[1], L["up"]), "relu2"), L["down"]))

            if spec.attn is not None:
                a = spec.attn
                cw = a.q_width + a.k_width + a.v_width
                n = s.heads * s.dim

                def recurrent_branch():
                    q32, k32, g32 = ops.hgrn2_prepare(y, cw, cw + n, s.heads, s.dim, L["f_bias"], L["lower"])
                    o32 = ops.gated_state_scan(q32, k32, g32, y[:, cw + 2 * n:cw + 2 * n + s.heads * s.vdim], None, meta,
                                               S["S"], False)
                    if sel is not None:
                        o32 = o32.index_select(0, sel)
                    return ops.head_norm_gate(o32, L["head_norm"], eps, None, dt)

                join = self._fork(overlap, recurrent_branch)
                u = ops.short_conv(y, cw, L["conv_w"], meta, S["conv"]) if a.conv else y
                q = ops.rope_pairs_kv_write(u, pos, meta.slots, a.heads, a.kv_heads, a.dim, a.vdim, L["q_norm"], L["k_norm"],
                                            eps, L["inv_freq"], L["v_inv_freq"], k_cache[i], v_cache[i])
                att = ops.multimap_attention(q, k_cache[i], v_cache[i], meta, a.scale, 1, 0.0, -1.0, 1.0, a.vdim,
                                             a.window, L["sink"])
                if sel is not None:
                    att, pos = att.index_select(0, sel), pos.index_select(0, sel)
                att = ops.rotate_pairs(att, pos, L["v_inv_freq"], -1.0, a.heads)
                normed = [(ops.linear(att, L["o_left"]), L["out_left"])]
                feed_forward()
                normed.append((ops.linear(join(), L["o_right"]), L["out_right"]))
            else:
                nqk = s.kv_heads * s.dim
                cw = 2 * nqk + s.heads * s.vdim
                u = ops.short_conv(y, cw, L["conv_w"], meta, S["conv"], "silu") if s.conv else ops.act_fn(y[:, :cw], "silu")
                off_a = cw + s.heads
                off_g = off_a + L["rank_a"]
                decay = ops.linear(y[:, off_a:off_g].contiguous(), L["a2"])
                q32, k32, g32, beta = ops.delta_prepare(u, y, cw, decay, L["a_log"], L["dt_bias"], s.heads, s.kv_heads, s.dim)

                def recurrent_branch():
                    o32 = ops.gated_state_scan(q32, k32, g32, u[:, 2 * nqk:], beta, meta, S["S"], True)
                    return o32 if sel is None else o32.index_select(0, sel)

                join = self._fork(overlap, recurrent_branch)
                gate_in = y[:, off_g:off_g + L["rank_g"]]
                if sel is not None:
                    gate_in = gate_in.index_select(0, sel)
                gate = ops.linear(gate_in.contiguous(), L["g2"])
                feed_forward()
                plain.insert(0, ops.linear(ops.head_norm_gate(join(), L["head_norm"], eps, gate, dt), L["o"]))
            hs = ops.residual_mix_norm(x, normed, 0.5, plain, mult, eps, self._gains(i + 1), dt)
            if trace is not None:
                trace.append(x.clone())
        return ops.linear(hs[0], self.lm_head).float()
