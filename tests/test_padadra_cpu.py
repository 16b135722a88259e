"""Padadra on the torch backend (CPU, fp32) against the float64 oracle (tests/padadra_oracle.py):
mechanisms one by one, then the engine's packed steps, paging, state-row reuse and generation."""
import numpy as np
import pytest
import torch

import padadra_cases as C
import padadra_oracle as O
from byzantine_consensus_llm_agents_amd.models.config import PadadraConfig, from_hf_config
from byzantine_consensus_llm_agents_amd.ops import reference as ref

TOL = dict(atol=2e-4, rtol=2e-4)


def _np(t):
    return t.detach().double().cpu().numpy()


def _close(got, want, tol=2e-3):
    np.testing.assert_allclose(_np(got), np.asarray(want), atol=tol, rtol=tol)


# ------------------------------------------------------------------ mechanisms
def test_scalar_gain_norms_and_residual_mix():
    g = torch.Generator().manual_seed(0)
    x, a, b, p = (torch.randn(7, 40, generator=g) for _ in range(4))
    wa, wb = torch.randn(40, generator=g), torch.randn(40, generator=g)
    want_x = _np(x) + 0.7 * (0.5 * (O.unit_rms(_np(a), 1e-5) * _np(wa) + O.unit_rms(_np(b), 1e-5) * _np(wb)) + _np(p))
    h1, h2 = ref.residual_mix_norm(x, [(a, wa), (b, wb)], 0.5, [p], 0.7, 1e-5, (1.3, -0.4), torch.float32)
    _close(x, want_x, 1e-5)
    _close(h1, O.unit_rms(want_x, 1e-5) * 1.3, 1e-5)
    _close(h2, O.unit_rms(want_x, 1e-5) * -0.4, 1e-5)


def test_bigram_rows_across_segments():
    """The first token of a sequence takes the last row; a portion's first token hashes with the
    state row's token; rows are independent."""
    cfg = {"embedding": {"scale": 1.5, "bigram": {"buckets": 11, "mul_prev": 7, "mul_cur": 3}}}
    g = torch.Generator().manual_seed(1)
    sd = {"embed": torch.randn(20, 6, generator=g), "bigram": torch.randn(12, 6, generator=g)}
    sdn = {k: _np(v) for k, v in sd.items()}
    a, b = C.tokens(9, 20, 1), C.tokens(5, 20, 2)
    prev = torch.full((4,), 19, dtype=torch.int32)   # stale tokens of earlier owners
    want_a, want_b = O.embed(sdn, cfg, a), O.embed(sdn, cfg, b)
    m = C.segments([(0, 4), (0, 5)], [2, 0])
    x = ref.embed_hashed_bigram(torch.tensor(a[:4] + b, dtype=torch.int32), m, prev, sd["embed"], 1.5, sd["bigram"], (7, 3))
    _close(x, np.concatenate([want_a[:4], want_b]), 1e-5)
    assert prev.tolist() == [b[-1], 19, a[3], 19]
    m = C.segments([(4, 1)], [2])
    _close(ref.embed_hashed_bigram(torch.tensor(a[4:5], dtype=torch.int32), m, prev, sd["embed"], 1.5, sd["bigram"], (7, 3)),
           want_a[4:5], 1e-5)
    m = C.segments([(5, 4)], [2])
    _close(ref.embed_hashed_bigram(torch.tensor(a[5:], dtype=torch.int32), m, prev, sd["embed"], 1.5, sd["bigram"], (7, 3)),
           want_a[5:], 1e-5)


@pytest.mark.parametrize("taps,cuts", [(4, [1, 1, 2, 5, 1, 3]), (2, [3, 1, 9]), (5, [2, 2, 2, 7]), (1, [6, 7]), (3, [13])])
def test_short_convolution_continues_from_its_state_row(taps, cuts):
    g = torch.Generator().manual_seed(taps)
    n, C_ = sum(cuts), 10
    u = torch.randn(n, C_ + 3, generator=g)
    w = torch.randn(C_, taps, generator=g)
    want = O.short_conv(_np(u[:, :C_]), _np(w))
    state = torch.randn(3, max(taps - 1, 0), C_, generator=g) if taps > 1 else None   # stale contents
    at = 0
    for c in cuts:
        # another sequence starts in the same step on another row
        m = C.segments([(at, c), (0, 2)], [1, 2])
        y = ref.short_conv(torch.cat([u[at:at + c], u[:2]]), C_, w, m, state)
        _close(y[:c], want[at:at + c], 1e-5)
        _close(y[c:], want[:2], 1e-5)
        at += c
    z = torch.randn(4, C_, generator=g)
    got = ref.short_conv(z, C_, w, C.segments([(0, 4)], [0]), state, "silu")
    _close(got, O.silu(O.short_conv(_np(z), _np(w))), 1e-5)


def test_frequency_scaling_bands():
    for dims, base, sc in ((32, 20000.0, (4.0, 1.0, 4.0, 1024)), (8, 5000.0, (3.0, 1.0, 3.0, 48)), (16, 100.0, (8.0, 2.0, 5.0, 60)), (12, 777.0, None)):
        want = O.scaled_freqs(dims, base, dict(zip(("factor", "low", "high", "original"), sc)) if sc else None)
        _close(ref.scaled_inv_freq(dims, base, sc), want, 1e-6)
    kept, mid, cut = (O.scaled_freqs(16, 100.0, {"factor": 8.0, "low": 2.0, "high": 5.0, "original": 60}) /
                      O.scaled_freqs(16, 100.0, None))[[0, 2, 7]]
    assert kept == 1.0 and 1 / 8 < mid < 1.0 and abs(cut - 1 / 8) < 1e-12   # all three bands occur


def _left_case(m, T, seed, craft=None, cuts=None):
    """The left mixer alone through the product ops over a paged cache with shuffled pages."""
    g = torch.Generator().manual_seed(seed)
    W, H, G, d, e = 32, m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    sd = {}
    for n, width in (("q", H * d), ("k", G * d), ("v", G * e)):
        sd[n] = torch.randn(width, W, generator=g) * 0.3
        sd[n + ".b"] = torch.randn(width, generator=g) * 0.2
        if m.get("conv"):
            sd[n + ".conv"] = torch.randn(width, m["conv"], generator=g) * 0.5
    sd.update({"q.norm": 1 + 0.3 * torch.randn(H * d, generator=g), "k.norm": 1 + 0.3 * torch.randn(G * d, generator=g),
               "sink": torch.randn(H, generator=g), "o": torch.randn(W, H * e, generator=g) * 0.3})
    h = torch.randn(T, W, generator=g)
    if craft is not None:
        craft(sd, h)
    want = O.left_mixer({k: _np(v) for k, v in sd.items()}, "", m, _np(h), 1e-5)
    BS = 16
    nblk = (T + BS - 1) // BS
    pages = torch.randperm(nblk + 2, generator=g)[:nblk] + 1
    k_cache, v_cache = torch.zeros(nblk + 4, G, BS, d), torch.zeros(nblk + 4, G, e, BS)
    rot = m["rot"]
    sc = rot.get("scaling")
    inv = ref.scaled_inv_freq(rot["dims"], rot["base"], tuple(sc[k] for k in ("factor", "low", "high", "original")) if sc else None)
    vinv = ref.rope_inv_freq(e, rot["base"])
    cw = (H + G) * d + G * e
    state = torch.randn(2, m["conv"] - 1, cw, generator=g) if m.get("conv", 0) > 1 else None
    outs, at = [], 0
    for c in cuts or [T]:
        meta = C.segments([(at, c)], [1])
        pos = meta.positions
        meta.slots = (pages[pos.long() // BS] * BS + pos % BS).to(torch.int32)
        meta.block_tables, meta.seq_lens = pages[None].to(torch.int32), torch.tensor([at + c], dtype=torch.int32)
        y = h[at:at + c] @ torch.cat([sd["q"], sd["k"], sd["v"]]).T + torch.cat([sd["q.b"], sd["k.b"], sd["v.b"]])
        if m.get("conv"):
            y = ref.short_conv(y, cw, torch.cat([sd["q.conv"], sd["k.conv"], sd["v.conv"]]), meta, state)
        q = ref.rope_pairs_kv_write(y, pos, meta.slots, H, G, d, e, sd["q.norm"], sd["k.norm"], 1e-5, inv, vinv, k_cache, v_cache)
        a = ref.multimap_attention(q, k_cache, v_cache, meta.block_tables, meta.q_start, meta.seq_lens, m["scale"], 1, 0.0,
                                   -1.0, 1.0, e, m.get("mask", {}).get("size", 0), sd["sink"])
        outs.append(ref.rotate_pairs(a, pos, vinv, -1.0, H) @ sd["o"].T)
        at += c
    return torch.cat(outs), want


@pytest.mark.parametrize("m", [C.left(), C.left(2, 1, 24, 16, 2, 7, 24, 900.0, None), C.left(3, 3, 10, 12, 0, 0, 0, 10000.0, None),
                               C.left(2, 2, 16, 8, 4, 16, 16)], ids=["gqa", "full-rot", "bare", "page-window"])
def test_left_mixer_whole_and_in_portions(m):
    got, want = _left_case(m, 45, 3)
    _close(got, want)
    got, want = _left_case(m, 45, 3, cuts=[2, 14, 1, 1, 17, 2, 8])
    _close(got, want)


def test_window_edge_shows_with_one_loud_key():
    """One key is made to dominate every later query: the outputs just inside and just outside the
    window differ by far more than the tolerance, in a prompt and token by token."""
    m = C.left(2, 1, 16, 16, 0, 9, 0, 10000.0, None)
    loud = 5

    def craft(sd, h):
        sd["q.b"].zero_(); sd["k.b"].zero_()
        h[loud] *= 6.0
        sd["k"].copy_(sd["q"][:16])          # keys line up with head 0's queries

    got, want = _left_case(m, 30, 5, craft)
    _close(got, want)
    got, want = _left_case(m, 30, 5, craft, cuts=[10] + [1] * 20)
    _close(got, want)
    inside, outside = want[loud + 8], want[loud + 9]
    assert np.abs(inside - outside).max() > 0.05


def test_sink_takes_weight_without_a_value():
    m = C.left(2, 2, 8, 8, 0, 0, 0, 10000.0, None)
    a, want_a = _left_case(m, 12, 7)
    _close(a, want_a)

    def craft(sd, h):
        sd["sink"].fill_(9.0)               # almost all the weight: outputs shrink towards zero

    b, want_b = _left_case(m, 12, 7, craft)
    _close(b, want_b)
    assert np.abs(want_b).max() < 0.2 * np.abs(want_a).max()


@pytest.mark.parametrize("H,d,e", [(2, 12, 20), (1, 16, 16), (3, 8, 5)])
def test_hgrn2_recurrence_in_portions(H, d, e):
    g = torch.Generator().manual_seed(H)
    W, T = 24, 33
    sd = {"q": torch.randn(H * d, W, generator=g) * 0.3, "f": torch.randn(H * d, W, generator=g) * 0.3,
          "f.b": torch.randn(H * d, generator=g), "lower": torch.rand(H * d, generator=g),
          "v": torch.randn(H * e, W, generator=g) * 0.3, "norm": 1 + 0.2 * torch.randn(e, generator=g),
          "o": torch.randn(W, H * e, generator=g) * 0.3}
    h = torch.randn(T, W, generator=g)
    want = O.hgrn2_mixer({k: _np(v) for k, v in sd.items()}, "", {"heads": H, "dim": d, "vdim": e}, _np(h), 1e-5)
    state = torch.randn(3, H, d, e, generator=g)   # stale
    outs, at = [], 0
    for c in (4, 1, 1, 2, 20, 5):
        meta = C.segments([(at, c)], [2])
        y = h[at:at + c] @ torch.cat([sd["q"], sd["f"], sd["v"]]).T
        q32, k32, g32 = ref.hgrn2_prepare(y, 0, H * d, H, d, sd["f.b"], sd["lower"])
        o = ref.gated_state_scan(q32, k32, g32, y[:, 2 * H * d:], None, meta, state, False)
        outs.append(ref.head_norm_gate(o, sd["norm"], 1e-5, None, torch.float32) @ sd["o"].T)
        at += c
    _close(torch.cat(outs), want)


@pytest.mark.parametrize("H,G,d,e,taps", [(4, 2, 16, 12, 4), (3, 3, 20, 18, 2), (2, 1, 8, 8, 0)])
def test_gated_delta_rule_in_portions(H, G, d, e, taps):
    g = torch.Generator().manual_seed(H + taps)
    W, T, ra, rg = 24, 33, 5, 4
    sd = {"q": torch.randn(G * d, W, generator=g) * 0.4, "k": torch.randn(G * d, W, generator=g) * 0.4,
          "v": torch.randn(H * e, W, generator=g) * 0.4, "b": torch.randn(H, W, generator=g) * 0.3,
          "A_log": torch.randn(H, generator=g) * 0.5 - 1, "norm": 1 + 0.2 * torch.randn(e, generator=g),
          "a1": torch.randn(ra, W, generator=g) * 0.3, "a2": torch.randn(H * d, ra, generator=g) * 0.5,
          "dt_bias": torch.randn(H * d, generator=g), "g1": torch.randn(rg, W, generator=g) * 0.3,
          "g2": torch.randn(H * e, rg, generator=g) * 0.5, "o": torch.randn(W, H * e, generator=g) * 0.3}
    if taps:
        for n, width in (("q", G * d), ("k", G * d), ("v", H * e)):
            sd[n + ".conv"] = torch.randn(width, taps, generator=g) * 0.5
    h = torch.randn(T, W, generator=g)
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": e, "conv": taps}
    want = O.channel_delta_mixer({k: _np(v) for k, v in sd.items()}, "", m, _np(h), 1e-5)
    cw = 2 * G * d + H * e
    state = torch.randn(2, H, d, e, generator=g)
    conv_state = torch.randn(2, taps - 1, cw, generator=g) if taps > 1 else None
    fused = torch.cat([sd["q"], sd["k"], sd["v"], sd["b"], sd["a1"], sd["g1"]])
    outs, at = [], 0
    for c in (2, 1, 1, 9, 2, 18):
        meta = C.segments([(at, c)], [1])
        y = h[at:at + c] @ fused.T
        if taps:
            u = ref.short_conv(y, cw, torch.cat([sd["q.conv"], sd["k.conv"], sd["v.conv"]]), meta, conv_state, "silu")
        else:
            u = ref.act_fn(y[:, :cw], "silu")
        a = y[:, cw + H:cw + H + ra] @ sd["a2"].T
        q32, k32, g32, beta = ref.delta_prepare(u, y, cw, a, sd["A_log"], sd["dt_bias"], H, G, d)
        o = ref.gated_state_scan(q32, k32, g32, u[:, 2 * G * d:], beta, meta, state, True)
        gate = y[:, cw + H + ra:] @ sd["g2"].T
        outs.append(ref.head_norm_gate(o, sd["norm"], 1e-5, gate, torch.float32) @ sd["o"].T)
        at += c
    _close(torch.cat(outs), want)


def test_config_round_trip(tmp_path):
    for name, cfg in C.CASES.items():
        path = str(tmp_path / name)
        C.checkpoint(cfg, path)
        read = from_hf_config(path)
        assert isinstance(read, PadadraConfig) and read.family == "padadra"
        assert PadadraConfig.from_dict(read.to_dict(), "x").layers == read.layers
        assert read.to_dict()["embedding"] == cfg["embedding"] and read.residual_mult == cfg["residual_mult"]


# ------------------------------------------------------------------ the engine
@pytest.fixture(scope="module", params=list(C.CASES))
def case(request, tmp_path_factory):
    path = str(tmp_path_factory.mktemp(request.param))
    cfg = C.CASES[request.param]
    sd = O.to_f64(C.checkpoint(cfg, path, seed=len(request.param)))
    eng = C.engine(path)
    yield cfg, sd, eng
    eng.shutdown()


def test_whole_prompt_every_position(case):
    cfg, sd, eng = case
    toks = C.tokens(45, cfg["vocab"], 1)
    got = eng.stream_step([("a", toks, list(range(45)))], end=["a"])
    _close(got, O.forward(sd, cfg, toks))


def test_residual_stream_after_every_layer(case):
    cfg, sd, eng = case
    toks = C.tokens(19, cfg["vocab"], 2)
    want = []
    O.forward(sd, cfg, toks, want)
    from byzantine_consensus_llm_agents_amd.models.batch import prefill_batch
    tokens, meta, nblk = prefill_batch([toks])
    meta.logits_idx = None
    meta.state, meta.state_rows = eng.model.alloc_state(2), torch.tensor([1], dtype=torch.int32)
    meta.token_seq = torch.zeros(19, dtype=torch.int32)
    k, v = eng.model.alloc_kv(nblk + 1, 16, torch.float32)
    got = []
    eng.model.forward(tokens, meta, k, v, trace=got)
    assert len(got) == len(want) == len(cfg["layers"])
    for a, b in zip(got, want):
        _close(a, b)


def test_prefill_then_token_by_token(case):
    cfg, sd, eng = case
    toks = C.tokens(70, cfg["vocab"], 3)
    want = O.forward(sd, cfg, toks)
    _close(eng.stream_step([("d", toks[:30], [0, 1, 29])]), want[[0, 1, 29]])
    for p in range(30, 70):   # crosses page borders at 32, 48, 64 and every window's edge
        _close(eng.stream_step([("d", toks[p:p + 1], [0])], end=["d"] if p == 69 else []), want[p:p + 1])


def test_first_tokens_one_by_one(case):
    cfg, sd, eng = case
    toks = C.tokens(7, cfg["vocab"], 4)
    want = O.forward(sd, cfg, toks)
    for p in range(7):
        _close(eng.stream_step([("f", toks[p:p + 1], [0])], end=["f"] if p == 6 else []), want[p:p + 1])


@pytest.mark.parametrize("sizes", [[2, 2, 3, 17, 16, 1, 31, 2, 5], [15, 1, 1, 16, 33, 11]])
def test_portions_of_changing_size(case, sizes):
    cfg, sd, eng = case
    n = sum(sizes)
    toks = C.tokens(n, cfg["vocab"], 5)
    want = O.forward(sd, cfg, toks)
    at = 0
    for i, s in enumerate(sizes):
        got = eng.stream_step([("p", toks[at:at + s], list(range(s)))], end=["p"] if i == len(sizes) - 1 else [])
        _close(got, want[at:at + s])
        at += s


def test_mixed_batches_equal_each_alone_and_reuse_pages_and_rows(case):
    """Four live requests of unequal progress per step (prompt portions beside single tokens);
    the pool holds far fewer tokens than all requests together and there are twice as many
    requests as state rows, so pages and rows come back with their old contents."""
    cfg, sd, eng = case
    lens = [50, 33, 18, 64, 41, 27, 5, 36]
    reqs = {f"r{i}": C.tokens(n, cfg["vocab"], 10 + i) for i, n in enumerate(lens)}
    want = {k: O.forward(sd, cfg, t) for k, t in reqs.items()}
    at = {k: 0 for k in reqs}
    waiting, live, step = list(reqs), [], 0
    free_at_start = eng.blocks.num_free_blocks
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
        entries, end, expect = [], [], []
        for j, k in enumerate(live):
            if (step + j) % 3 == 2 and at[k] > 0:
                continue  # a request may sit a step out
            take = [1, 2, 16, 7, 1, 19][(step + j) % 6] if at[k] > 0 else [20, 3, 16][j % 3]
            take = min(take, len(reqs[k]) - at[k])
            entries.append((k, reqs[k][at[k]:at[k] + take], list(range(take))))
            expect.append(want[k][at[k]:at[k] + take])
            at[k] += take
            if at[k] == len(reqs[k]):
                end.append(k)
        if entries:
            _close(eng.stream_step(entries, end), np.concatenate(expect))
        live = [k for k in live if k not in end]
        step += 1
    assert eng.blocks.num_free_blocks == free_at_start and not any(eng.slots)
    assert sum(lens) > 16 * free_at_start / 2


def test_long_decoding(case):
    cfg, sd, eng = case
    toks = C.tokens(150, cfg["vocab"], 6)
    want = O.forward(sd, cfg, toks)
    eng.stream_step([("l", toks[:4], [])])
    for p in range(4, 150):
        got = eng.stream_step([("l", toks[p:p + 1], [0])], end=["l"] if p == 149 else [])
        if p % 9 == 0 or p > 140:
            _close(got, want[p:p + 1])


def test_greedy_generation_through_the_scheduler(case):
    """`generate_ids`: admission, paged prefill, decode bursts and the sampler; more requests than
    state rows, so finished rows are compacted and reused while others still decode."""
    cfg, sd, eng = case
    prompts = [C.tokens(n, cfg["vocab"], 20 + n) for n in (9, 31, 16, 2, 40, 23)]
    budgets = (6, 4, 17, 5, 3, 11)
    outs = eng.generate_ids(prompts, max_tokens=list(budgets), temperature=0.0)
    for p, out, n in zip(prompts, outs, budgets):
        assert len(out) == n
        seq = list(p)
        for tok in out:
            logits = O.forward(sd, cfg, seq)[-1]
            top2 = np.sort(logits)[-2:]
            if float(top2[1] - top2[0]) < 1e-3:
                break  # a near tie: either token is a correct greedy step
            assert tok == int(logits.argmax())
            seq.append(tok)


def test_generate_command_line(tmp_path, capsys):
    from byzantine_consensus_llm_agents_amd.engine.generate import main
    cfg = C.CASES["mixed"]
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=6))
    prompts = [C.tokens(7, cfg["vocab"], 1), C.tokens(20, cfg["vocab"], 2)]
    argv = ["--weights", path, "--backend", "torch", "--dtype", "float32", "--max-tokens", "3", "--max-model-len", "64"]
    for p in prompts:
        argv += ["--prompt", " ".join(map(str, p))]
    assert main(argv) == 0
    lines = [l for l in capsys.readouterr().out.strip().splitlines() if l.strip()]
    assert len(lines) == 2
    for p, line in zip(prompts, lines):
        ids = [int(t) for t in line.split()]
        assert len(ids) == 3 and ids[0] == int(O.forward(sd, cfg, p)[-1].argmax())


@pytest.mark.parametrize("seed", range(8, 13))
def test_drawn_configurations(tmp_path, seed):
    """Configurations drawn from a seed (sizes, head counts, layer order, windows, taps, constants):
    a whole prompt against the same prompt in portions beside another request."""
    cfg = C.random_config(seed)
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=seed))
    eng = C.engine(path, pool_tokens=256)
    try:
        a, b = C.tokens(60, cfg["vocab"], seed), C.tokens(23, cfg["vocab"], seed + 100)
        wa, wb = O.forward(sd, cfg, a), O.forward(sd, cfg, b)
        _close(eng.stream_step([("w", a, list(range(60)))], end=["w"]), wa)
        at = 0
        for i, s in enumerate([3, 2, 30, 1, 1, 17, 2, 4]):
            entries, want = [("a", a[at:at + s], list(range(s)))], [wa[at:at + s]]
            at += s
            if i < 23:
                entries.append(("b", b[i:i + 1], [0]))
                want.append(wb[i:i + 1])
            _close(eng.stream_step(entries), np.concatenate(want))
        assert at == 60
        eng.stream_step([("b", b[8:], [])], end=["a", "b"])
        assert not any(eng.slots)
    finally:
        eng.shutdown()


def test_text_entry_point_with_id_prompts(tmp_path):
    from byzantine_consensus_llm_agents_amd.engine import LLM, SamplingParams
    cfg = C.CASES["plain"]
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=4))
    llm = LLM(path, backend="torch", weights=path, seed=1, max_model_len=128, kv_cache_gb=0.01, max_batch_seqs=4, dtype=torch.float32)
    try:
        prompt = C.tokens(12, cfg["vocab"], 8)
        out = llm.generate(" ".join(map(str, prompt)), SamplingParams(temperature=0.0, max_tokens=5))[0].outputs[0].text
        ids = [int(t) for t in out.split()]
        assert len(ids) == 5 and ids[0] == int(O.forward(sd, cfg, prompt)[-1].argmax())
    finally:
        llm.shutdown()
