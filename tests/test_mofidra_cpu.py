"""Mofidra on the torch backend (CPU, fp32) against the float64 oracle (tests/mofidra_oracle.py):
mechanisms one by one, then the engine's packed steps, paging, row reuse and generation."""
import math

import pytest
import torch

import mofidra_cases as C
import mofidra_oracle as O
from byzantine_consensus_llm_agents_amd.models.config import MofidraConfig, from_hf_config
from byzantine_consensus_llm_agents_amd.ops import reference as ref

TOL = dict(atol=2e-4, rtol=2e-4)


def _f64(sd):
    return {k: v.to(torch.float64) for k, v in sd.items()}


# ------------------------------------------------------------------ mechanisms
def test_norm_weight_is_an_offset_from_one():
    x = torch.randn(5, 40, dtype=torch.float64)
    w = torch.randn(40) * 0.2
    got = ref.rmsnorm32(x.float(), w, 1e-5, 1.0, torch.float32)
    torch.testing.assert_close(got.double(), O.layer_norm(x, w, 1e-5), **TOL)
    # a zero weight leaves the unit-RMS rows
    torch.testing.assert_close(ref.rmsnorm32(x.float(), torch.zeros(40), 1e-5, 1.0, torch.float32).double(),
                               O.unit_rms(x, 1e-5), **TOL)


def test_activations():
    z = torch.linspace(-6, 6, 101, dtype=torch.float64)
    torch.testing.assert_close(ref.act_fn(z.float(), "gelu_tanh").double(), O.gelu_tanh(z), **TOL)
    torch.testing.assert_close(ref.act_fn(z.float(), "relu2").double(), O.relu_squared(z), **TOL)


@pytest.mark.parametrize("dims,dim", [(8, 16), (16, 16), (0, 12), (6, 20)])
def test_partial_rotary_and_cache_write(dims, dim):
    T, n_q, n_kv, maps, vdim, BS = 21, 3, 1, 2, 10, 16
    x = torch.randn(T, (n_q + n_kv) * maps * dim + n_kv * vdim + 5)
    pos = torch.arange(100, 100 + T, dtype=torch.int32)
    slots = (torch.randperm(4 * BS)[:T] + BS).to(torch.int32)
    k_cache, v_cache = torch.zeros(6, n_kv, BS, maps * dim), torch.zeros(6, n_kv, vdim, BS)
    q = ref.rope_multi_kv_write(x, pos, slots, n_q, n_kv, maps, dim, vdim, ref.rope_inv_freq(dims, 777.0), k_cache, v_cache)
    qw = n_q * maps * dim
    want_q = torch.stack([O.rotate(x[:, :qw].double().view(T, n_q, maps, dim)[:, :, j], pos, dims, 777.0) for j in range(maps)], 2)
    torch.testing.assert_close(q.double().view(T, n_q, maps, dim), want_q, **TOL)
    want_k = torch.stack([O.rotate(x[:, qw:qw + n_kv * maps * dim].double().view(T, n_kv, maps, dim)[:, :, j], pos, dims, 777.0)
                          for j in range(maps)], 2).reshape(T, n_kv, maps * dim)
    blk, off = (slots // BS).long(), (slots % BS).long()
    torch.testing.assert_close(k_cache[blk, :, off].double(), want_k, **TOL)
    torch.testing.assert_close(v_cache[blk, :, :, off], x[:, qw + n_kv * maps * dim:-5].view(T, n_kv, vdim))


def _attention_case(m, T, seed, craft=None):
    """The mixer alone: product ops over a paged cache with shuffled pages against the oracle."""
    g = torch.Generator().manual_seed(seed)
    W = 32
    sd = {"q": torch.randn(m["heads"] * 2 * m["dim"], W, generator=g) * 0.3, "k": torch.randn(m["kv_heads"] * 2 * m["dim"], W, generator=g) * 0.3,
          "v": torch.randn(m["kv_heads"] * m["vdim"], W, generator=g) * 0.3, "o": torch.randn(W, m["heads"] * m["vdim"], generator=g) * 0.3}
    sd.update({n: torch.randn(m["dim"], generator=g) * 0.3 for n in ("lq1", "lk1", "lq2", "lk2")})
    h = torch.randn(T, W, generator=g)
    if craft is not None:
        craft(h)
    want = O.differential_attention(h.double(), _f64(sd), "", m, 1e-5)
    BS = 16
    nblk = (T + BS - 1) // BS
    pages = torch.randperm(nblk + 2, generator=g)[:nblk] + 1
    k_cache = torch.zeros(nblk + 4, m["kv_heads"], BS, 2 * m["dim"])
    v_cache = torch.zeros(nblk + 4, m["kv_heads"], m["vdim"], BS)
    pos = torch.arange(T, dtype=torch.int32)
    slots = (pages[pos.long() // BS] * BS + pos % BS).to(torch.int32)
    y = h @ torch.cat([sd["q"], sd["k"], sd["v"]]).T
    q = ref.rope_multi_kv_write(y, pos, slots, m["heads"], m["kv_heads"], 2, m["dim"], m["vdim"],
                                ref.rope_inv_freq(m["rot"]["dims"], m["rot"]["base"]), k_cache, v_cache)
    lam = O.differential_lambda(_f64(sd), "", m["diff"])
    a = ref.multimap_attention(q, k_cache, v_cache, pages[None].to(torch.int32), torch.tensor([0, T]), torch.tensor([T]),
                               m["scale"], 2, lam, 1e-5, 1.0 - m["diff"], m["vdim"])
    return (a @ sd["o"].T).double(), want


@pytest.mark.parametrize("m", [C.mixer(), C.mixer(4, 4, 16, 16, 16), C.mixer(2, 1, 24, 40, 12, diff=0.8), C.mixer(3, 3, 20, 18, 0)])
def test_differential_attention_alone(m):
    got, want = _attention_case(m, 50, seed=m["dim"])
    torch.testing.assert_close(got, want, atol=1e-3, rtol=1e-3)


def test_differential_attention_far_key():
    """Token 2's input is made to dominate the last query's scores from 300 tokens away."""
    def craft(h):
        h[2] = 4.0 * h[-1]
    got, want = _attention_case(C.mixer(2, 1, 16, 24, 0, scale=0.5), 303, seed=9, craft=craft)
    torch.testing.assert_close(got, want, atol=1e-3, rtol=1e-3)


@pytest.mark.parametrize("f", [C.moe(), C.moe(3, 1, 16, 0), C.moe(5, 5, 12, 8), C.dense(40)])
def test_feed_forward_alone(f):
    g = torch.Generator().manual_seed(3)
    W, T = 32, 40
    names = {}
    if f["kind"] == "dense":
        names = {"up": (f["ff"], W), "down": (W, f["ff"])}
    else:
        for e in range(f["router"]["experts"]):
            names.update({f"e{e}.up": (f["expert"]["ff"], W), f"e{e}.down": (W, f["expert"]["ff"])})
        names.update({"router": (f["router"]["experts"], W), "router.b": (f["router"]["experts"],)})
        if f.get("shared"):
            names.update({"shared.up": (f["shared"]["ff"], W), "shared.down": (W, f["shared"]["ff"]), "shared.sg": (1, W)})
    sd = {k: torch.randn(s, generator=g) * 0.3 for k, s in names.items()}
    h = torch.randn(T, W, generator=g)
    want = O.feed_forward(h.double(), _f64(sd), "", f)
    if f["kind"] == "dense":
        got = ref.act_fn(h @ sd["up"].T, "gelu_tanh") @ sd["down"].T
    else:
        E = f["router"]["experts"]
        idx, wts, gate = ref.moe_route(h, sd["router"], sd["router.b"], f["router"]["top"],
                                       sd["shared.sg"].reshape(-1) if f.get("shared") else None)
        got = ref.moe_experts(h, torch.stack([sd[f"e{e}.up"] for e in range(E)]), torch.stack([sd[f"e{e}.down"] for e in range(E)]),
                              idx, wts, "relu2")
        if f.get("shared"):
            got = got + torch.sigmoid(gate)[:, None] * (ref.act_fn(h @ sd["shared.up"].T, "relu2") @ sd["shared.down"].T)
    torch.testing.assert_close(got.double(), want, atol=1e-3, rtol=1e-3)


def test_config_reader_roundtrip(tmp_path):
    for name, cfg in C.CASES.items():
        C.checkpoint(cfg, str(tmp_path / name))
        read = from_hf_config(str(tmp_path / name))
        assert isinstance(read, MofidraConfig) and read.layer_runs == tuple(O.layer_order(cfg))
        assert MofidraConfig.from_dict(read.to_dict(), "x").layers == read.layers


# ------------------------------------------------------------------ the engine
@pytest.fixture(scope="module", params=list(C.CASES))
def case(request, tmp_path_factory):
    path = str(tmp_path_factory.mktemp(request.param))
    cfg = C.CASES[request.param]
    sd = _f64(C.checkpoint(cfg, path, seed=len(request.param)))
    eng = C.engine(path)
    yield cfg, sd, eng
    eng.shutdown()


def _oracle(cfg, sd, toks):
    assert O.router_margin(cfg, sd, toks) > 1e-6
    return O.forward(cfg, sd, toks)


def _close(got, want):
    torch.testing.assert_close(got.double().cpu(), want, atol=2e-3, rtol=2e-3)


def test_whole_prompt_every_position(case):
    cfg, sd, eng = case
    toks = C.tokens(45, cfg["vocab"], 1)
    got = eng.stream_step([("a", toks, list(range(45)))], end=["a"])
    _close(got, _oracle(cfg, sd, toks))


def test_residual_stream_after_every_layer_run(case):
    cfg, sd, eng = case
    toks = C.tokens(19, cfg["vocab"], 2)
    want = []
    O.forward(cfg, sd, toks, stream=want)
    from byzantine_consensus_llm_agents_amd.models.batch import prefill_batch
    tokens, meta, nblk = prefill_batch([toks])
    meta.logits_idx = None
    k, v = eng.model.alloc_kv(nblk + 1, 16, torch.float32)
    got = []
    eng.model.forward(tokens, meta, k, v, trace=got)
    assert len(got) == len(want) == len(O.layer_order(cfg))
    for a, b in zip(got, want):
        _close(a, b)


def test_prefill_then_token_by_token(case):
    cfg, sd, eng = case
    toks = C.tokens(70, cfg["vocab"], 3)
    want = _oracle(cfg, sd, toks)
    _close(eng.stream_step([("d", toks[:30], [0, 1, 29])]), want[[0, 1, 29]])
    for p in range(30, 70):   # crosses the page borders at 32, 48, 64
        _close(eng.stream_step([("d", toks[p:p + 1], [0])], end=["d"] if p == 69 else []), want[p:p + 1])


def test_first_tokens_one_by_one(case):
    cfg, sd, eng = case
    toks = C.tokens(6, cfg["vocab"], 4)
    want = _oracle(cfg, sd, toks)
    for p in range(6):
        _close(eng.stream_step([("f", toks[p:p + 1], [0])], end=["f"] if p == 5 else []), want[p:p + 1])


@pytest.mark.parametrize("sizes", [[2, 2, 3, 17, 16, 1, 31, 2, 5], [15, 1, 1, 16, 33, 11]])
def test_portions_of_changing_size(case, sizes):
    cfg, sd, eng = case
    n = sum(sizes)
    toks = C.tokens(n, cfg["vocab"], 5)
    want = _oracle(cfg, sd, toks)
    at = 0
    for i, s in enumerate(sizes):
        got = eng.stream_step([("p", toks[at:at + s], list(range(s)))], end=["p"] if i == len(sizes) - 1 else [])
        _close(got, want[at:at + s])
        at += s


def test_mixed_batches_equal_each_alone_and_reuse_pages(case):
    """Four live requests of unequal progress per step (prompt portions beside single tokens);
    the pool holds far fewer tokens than all requests together, so pages and rows come back."""
    cfg, sd, eng = case
    lens = [50, 33, 18, 64, 41, 27, 5, 36]
    reqs = {f"r{i}": C.tokens(n, cfg["vocab"], 10 + i) for i, n in enumerate(lens)}
    want = {k: _oracle(cfg, sd, t) for k, t in reqs.items()}
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
            _close(eng.stream_step(entries, end), torch.cat(expect))
        live = [k for k in live if k not in end]
        step += 1
    assert eng.blocks.num_free_blocks == free_at_start and not any(eng.slots)
    assert sum(lens) > 16 * free_at_start / 2  # the pool was worked through more than once over


def test_long_decoding(case):
    cfg, sd, eng = case
    toks = C.tokens(150, cfg["vocab"], 6)
    want = _oracle(cfg, sd, toks)
    eng.stream_step([("l", toks[:4], [])])
    for p in range(4, 150):
        got = eng.stream_step([("l", toks[p:p + 1], [0])], end=["l"] if p == 149 else [])
        if p % 9 == 0 or p > 140:
            _close(got, want[p:p + 1])


def test_pool_exhaustion_is_an_error_not_a_wrong_answer(case):
    cfg, sd, eng = case
    free = eng.blocks.num_free_blocks
    toks = C.tokens(100, cfg["vocab"], 7)
    eng.stream_step([("w", toks[:60], [])])
    with pytest.raises(RuntimeError):   # refused as a whole: "w" keeps its 60 tokens, "x" never opens
        eng.stream_step([("w", toks[60:70], [0]), ("x", C.tokens(16 * free - 50, cfg["vocab"], 7), [])])
    assert "x" not in eng._streams and len(eng._streams["w"].seq.prompt_ids) == 60
    _close(eng.stream_step([("w", toks[60:], [39])], end=["w"]), _oracle(cfg, sd, toks)[99:100])
    assert eng.blocks.num_free_blocks == free and not any(eng.slots)


def test_greedy_generation_through_the_scheduler(case):
    """`generate_ids`: admission, paged prefill, decode bursts and the sampler; more requests than rows."""
    cfg, sd, eng = case
    prompts = [C.tokens(n, cfg["vocab"], 20 + n) for n in (9, 31, 16, 2, 40, 23)]
    outs = eng.generate_ids(prompts, max_tokens=[6, 4, 7, 5, 3, 6], temperature=0.0)
    for p, out, n in zip(prompts, outs, (6, 4, 7, 5, 3, 6)):
        assert len(out) == n
        seq = list(p)
        for tok in out:
            logits = O.forward(cfg, sd, seq)[-1]
            top2 = torch.topk(logits, 2).values
            if float(top2[0] - top2[1]) < 1e-3:
                break  # a near tie: either token is a correct greedy step
            assert tok == int(logits.argmax())
            seq.append(tok)


def test_text_entry_point_with_id_prompts(tmp_path):
    from byzantine_consensus_llm_agents_amd.engine import LLM, SamplingParams
    cfg = C.CASES["plain"]
    path = str(tmp_path / "m")
    sd = _f64(C.checkpoint(cfg, path, seed=4))
    llm = LLM(path, backend="torch", weights=path, seed=1, max_model_len=128, kv_cache_gb=0.01, max_batch_seqs=4, dtype=torch.float32)
    try:
        prompt = C.tokens(12, cfg["vocab"], 8)
        out = llm.generate(" ".join(map(str, prompt)), SamplingParams(temperature=0.0, max_tokens=5))[0].outputs[0].text
        ids = [int(t) for t in out.split()]
        assert len(ids) == 5 and ids[0] == int(O.forward(cfg, sd, prompt)[-1].argmax())
    finally:
        llm.shutdown()


def test_generate_command_line(tmp_path, capsys):
    from byzantine_consensus_llm_agents_amd.engine.generate import main
    cfg = C.CASES["plain"]
    path = str(tmp_path / "m")
    sd = _f64(C.checkpoint(cfg, path, seed=6))
    prompts = [C.tokens(7, cfg["vocab"], 1), C.tokens(20, cfg["vocab"], 2)]
    argv = ["--weights", path, "--backend", "torch", "--dtype", "float32", "--max-tokens", "3", "--max-model-len", "64"]
    for p in prompts:
        argv += ["--prompt", " ".join(map(str, p))]
    assert main(argv) == 0
    lines = [l for l in capsys.readouterr().out.strip().splitlines() if l.strip()]
    assert len(lines) == 2
    for p, line in zip(prompts, lines):
        ids = [int(t) for t in line.split()]
        assert len(ids) == 3 and ids[0] == int(O.forward(cfg, sd, p)[-1].argmax())


def test_bench_option_leaves_the_default_workload():
    import bench
    assert bench.parse([]).family_compare is False and bench.parse(["--family-compare"]).family_compare is True
