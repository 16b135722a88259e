"""Padadra on the HIP backend against the float64 oracle: packed steps of the engine (prompt
portions beside single tokens, page and state-row reuse), fp32 (exact mode) and bf16, and greedy
generation through the scheduler with captured decode graphs."""
import numpy as np
import pytest
import torch

import padadra_cases as C
import padadra_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=[(n, d) for n in C.CASES for d in ("float32", "bfloat16")],
                ids=lambda p: f"{p[0]}-{p[1]}")
def case(request, tmp_path_factory):
    name, dtype = request.param
    path = str(tmp_path_factory.mktemp(name))
    cfg = C.CASES[name]
    sd = O.to_f64(C.checkpoint(cfg, path, seed=len(name)))
    eng = C.engine(path, backend="hip", dtype=getattr(torch, dtype))
    assert eng.ops.name == "hip"
    yield cfg, sd, eng, dtype
    eng.shutdown()


def _close(got, want, dtype):
    got = got.double().cpu().numpy()
    if dtype == "float32":
        np.testing.assert_allclose(got, want, atol=3e-3, rtol=3e-3)
    else:  # bf16 activations: error relative to the spread of the logits
        err = np.sqrt(((got - want) ** 2).mean(-1)) / want.std()
        assert float(err.max()) < 0.08, float(err.max())
        assert float(np.median(err)) < 0.03


def test_whole_prompt_every_position(case):
    cfg, sd, eng, dtype = case
    toks = C.tokens(150, cfg["vocab"], 1)
    got = eng.stream_step([("a", toks, list(range(150)))], end=["a"])
    _close(got, O.forward(sd, cfg, toks), dtype)


def test_portions_then_single_tokens(case):
    cfg, sd, eng, dtype = case
    toks = C.tokens(140, cfg["vocab"], 2)
    want = O.forward(sd, cfg, toks)
    at = 0
    for s in [2, 3, 64, 1, 17, 2, 1]:
        _close(eng.stream_step([("p", toks[at:at + s], list(range(s)))]), want[at:at + s], dtype)
        at += s
    got = [eng.stream_step([("p", toks[p:p + 1], [0])], end=["p"] if p == 139 else []) for p in range(at, 140)]
    _close(torch.cat(got), want[at:140], dtype)


def test_first_tokens_one_by_one(case):
    cfg, sd, eng, dtype = case
    toks = C.tokens(6, cfg["vocab"], 4)
    want = O.forward(sd, cfg, toks)
    for p in range(6):
        _close(eng.stream_step([("f", toks[p:p + 1], [0])], end=["f"] if p == 5 else []), want[p:p + 1], dtype)


def test_mixed_batches_and_reuse(case):
    cfg, sd, eng, dtype = case
    lens = [70, 33, 18, 64, 41, 90, 5, 36, 120]
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
            if (step + j) % 5 == 4 and at[k] > 0:
                continue
            take = [1, 2, 16, 7, 1, 19][(step + j) % 6] if at[k] > 0 else [20, 3, 16][j % 3]
            take = min(take, len(reqs[k]) - at[k])
            entries.append((k, reqs[k][at[k]:at[k] + take], list(range(take))))
            expect.append(want[k][at[k]:at[k] + take])
            at[k] += take
            if at[k] == len(reqs[k]):
                end.append(k)
        if entries:
            _close(eng.stream_step(entries, end), np.concatenate(expect), dtype)
        live = [k for k in live if k not in end]
        step += 1
    assert eng.blocks.num_free_blocks == free_at_start and not any(eng.slots)


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation(tmp_path, graphs):
    """Captured decode graphs: replays advance the recurrent state exactly once per step (the
    capture's warm-up runs are rolled back), finished rows write the scratch state row."""
    cfg = C.CASES["mixed"]
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=2))
    eng = C.engine(path, backend="hip", dtype=torch.float32, rows=4, use_hip_graphs=graphs, precapture_graphs=False)
    try:
        prompts = [C.tokens(n, cfg["vocab"], 20 + n) for n in (9, 31, 16, 2, 40, 23)]
        budget = [6, 12, 19, 5, 3, 10]
        outs = eng.generate_ids(prompts, max_tokens=budget, temperature=0.0)
        for p, out, n in zip(prompts, outs, budget):
            assert len(out) == n
            seq = list(p)
            for tok in out:
                logits = O.forward(sd, cfg, seq)[-1]
                top2 = np.sort(logits)[-2:]
                if float(top2[1] - top2[0]) < 0.05 * float(logits.std()):
                    break  # the sampler reads bf16 rows: a near tie may go either way
                assert tok == int(logits.argmax())
                seq.append(tok)
    finally:
        eng.shutdown()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(8))
def test_drawn_configurations(tmp_path, seed, dtype):
    """Configurations drawn from a seed (sizes, head counts, layer order, windows, taps, constants):
    a whole prompt, the same prompt in portions and token by token, and two requests side by side."""
    cfg = C.random_config(seed)
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=seed))
    eng = C.engine(path, backend="hip", dtype=getattr(torch, dtype), pool_tokens=256)
    try:
        a, b = C.tokens(90, cfg["vocab"], seed), C.tokens(41, cfg["vocab"], seed + 100)
        wa, wb = O.forward(sd, cfg, a), O.forward(sd, cfg, b)
        _close(eng.stream_step([("w", a, list(range(90)))], end=["w"]), wa, dtype)
        at, bt = 0, 0
        for i, s in enumerate([3, 2, 30, 1, 1, 17, 2, 16, 1] + [1] * 17):
            entries, want = [("a", a[at:at + s], list(range(s)))], [wa[at:at + s]]
            at += s
            if bt < 41:
                n = min([1, 7, 2, 16][i % 4], 41 - bt)
                entries.append(("b", b[bt:bt + n], list(range(n))))
                want.append(wb[bt:bt + n])
                bt += n
            _close(eng.stream_step(entries, [k for k, done in (("a", at == 90), ("b", bt == 41 and n > 0)) if done and any(e[0] == k for e in entries)]),
                   np.concatenate(want), dtype)
        assert at == 90
    finally:
        eng.shutdown()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_context_window_across_decode_splits(tmp_path, dtype):
    """A window longer than a decode split and a context several windows long: the decode kernel
    starts at the window's first split, the recurrences run hundreds of tokens."""
    cfg = C.config([C.parallel(C.left(4, 2, 32, 32, 4, 200, 16, 50000.0, (4.0, 1.0, 4.0, 128)), 2, 16, 32, 48),
                    C.delta(2, 2, 32, 16, 4, 48)], width=64, vocab=80)
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=11))
    eng = C.engine(path, backend="hip", dtype=getattr(torch, dtype), pool_tokens=1024, max_len=1024)
    try:
        toks = C.tokens(700, cfg["vocab"], 3)
        want = O.forward(sd, cfg, toks)
        idx = list(range(0, 520, 7)) + [519]
        _close(eng.stream_step([("x", toks[:520], idx)]), want[idx], dtype)
        got = [eng.stream_step([("x", toks[p:p + 1], [0])]) for p in range(520, 600)]
        _close(torch.cat(got), want[520:600], dtype)
        _close(eng.stream_step([("x", toks[600:], list(range(100)))], end=["x"]), want[600:], dtype)
    finally:
        eng.shutdown()


@pytest.mark.parametrize("name", list(C.CASES))
def test_recurrent_branch_on_the_second_stream(tmp_path, name):
    """Large prefill steps run the recurrence beside the attention branch and the feed-forward on
    a second stream; here every step does, several times over, against the one-stream result."""
    cfg = C.CASES[name]
    path = str(tmp_path / "m")
    sd = O.to_f64(C.checkpoint(cfg, path, seed=9))
    eng = C.engine(path, backend="hip", dtype=torch.float32, pool_tokens=1024)
    try:
        eng.model.overlap_min_rows = 1
        toks = [C.tokens(n, cfg["vocab"], 30 + n) for n in (200, 77, 130)]
        want = [O.forward(sd, cfg, t) for t in toks]
        for rep in range(4):
            got = eng.stream_step([(f"s{i}", t[:50], list(range(50))) for i, t in enumerate(toks)])
            _close(got, np.concatenate([w[:50] for w in want]), "float32")
            got = eng.stream_step([(f"s{i}", t[50:], list(range(len(t) - 50))) for i, t in enumerate(toks)],
                                  end=[f"s{i}" for i in range(3)])
            _close(got, np.concatenate([w[50:] for w in want]), "float32")
    finally:
        eng.shutdown()
