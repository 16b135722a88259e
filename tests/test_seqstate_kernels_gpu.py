"""Every HIP op of the per-sequence-state mixers against its fp32 reference (ops/reference.py),
for float and bf16 activations, with segment tables that mix fresh sequences, continued ones and
single tokens, and with inputs made so that a wrong window edge, a dropped sink or a stale state
row shows."""
import pytest
import torch

import padadra_cases as C
from byzantine_consensus_llm_agents_amd.ops import reference as ref

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def ops():
    from byzantine_consensus_llm_agents_amd.ops import get_ops
    return get_ops("hip")


def _tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def _meta(parts, rows):
    return C.segments(parts, rows), C.segments(parts, rows, DEV)


PARTS, ROWS = [(0, 5), (7, 1), (3, 20), (0, 1), (40, 2)], [3, 0, 4, 1, 2]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gains", [(1.2,), (0.7, -1.1)])
def test_embed_hashed_bigram_norm(ops, dtype, gains):
    g = torch.Generator().manual_seed(0)
    table, bigram = torch.randn(50, 72, generator=g).to(dtype), torch.randn(14, 72, generator=g).to(dtype)
    mc, md = _meta(PARTS, ROWS)
    T = mc.positions.numel()
    toks = torch.randint(0, 50, (T,), generator=g, dtype=torch.int32)
    prev = torch.randint(0, 50, (6,), generator=g, dtype=torch.int32)
    prev_d = prev.to(DEV)
    x, hs = ref.embed_hashed_bigram_norm(toks, mc, prev, table, 1.7, bigram, (1009, 31), 1e-5, gains, dtype)
    xd, hd = ops.embed_hashed_bigram_norm(toks.to(DEV), md, prev_d, table.to(DEV), 1.7, bigram.to(DEV), (1009, 31), 1e-5, gains, dtype)
    torch.testing.assert_close(xd.cpu(), x, atol=1e-5, rtol=1e-5)
    assert prev_d.cpu().tolist() == prev.tolist()
    for a, b in zip(hd, hs):
        torch.testing.assert_close(a.cpu().float(), b.float(), **_tol(dtype))
    x2, _ = ops.embed_hashed_bigram_norm(toks.to(DEV), md, prev_d, table.to(DEV), 1.7, None, None, 1e-5, gains, dtype)
    torch.testing.assert_close(x2.cpu(), table[toks.long()].float() * 1.7, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_residual_mix_norm(ops, dtype):
    g = torch.Generator().manual_seed(1)
    T, W = 9, 200
    x = torch.randn(T, W, generator=g)
    a, b, p, q = (torch.randn(T, W, generator=g).to(dtype) for _ in range(4))
    wa, wb = torch.randn(W, generator=g), torch.randn(W, generator=g)
    for normed, plain, gains in (([(a, wa), (b, wb)], [p], (1.1, 0.3)), ([], [p, q], (0.9,)), ([(a, wa)], [], (2.0, 1.0)), ([], [], (1.5,))):
        xr, xd = x.clone(), x.clone().to(DEV)
        want = ref.residual_mix_norm(xr, normed, 0.5, plain, 0.7, 1e-5, gains, dtype)
        got = ops.residual_mix_norm(xd, [(t.to(DEV), w.to(DEV)) for t, w in normed], 0.5, [t.to(DEV) for t in plain], 0.7, 1e-5, gains, dtype)
        torch.testing.assert_close(xd.cpu(), xr, atol=1e-5, rtol=1e-5)
        for u, v in zip(got, want):
            torch.testing.assert_close(u.cpu().float(), v.float(), **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,act,Cn,pad", [(4, None, 300, 11), (2, "silu", 304, 8), (7, None, 300, 11), (1, "silu", 300, 11),
                                             (3, None, 512, 0), (4, "silu", 2056, 8)])
def test_short_conv_and_its_state(ops, dtype, taps, act, Cn, pad):
    """Widths and strides on and off the 16-byte grid (vector and element kernels)."""
    g = torch.Generator().manual_seed(taps)
    mc, md = _meta(PARTS, ROWS)
    T = mc.positions.numel()
    y = torch.randn(T, Cn + pad, generator=g).to(dtype)
    w = torch.randn(Cn, taps, generator=g)
    state = torch.randn(6, taps - 1, Cn, generator=g).to(dtype) if taps > 1 else None
    sd = state.to(DEV) if taps > 1 else None
    want = ref.short_conv(y, Cn, w, mc, state, act)
    got = ops.short_conv(y.to(DEV), Cn, w.to(DEV), md, sd, act)
    torch.testing.assert_close(got.cpu().float(), want.float(), **_tol(dtype))
    if taps > 1:
        assert torch.equal(sd.cpu(), state)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,e,rot", [(4, 2, 16, 24, 8), (2, 1, 24, 16, 24), (3, 3, 10, 12, 0), (6, 2, 72, 40, 36), (2, 2, 6, 10, 6)])
def test_rope_pairs_kv_write_and_rotate_back(ops, dtype, H, G, d, e, rot):
    g = torch.Generator().manual_seed(H)
    T, BS = 37, 16
    x = torch.randn(T, (H + G) * d + G * e + 3, generator=g).to(dtype)
    pos = torch.randint(0, 5000, (T,), generator=g, dtype=torch.int32)
    slots = (torch.randperm(5 * BS, generator=g)[:T] + BS).to(torch.int32)
    qn, kn = 1 + 0.3 * torch.randn(H * d, generator=g), 1 + 0.3 * torch.randn(G * d, generator=g)
    inv, vinv = ref.scaled_inv_freq(rot, 20000.0, (4.0, 1.0, 4.0, 256)), ref.rope_inv_freq(e, 20000.0)
    kc, vc = torch.zeros(7, G, BS, d, dtype=dtype), torch.zeros(7, G, e, BS, dtype=dtype)
    kd, vd = kc.to(DEV), vc.to(DEV)
    want = ref.rope_pairs_kv_write(x, pos, slots, H, G, d, e, qn, kn, 1e-5, inv, vinv, kc, vc)
    got = ops.rope_pairs_kv_write(x.to(DEV), pos.to(DEV), slots.to(DEV), H, G, d, e, qn.to(DEV), kn.to(DEV), 1e-5, inv.to(DEV),
                                  vinv.to(DEV), kd, vd)
    tol = _tol(dtype) if dtype == torch.bfloat16 else dict(atol=2e-3, rtol=2e-3)   # fp32 sin / cos at positions in the thousands
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol)
    kl, vl = ops.kv_to_logical(kd, vd)
    torch.testing.assert_close(kl.cpu().float(), kc.float(), **tol)
    torch.testing.assert_close(vl.cpu().float(), vc.float(), **tol)
    o = torch.randn(T, H * e, generator=g).to(dtype)
    torch.testing.assert_close(ops.rotate_pairs(o.to(DEV), pos.to(DEV), vinv.to(DEV), -1.0, H).cpu().float(),
                               ref.rotate_pairs(o, pos, vinv, -1.0, H).float(), **tol)


def _attention_inputs(H, G, d, e, lens, q_lens, dtype, seed, loud=None):
    """Paged K / V of sequences of ``lens`` tokens (shuffled pages), queries for their last
    ``q_lens`` positions; ``loud`` = (sequence, key position): that key lines up with the sequence's last query."""
    g = torch.Generator().manual_seed(seed)
    BS = 16
    nblk = [(n + BS - 1) // BS for n in lens]
    pages = torch.randperm(sum(nblk) + 3, generator=g) + 1
    tables = torch.zeros(len(lens), max(nblk), dtype=torch.int32)
    kc, vc = torch.zeros(sum(nblk) + 5, G, BS, d), torch.zeros(sum(nblk) + 5, G, e, BS)
    q = torch.randn(sum(q_lens), H, d, generator=g)
    at = 0
    for b, n in enumerate(lens):
        tables[b, :nblk[b]] = pages[at:at + nblk[b]].to(torch.int32)
        at += nblk[b]
        k, v = torch.randn(n, G, d, generator=g), torch.randn(n, G, e, generator=g)
        if loud is not None and loud[0] == b:
            k[loud[1]] = 4.0 * q[sum(q_lens[:b + 1]) - 1, ::H // G]   # lines up with the first head of every group
            v[loud[1]] = 5.0
        for p in range(n):
            kc[tables[b, p // BS], :, p % BS] = k[p]
            vc[tables[b, p // BS], :, :, p % BS] = v[p]
    qs = [0]
    for n in q_lens:
        qs.append(qs[-1] + n)
    return q.to(dtype), kc.to(dtype), vc.to(dtype), tables, torch.tensor(qs, dtype=torch.int32), torch.tensor(lens, dtype=torch.int32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,e", [(8, 1, 64, 64), (4, 2, 16, 24), (6, 2, 72, 40), (34, 2, 32, 32), (4, 2, 128, 128),
                                     (2, 1, 64, 128), (3, 1, 96, 96), (2, 1, 18, 10)])
@pytest.mark.parametrize("window", [0, 1, 16, 37, 96, 400])
def test_window_and_sink_attention(ops, dtype, H, G, d, e, window):
    """Prefill tiles and single rows in one step; the loud key sits just outside the last query's
    window of one sequence and just inside another's."""
    from byzantine_consensus_llm_agents_amd.models.transformer import AttnMeta
    lens, q_lens = [300, 139, 64, 17, 210], [130, 1, 64, 1, 2]
    loud = (1, 138 - window) if 0 < window < 138 else (0, 3)        # the last key outside the window of sequence 1's query
    q, kc, vc, tables, qs, sl = _attention_inputs(H, G, d, e, lens, q_lens, dtype, window + H, loud)
    sink = 3.0 + torch.randn(H, generator=torch.Generator().manual_seed(5)) * 2
    want = ref.multimap_attention(q, kc, vc, tables, qs, sl, d ** -0.5, 1, 0.0, -1.0, 1.0, e, window, sink)
    kd, vd = ops.kv_from_logical(kc.to(DEV), vc.to(DEV))
    tiles, single = [], []
    for b, n in enumerate(q_lens):
        if n == 1:
            single.append((int(qs[b]), b))
        else:
            tiles += [(b, t, min(t + 64, int(qs[b + 1]))) for t in range(int(qs[b]), int(qs[b + 1]), 64)]
    i32 = dict(dtype=torch.int32, device=DEV)
    meta = AttnMeta(positions=None, slots=None, block_tables=tables.to(DEV), seq_lens=sl.to(DEV), q_start=qs.to(DEV),
                    tiles=torch.tensor(tiles, **i32), single=torch.tensor(single, **i32), tile_rows=64)
    got = ops.multimap_attention(q.to(DEV), kd, vd, meta, d ** -0.5, 1, 0.0, -1.0, 1.0, e, window, sink.to(DEV))
    tol = dict(atol=2e-4, rtol=2e-4) if dtype == torch.float32 else dict(atol=4e-2, rtol=4e-2)
    torch.testing.assert_close(got.cpu().float(), want.float(), **tol)
    if 0 < window < 138:   # one key further in and the answer changes by far more than the tolerance
        inside = ref.multimap_attention(q, kc, vc, tables, qs, sl, d ** -0.5, 1, 0.0, -1.0, 1.0, e, window + 1, sink)
        assert float((inside[130] - want[130]).abs().max()) > 0.5
    # the same rows as a pure decode step (every sequence's last token)
    last = torch.tensor([int(qs[b + 1]) - 1 for b in range(len(lens))])
    dmeta = AttnMeta(positions=None, slots=None, block_tables=tables.to(DEV), seq_lens=sl.to(DEV), decode=True)
    gd = ops.multimap_attention(q[last].contiguous().to(DEV), kd, vd, dmeta, d ** -0.5, 1, 0.0, -1.0, 1.0, e, window, sink.to(DEV))
    torch.testing.assert_close(gd.cpu().float(), want[last].float(), **tol)
    no_sink = ops.multimap_attention(q[last].contiguous().to(DEV), kd, vd, dmeta, d ** -0.5, 1, 0.0, -1.0, 1.0, e, window, None)
    assert float((no_sink.cpu().float() - want[last].float())[2:].abs().max()) > 0.1   # the sink is not a no-op here


@pytest.mark.parametrize("window", [0, 100, 513, 1290])
def test_window_over_long_contexts(ops, window):
    """Contexts of many decode splits: the window's first split is far from the sequence's first."""
    from byzantine_consensus_llm_agents_amd.models.transformer import AttnMeta
    H, G, d, e, dtype = 4, 2, 32, 48, torch.float32
    lens, q_lens = [1500, 700, 129], [70, 1, 1]
    q, kc, vc, tables, qs, sl = _attention_inputs(H, G, d, e, lens, q_lens, dtype, window, None)
    sink = torch.randn(H, generator=torch.Generator().manual_seed(2))
    want = ref.multimap_attention(q, kc, vc, tables, qs, sl, d ** -0.5, 1, 0.0, -1.0, 1.0, e, window, sink)
    kd, vd = ops.kv_from_logical(kc.to(DEV), vc.to(DEV))
    i32 = dict(dtype=torch.int32, device=DEV)
    meta = AttnMeta(positions=None, slots=None, block_tables=tables.to(DEV), seq_lens=sl.to(DEV), q_start=qs.to(DEV),
                    tiles=torch.tensor([(0, 0, 64), (0, 64, 70)], **i32), single=torch.tensor([(70, 1), (71, 2)], **i32), tile_rows=64)
    got = ops.multimap_attention(q.to(DEV), kd, vd, meta, d ** -0.5, 1, 0.0, -1.0, 1.0, e, window, sink.to(DEV))
    torch.testing.assert_close(got.cpu(), want, atol=2e-4, rtol=2e-4)
    last = torch.tensor([69, 70, 71])
    dmeta = AttnMeta(positions=None, slots=None, block_tables=tables.to(DEV), seq_lens=sl.to(DEV), decode=True)
    gd = ops.multimap_attention(q[last].contiguous().to(DEV), kd, vd, dmeta, d ** -0.5, 1, 0.0, -1.0, 1.0, e, window, sink.to(DEV))
    torch.testing.assert_close(gd.cpu(), want[last], atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,Gq,d,e,delta", [(4, 4, 48, 64, False), (6, 6, 64, 32, True), (4, 2, 16, 12, True), (2, 1, 96, 72, True),
                                            (3, 3, 20, 130, False), (2, 2, 128, 8, True), (2, 1, 160, 24, True), (1, 1, 256, 40, False)])
def test_gated_state_scan(ops, dtype, H, Gq, d, e, delta):
    g = torch.Generator().manual_seed(H * d)
    mc, md = _meta(PARTS, ROWS)
    T = mc.positions.numel()
    q, k = torch.randn(T, Gq, d, generator=g) * 0.3, torch.randn(T, Gq, d, generator=g) * 0.3
    gg = torch.rand(T, H, d, generator=g)
    v = torch.randn(T, H * e + 5, generator=g).to(dtype)[:, 2:2 + H * e]
    beta = torch.rand(T, H, generator=g) if delta else None
    state = torch.randn(6, H, d, e, generator=g)
    sd = state.to(DEV)
    want = ref.gated_state_scan(q, k, gg, v, beta, mc, state, delta)
    got = ops.gated_state_scan(q.to(DEV), k.to(DEV), gg.to(DEV), v.to(DEV), beta.to(DEV) if delta else None, md, sd, delta)
    torch.testing.assert_close(got.cpu(), want, atol=2e-4, rtol=2e-4)
    torch.testing.assert_close(sd.cpu(), state, atol=2e-4, rtol=2e-4)   # rows of segments moved on, row 5 untouched


@pytest.mark.parametrize("d,delta", [(64, False), (128, True), (40, True)])
def test_gated_state_scan_many_workgroups(ops, d, delta):
    """Enough (segment, head, column) work that the kernel takes its 8-columns-per-wave form."""
    g = torch.Generator().manual_seed(d)
    H, Gq, e = 16, 8, 128
    parts = [(0, 3), (5, 1), (2, 6), (0, 1), (9, 2), (1, 1), (0, 5), (3, 4)]
    mc, md = _meta(parts, [1, 0, 3, 2, 5, 4, 7, 6])
    T = mc.positions.numel()
    q, k = torch.randn(T, Gq, d, generator=g) * 0.3, torch.randn(T, Gq, d, generator=g) * 0.3
    gg, v = torch.rand(T, H, d, generator=g), torch.randn(T, H * e, generator=g).to(torch.bfloat16)
    beta = torch.rand(T, H, generator=g) if delta else None
    state = torch.randn(9, H, d, e, generator=g)
    sd = state.to(DEV)
    want = ref.gated_state_scan(q, k, gg, v, beta, mc, state, delta)
    got = ops.gated_state_scan(q.to(DEV), k.to(DEV), gg.to(DEV), v.to(DEV), beta.to(DEV) if delta else None, md, sd, delta)
    torch.testing.assert_close(got.cpu(), want, atol=2e-4, rtol=2e-4)
    torch.testing.assert_close(sd.cpu(), state, atol=2e-4, rtol=2e-4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prepare_and_head_norm(ops, dtype):
    g = torch.Generator().manual_seed(3)
    T, H, G, d, e = 11, 4, 2, 20, 70
    y = torch.randn(T, 3 * H * d + 9, generator=g).to(dtype)
    fb, low = torch.randn(H * d, generator=g), torch.rand(H * d, generator=g)
    for a, b in zip(ops.hgrn2_prepare(y.to(DEV), 4, 4 + H * d, H, d, fb.to(DEV), low.to(DEV)), ref.hgrn2_prepare(y, 4, 4 + H * d, H, d, fb, low)):
        torch.testing.assert_close(a.cpu(), b, atol=1e-5, rtol=1e-5)
    c = torch.randn(T, 2 * G * d + 7, generator=g).to(dtype)
    a_in = torch.randn(T, H * d, generator=g).to(dtype) * 3
    alog, dtb = torch.randn(H, generator=g), torch.randn(H * d, generator=g)
    got = ops.delta_prepare(c.to(DEV), y.to(DEV), 5, a_in.to(DEV), alog.to(DEV), dtb.to(DEV), H, G, d)
    for a, b in zip(got, ref.delta_prepare(c, y, 5, a_in, alog, dtb, H, G, d)):
        torch.testing.assert_close(a.cpu(), b, atol=1e-5, rtol=1e-4)
    o = torch.randn(T, H, e, generator=g)
    w = torch.randn(e, generator=g)
    gate = torch.randn(T, H * e + 3, generator=g).to(dtype)[:, 1:1 + H * e]
    for gt in (None, gate):
        torch.testing.assert_close(ops.head_norm_gate(o.to(DEV), w.to(DEV), 1e-5, gt.to(DEV) if gt is not None else None, dtype).cpu().float(),
                                   ref.head_norm_gate(o, w, 1e-5, gt, dtype).float(), **_tol(dtype))
    z = torch.randn(T, 50, generator=g).to(dtype)
    torch.testing.assert_close(ops.act_fn(z.to(DEV), "silu").cpu().float(), ref.act_fn(z, "silu").float(), **_tol(dtype))
