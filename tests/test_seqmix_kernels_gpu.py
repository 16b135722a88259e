"""HIP kernels of the fp32-stream mixers against the PyTorch fp32 references of the same ops."""
import math

import pytest
import torch

from byzantine_consensus_llm_agents_amd.models.transformer import AttnMeta
from byzantine_consensus_llm_agents_amd.ops import reference as ref

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def ops():
    from byzantine_consensus_llm_agents_amd.ops import get_ops
    return get_ops("hip")


def _tol(dtype):
    return dict(atol=2e-2, rtol=2e-2) if dtype == torch.bfloat16 else dict(atol=2e-5, rtol=2e-5)


DTYPES = [torch.bfloat16, torch.float32]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [96, 256, 1000])
def test_embed_and_residual_norm(ops, dtype, W):
    g = torch.Generator().manual_seed(W)
    T, V = 37, 50
    table = torch.randn(V, W, generator=g).to(dtype).to(DEV)
    w = (torch.randn(W, generator=g) * 0.1).to(DEV)
    tokens = torch.randint(0, V, (T,), generator=g, dtype=torch.int32).to(DEV)
    h, x = ops.embed_scale_rmsnorm(tokens, table, 7.5, w, 1e-5, 1.0, dtype)
    h_r, x_r = ref.embed_scale_rmsnorm(tokens, table, 7.5, w, 1e-5, 1.0, dtype)
    torch.testing.assert_close(x, x_r, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(h.float(), h_r.float(), **_tol(dtype))
    parts = [torch.randn(T, W, generator=g).to(dtype).to(DEV) for _ in range(2)]
    moe = torch.randn(T, W, generator=g).to(DEV)
    gate = torch.randn(T, generator=g).to(DEV)
    gated = torch.randn(T, W, generator=g).to(dtype).to(DEV)
    x2, x2_r = x.clone(), x_r.clone()
    h2 = ops.residual_add_rmsnorm32(x2, parts[:1] + [moe], w, 1e-5, 1.0, dtype, gate, gated)
    h2_r = ref.residual_add_rmsnorm32(x2_r, parts[:1] + [moe], w, 1e-5, 1.0, dtype, gate, gated)
    torch.testing.assert_close(x2, x2_r, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(h2.float(), h2_r.float(), **_tol(dtype))
    assert ops.residual_add_rmsnorm32(x2, parts, None, 1e-5, 1.0, dtype) is None
    ref.residual_add_rmsnorm32(x2_r, parts, None, 1e-5, 1.0, dtype)
    torch.testing.assert_close(x2, x2_r, atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["gelu_tanh", "relu2"])
def test_act_fn_strided(ops, dtype, kind):
    x = (torch.randn(33, 300) * 3).to(dtype).to(DEV)
    view = x[:, 17:217]
    torch.testing.assert_close(ops.act_fn(view, kind).float(), ref.act_fn(view, kind).float(), **_tol(dtype))


def _paged(seq_lens, q_lens, BS, G, KD, VD, dtype, seed, shuffle=True, tile_rows=64):
    """Random paged cache + metadata of a packed step: sequence b holds seq_lens[b] tokens, the last q_lens[b] are queries."""
    g = torch.Generator().manual_seed(seed)
    nblk = [(n + BS - 1) // BS for n in seq_lens]
    NB = sum(nblk) + 3
    ids = torch.randperm(NB - 1, generator=g)[:sum(nblk)] + 1 if shuffle else torch.arange(1, sum(nblk) + 1)
    bt = torch.zeros(len(seq_lens), max(nblk) + 1, dtype=torch.int32)
    o = 0
    for b, n in enumerate(nblk):
        bt[b, :n] = ids[o:o + n].to(torch.int32)
        o += n
    k = torch.randn(NB, G, BS, KD, generator=g).to(dtype)
    v = torch.randn(NB, G, VD, BS, generator=g).to(dtype)
    q_start = [0]
    tiles, single = [], []
    for b, ql in enumerate(q_lens):
        if ql == 1:
            single.append((q_start[-1], b))
        else:
            for t in range(q_start[-1], q_start[-1] + ql, tile_rows):
                tiles.append((b, t, min(t + tile_rows, q_start[-1] + ql)))
        q_start.append(q_start[-1] + ql)
    i32 = torch.int32
    meta = AttnMeta(positions=None, slots=None, block_tables=bt.to(DEV), seq_lens=torch.tensor(seq_lens, dtype=i32, device=DEV),
                    q_start=torch.tensor(q_start, dtype=i32, device=DEV), decode=False, tile_rows=tile_rows,
                    tiles=torch.tensor(tiles, dtype=i32, device=DEV).reshape(-1, 3),
                    single=torch.tensor(single, dtype=i32, device=DEV).reshape(-1, 2))
    return k.to(DEV), v.to(DEV), meta, q_start[-1]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,maps,dim,vdim,BS", [(4, 2, 2, 32, 64, 16), (3, 3, 2, 24, 40, 16), (4, 1, 1, 64, 128, 32),
                                                 (2, 2, 2, 80, 144, 16), (2, 1, 2, 20, 18, 16), (8, 2, 2, 64, 128, 16),
                                                 (6, 2, 2, 48, 96, 16), (2, 2, 2, 64, 64, 16), (40, 2, 2, 32, 32, 16), (2, 1, 2, 9, 10, 16),
                                                 (3, 1, 1, 7, 5, 16)])
def test_multimap_attention_mixed_step(ops, dtype, H, G, maps, dim, vdim, BS):
    seq_lens = [300, 17, 1, 129, 64, 513, 40, 400]
    q_lens = [70, 17, 1, 1, 2, 1, 16, 301]
    k, v, meta, T = _paged(seq_lens, q_lens, BS, G, maps * dim, vdim, dtype, seed=dim,
                           tile_rows=ops.multimap_tile_rows(dim, vdim))
    q = torch.randn(T, H, maps * dim, generator=torch.Generator().manual_seed(1)).to(dtype).to(DEV)
    args = (0.17, maps, 0.35, 1e-5, 0.4, vdim)
    kp, vp = ops.kv_from_logical(k, v)   # the kernels' slab order
    got = ops.multimap_attention(q, kp, vp, meta, *args)
    want = ref.multimap_attention(q, k, v, meta.block_tables, meta.q_start, meta.seq_lens, *args)
    torch.testing.assert_close(got.float(), want.float(), **(dict(atol=3e-2, rtol=3e-2) if dtype == torch.bfloat16 else dict(atol=1e-4, rtol=1e-4)))
    # the same rows through the decode form of a step: every sequence one token
    B = len(seq_lens)
    dmeta = AttnMeta(positions=None, slots=None, block_tables=meta.block_tables, seq_lens=meta.seq_lens, decode=True)
    qd = q[(meta.q_start[1:] - 1).long()].contiguous()
    got_d = ops.multimap_attention(qd, kp, vp, dmeta, *args)
    want_d = ref.multimap_attention(qd, k, v, meta.block_tables, torch.arange(B + 1, dtype=torch.int32, device=DEV),
                                    meta.seq_lens, *args)
    torch.testing.assert_close(got_d.float(), want_d.float(), **(dict(atol=3e-2, rtol=3e-2) if dtype == torch.bfloat16 else dict(atol=1e-4, rtol=1e-4)))


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_far_key_stands_out(ops, dtype):
    """One key far back is made to dominate map 0 (and another map 1): dropping either shows."""
    H, G, maps, dim, vdim, BS = 2, 1, 2, 32, 48, 16
    n = 1200
    k, v, meta, T = _paged([n, n], [1, 90], BS, G, maps * dim, vdim, dtype, seed=5)
    q = torch.randn(T, H, maps * dim, generator=torch.Generator().manual_seed(2)).to(dtype).to(DEV)
    for b, far in ((0, 3), (1, 17)):
        blk = int(meta.block_tables[b, far // BS])
        k[blk, 0, far % BS, :dim] = 6.0 * q[0 if b == 0 else T - 1, 0, :dim]
        blk2 = int(meta.block_tables[b, (far + 300) // BS])
        k[blk2, 0, (far + 300) % BS, dim:] = 6.0 * q[0 if b == 0 else T - 1, 0, dim:]
    args = (0.2, maps, 0.5, 1e-5, 1.0, vdim)
    got = ops.multimap_attention(q, *ops.kv_from_logical(k, v), meta, *args)
    want = ref.multimap_attention(q, k, v, meta.block_tables, meta.q_start, meta.seq_lens, *args)
    torch.testing.assert_close(got.float(), want.float(), **(dict(atol=3e-2, rtol=3e-2) if dtype == torch.bfloat16 else dict(atol=1e-4, rtol=1e-4)))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n_q,n_kv,maps,dim,vdim,rot", [(4, 2, 2, 32, 64, 32), (3, 1, 2, 24, 20, 8), (2, 2, 1, 64, 64, 0),
                                                        (2, 1, 2, 9, 10, 4)])
def test_rope_multi_kv_write(ops, dtype, n_q, n_kv, maps, dim, vdim, rot):
    T, BS, NB = 45, 16, 9
    g = torch.Generator().manual_seed(rot)
    width = n_q * maps * dim + n_kv * maps * dim + n_kv * vdim + 13
    qkv = torch.randn(T, width, generator=g).to(dtype).to(DEV)
    pos = torch.randint(0, 5000, (T,), generator=g, dtype=torch.int32).to(DEV)
    slots = (torch.randperm((NB - 1) * BS, generator=g)[:T] + BS).to(torch.int32).to(DEV)
    inv = ref.rope_inv_freq(rot, 30000.0, DEV)
    caches = [[torch.zeros(NB, n_kv, BS, maps * dim, dtype=dtype, device=DEV),
               torch.zeros(NB, n_kv, vdim, BS, dtype=dtype, device=DEV)] for _ in range(2)]
    q = ops.rope_multi_kv_write(qkv, pos, slots, n_q, n_kv, maps, dim, vdim, inv, *caches[0])
    q_r = ref.rope_multi_kv_write(qkv, pos, slots, n_q, n_kv, maps, dim, vdim, inv, *caches[1])
    tol = dict(atol=3e-2, rtol=2e-2) if dtype == torch.bfloat16 else dict(atol=2e-3, rtol=1e-3)  # fp32 sin/cos at large angles
    torch.testing.assert_close(q.float(), q_r.float(), **tol)
    k_l, v_l = ops.kv_to_logical(*caches[0])
    torch.testing.assert_close(k_l.float(), caches[1][0].float(), **tol)
    torch.testing.assert_close(v_l.float(), caches[1][1].float(), atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,W,E,top,ff", [(1, 64, 4, 1, 32), (5, 128, 8, 2, 48), (333, 256, 6, 3, 100), (64, 96, 3, 3, 36),
                                          (700, 512, 8, 2, 320), (130, 72, 5, 2, 40)])
def test_moe_route_and_experts(ops, dtype, T, W, E, top, ff):
    g = torch.Generator().manual_seed(T + E)
    h = torch.randn(T, W, generator=g).to(dtype).to(DEV)
    rw = torch.randn(E, W, generator=g).to(DEV) / math.sqrt(W)
    rb = torch.randn(E, generator=g).to(DEV)
    gw = torch.randn(W, generator=g).to(DEV) / math.sqrt(W)
    up = (torch.randn(E, ff, W, generator=g) / math.sqrt(W)).to(dtype).to(DEV)
    down = (torch.randn(E, W, ff, generator=g) / math.sqrt(ff)).to(dtype).to(DEV)
    idx, wts, gate = ops.moe_route(h, rw, rb, top, gw)
    idx_r, wts_r, gate_r = ref.moe_route(h, rw, rb, top, gw)
    z = h.float() @ rw.t() + rb
    margin = (torch.sort(z, -1, descending=True).values[:, :top + 1].diff(dim=-1).abs().min(-1).values > 1e-4
              if top < E else torch.ones(T, dtype=torch.bool, device=DEV))
    assert torch.equal(idx[margin], idx_r[margin])   # (rows with a near tie may order differently)
    torch.testing.assert_close(wts[margin], wts_r[margin], atol=1e-5, rtol=1e-4)
    torch.testing.assert_close(gate, gate_r, atol=1e-4, rtol=1e-4)
    got = ops.moe_experts(h, up, down, idx_r, wts_r, "relu2")
    want = ref.moe_experts(h, up, down, idx_r, wts_r, "relu2")
    torch.testing.assert_close(got, want, **(dict(atol=3e-2, rtol=3e-2) if dtype == torch.bfloat16 else dict(atol=1e-4, rtol=1e-4)))
