"""The HIP kernels the Pudizen design added or extended, each against the
eager torch op of ops/reference.py, in both activation types: grouped RMS norm
over the parallel residual (register path, scalar path, strided branches),
pair-hash embedding, squared relu, rotation of head rows, the cache store with
a whole-row norm, either pair layout and rotated values, row attention with a
window and sigmoid weights, with fp32 results, and over rows whose values are
their keys (per-token kernel and matrix-core kernel)."""

import pytest
import torch

from parallax_amd import ops
from parallax_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda")
TOLS = {torch.float32: 2e-5, torch.bfloat16: 1.6e-2}
DTYPES = [torch.float32, torch.bfloat16]


def close(got, want, tol):
    err = (got.float().cpu() - want.float().cpu()).abs().max().item()
    return err <= tol * max(1.0, want.float().abs().max().item())


def gpu(x):
    return x.to(DEV) if torch.is_tensor(x) else x


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W,G", [(224, 7), (256, 1), (100, 5), (4096, 8), (6144, 3), (40, 40)])
def test_group_rmsnorm_add(dt, W, G):
    assert ops.has_mix_extension()
    g = torch.Generator().manual_seed(W + G)
    T = 7
    x = torch.randn(T, W, generator=g) * 3
    x[:, : W // 2] *= 20.0
    y1 = torch.randn(T, W, generator=g).to(dt)
    y2 = torch.randn(T, W + 8, generator=g).to(dt)[:, 4:4 + W]     # a strided view
    w = torch.randn(W, generator=g).to(dt)
    for ys in ((None, None), (y1, None), (y1, y2)):
        xc, xg = x.clone(), x.clone().to(DEV)
        hc = ref.group_rmsnorm_add(xc, ys[0], ys[1], w, G, 1e-5, dt)
        hg = ops.group_rmsnorm_add(xg, gpu(ys[0]), gpu(ys[1]), w.to(DEV), G, 1e-5, dt)
        assert close(hg, hc, TOLS[dt]) and close(xg, xc, 1e-6)
    xc, xg = x.clone(), x.clone().to(DEV)
    assert ops.group_rmsnorm_add(xg, y1.to(DEV), y2.to(DEV), None, G, 1e-5, dt) is None
    ref.group_rmsnorm_add(xc, y1, y2, None, G, 1e-5, dt)
    assert close(xg, xc, 1e-6)


@pytest.mark.parametrize("dt", DTYPES)
def test_pair_hash_embedding_relu_and_rotation(dt):
    g = torch.Generator().manual_seed(1)
    V, W, B = 50, 72, 13
    tab, pair = torch.randn(V, W, generator=g).to(dt), torch.randn(B + 1, W, generator=g).to(dt)
    ids = torch.randint(0, V, (9,), generator=g)
    prev = torch.randint(0, V, (9,), generator=g)
    prev[0] = prev[5] = -1
    for mp, mc in ((29, 3), (1000003, 999983)):
        got = ops.pair_hash_embedding(ids.to(DEV), prev.to(DEV), tab.to(DEV), 2.5,
                                      pair.to(DEV), B, mp, mc)
        assert close(got, ref.pair_hash_embedding(ids, prev, tab, 2.5, pair, B, mp, mc), 1e-6)
    for I in (352, 50):
        xx = torch.randn(5, I + 20, generator=g).to(dt)
        assert close(ops.relu_squared(xx.to(DEV)[:, 12:12 + I]),
                     ref.relu_squared(xx[:, 12:12 + I]), TOLS[dt] / 2)
    pos = torch.tensor([0, 1, 5, 1000, 77, 3], dtype=torch.int32)
    for inter in (False, True):
        for D in (24, 2, 130):
            x, fr = torch.randn(6, 3, D, generator=g), torch.rand(D // 2, generator=g)
            for sign in (-1.0, 1.0):
                assert close(ops.rotate_heads(x.to(DEV), pos.to(DEV), fr.to(DEV), inter, sign, dt),
                             ref.rotate_heads(x, pos, fr, inter, sign, dt), TOLS[dt])


def _paged(lens, bs, nblk, g):
    pos = torch.cat([torch.arange(n) for n in lens]).int()
    seq = torch.cat([torch.full((n,), i) for i, n in enumerate(lens)]).int()
    perm = torch.randperm(nblk, generator=g)
    bt = torch.zeros(len(lens), max((n + bs - 1) // bs for n in lens), dtype=torch.int32)
    o = 0
    for i, n in enumerate(lens):
        nb = (n + bs - 1) // bs
        bt[i, :nb] = perm[o:o + nb]
        o += nb
    slots = bt[seq.long(), (pos // bs).long()].long() * bs + pos % bs
    bounds = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    return pos, seq, bt, slots, bounds


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,G,d,dv,rot,inter,whole,vrot,win,sig", [
    (6, 2, 128, 128, 48, True, False, False, 70, True),
    (6, 3, 96, 96, 32, False, True, True, 0, False),
    (4, 2, 40, 24, 40, False, True, True, 0, False),
    (3, 3, 20, 12, 8, True, False, False, 5, True),      # widths off the vector paths
    (8, 2, 64, 64, 64, False, True, True, 0, False),
    (2, 1, 16, 256, 0, False, True, True, 33, False),
    (4, 4, 32, 48, 16, True, False, True, 0, False),     # neighbouring value pairs
    (5, 1, 24, 20, 0, False, False, True, 0, True),
])
def test_store_and_attention(dt, H, G, d, dv, rot, inter, whole, vrot, win, sig):
    g = torch.Generator().manual_seed(H * d + dv)
    bs, nblk = 16, 40
    lens = [37, 150, 1]
    T = sum(lens)
    pos, seq, bt, slots, bounds = _paged(lens, bs, nblk, g)
    q = torch.randn(T, H * d + 16, generator=g).to(dt)[:, 8:8 + H * d]
    k, v = torch.randn(T, G * d, generator=g).to(dt), torch.randn(T, G * dv, generator=g).to(dt)
    cache_c = torch.zeros(nblk, bs, G * d + G * dv, dtype=dt)
    cache_g = cache_c.to(DEV)
    kw = dict(rot_freq=torch.rand(rot // 2, generator=g) if rot else None, rot_mult=1.0,
              rot_dims=rot, norm_whole=whole, rot_interleaved=inter, v_seg=dv,
              v_rot_freq=torch.rand(dv // 2, generator=g) if vrot else None,
              q_weight=torch.randn(H * d, generator=g) if whole else None,
              k_weight=torch.randn(G * d, generator=g) if whole else None)
    eps = 1e-5 if whole else None
    # the cos/sin of the value rotation, for the attention's turn back
    cs_c = torch.zeros(T, dv) if vrot else None
    cs_g = torch.zeros(T, dv, device=DEV) if vrot else None
    qc = ref.qkv_store(q, k, v, pos, slots, cache_c, d, eps, 0.0, 0, v_cs_out=cs_c, **kw)
    qg = ops.qkv_store(q.to(DEV), k.to(DEV), v.to(DEV), pos.to(DEV), slots.to(DEV), cache_g,
                       d, eps, 0.0, 0, v_cs_out=cs_g, **{a: gpu(b) for a, b in kw.items()})
    assert close(qg, qc, 2e-5) and close(cache_g, cache_c, TOLS[dt])
    if vrot:
        assert close(cs_g, cs_c, 1e-4)      # angles up to 150 rad in fp32
    bias = torch.randn(H, generator=g) - 2 if sig else None
    for odt in (dt, torch.float32):
        want = ref.row_attention(qc, cache_c, None, bt, seq, pos, H, G, 1, d, dv, win, 0, 0.1,
                                 0.0, 0.0, None, 1.0, odt, bias, None, False, cs_c, inter)
        if vrot:
            # the table is what a separate pass over fp32 results would use
            plain = ref.row_attention(qc, cache_c, None, bt, seq, pos, H, G, 1, d, dv, win, 0,
                                      0.1, 0.0, 0.0, None, 1.0, torch.float32, bias)
            turned = ref.rotate_heads(plain.view(T, H, dv), pos, kw["v_rot_freq"], inter,
                                      -1.0, torch.float32)
            assert close(want, turned, 1e-4 if odt == torch.float32 else TOLS[dt])
        for tiled in (True, False):     # the matrix-core kernel, the per-token kernel
            got = ops.row_attention(
                qc.to(DEV), cache_c.to(DEV), None, bt.to(DEV), seq.to(DEV), pos.to(DEV), H, G, 1,
                d, dv, win, 0, 0.1, 0.0, 0.0, None, 1.0, odt, max_seq_len=max(lens),
                query_bounds=bounds.to(DEV) if tiled else None, head_bias=gpu(bias),
                out_rot_cs=gpu(cs_c), out_rot_interleaved=inter)
            assert got.dtype == odt
            assert close(got, want, 2e-5 if odt == torch.float32 else TOLS[dt]), (odt, tiled)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,r", [(8, 64), (3, 24), (5, 20), (2, 256), (2, 320)])
def test_rows_whose_values_are_their_keys(dt, H, r):
    g = torch.Generator().manual_seed(H + r)
    bs = 16
    lens = [70, 9, 1]
    T = sum(lens)
    pos, seq, bt, slots, bounds = _paged(lens, bs, 9, g)
    dkv = torch.randn(T, r + 8, generator=g).to(dt)[:, :r]
    nw = torch.randn(r, generator=g).to(dt)
    cc = torch.zeros(9, bs, r, dtype=dt)
    cg = cc.to(DEV)
    none = torch.empty(0)
    ref.latent_kv_store(dkv, nw, 1e-5, none, 1.0, 0, pos, slots, cc, r)
    ops.latent_kv_store(dkv.to(DEV), nw.to(DEV), 1e-5, none.to(DEV), 1.0, 0, pos.to(DEV),
                        slots.to(DEV), cg, r)
    assert close(cg, cc, TOLS[dt])
    ql = torch.randn(T, H * r, generator=g)
    gate = torch.randn(T, H + 4, generator=g).to(dt)[:, :H]
    want = ref.row_attention(ql, cc, None, bt, seq, pos, H, 1, 1, r, r, 0, 0, 0.2, 0.0, 0.0,
                             None, 1.0, torch.float32, None, gate, True)
    for tiled in (True, False):
        if r > 256:      # more value columns than a head sums in one call
            with pytest.raises(RuntimeError):
                ops.row_attention(ql.to(DEV), cc.to(DEV), None, bt.to(DEV), seq.to(DEV),
                                  pos.to(DEV), H, 1, 1, r, r, 0, 0, 0.2, 0.0, 0.0, None, 1.0,
                                  torch.float32, gate=gate.to(DEV), shared_kv=True)
            break
        got = ops.row_attention(ql.to(DEV), cc.to(DEV), None, bt.to(DEV), seq.to(DEV),
                                pos.to(DEV), H, 1, 1, r, r, 0, 0, 0.2, 0.0, 0.0, None, 1.0,
                                torch.float32, max_seq_len=70,
                                query_bounds=bounds.to(DEV) if tiled else None,
                                gate=gate.to(DEV), shared_kv=True)
        assert close(got, want, 2e-5), tiled
    # a share of the row's columns as values
    if r >= 24:
        c0, cols = (8, r - 16) if r <= 256 else (256, r - 256)
        want = ref.row_attention(ql, cc, None, bt, seq, pos, H, 1, 1, r, cols, 0, 0, 0.2, 0.0,
                                 0.0, None, 1.0, torch.float32, None, gate, True, None, False,
                                 c0)
        for tiled in (True, False):
            got = ops.row_attention(ql.to(DEV), cc.to(DEV), None, bt.to(DEV), seq.to(DEV),
                                    pos.to(DEV), H, 1, 1, r, cols, 0, 0, 0.2, 0.0, 0.0, None,
                                    1.0, torch.float32, max_seq_len=70,
                                    query_bounds=bounds.to(DEV) if tiled else None,
                                    gate=gate.to(DEV), shared_kv=True, value_col=c0)
            assert close(got, want, 2e-5), (tiled, "share")


@pytest.mark.parametrize("H,G,d,dv,win,sig", [
    (8, 2, 128, 128, 0, False),
    (4, 4, 64, 64, 200, True),
    (6, 1, 40, 96, 0, True),
    (3, 3, 128, 32, 333, False),
])
def test_three_part_bf16_products_are_exact(H, G, d, dv, win, sig):
    """Prompt portions over bf16 rows run both products on the bf16 matrix
    cores with the fp32 operand split into three bf16 parts: the result must
    equal the fp32 arithmetic of the reference (and of the per-token kernel)
    to rounding, over many key steps, ragged tiles and portions that start
    in the middle of a sequence."""
    g = torch.Generator().manual_seed(d + dv)
    bs, nblk = 32, 40
    lens = [700, 45, 290]
    starts = [0, 13, 258]           # the portions' first positions
    pos = torch.cat([torch.arange(s0, n) for s0, n in zip(starts, lens)]).int()
    seq = torch.cat([torch.full((n - s0,), i) for i, (s0, n) in enumerate(zip(starts, lens))]).int()
    T = pos.numel()
    perm = torch.randperm(nblk, generator=g)
    bt = torch.zeros(3, 22, dtype=torch.int32)
    o = 0
    for i, n in enumerate(lens):
        nb = (n + bs - 1) // bs
        bt[i, :nb] = perm[o:o + nb]
        o += nb
    bounds = torch.tensor([0] + torch.tensor([n - s0 for s0, n in zip(starts, lens)])
                          .cumsum(0).tolist(), dtype=torch.int32)
    cache = (torch.randn(nblk, bs, G * d + G * dv, generator=g) * 0.7).to(torch.bfloat16)
    q = torch.randn(T, H * d, generator=g) * 1.3
    bias = torch.randn(H, generator=g) - 3 if sig else None
    want = ref.row_attention(q, cache, None, bt, seq, pos, H, G, 1, d, dv, win, 0, d ** -0.5,
                             0.0, 0.0, None, 1.0, torch.float32, bias)
    for tiled in (True, False):
        got = ops.row_attention(q.to(DEV), cache.to(DEV), None, bt.to(DEV), seq.to(DEV),
                                pos.to(DEV), H, G, 1, d, dv, win, 0, d ** -0.5, 0.0, 0.0, None,
                                1.0, torch.float32, max_seq_len=max(lens),
                                query_bounds=bounds.to(DEV) if tiled else None,
                                head_bias=gpu(bias))
        assert close(got, want, 3e-5), tiled
