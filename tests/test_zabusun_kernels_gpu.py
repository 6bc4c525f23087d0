"""GPU numerics of the kernels the Zabusun design added to extension _mix
(post-norm residual step, clamped gated linear unit, minGRU scan, q/k norm
with rotation in the cache store, sigmoid-weighted row attention with an
output gate) and of the grouped expert GEMMs with the routing weight on the
input: each against the eager fp32 torch version of the same op
(ops/reference.py), for bf16 and float32 activations, on sizes that are not
multiples of the kernels' tiles (and some that are)."""

import pytest
import torch

from parallax_amd import ops
from parallax_amd.models.rope import yarn_ramp_frequencies
from parallax_amd.ops import reference as ref

pytestmark = pytest.mark.gpu

DEV = "cuda"


def _rand(*shape, dtype=torch.float32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def _tol(dtype):
    return (2e-2, 2e-2) if dtype == torch.bfloat16 else (3e-5, 3e-5)


def _dev(t):
    return t.to(DEV) if t is not None else None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W", [40, 46, 256, 1000, 4500])
def test_branch_rmsnorm_add(dtype, W):
    T = 5
    x = _rand(T, W, seed=1) + 0.3
    a = _rand(T, W, dtype=dtype, seed=2, scale=3.0)
    b = _rand(T, W + 8, dtype=dtype, seed=3)[:, 4:4 + W]       # a strided view
    a32 = _rand(T, W, seed=4, scale=2.0)                       # fp32 branch
    wn = (1.0 + _rand(W, seed=5, scale=0.2)).to(dtype)
    rt, at = _tol(dtype)

    def both(x_in, y1, y2, ca, cb, keep=True):
        xr = x_in.clone() if x_in is not None else None
        wx, wh = ref.branch_rmsnorm_add(xr, y1, y2, ca, cb, wn, 1e-5, dtype, keep)
        xg = x_in.to(DEV) if x_in is not None else None
        gx, gh = ops.branch_rmsnorm_add(xg, _dev(y1), _dev(y2), ca, cb, _dev(wn),
                                        1e-5, dtype, keep)
        if keep:
            assert gx.dtype == torch.float32
            if x_in is not None:
                assert gx is xg
            torch.testing.assert_close(gx.cpu(), wx, rtol=3e-6, atol=3e-6)
        else:
            assert gx is None
            if x_in is not None:
                assert torch.equal(xg.cpu(), x_in)
        assert gh.dtype == dtype
        torch.testing.assert_close(gh.float().cpu(), wh.float(), rtol=rt, atol=at)

    both(x, a, b, 0.6, 1.7)            # two branches, one strided
    both(x, a32 if dtype == torch.bfloat16 else a, None, 1.0, 0.0)   # fp32 branch
    both(None, a, None, 1.0, 0.0)      # a stream that starts here
    both(None, x.clone(), None, 1.0, 0.0, keep=False)   # the norm alone, fp32 in


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T,I", [(3, 5), (7, 96), (33, 1024)])
def test_clamped_glu(dtype, T, I):
    x = _rand(T, 2 * I + 8, dtype=dtype, seed=6, scale=2.0)
    for view in (x[:, :2 * I].contiguous(), x[:, 4:4 + 2 * I], x[:, 1:1 + 2 * I]):
        want = ref.clamped_glu(view, 1.5)
        got = ops.clamped_glu(view.to(DEV), 1.5)
        rt, at = _tol(dtype)
        torch.testing.assert_close(got.float().cpu(), want.float(), rtol=rt, atol=at)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("width", [1, 33, 200, 700])
@pytest.mark.parametrize("lens", [[37, 20, 1], [700, 333, 1]])
def test_mingru_scan(dtype, width, lens):
    # three sequences in one packed step: a fresh one, a continued one, a
    # single token (short steps run token-serial, long ones in chunks side by
    # side); then single-token rows (decode); slots out of order
    pos0, slots = [0, 11, 5], [4, 0, 2]
    T = sum(lens)
    zug = _rand(T, 3 * width + 6, dtype=dtype, seed=7, scale=2.0)[:, 3:3 + 3 * width]
    zb, ub = _rand(width, seed=8), _rand(width, seed=9, scale=0.5)
    state = _rand(6, width, seed=10)
    cu = torch.tensor([0, lens[0], lens[0] + lens[1], T], dtype=torch.int32)
    positions = torch.cat([torch.arange(p, p + n) for p, n in zip(pos0, lens)]).int()
    sl = torch.tensor(slots, dtype=torch.int64)
    rt, at = _tol(dtype)
    sr, sg = state.clone(), state.to(DEV)
    want = ref.mingru_scan(zug, zb, ub, sr, sl, cu, positions, dtype)
    got = ops.mingru_scan(zug.to(DEV), zb.to(DEV), ub.to(DEV), sg, sl.to(DEV),
                          cu.to(DEV), positions.to(DEV), dtype)
    torch.testing.assert_close(got.float().cpu(), want.float(), rtol=rt, atol=at)
    torch.testing.assert_close(sg.cpu(), sr, rtol=2e-5, atol=2e-5)
    assert torch.equal(sg.cpu()[[1, 3, 5]], state[[1, 3, 5]])
    # decode rows
    z1 = zug[:3]
    p1 = torch.tensor([58, 0, 7], dtype=torch.int32)
    want = ref.mingru_scan(z1, zb, ub, sr, sl, None, p1, dtype)
    got = ops.mingru_scan(z1.to(DEV), zb.to(DEV), ub.to(DEV), sg, sl.to(DEV),
                          None, p1.to(DEV), dtype)
    torch.testing.assert_close(got.float().cpu(), want.float(), rtol=rt, atol=at)
    torch.testing.assert_close(sg.cpu(), sr, rtol=1e-5, atol=1e-5)


class _Paged:
    """A paged cache with shuffled pages for sequences of given lengths."""

    def __init__(self, lens, width, bs, dtype, seed=0):
        pages = [(n + bs - 1) // bs for n in lens]
        total = sum(pages) + 3
        perm = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
        self.bs = bs
        self.tables, at = [], 0
        for n in pages:
            self.tables.append(perm[at:at + n])
            at += n
        self.cache = torch.full((total, bs, width), 3.0, dtype=dtype)
        self.bt = torch.zeros(len(lens), max(pages), dtype=torch.int32)
        for i, t in enumerate(self.tables):
            self.bt[i, :len(t)] = torch.tensor(t, dtype=torch.int32)

    def slots(self, seq, positions):
        t = torch.tensor(self.tables[seq])
        p = torch.as_tensor(positions)
        return t[p // self.bs] * self.bs + p % self.bs


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,G,d,dv,rot", [(6, 2, 12, 20, 8), (8, 2, 96, 80, 32),
                                          (4, 4, 16, 8, 16), (3, 1, 24, 24, 0),
                                          (2, 1, 136, 264, 100), (50, 2, 256, 8, 64)])
def test_qk_norm_rotation_store(dtype, H, G, d, dv, rot):
    """Rows that are staged in LDS by 16-byte loads (widths in multiples of
    8), by scalar loads (12 / 20), and rows too wide to stage (50 heads of
    256)."""
    T, bs = 9, 4
    q = _rand(T, H * d + 8, dtype=dtype, seed=11)[:, 8:]
    k = _rand(T, G * d, dtype=dtype, seed=12, scale=3.0)
    v = _rand(T, G * dv, dtype=dtype, seed=13)
    wq, wk = 1.0 + _rand(d, seed=14, scale=0.3), 1.0 + _rand(d, seed=15, scale=0.3)
    freq, mult = (None, 1.0)
    if rot:
        freq, mult = yarn_ramp_frequencies(rot, 500.0, 4.0, 64, 8.0, 1.0)
    pg = _Paged([1200], G * d + G * dv, bs, dtype, seed=1)
    positions = torch.tensor([0, 1, 2, 3, 500, 501, 1100, 1101, 1102], dtype=torch.int32)
    slots = pg.slots(0, positions.long())
    slots[4] = -1                               # a pad row stores nothing
    cr, cg = pg.cache.clone(), pg.cache.to(DEV)
    want = ref.qkv_store(q, k, v, positions, slots, cr, d, 1e-5, 0.0, 0, wq, wk,
                         freq, mult, rot)
    got = ops.qkv_store(q.to(DEV), k.to(DEV), v.to(DEV), positions.to(DEV),
                        slots.to(DEV), cg, d, 1e-5, 0.0, 0, wq.to(DEV), wk.to(DEV),
                        _dev(freq), mult, rot)
    # angles of about a thousand radians in fp32: 1e-4 of absolute room
    torch.testing.assert_close(got.cpu(), want, rtol=1e-4, atol=3e-4)
    rt, at = _tol(dtype)
    torch.testing.assert_close(cg.float().cpu(), cr.float(), rtol=rt, atol=max(at, 3e-4))
    assert torch.all(cg.cpu().view(-1, cr.shape[-1])[pg.slots(0, [500])] == 3.0)


def _attention_case(dtype, H, G, d, dv, lens, new, bs, seed):
    """Sequences of `lens` cached tokens of which the last `new` are this
    step's queries. Returns the operands on the CPU."""
    E = G * d + G * dv
    pg = _Paged(lens, E, bs, dtype, seed)
    for b, n in enumerate(lens):
        rows = _rand(n, E, dtype=dtype, seed=seed + 10 + b)
        pg.cache.view(-1, E)[pg.slots(b, torch.arange(n))] = rows
    T = sum(new)
    q = _rand(T, H * d, seed=seed + 1, scale=1.5)
    token_seq = torch.cat([torch.full((m,), b) for b, m in enumerate(new)]).int()
    positions = torch.cat([torch.arange(n - m, n) for n, m in zip(lens, new)]).int()
    bounds = torch.tensor([0] + list(torch.tensor(new).cumsum(0)), dtype=torch.int32)
    bias = _rand(H, seed=seed + 2) - 3.0
    gate = _rand(T, H + 3, dtype=dtype, seed=seed + 3, scale=2.0)[:, 2:2 + H]
    return pg, q, token_seq, positions, bounds, bias, gate


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,G,d,dv", [(6, 2, 12, 20), (8, 2, 96, 80), (4, 4, 16, 8),
                                      (5, 1, 40, 72), (3, 3, 128, 256), (2, 1, 136, 24)])
def test_sigmoid_attention_prompt_portions(dtype, H, G, d, dv):
    """Portions of several sequences in one step (the matrix-core kernel where
    the widths allow it, the per-token kernel elsewhere), queries that start
    in the middle of a page and of a 32-token tile."""
    lens, new, bs = [150, 37, 1, 70], [150, 5, 1, 33], 8
    pg, q, token_seq, positions, bounds, bias, gate = _attention_case(
        dtype, H, G, d, dv, lens, new, bs, 20)
    args = (H, G, 1, d, dv, 0, 0, 0.11, 0.0, 0.0, None, 1.0, dtype)
    want = ref.row_attention(q, pg.cache, None, pg.bt, token_seq, positions, *args,
                             head_bias=bias, gate=gate)
    got = ops.row_attention(q.to(DEV), pg.cache.to(DEV), None, pg.bt.to(DEV),
                            token_seq.to(DEV), positions.to(DEV), *args,
                            max_seq_len=max(lens), query_bounds=bounds.to(DEV),
                            head_bias=bias.to(DEV), gate=gate.to(DEV))
    rt, at = _tol(dtype)
    torch.testing.assert_close(got.float().cpu(), want.float(), rtol=rt, atol=at * 3)
    # the per-token kernel on the same step (no token bounds given)
    got = ops.row_attention(q.to(DEV), pg.cache.to(DEV), None, pg.bt.to(DEV),
                            token_seq.to(DEV), positions.to(DEV), *args,
                            max_seq_len=max(lens), head_bias=bias.to(DEV),
                            gate=gate.to(DEV))
    torch.testing.assert_close(got.float().cpu(), want.float(), rtol=rt, atol=at * 3)
    # no gate, and the softmax path through the same kernels is untouched
    for kw in ({"head_bias": bias}, {"gate": gate}, {}):
        want = ref.row_attention(q, pg.cache, None, pg.bt, token_seq, positions, *args, **kw)
        got = ops.row_attention(q.to(DEV), pg.cache.to(DEV), None, pg.bt.to(DEV),
                                token_seq.to(DEV), positions.to(DEV), *args,
                                max_seq_len=max(lens), query_bounds=bounds.to(DEV),
                                **{k: v.to(DEV) for k, v in kw.items()})
        torch.testing.assert_close(got.float().cpu(), want.float(), rtol=rt, atol=at * 3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,G,d,dv", [(6, 2, 12, 20), (8, 2, 96, 80), (3, 3, 128, 256)])
def test_sigmoid_attention_decode_rows_split_keys(dtype, H, G, d, dv):
    """Single-token rows over long contexts: the key list is split over
    several workgroups and the shares' sums add up."""
    lens, bs = [1500, 1, 257, 64], 32
    pg, q, _, positions, _, bias, gate = _attention_case(
        dtype, H, G, d, dv, lens, [1, 1, 1, 1], bs, 30)
    args = (H, G, 1, d, dv, 0, 0, 0.08, 0.0, 0.0, None, 1.0, dtype)
    want = ref.row_attention(q, pg.cache, None, pg.bt, None, positions, *args,
                             head_bias=bias, gate=gate)
    got = ops.row_attention(q.to(DEV), pg.cache.to(DEV), None, pg.bt.to(DEV), None,
                            positions.to(DEV), *args, max_seq_len=max(lens),
                            head_bias=bias.to(DEV), gate=gate.to(DEV))
    rt, at = _tol(dtype)
    torch.testing.assert_close(got.float().cpu(), want.float(), rtol=rt, atol=at * 3)


@pytest.mark.parametrize("I,top", [(96, 1), (64, 2), (160, 3)])
def test_grouped_experts_weight_on_input(I, top):
    """The grouped-GEMM expert kernels (bf16) with the routing weight applied
    to the expert's input, on expert widths that are multiples of 32 but not
    of 64, against a per-expert loop in fp32."""
    T, W, E, L = 50, 64, 5, 1.5
    x = _rand(T, W, dtype=torch.bfloat16, seed=40, scale=2.0)
    gu = _rand(E, 2 * I, W, dtype=torch.bfloat16, seed=41, scale=0.3)
    dn = _rand(E, W, I, dtype=torch.bfloat16, seed=42, scale=0.2)
    g = torch.Generator().manual_seed(43)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)])
    wts = torch.rand(T, top, generator=g) * 0.9 + 0.05
    for on_input in (True, False):
        want = torch.zeros(T, W, dtype=torch.float64)
        for t in range(T):
            for j in range(top):
                e, wt = int(ids[t, j]), float(wts[t, j])
                xin = x[t].double() * (wt if on_input else 1.0)
                h = gu[e].double() @ xin
                a = ref.clamped_glu(h[None].float(), L)[0].to(torch.bfloat16).double()
                want[t] += (dn[e].double() @ a) * (1.0 if on_input else wt)
        got = ops.fused_moe_forward(x.to(DEV), gu.to(DEV), dn.to(DEV), ids.to(DEV),
                                    wts.to(DEV), limit=L, weight_on_input=on_input)
        torch.testing.assert_close(got.double().cpu(), want, rtol=3e-2, atol=3e-2)
