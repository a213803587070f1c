"""The Dogidra mechanisms one at a time.

CPU part: the reference ops against the float64 oracle's per-mechanism
functions (tests/oracle_dogidra.py), fed in ragged portions through paged
caches and state slots that held another sequence before. GPU part (marked
gpu): every new or extended HIP kernel against the PyTorch fp32 reference of
the same op over odd sizes, ragged batches, single tokens and used slots."""

import math

import pytest
import torch

import oracle_dogidra as O
from production_stack_amd import ops
from production_stack_amd.ops import reference as R

F64 = torch.float64


def rnd(g, *shape, scale=1.0):
    return torch.randn(*shape, generator=g) * scale


def segments(lens, pos0s, slots):
    rows, t0 = [], 0
    for n, p, s in zip(lens, pos0s, slots):
        rows.append([t0, n, p, s])
        t0 += n
    return torch.tensor(rows, dtype=torch.int32), t0


def relerr(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


# ---------------------------------------------------------------------------
# paged attention helper: one sequence through attn_prep / pool_append /
# talk_attention in portions
# ---------------------------------------------------------------------------
class PagedAttention:
    def __init__(self, m, Wq, Wk, Wv, qn, kn, eps, bs=8, pages=None,
                 device="cpu", dtype=torch.float32, n_pages=64, seed=0):
        self.m, self.eps, self.bs = m, eps, bs
        self.dev, self.dt = device, dtype
        self.H, self.G = m["heads"], m.get("kv_heads", m["heads"])
        self.D, self.DV = m["dim"], m.get("vdim", m["dim"])
        self.W = [w.to(dtype).to(device) for w in (Wq, Wk, Wv)]
        self.qn, self.kn = qn.float().to(device), kn.float().to(device)
        mask = m.get("mask") or {}
        self.window = int(mask.get("size", 0))
        self.P = int(mask.get("pool", 0))
        rot = m.get("rot") or {}
        self.rot_dims = int(rot.get("dims", 0))
        sc = rot.get("scaling")
        self.cs = None
        if self.rot_dims:
            self.cs = ops.rope_table(
                4096, self.rot_dims, rot["base"], device, 1.0,
                (sc["factor"], sc["original"], sc["fast"], sc["slow"])
                if sc else None)
        g = torch.Generator().manual_seed(seed)
        # caches start full of another owner's numbers
        def mk(r, w):
            return (torch.randn(n_pages, self.G, r, w, generator=g)
                    * 3).to(dtype).to(device)

        self.kc, self.vc = mk(bs, self.D), mk(bs, self.DV)
        self.pool = None
        if self.P:
            pr = (bs + self.P - 1) // self.P
            self.pool = (mk(pr, self.D), mk(pr, self.DV), self.P)
        # scattered pages
        self.table = (pages if pages is not None else
                      torch.randperm(n_pages, generator=g)).to(torch.int32)
        self.at = 0

    def step(self, h):
        n = h.shape[0]
        dev, bs = self.dev, self.bs
        h = h.to(self.dt).to(dev)
        q, k, v = (h @ w.t() for w in self.W)
        pos = torch.arange(self.at, self.at + n)
        slots = (self.table[(pos // bs)].long() * bs + pos % bs).to(dev)
        pos32 = pos.to(torch.int32).to(dev)
        ops.attn_prep(q, k, v, self.qn, self.kn, self.eps, None, None,
                      self.kc, self.vc, slots, self.H, cos_sin=self.cs,
                      positions=pos32 if self.cs is not None else None,
                      rot_dims=self.rot_dims, norm_all=True, half=True)
        tables = self.table[None].contiguous().to(dev)
        sr = torch.tensor([[0, n, self.at, 0]], dtype=torch.int32).to(dev)
        if self.pool:
            ops.pool_append(self.kc, self.vc, self.pool[0], self.pool[1],
                            tables, sr, self.P, n)
        seq = torch.zeros(n, dtype=torch.int32, device=dev)
        o = ops.talk_attention(
            q, self.kc, self.vc, tables, seq, pos32, self.m["scale"], self.H,
            window=self.window, softcap=float(self.m.get("softcap") or 0),
            pool=self.pool, variant=0 if n > 1 else 3)
        self.at += n
        return o.float().cpu()


def attention_case(g, heads=4, kv_heads=2, dim=16, vdim=8, size=11, pool=3,
                   rot_dims=8, scaling=True, softcap=20.0, width=32):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": 0.3, "softcap": softcap}
    if size:
        m["mask"] = {"size": size}
        if pool:
            m["mask"]["pool"] = pool
    if rot_dims:
        m["rot"] = {"base": 100.0, "dims": rot_dims}
        if scaling:
            m["rot"]["scaling"] = {"factor": 3.0, "original": 32,
                                   "fast": 4.0, "slow": 1.0}
    W = {"q": rnd(g, heads * dim, width, scale=width ** -0.5),
         "k": rnd(g, kv_heads * dim, width, scale=width ** -0.5),
         "v": rnd(g, kv_heads * vdim, width, scale=width ** -0.5),
         "q.norm": 1 + 0.3 * rnd(g, heads * dim),
         "k.norm": 1 + 0.3 * rnd(g, kv_heads * dim),
         "o": torch.eye(heads * vdim)}
    return m, W


def oracle_attention(m, W, h, eps):
    return O.pooled_window_attention(W, "", m, h.to(F64), eps)


@pytest.mark.parametrize("case", [
    dict(),                                        # everything on
    dict(pool=1),                                  # blocks of one position
    dict(pool=16, size=5),                         # blocks longer than a page
    dict(pool=0),                                  # window only
    dict(size=0, pool=0),                          # plain causal
    dict(rot_dims=16),                             # rotary over the whole head
    dict(rot_dims=0),                              # no rotary code
    dict(scaling=False, softcap=0.0),
    dict(heads=3, kv_heads=3, dim=8, vdim=16, size=1, pool=2),
    dict(heads=6, kv_heads=1, size=8, pool=8),
])
@pytest.mark.parametrize("cuts", [[70], [1] * 40, [2, 3, 17, 1, 1, 30, 2, 9]])
def test_attention_portions_vs_oracle(case, cuts):
    g = torch.Generator().manual_seed(5)
    m, W = attention_case(g, **case)
    T = sum(cuts)
    h = rnd(g, T, 32)
    want = oracle_attention(m, W, h, 1e-5)
    pa = PagedAttention(m, W["q"], W["k"], W["v"], W["q.norm"], W["k.norm"],
                        1e-5)
    got, at = [], 0
    for n in cuts:
        got.append(pa.step(h[at:at + n]))
        at += n
    assert relerr(torch.cat(got), want) < 2e-5


def test_pooled_block_edges_stand_out():
    """One far key block is made to dominate: the query must see it exactly
    from the position at which the whole block has left the window."""
    g = torch.Generator().manual_seed(6)
    m, W = attention_case(g, heads=2, kv_heads=1, dim=8, vdim=8, size=6,
                          pool=4, rot_dims=0, softcap=0.0, width=8)
    m["scale"] = 1.0
    W["q"] = torch.cat([torch.eye(8)] * 2)
    W["k"], W["v"] = torch.eye(8), torch.eye(8)
    W["q.norm"] = torch.ones(16)
    W["k.norm"] = torch.ones(8)
    T = 40
    h = rnd(g, T, 8, scale=0.05)
    # block 2 (positions 8..11) gets a large shared key/value direction;
    # unit-rms norm keeps the rest small next to it
    h[8:12, 0] += 6.0
    h[12:, 0] += 2.0
    want = oracle_attention(m, W, h, 1e-5)
    pa = PagedAttention(m, W["q"], W["k"], W["v"], W["q.norm"], W["k.norm"],
                        1e-5, bs=4)
    got = torch.cat([pa.step(h[:13]), pa.step(h[13:15])]
                    + [pa.step(h[t:t + 1]) for t in range(15, T)])
    assert relerr(got, want) < 2e-5
    # positions 12..16 still hold part of the block in the window; at 17 the
    # window starts at 12 and block 2 is seen pooled (11 <= 17 - 6)
    col = want[:, 0]
    assert col[16] > 0.5 and col[17] > 0.5 and col[16] != col[17]


@pytest.mark.parametrize("K", [1, 2, 4, 7])
@pytest.mark.parametrize("cuts", [[23], [1] * 9, [2, 5, 1, 1, 3, 11]])
def test_layer_norm_conv_portions(K, cuts):
    g = torch.Generator().manual_seed(K)
    W_ = 24
    T = sum(cuts)
    x = rnd(g, T, W_, scale=2.0) + 0.7
    d0, d1 = rnd(g, T, W_), rnd(g, T, W_)
    w, b = 1 + 0.2 * rnd(g, W_), 0.3 * rnd(g, W_)
    cw = rnd(g, W_, K, scale=0.5)
    xs = x.to(F64) + 0.8 * d0.to(F64) + 0.5 * d1.to(F64)
    want = O.input_conv(O.layer_norm(xs, w, b, 1e-5), cw)
    state = torch.full((3, K - 1, W_), 9.0)
    got, at = [], 0
    x32 = x.clone()
    for n in cuts:
        sr = torch.tensor([[0, n, at, 2]], dtype=torch.int32)
        part = x32[at:at + n].clone()
        got.append(ops.add_layer_norm_conv32(
            part, [d0[at:at + n], d1[at:at + n]], [0.8, 0.5], w, b, 1e-5,
            cw, state, sr, torch.float32))
        assert relerr(part, xs[at:at + n]) < 1e-6
        at += n
    assert relerr(torch.cat(got), want) < 1e-5


@pytest.mark.parametrize("cuts", [[50], [1] * 12, [2, 1, 9, 1, 30]])
def test_mingru_portions(cuts):
    g = torch.Generator().manual_seed(3)
    C, width = 20, 12
    T = sum(cuts)
    h = rnd(g, T, width)
    W = {"z": rnd(g, C, width, scale=0.5), "z.b": rnd(g, C),
         "x": rnd(g, C, width), "x.b": rnd(g, C),
         "g": rnd(g, C, width, scale=0.5), "o": torch.eye(C)}
    want = O.min_gru(W, "", h.to(F64))
    state = torch.full((2, C), -4.0)
    got, at = [], 0
    for n in cuts:
        hh = h[at:at + n]
        sr = torch.tensor([[0, n, at, 1]], dtype=torch.int32)
        got.append(ops.mingru_scan(hh @ W["z"].t(), hh @ W["x"].t(),
                                   hh @ W["g"].t(), W["z.b"], W["x.b"],
                                   state, sr))
        at += n
    assert relerr(torch.cat(got), want) < 1e-5
    # both branches of the candidate were exercised
    u = h @ W["x"].t() + W["x.b"]
    assert (u >= 0).any() and (u < 0).any()


def test_router_choice_by_corrected_score_weights_without():
    g = torch.Generator().manual_seed(4)
    T, W_, E, top = 40, 16, 7, 3
    x = rnd(g, T, W_)
    rw = rnd(g, E, W_, scale=0.5)
    corr = torch.tensor([0.0, 0.9, -0.9, 0.0, 0.4, 0.0, -0.2])
    wts, sel, dense = ops.moe_route(x, rw, top, "sigmoid", False, corr, 2.5,
                                    0.0)
    s = torch.sigmoid(x.double() @ rw.double().t())
    want_sel = torch.topk(s + corr.double(), top, dim=-1).indices
    assert torch.equal(sel.sort(-1).values, want_sel.sort(-1).values)
    plain_sel = torch.topk(s, top, dim=-1).indices
    assert not torch.equal(plain_sel.sort(-1).values,
                           want_sel.sort(-1).values)
    assert relerr(wts, s.gather(-1, sel) * 2.5) < 1e-6
    assert relerr(dense.sum(-1), wts.sum(-1)) < 1e-6


def test_frequency_blend_matches_oracle():
    for dims, base, sc in [(8, 100.0, (4.0, 32, 4.0, 1.0)),
                           (64, 50000.0, (8.0, 1024, 32.0, 1.0)),
                           (6, 10.0, (2.0, 16, 2.0, 0.5)),
                           (16, 1000.0, None)]:
        rot = {"dims": dims, "base": base}
        if sc:
            rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"),
                                      sc))
        f, mag = O.yarn_frequencies(rot)
        tab = R.rope_table(50, dims, base, None, 1.0, sc)
        a = torch.arange(50, dtype=F64)[:, None] * f
        assert relerr(tab[..., 0], torch.cos(a) * mag) < 1e-6
        assert relerr(tab[..., 1], torch.sin(a) * mag) < 1e-6
        if sc:
            assert mag == pytest.approx(0.1 * math.log(sc[0]) + 1)


# ---------------------------------------------------------------------------
# GPU: kernels against the reference ops
# ---------------------------------------------------------------------------
def gtol(dtype):
    return 2e-2 if dtype == torch.bfloat16 else 3e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("K", [0, 1, 2, 4, 8, 11])
@pytest.mark.parametrize("W_", [328, 330])
def test_gpu_layer_norm_conv(dtype, K, W_):
    """Row widths with and without whole 16-byte vectors; tap counts with
    their own instantiation (up to 8) and above."""
    g = torch.Generator().manual_seed(10 + K)
    lens, pos0, slots = [70, 1, 3, 130, 1], [0, 5, 2, 64, 0], [3, 0, 2, 1, 4]
    sr, T = segments(lens, pos0, slots)
    x = rnd(g, T, W_, scale=2.0) + 0.5
    w, b = 1 + 0.2 * rnd(g, W_), 0.3 * rnd(g, W_)
    cw = rnd(g, W_, K, scale=0.5) if K else None
    for deltas, ddt in (([], dtype), ([rnd(g, T, W_)], torch.float32),
                        ([rnd(g, T, W_), rnd(g, T, W_)], dtype)):
        deltas = [d.to(ddt) for d in deltas]
        scales = [0.8, 0.5][:len(deltas)]
        st = rnd(g, 5, max(K - 1, 0), W_) if K else None
        x_ref, st_ref = x.clone(), (st.clone() if K else None)
        want = R.add_layer_norm_conv32(x_ref, deltas, scales, w, b, 1e-5, cw,
                                       st_ref, sr, dtype)
        x_gpu, st_gpu = x.cuda(), (st.cuda() if K else None)
        got = ops.add_layer_norm_conv32(
            x_gpu, [d.cuda() for d in deltas], scales, w.cuda(), b.cuda(),
            1e-5, cw.cuda() if K else None, st_gpu, sr.cuda(), dtype)
        assert got.dtype == dtype
        assert relerr(x_gpu, x_ref) < 1e-6
        assert relerr(got, want) < gtol(dtype)
        if K > 1:
            assert relerr(st_gpu, st_ref) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pad", [5, 0])
def test_gpu_mingru_scan(dtype, pad):
    """Ragged segments above and below the tile length; row strides and
    offsets with (pad 0) and without whole 16-byte vectors."""
    g = torch.Generator().manual_seed(11)
    C = 200
    lens, pos0, slots = [90, 1, 2, 300, 1], [0, 7, 0, 16, 3], [2, 4, 0, 1, 3]
    sr, T = segments(lens, pos0, slots)
    big = rnd(g, T, 3 * C + pad).to(dtype)
    z, u, gate = big[:, :C], big[:, C:2 * C], big[:, 2 * C + pad:]
    zb, ub = rnd(g, C), rnd(g, C)
    st = rnd(g, 5, C)
    st_ref = st.clone()
    want = R.mingru_scan(z, u, gate, zb, ub, st_ref, sr, dtype)
    st_gpu = st.cuda()
    bg = big.cuda()
    got = ops.mingru_scan(bg[:, :C], bg[:, C:2 * C], bg[:, 2 * C + pad:],
                          zb.cuda(), ub.cuda(), st_gpu, sr.cuda())
    assert relerr(got, want) < gtol(dtype)
    assert relerr(st_gpu, st_ref) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_plain_activation_and_router(dtype):
    g = torch.Generator().manual_seed(12)
    x = rnd(g, 37, 136).to(dtype)
    want = R.gated_act(x, None, "relu2", 0.0, dtype)
    got = ops.gated_act(x.cuda(), None, "relu2")
    assert relerr(got, want) < 1e-6
    up = rnd(g, 37, 136).to(dtype)
    want = R.gated_act(x, up, "relu2", 0.0, dtype)
    assert relerr(ops.gated_act(x.cuda(), up.cuda(), "relu2"), want) < 1e-2
    rw = rnd(g, 9, 136, scale=0.2).to(dtype)
    corr = 0.5 * rnd(g, 9)
    w0, s0, d0 = R.moe_route(x, rw, 4, "sigmoid", False, corr, 2.5, 0.0)
    w1, s1, d1 = ops.moe_route(x.cuda(), rw.cuda(), 4, "sigmoid", False,
                               corr.cuda(), 2.5, 0.0)
    assert torch.equal(s1.cpu().sort(-1).values, s0.sort(-1).values)
    assert relerr(d1, d0) < 1e-5
    y = rnd(g, 5, 37, 136).to(dtype)
    ys = rnd(g, 37, 136).to(dtype)
    want = R.moe_combine(y, d0[:, :5].contiguous(), x, 5, ys, None)
    got = ops.moe_combine(y.cuda(), d0[:, :5].contiguous().cuda(), x.cuda(),
                          5, ys.cuda(), None)
    assert relerr(got, want) < 1e-5


ATT_CASES = [
    dict(),
    dict(pool=1),
    dict(pool=16, size=5),
    dict(heads=16, kv_heads=2, dim=64, vdim=48, size=40, pool=8,
         rot_dims=32, width=64),
    dict(heads=4, kv_heads=2, dim=128, vdim=128, size=24, pool=8,
         rot_dims=128, width=64),
    dict(heads=3, kv_heads=3, dim=8, vdim=16, size=1, pool=2),
    # six query heads on one key/value head: outside the matrix-core
    # kernel's shapes, so bfloat16 takes the vector kernels too
    dict(heads=6, kv_heads=1, size=8, pool=8),
    dict(pool=0),
    dict(size=0, pool=0, rot_dims=0),
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", ATT_CASES)
def test_gpu_attention_portions(dtype, case):
    """attn_prep (whole-projection norms, half-split rotary pairs),
    pool_append and the attention kernels (prompt and single-token forms)
    against the same ops on the CPU, through scattered pages that held other
    numbers."""
    g = torch.Generator().manual_seed(13)
    m, W = attention_case(g, **case)
    width = W["q"].shape[1]
    cuts = [37, 1, 1, 2, 50, 1, 1, 1, 26, 1]
    h = rnd(g, sum(cuts), width)
    kw = dict(bs=16, n_pages=24, seed=1)
    ref = PagedAttention(m, W["q"], W["k"], W["v"], W["q.norm"], W["k.norm"],
                         1e-5, dtype=dtype, **kw)
    dev = PagedAttention(m, W["q"], W["k"], W["v"], W["q.norm"], W["k.norm"],
                         1e-5, device="cuda", dtype=dtype, **kw)
    at = 0
    for n in cuts:
        want = ref.step(h[at:at + n])
        got = dev.step(h[at:at + n])
        assert relerr(got, want) < gtol(dtype), (at, n)
        at += n
    assert relerr(dev.kc, ref.kc) < gtol(dtype) / 4
    if ref.pool:
        assert relerr(dev.pool[0], ref.pool[0]) < gtol(dtype) / 4
        assert relerr(dev.pool[1], ref.pool[1]) < gtol(dtype) / 4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_attention_ragged_batch(dtype):
    """Several sequences of one step (two prompt portions, three single
    tokens) against each of them alone."""
    g = torch.Generator().manual_seed(14)
    m, W = attention_case(g, heads=8, kv_heads=2, dim=32, vdim=16, size=20,
                          pool=4, rot_dims=16, width=48)
    H, G, D, DV = 8, 2, 32, 16
    bs, n_pages = 16, 40
    ctx = [0, 33, 70, 5, 64]         # tokens already cached
    new = [45, 9, 1, 1, 1]
    hs = [rnd(g, c + n, 48) for c, n in zip(ctx, new)]
    want = []
    for h, c in zip(hs, ctx):
        pa = PagedAttention(m, W["q"], W["k"], W["v"], W["q.norm"],
                            W["k.norm"], 1e-5, bs=bs, dtype=dtype)
        if c:
            pa.step(h[:c])
        want.append(pa.step(h[c:]))
    # one batch on the GPU: contexts first (each alone), then one step
    pas = []
    perm = torch.randperm(n_pages, generator=g)
    for i, (h, c) in enumerate(zip(hs, ctx)):
        pa = PagedAttention(m, W["q"], W["k"], W["v"], W["q.norm"],
                            W["k.norm"], 1e-5, bs=bs, device="cuda",
                            dtype=dtype, pages=perm[8 * i:8 * i + 8],
                            n_pages=n_pages, seed=2)
        if i:
            pa.kc, pa.vc, pa.pool = pas[0].kc, pas[0].vc, pas[0].pool
        if c:
            pa.step(h[:c])
        pas.append(pa)
    p0 = pas[0]
    hcat = torch.cat([h[c:] for h, c in zip(hs, ctx)]).to(dtype).cuda()
    q, k, v = (hcat @ w.t() for w in p0.W)
    pos = torch.cat([torch.arange(c, c + n) for c, n in zip(ctx, new)])
    seq = torch.cat([torch.full((n,), i) for i, n in enumerate(new)])
    tables = torch.stack([pa.table for pa in pas]).contiguous()
    slots = (tables[seq, pos // bs].long() * bs + pos % bs).cuda()
    pos32, seq32 = pos.to(torch.int32).cuda(), seq.to(torch.int32).cuda()
    ops.attn_prep(q, k, v, p0.qn, p0.kn, 1e-5, None, None, p0.kc, p0.vc,
                  slots, H, cos_sin=p0.cs, positions=pos32, rot_dims=16,
                  norm_all=True, half=True)
    sr, T = segments(new, ctx, [0] * 5)
    ops.pool_append(p0.kc, p0.vc, p0.pool[0], p0.pool[1], tables.cuda(),
                    sr.cuda(), 4, T)
    npt = 54
    out = torch.empty(T, H * DV, dtype=dtype, device="cuda")
    for a, b, variant in ((0, npt, 0), (npt, T, 3)):
        ops.talk_attention(q[a:b], p0.kc, p0.vc, tables.cuda(), seq32[a:b],
                           pos32[a:b], m["scale"], H, window=20,
                           softcap=20.0, pool=p0.pool, out=out[a:b],
                           variant=variant)
    assert relerr(out, torch.cat(want)) < gtol(dtype)
