"""Sosepel on the GPU against the plain implementation: every mechanism alone through its
kernel, then whole models (four small configurations, in 32-bit and in bfloat16) layer by
layer, whole, decoded token by token, in portions down to two tokens, in mixed batches with
pages and state slots that are given back and used again, from a captured graph, generated
greedily through the scheduler, through the command line and the trace replay program, and
configurations drawn at random. bfloat16 is compared
with the plain implementation on the bfloat16-rounded weights. Prompts are chosen so that no
routing decision of the plain implementation is a close call."""
import json
import math
import os
import random
import subprocess
import sys

import pytest
import torch

import plain_sosepel
import sosepel_cases
import util

pytestmark = pytest.mark.gpu
DEV = "cuda"
STD = 0.25


@pytest.fixture(scope="module")
def ops():
    from ninfer_amd.kernels import load_ops
    return load_ops()


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return ((got - want).norm() / want.norm().clamp_min(1e-30)).item()


def _steps(ops, dtype, lengths_by_step, slots):
    """StepContexts for requests that go on from step to step: lengths_by_step[i][r] rows of
    request r in step i (0: left out)."""
    done = [0] * len(slots)
    for lengths in lengths_by_step:
        seqs, who = [], []
        for r, n in enumerate(lengths):
            if n:
                seqs.append((done[r], n))
                who.append(r)
        ctx = util.make_context(ops, dtype, seqs)
        ctx.seq_slots = torch.tensor([slots[r] for r in who], dtype=torch.int32, device=DEV)
        yield ctx, who, [done[r] for r in who], [lengths[r] for r in who]
        for r, n in enumerate(lengths):
            done[r] += n


# ---- mechanisms alone ------------------------------------------------------------------------

def _step_tokens(ctx, toks, who, starts, counts):
    ctx.tokens = torch.tensor(sum((toks[r][s:s + n] for r, s, n in zip(who, starts, counts)), []),
                              dtype=torch.int32, device=DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("buckets,mul_prev,mul_cur,scale", [(37, 31, 5, 1.5), (1, 1, 1, 1.0), (0, 0, 0, 2.0)])
def test_hashed_pairs_in_portions(ops, dtype, buckets, mul_prev, mul_cur, scale):
    """The pair table's row of a step's first token comes from the request's state, also when
    the step brings one token; a request's first token takes the table's last row; the state's
    column lies inside wider rows, and the requests hold slots 2 and 0. Without a table
    (buckets 0) only the scale is left."""
    torch.manual_seed(buckets)
    vocab, width, lens = 90, 40, [23, 9]
    toks = [util.random_tokens(n, vocab, 3 + n) for n in lens]
    table = torch.randn(vocab, width).to(dtype)
    cfg, w = {"embedding": {"scale": scale}}, {"embed": table.float()}
    pair = None
    if buckets:
        pair = torch.randn(buckets + 1, width).to(dtype)
        cfg["embedding"]["bigram"] = {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}
        w["bigram"] = pair.float()
    want = [plain_sosepel.embed(w, cfg, t) for t in toks]
    state_all = torch.zeros(3, 7, device=DEV)
    state = state_all[:, 3:4]
    steps = [[3, 0], [2, 2], [1, 1], [1, 1], [7, 2], [1, 0], [2, 3], [6, 0]]
    assert [sum(s[r] for s in steps) for r in range(2)] == lens
    got = [torch.zeros(n, width) for n in lens]
    for ctx, who, starts, counts in _steps(ops, dtype, steps, slots=[2, 0]):
        _step_tokens(ctx, toks, who, starts, counts)
        out = torch.empty(ctx.T, width, device=DEV)
        ops.embed_pairs(ctx, table.to(DEV), out, scale, None if pair is None else pair.to(DEV), buckets,
                        mul_prev, mul_cur, state if buckets else None)
        o = 0
        for r, s, n in zip(who, starts, counts):
            got[r][s:s + n] = out[o:o + n].cpu()
            o += n
    for g, wnt in zip(got, want):
        torch.testing.assert_close(g.double(), wnt, atol=1e-6, rtol=1e-6)
    assert state_all[1].abs().max() == 0 and state_all[:, :3].abs().max() == 0   # nobody else's
    assert state_all[:, 4:].abs().max() == 0


def test_pair_hash_of_large_numbers(ops):
    """Token ids, multipliers and buckets whose products pass 2^31: the row is that of the
    hash in integers of any size (a table whose row r holds the number r says which was read)."""
    buckets, mul_prev, mul_cur, vocab = 1000003, 65537, 257, 70000
    toks = [util.random_tokens(23, vocab, 5), util.random_tokens(9, vocab, 6)]
    assert max(p * mul_prev + c * mul_cur for t in toks for p, c in zip(t[:-1], t[1:])) > 2 ** 31
    big = torch.arange(buckets + 1, dtype=torch.float32)[:, None].expand(buckets + 1, 2).contiguous().to(DEV)
    zero = torch.zeros(vocab, 2, device=DEV)
    state = torch.zeros(3, 1, device=DEV)
    seen = {0: [], 1: []}
    for ctx, who, starts, counts in _steps(ops, torch.float32, [[5, 0], [1, 2], [17, 7]], [2, 0]):
        _step_tokens(ctx, toks, who, starts, counts)
        out = torch.empty(ctx.T, 2, device=DEV)
        ops.embed_pairs(ctx, zero, out, 1.0, big, buckets, mul_prev, mul_cur, state)
        o = 0
        for r, n in zip(who, counts):
            seen[r] += out[o:o + n, 0].cpu().tolist()
            o += n
    for r in (0, 1):
        assert seen[r] == [float(x) for x in plain_sosepel.pair_rows(toks[r], buckets, mul_prev, mul_cur)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [72, 256, 1100])
def test_scaled_sum_add(ops, dtype, width):
    from ninfer_amd.parts import PendingRows
    torch.manual_seed(width)
    t, k = 5, 3
    x = torch.randn(t, width)
    a, f = torch.randn(t, width).to(dtype), torch.randn(t, width).to(dtype)
    y, sh = torch.randn(t * k, width).to(dtype), torch.randn(t, width).to(dtype)
    wts, gate_wide = torch.rand(t, k), torch.randn(t, 4)
    s1, s2 = torch.randn(width), torch.randn(width)
    D = lambda v: v.double()
    moe = (D(wts)[:, :, None] * D(y).view(t, k, width)).sum(1) + torch.sigmoid(D(gate_wide[:, 2:3])) * D(sh)
    gw = gate_wide.to(DEV)
    for want, args in (
            (D(x) + D(a) * D(s1) + D(f) * D(s2), (a.to(DEV), s1.to(DEV), f.to(DEV), s2.to(DEV))),
            (D(x) + D(a) * D(s1), (a.to(DEV), s1.to(DEV), None, s2.to(DEV))),
            (D(x) + D(a) + D(f), (a.to(DEV), None, f.to(DEV), None)),
            (D(x) + D(a) * D(s1) + moe * D(s2),
             (a.to(DEV), s1.to(DEV), PendingRows(y.to(DEV), wts.to(DEV), sh.to(DEV), gw[:, 2]), s2.to(DEV))),
            (D(x) + D(a) + (D(wts)[:, :, None] * D(y).view(t, k, width)).sum(1),
             (a.to(DEV), None, PendingRows(y.to(DEV), wts.to(DEV)), None))):
        res = x.to(DEV)
        ops.scaled_sum_add(res, *args)
        torch.testing.assert_close(res.cpu().double(), want, atol=1e-5, rtol=1e-5)


def test_small_row_kernels(ops):
    torch.manual_seed(1)
    a, b = torch.randn(6, 50), torch.randn(6, 50)
    for dtype in (torch.float32, torch.bfloat16):
        out = torch.empty(6, 100, dtype=dtype, device=DEV)
        ops.concat_rows(a.to(DEV), b.to(DEV), out)
        assert torch.equal(out.cpu(), torch.cat([a, b], -1).to(dtype))
        x = (torch.randn(7, 33) * 3).to(dtype)
        y = x.to(DEV).clone()
        ops.relu_square(y)
        assert rel_err(y, torch.relu(x.double()) ** 2) < (1e-6 if dtype == torch.float32 else 4e-3)
    x = torch.randn(5, 77) * 20
    y = x.to(DEV).clone()
    ops.tanh_cap(y, 7.5)
    torch.testing.assert_close(y.cpu().double(), 7.5 * torch.tanh(x.double() / 7.5), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [1, 5, 20, 40, 70, 300])
def test_product_with_the_square_of_relu(ops, dtype, rows):
    """The activation runs in the product's epilogue, whichever kernel the row count picks."""
    torch.manual_seed(rows)
    for k, n in ((72, 100), (256, 512), (2048, 1408)):
        x, w = (torch.randn(rows, k) * 0.5).to(dtype), (torch.randn(n, k) * 0.1).to(dtype)
        want = torch.relu(x.double() @ w.double().T) ** 2
        out = torch.empty(rows, n, dtype=dtype, device=DEV)
        ops.linear(x.to(DEV), w.to(DEV), out, act="relu2")
        assert rel_err(out, want) < (1e-5 if dtype == torch.float32 else 6e-3)
        with ops.tuned(force_kernel=0):
            ops.force_generic = True
            try:
                ops.linear(x.to(DEV), w.to(DEV), out, act="relu2")
            finally:
                ops.force_generic = False
        assert rel_err(out, want) < (1e-5 if dtype == torch.float32 else 6e-3)


@pytest.mark.parametrize("experts,top,count,keep", [(6, 3, 3, 2), (16, 4, 2, 1), (9, 2, 3, 1), (4, 2, 4, 3),
                                                     (128, 6, 8, 3), (12, 5, 1, 1), (70, 2, 7, 2)])
def test_choice_limited_to_groups_by_their_two_best(ops, experts, top, count, keep):
    """Sigmoid scores, groups scored by the sum of their two largest, the choice among the kept
    groups' experts, weights divided by their sum: for few rows (one block routes them), for
    some dozens and for thousands (the kernels of many rows)."""
    for t in (3, 40, 2100):
        g = torch.Generator().manual_seed(experts * 7 + t)
        logits = torch.randn(t, experts + 2, generator=g) * 2
        r = {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}
        chosen, weights, margin = plain_sosepel.route(torch.sigmoid(logits[:, :experts].double()), r)
        ids = torch.empty(t, top, dtype=torch.int32, device=DEV)
        wts = torch.empty(t, top, dtype=torch.float32, device=DEV)
        ops.router_topk(logits.to(DEV), experts, top, True, ids, wts, score="sigmoid", n_group=count,
                        topk_group=keep, group_top=min(2, experts // count), renorm_eps=1e-20)
        clear = margin > 1e-5
        assert clear.float().mean() > 0.9
        # (the order among the chosen may differ where two of them score alike: by expert)
        got_ids, at = ids.cpu().long().sort(-1)
        want_ids, at2 = chosen.sort(-1)
        assert torch.equal(got_ids[clear], want_ids[clear])
        torch.testing.assert_close(wts.cpu().double().gather(1, at)[clear], weights.gather(1, at2)[clear],
                                   atol=1e-6, rtol=1e-5)


class _Paged:
    """A cache of keys and values for requests that go on from step to step, with pages dealt
    out of order, fed through the mixer's own kernels (write and attention)."""

    def __init__(self, ops, dtype, heads, kv_heads, dim, vdim, page_size, lens, seed):
        self.ops, self.dtype = ops, dtype
        self.H, self.G, self.d, self.vd, self.ps = heads, kv_heads, dim, vdim, page_size
        g = torch.Generator().manual_seed(seed)
        per = [-(-n // page_size) for n in lens]
        pages = sum(per) + 3
        perm = torch.randperm(pages, generator=g)
        self.table = torch.full((len(lens), max(per)), -1, dtype=torch.int32)
        at = 0
        for r, n in enumerate(per):
            self.table[r, :n] = perm[at:at + n]
            at += n
        nan = float("nan")   # what is not written is not to be read
        self.k = torch.full((pages, kv_heads, page_size, 2 * dim), nan, dtype=dtype, device=DEV)
        self.v = torch.full((pages, kv_heads, page_size, vdim), nan, dtype=dtype, device=DEV)
        width = (heads + kv_heads) * 2 * dim + kv_heads * vdim
        self.rows = [(torch.randn(n, width, generator=g)).to(dtype) for n in lens]

    def run(self, steps, m, lam, eps, force_plain=False):
        got = [torch.zeros(r.shape[0], self.H * self.vd) for r in self.rows]
        t = m.get("q_temp") or {"coef": 0.0, "every": 1}
        self.ops.force_generic = force_plain
        try:
            for ctx, who, starts, counts in _steps(self.ops, self.dtype, steps, list(range(len(self.rows)))):
                qkv = torch.cat([self.rows[r][s:s + n] for r, s, n in zip(who, starts, counts)]).to(DEV)
                out = torch.empty(ctx.T, self.H * self.vd, dtype=self.dtype, device=DEV)
                self.ops.diff_attention(qkv, self.k, self.v, self.table[who].contiguous().to(DEV), ctx, self.H,
                                        self.G, self.d, self.vd, self.ps, m["scale"], m.get("softcap", 0.0),
                                        t["coef"], t["every"], lam, eps, 1.0 - m["diff"], out)
                o = 0
                for r, s, n in zip(who, starts, counts):
                    got[r][s:s + n] = out[o:o + n].float().cpu()
                    o += n
        finally:
            self.ops.force_generic = False
        return got

    def plain(self, m, lam, eps):
        out = []
        nq, nk = self.H * 2 * self.d, self.G * 2 * self.d
        for r in self.rows:
            x = r.double()
            n = x.shape[0]
            out.append(plain_sosepel.differential_attention(
                x[:, :nq].view(n, self.H, 2, self.d), x[:, nq:nq + nk].view(n, self.G, 2, self.d),
                x[:, nq + nk:].view(n, self.G, self.vd), m, lam, eps).reshape(n, -1))
        return out


def _cut(n, sizes, tail):
    """n rows as portions of the given sizes in turn, the last `tail` one by one."""
    out, i, j = [], 0, 0
    while i < n - tail:
        s = min(sizes[j % len(sizes)], n - tail - i)
        out.append(s)
        i += s
        j += 1
    return out + [1] * tail


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,ps", [(6, 3, 12, 20, 8), (4, 1, 32, 64, 16), (2, 2, 16, 32, 4),
                                                        (4, 2, 64, 128, 16), (6, 2, 40, 72, 32),
                                                        (1, 1, 128, 8, 16), (8, 2, 24, 96, 2),
                                                        (2, 1, 136, 160, 8), (4, 2, 16, 40, 12), (40, 1, 8, 16, 16)])
def test_differential_attention_in_portions(ops, dtype, heads, kv_heads, dim, vdim, ps):
    """Three requests of unequal length side by side: portions that end before, at and after
    the borders of pages and of the kernels' tiles of 64 keys, down to two rows, then rows one
    by one; against the plain implementation and with every kernel (plain, matrix cores,
    contexts in chunks) against the others."""
    lens = [200, 67, 331]
    m = {"scale": 0.9 / math.sqrt(dim), "softcap": 6.0, "diff": 0.35, "q_temp": {"coef": 0.4, "every": 16}}
    lam, eps = 0.62, 1e-5
    cache = _Paged(ops, dtype, heads, kv_heads, dim, vdim, ps, lens, seed=dim + vdim)
    cuts = [_cut(200, [63, 2, 64, 5], 30), _cut(67, [3, 61], 3), _cut(331, [128, 2, 65, 100], 20)]
    n_steps = max(len(c) for c in cuts)
    steps = [[c[i] if i < len(c) else 0 for c in cuts] for i in range(n_steps)]
    want = cache.plain(m, lam, eps)
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    for force_plain in (False, True):
        got = cache.run(steps, m, lam, eps, force_plain)
        for g, w_ in zip(got, want):
            assert torch.isfinite(g).all()
            assert rel_err(g, w_) < tol
            assert (g - w_.float()).abs().max() < (1e-4 if dtype == torch.float32 else 0.08)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_differential_attention_whole_against_rows(ops, dtype):
    """A whole prompt in one step, and the same rows one by one (single rows of long contexts
    run with the context cut into chunks in bfloat16): no cap, no temperature, no norm."""
    heads, kv_heads, dim, vdim, ps, n = 4, 2, 32, 64, 16, 700
    m = {"scale": 1.0 / math.sqrt(dim), "diff": 0.5}
    cache = _Paged(ops, dtype, heads, kv_heads, dim, vdim, ps, [n], seed=8)
    want = cache.plain(m, 0.8, 1e-6)[0]
    whole = cache.run([[n]], m, 0.8, 1e-6)[0]
    rows = cache.run([[n - 150]] + [[1]] * 150, m, 0.8, 1e-6)[0]
    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    assert rel_err(whole, want) < tol and rel_err(rows, want) < tol
    if dtype == torch.float32:
        assert torch.equal(whole, rows)   # the 32-bit sums depend on the row alone


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("first,second", [(0, 498), (1, 0), (15, 16), (16, 15), (63, 64), (64, 63), (300, 2),
                                          (511, 512), (512, 255), (640, 639)])
def test_each_map_finds_its_key(ops, dtype, first, second):
    """Among hundreds of keys one matches the query of map 1 and another that of map 2: the
    result is the first one's value minus lam times the second one's, wherever they lie (the
    first positions, a page's and a tile's border, far back), for the last rows of a prompt
    portion and for single rows."""
    heads, kv_heads, dim, vdim, ps, n = 2, 1, 16, 32, 16, 644
    m = {"scale": 1.0, "diff": 0.0}
    lam = 0.5
    cache = _Paged(ops, dtype, heads, kv_heads, dim, vdim, ps, [n], seed=first * 1000 + second)
    rows = cache.rows[0].float()
    nq = heads * 2 * dim
    rows[:, :nq + 2 * dim] *= 0.05                     # quiet queries and keys everywhere
    for r in (n - 3, n - 1):                           # a loud query in both heads, both maps
        for h in range(heads):
            rows[r, h * 2 * dim:(h + 1) * 2 * dim] = 4.0 * torch.sign(torch.randn(2 * dim))
        for h in range(1, heads):
            rows[r, h * 2 * dim:(h + 1) * 2 * dim] = rows[r, :2 * dim]
    rows[n - 3, :nq] = rows[n - 1, :nq]
    q = rows[n - 1, :2 * dim]
    rows[first, nq:nq + dim] = q[:dim] * 2              # key of map 1 at `first`
    rows[second, nq + dim:nq + 2 * dim] = q[dim:] * 2   # key of map 2 at `second`
    cache.rows[0] = rows.to(dtype)
    want = cache.plain(m, lam, 1e-6)[0]
    v = cache.rows[0].double()[:, nq + 2 * dim:]
    expect = plain_sosepel.rms(v[first] - lam * v[second], 1e-6)
    for steps in ([[n]], [[n - 2], [1], [1]]):
        got = cache.run(steps, m, lam, 1e-6)[0]
        assert rel_err(got[n - 1], want[n - 1]) < (1e-4 if dtype == torch.float32 else 1.5e-2)
        assert rel_err(got[n - 1].view(heads, vdim)[0], expect) < 0.03   # the two keys have all the weight
        assert rel_err(got[n - 3], want[n - 3]) < (1e-4 if dtype == torch.float32 else 1.5e-2)


# ---- whole models ----------------------------------------------------------------------------

PROMPT_LENGTHS = [70, 1, 23, 97, 40, 64]


def safe_prompt(w, cfg, n, seed, rel_margin=0.05):
    """n tokens drawn so that every routing decision of the plain implementation is clear by
    `rel_margin` (a close call may fall the other way under rounding, which no test is about)."""
    rng = random.Random(seed)
    toks = []
    tries = 0
    while len(toks) < n:
        cand = rng.randrange(cfg["vocab"])
        margins = []
        plain_sosepel.forward(w, cfg, toks + [cand], margins=margins)
        tries += 1
        if all(float(m[-1]) >= rel_margin for m in margins):
            toks.append(cand)
        elif tries % (10 * n + 50) == 0:
            rel_margin /= 2   # (many sparse layer runs: settle for less)
            if rel_margin < 2e-3:
                raise RuntimeError("no prompt with clear routing found")
    return toks


def row_errors(got, ref):
    d = (got - ref).double()
    return (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt() / ref.double().std()


def noise_of(cfg, w, toks, ref):
    """How far the plain implementation's logits move when every weight is disturbed by one
    part in 2^9 (what rounding to bfloat16 does to a number): median, ninth decile and largest
    of the rows' errors. The comparisons' bounds come from the model at hand."""
    g = torch.Generator().manual_seed(len(toks))
    w2 = {k: v * (1 + torch.randn(v.shape, generator=g) * 2.0 ** -9) if v.is_floating_point() else v
          for k, v in w.items()}
    e = row_errors(plain_sosepel.forward(w2, cfg, toks), ref)
    return e.median().item(), e.kthvalue(max(1, int(0.9 * len(e)))).values.item(), e.max().item()


@pytest.fixture(scope="module", params=list(sosepel_cases.CASES))
def case(request, tmp_path_factory):
    import ninfer_amd
    name = request.param
    make, seed = sosepel_cases.CASES[name]
    raw = make()
    out = {"name": name, "cfg": raw, "dirs": {}, "ref": {}, "reqs": {}, "noise": {}}
    for dtype in ("float32", "bfloat16"):
        d = str(tmp_path_factory.mktemp(f"sosepel_{name}_{dtype}"))
        ninfer_amd.write_random_model(d, raw, seed, dtype=dtype, std=STD)
        out["dirs"][dtype] = d
    cfg, w = util.read_folder(out["dirs"]["bfloat16"])
    for i, n in enumerate(PROMPT_LENGTHS):
        out["reqs"][f"r{i}"] = safe_prompt(w, cfg, n, 50 + i)
    for dtype in ("float32", "bfloat16"):
        cfg, w = util.read_folder(out["dirs"][dtype])
        out["ref"][dtype] = {k: plain_sosepel.forward(w, cfg, v) for k, v in out["reqs"].items()}
        out["noise"][dtype] = {k: noise_of(cfg, w, v, out["ref"][dtype][k]) for k, v in out["reqs"].items()}
    return out


def make_runner(case, dtype, page_size=8, num_pages=40, seqs=4, **more):
    from ninfer_amd import EngineOptions, load_model
    opt = EngineOptions(dtype=dtype, max_context=128, num_sequences=seqs, page_size=page_size,
                        num_pages=num_pages, check_pages=True, poison_freed_pages=True, **more)
    return load_model(case["dirs"][dtype], opt)


def check_logits(case, dtype, got, what):
    for rid, g in got.items():
        ref = case["ref"][dtype][rid]
        who = f"{case['name']} {rid} {what}"
        assert g.shape == ref.shape, who
        assert torch.isfinite(g).all(), f"{who}: not finite"
        err = row_errors(g, ref)
        n50, n90, nmax = case["noise"][dtype][rid]
        f50, f90, fmax, floor = (3, 3, 3, 0.03) if dtype == "bfloat16" else \
            (8 * 2.0 ** -15, 8 * 2.0 ** -15, 16 * 2.0 ** -15, 3e-6)
        e50 = err.median().item()
        e90 = err.kthvalue(max(1, int(0.9 * len(err)))).values.item()
        if len(err) >= 20:
            assert e50 <= max(f50 * n50, floor), f"{who}: median row error {e50:.2e} (disturbance {n50:.2e})"
            assert e90 <= max(f90 * n90, floor), f"{who}: ninth decile {e90:.2e} (disturbance {n90:.2e})"
        assert err.max().item() <= max(fmax * nmax, 4 * floor), \
            f"{who}: row {err.argmax()} is off by {err.max():.2e} (disturbance {nmax:.2e})"


def test_layer_by_layer(case):
    """The 32-bit residual stream after every run of a layer (a looped layer counts each
    time), for a prompt in one step and in portions."""
    from ninfer_amd.engine import Chunk
    cfg, w = util.read_folder(case["dirs"]["float32"])
    toks = case["reqs"]["r4"]
    streams = []
    plain_sosepel.forward(w, cfg, toks, streams)
    runner = make_runner(case, "float32")
    assert len(runner.spec.plan) == len(streams) == len(plain_sosepel.layer_order(cfg))
    for cuts in ([len(toks)], [17, 2, len(toks) - 19]):
        slot = runner.open()
        got = [[] for _ in streams]
        runner.tap = lambda i, residual, pending: got[i].append(residual.cpu().clone())
        o = 0
        for n in cuts:
            runner.step([Chunk(slot, toks[o:o + n], [])])
            o += n
        runner.tap = None
        runner.close(slot)
        for i, want in enumerate(streams):
            g = torch.cat(got[i]).double()
            assert (g - want).abs().max() <= 2e-5 * max(1.0, want.abs().max().item()), f"layer run {i}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_tail_portions(case, dtype):
    runner = make_runner(case, dtype)
    for rid, toks in case["reqs"].items():
        for what, sched in (("whole", util.schedule_whole(rid, toks)),
                            ("tail", util.schedule_tail(rid, toks, 48)),
                            ("portions", util.schedule_portions(rid, toks, seed=len(toks)))):
            if what == "tail" and len(toks) == 1:
                continue
            check_logits(case, dtype, util.run_schedule(runner, sched), what)
    runner.cache.check()
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)


def test_cut_does_not_matter_in_32_bit(case):
    """Every way of cutting a request gives the same logits to the bit in 32-bit: all kernels
    of that path sum in an order that depends on the row alone."""
    runner = make_runner(case, "float32")
    toks = case["reqs"]["r3"]
    whole = util.run_schedule(runner, util.schedule_whole("a", toks))["a"]
    for sched in (util.schedule_tail("a", toks, 40), util.schedule_portions("a", toks, seed=3)):
        assert torch.equal(util.run_schedule(runner, sched)["a"], whole)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_reuse_pages_and_slots(case, dtype):
    """Up to four live requests, prompt portions beside single tokens, in a pool so small that
    pages are used again (freed pages are filled with NaN), then schedules drawn at random;
    every request's logits equal those of the request alone."""
    runner = make_runner(case, dtype, page_size=8, num_pages=34)
    reqs = dict(case["reqs"])
    reqs.update({k + "again": v for k, v in case["reqs"].items()})
    ref, noise = case["ref"][dtype], case["noise"][dtype]
    case["ref"][dtype] = {**ref, **{k + "again": v for k, v in ref.items()}}
    case["noise"][dtype] = {**noise, **{k + "again": v for k, v in noise.items()}}
    try:
        check_logits(case, dtype, util.run_schedule(runner, util.schedule_mixed(reqs, seed=1)), "mixed")
        for seed in (2, 3):
            steps = util.schedule_random(reqs, seed)
            got = util.run_schedule(runner, steps)
            wanted = {}
            for entries, _ in steps:
                for rid, toks, want in entries:
                    wanted.setdefault(rid, [0, []])
                    wanted[rid][1] += [wanted[rid][0] + w_ for w_ in want]
                    wanted[rid][0] += len(toks)
            full = case["ref"][dtype]
            case["ref"][dtype] = {rid: full[rid][rows] for rid, (_, rows) in wanted.items() if rows}
            check_logits(case, dtype, got, f"random {seed}")
            case["ref"][dtype] = full
    finally:
        case["ref"][dtype], case["noise"][dtype] = ref, noise
    assert runner.cache.pages_reused() > 0
    runner.cache.check()


def test_a_slot_used_again_starts_empty(case):
    """One state slot: every request gets the slot the last one left, with that request's last
    token still in it unless it is cleared (the pair table's row of a first token is its own)."""
    runner = make_runner(case, "float32", seqs=1)
    for rid in ("r3", "r0", "r1", "r2"):
        toks = case["reqs"][rid]
        sched = util.schedule_tail(rid, toks, 5) if len(toks) > 1 else util.schedule_whole(rid, toks)
        check_logits(case, "float32", util.run_schedule(runner, sched), "slot used again")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(case, dtype):
    """A few tokens of prompt, then hundreds of single steps: across pages, across the
    attention kernels' tiles and chunks of keys, across many steps of the temperature."""
    if case["name"] in ("ones", "straight") and dtype == "bfloat16":
        pytest.skip("covered by the other two")
    from ninfer_amd import EngineOptions, load_model
    n = 330
    cfg, w = util.read_folder(case["dirs"][dtype])
    toks = safe_prompt(w, cfg, n, 9, rel_margin=0.04)
    ref = plain_sosepel.forward(w, cfg, toks)
    runner = load_model(case["dirs"][dtype], EngineOptions(
        dtype=dtype, max_context=352, num_sequences=2, page_size=16, num_pages=24, check_pages=True))
    got = util.run_schedule(runner, util.schedule_tail("x", toks, n - 3))["x"]
    saved = case["ref"][dtype], case["noise"][dtype]
    case["ref"][dtype], case["noise"][dtype] = {"x": ref}, {"x": noise_of(cfg, w, toks, ref)}
    try:
        check_logits(case, dtype, {"x": got}, "long decoding")
    finally:
        case["ref"][dtype], case["noise"][dtype] = saved


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_from_a_captured_graph(case, dtype):
    """Decode-only steps replayed from a HIP graph (the first step of a shape runs eagerly, the
    second is captured, the rest are replays), two requests side by side, every replay against
    the plain implementation: the previous token travels in the state the graph reads and writes."""
    runner = make_runner(case, dtype, use_graph=True)
    reqs = {k: case["reqs"][k] for k in ("r0", "r4")}
    from ninfer_amd.engine import Chunk
    slots = {k: runner.open() for k in reqs}
    heads = {k: len(v) - 30 for k, v in reqs.items()}
    got = {k: [] for k in reqs}
    logits = runner.step([Chunk(slots[k], reqs[k][:heads[k]], list(range(heads[k]))) for k in reqs])
    o = 0
    for k in reqs:
        got[k].append(logits[o:o + heads[k]].float().cpu())
        o += heads[k]
    for i in range(30):
        logits = runner.step([Chunk(slots[k], [reqs[k][heads[k] + i]], [0]) for k in reqs])
        for j, k in enumerate(reqs):
            got[k].append(logits[j:j + 1].float().cpu().clone())
    assert len(runner._graphs) >= 1
    for k in reqs:
        runner.close(slots[k])
    check_logits(case, dtype, {k: torch.cat(v) for k, v in got.items()}, "graph replay")


@pytest.mark.parametrize("seed", list(range(9)))
def test_random_configurations(seed, tmp_path):
    """Configurations drawn at random (sizes, head counts, kinds and order of layers, what is
    absent), in both precisions: whole, in portions and in a mixed batch."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    raw = sosepel_cases.random_config(seed)
    for dtype in ("float32", "bfloat16"):
        d = str(tmp_path / dtype)
        ninfer_amd.write_random_model(d, raw, 100 + seed, dtype=dtype, std=STD)
        cfg, w = util.read_folder(d)
        if dtype == "float32":
            reqs = {f"q{i}": safe_prompt(w, cfg, n, 7 * seed + i) for i, n in enumerate([33, 1, 14, 50])}
        ref = {k: plain_sosepel.forward(w, cfg, v) for k, v in reqs.items()}
        case = {"name": f"random {seed}", "ref": {dtype: ref},
                "noise": {dtype: {k: noise_of(cfg, w, v, ref[k]) for k, v in reqs.items()}}}
        runner = load_model(d, EngineOptions(dtype=dtype, max_context=64, num_sequences=3, page_size=8,
                                             num_pages=20, check_pages=True, poison_freed_pages=True))
        for k, v in reqs.items():
            check_logits(case, dtype, util.run_schedule(runner, util.schedule_whole(k, v)), "whole")
            check_logits(case, dtype, util.run_schedule(runner, util.schedule_portions(k, v, seed=seed)), "portions")
        check_logits(case, dtype, util.run_schedule(runner, util.schedule_mixed(reqs, seed=seed, max_live=3)), "mixed")
        runner.release()


def test_greedy_generation_through_the_scheduler(case):
    """The framework's own entry point: prompts of unequal length generated greedily by the
    scheduler (admission, portions under a token budget, batched decoding, sampling kernel),
    token for token what the plain implementation chooses."""
    from ninfer_amd import Ninfer, SamplingParams
    cfg, w = util.read_folder(case["dirs"]["float32"])
    prompts = [case["reqs"][k][:n] for k, n in (("r0", 19), ("r2", 3), ("r3", 41))]
    new = 10
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(new):
            margins = []
            logits = plain_sosepel.forward(w, cfg, toks, margins=margins)[-1]
            top = torch.topk(logits, 2).values
            if top[0] - top[1] < 1e-3 or any(float(m[-1]) < 1e-3 for m in margins):
                break   # too close to call: the comparison ends here for this prompt
            toks.append(int(logits.argmax()))
        want.append(toks[len(p):])
    eng = Ninfer(case["dirs"]["float32"], max_context=128, prefill_chunk=16, num_sequences=2,
                 dtype="float32", page_size=8, num_pages=30)
    got = eng.generate(prompts, SamplingParams.greedy(new), stop_ids=[])
    eng.close()
    assert sum(len(x) for x in want) >= new
    assert [g[:len(x)] for g, x in zip(got, want)] == want


def test_command_line(case):
    """`ninfer <folder>` on a Sosepel folder: greedy from given and random prompts in 32-bit, the
    first against the plain choice; sampling with the defaults from a captured graph in
    bfloat16, the same seed the same tokens."""
    if case["name"] != "even":
        pytest.skip("one configuration is enough for the program")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg, w = util.read_folder(case["dirs"]["float32"])
    prompt = case["reqs"]["r2"][:9]
    want = list(prompt)
    for _ in range(4):
        want.append(int(plain_sosepel.forward(w, cfg, want)[-1].argmax()))
    run = lambda d, *more: subprocess.run(
        [sys.executable, os.path.join(root, "bin", "ninfer"), d, "--prompt-ids", ",".join(map(str, prompt)),
         "--max-context", "64", "--prefill-chunk", "8", *more], capture_output=True, text=True, timeout=300)
    proc = run(case["dirs"]["float32"], "--random-prompts", "5,12", "--max-new", "4", "--temperature", "0",
               "--dtype", "fp32", "--repeat-penalty", "1", "--eos-id", "-1")
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = proc.stdout.strip().splitlines()
    assert len(lines) == 3 and [int(x) for x in lines[0].split(",")] == want[len(prompt):]
    outs = []
    for _ in range(2):
        proc = run(case["dirs"]["bfloat16"], "--max-new", "12", "--seed", "7", "--graph", "--eos-id", "-1")
        assert proc.returncode == 0, proc.stderr[-2000:]
        outs.append(proc.stdout.strip())
    assert outs[0] == outs[1] and len(outs[0].split(",")) == 12


def test_trace_replay_program(case, tmp_path):
    """bin/trace_run on a model folder: a mixed schedule as JSON lines, the logits files
    against the plain implementation."""
    if case["name"] != "odd":
        pytest.skip("one configuration is enough for the program")
    reqs = {k: case["reqs"][k] for k in ("r0", "r2", "r4", "r1")}
    steps = util.schedule_mixed(reqs, seed=4)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out_dir = str(tmp_path / "out")
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model",
                        case["dirs"]["float32"], "--dtype", "float32", "--out", out_dir,
                        "--max-tokens", "256"], input=util.write_trace(steps), text=True,
                       capture_output=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(len(steps))]
    got = util.read_trace_output(out_dir, steps, case["cfg"]["vocab"])
    check_logits(case, "float32", got, "trace_run")
    stats = json.load(open(os.path.join(out_dir, "stats.json")))
    assert stats["groups"][0]["in_use"] == 0
