"""Getodra on the GPU against the plain implementation: every mechanism alone through its
kernel, then whole models (three small configurations, in 32-bit and in bfloat16) whole,
decoded token by token, in portions down to two tokens, in mixed batches with pages and
state slots that are given back and used again, and generated greedily through the
scheduler. bfloat16 is compared with the plain implementation on the bfloat16-rounded
weights; the 32-bit bound is that of rounding."""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

import getodra_cases
import plain_getodra
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


# ---- mechanisms alone ------------------------------------------------------------------------

def _portions(ops, dtype, lengths_by_step, slots):
    """StepContexts for requests that go on from step to step: lengths_by_step[i][r] rows of
    request r in step i (0: left out); rows of the step are taken from each request in order."""
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


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,width", [(4, 72), (2, 256), (1, 64), (6, 40)])
def test_short_conv_in_portions(ops, dtype, taps, width):
    torch.manual_seed(taps * 100 + width)
    lens = [23, 9]
    x = [torch.randn(n, width) for n in lens]
    w = torch.randn(width, taps) * 0.5
    want = [plain_getodra.input_conv(a.double(), w.double()) for a in x]
    # the state's columns lie inside wider rows, and the requests hold slots 2 and 0
    state_all = torch.zeros(3, (taps - 1) * width + 17, device=DEV)
    state = state_all[:, 5:5 + max((taps - 1) * width, 1)]
    steps = [[3, 0], [2, 2], [1, 1], [1, 1], [7, 2], [1, 0], [2, 3], [6, 0]]
    assert [sum(s[r] for s in steps) for r in range(2)] == lens
    got = [torch.zeros(n, width) for n in lens]
    for ctx, who, starts, counts in _portions(ops, dtype, steps, slots=[2, 0]):
        rows = torch.cat([x[r][s:s + n] for r, s, n in zip(who, starts, counts)]).to(DEV)
        out = torch.empty(rows.shape, dtype=dtype, device=DEV)
        ops.short_conv(rows, w.to(DEV), state, ctx, out)
        o = 0
        for r, s, n in zip(who, starts, counts):
            got[r][s:s + n] = out[o:o + n].float().cpu()
            o += n
    for g, wnt in zip(got, want):
        if dtype == torch.float32:
            torch.testing.assert_close(g.double(), wnt, atol=1e-5, rtol=1e-5)
        else:
            assert rel_err(g, wnt) < 6e-3
    assert state_all[1].abs().max() == 0 and state_all[:, :5].abs().max() == 0   # nobody else's


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,single", [(72, True), (256, False), (1100, True)])
def test_norm_add(ops, dtype, width, single):
    torch.manual_seed(width)
    x = torch.randn(5, width)
    y = (torch.randn(5, width) * 3).to(dtype)
    gain = torch.randn(1 if single else width)
    want = x.double() + plain_getodra.rms_unit(y.double(), 1e-5) * gain.double()
    res = x.to(DEV)
    ops.norm_add(res, y.to(DEV), gain.to(DEV), 1e-5)
    torch.testing.assert_close(res.cpu().double(), want, atol=2e-6, rtol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_rmsnorm(ops, dtype):
    torch.manual_seed(3)
    n = 100
    o = torch.randn(7, n) * 4
    wide = torch.randn(7, n + 60).to(dtype)
    w = torch.randn(n)
    want = plain_getodra.rms_unit(o.double(), 1e-5) * w.double() * torch.sigmoid(wide[:, 60:].double())
    out = torch.empty(7, n, dtype=dtype, device=DEV)
    ops.gated_rmsnorm(o.to(DEV), wide.to(DEV)[:, 60:], w.to(DEV), 1e-5, out)
    assert rel_err(out, want) < (2e-6 if dtype == torch.float32 else 5e-3)


def _plain_lightning(q, k, v, decay):
    n, H = q.shape[0], q.shape[1]
    out = torch.zeros(n, H, v.shape[2], dtype=torch.float64)
    for h in range(H):
        S = torch.zeros(q.shape[2], v.shape[2], dtype=torch.float64)
        for t in range(n):
            S = decay[h] * S + torch.outer(k[t, h], v[t, h])
            out[t, h] = S.T @ q[t, h]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,vdim", [(5, 12, 20), (2, 64, 48), (1, 16, 16), (3, 40, 300)])
def test_lightning_in_portions(ops, dtype, heads, dim, vdim):
    """Two requests cut into portions of many sizes against the recurrence run whole; one
    head does not decay at all, one forgets within a few tokens."""
    torch.manual_seed(heads * 7 + dim)
    lens = [330, 31] if dim == 64 else [150, 31]
    decay = ([1.0, 0.3, 0.9, 0.99, 0.97] * 2)[:heads]
    if dim == 16:
        decay = [0.0]    # a head that forgets everything at once
    qk, vw = heads * dim, heads * vdim
    rows = [(torch.randn(n, 2 * qk + vw + 11) * 1.5).to(dtype) for n in lens]
    silu = plain_getodra.silu
    want = []
    for r in rows:
        d = r.double()
        want.append(_plain_lightning(silu(d[:, 3:3 + qk]).reshape(-1, heads, dim),
                                     silu(d[:, 3 + qk:3 + 2 * qk]).reshape(-1, heads, dim),
                                     silu(d[:, 3 + 2 * qk:3 + 2 * qk + vw]).reshape(-1, heads, vdim),
                                     decay))
    state_all = torch.zeros(4, heads * dim * vdim + 9, device=DEV)
    state = state_all[:, 9:]
    # (bfloat16 steps whose longest portion has 8 rows or more run in chunks of 64 on the matrix
    # cores, the others token by token: both kinds follow each other on the same state)
    steps = [[64, 0], [1, 7], [1, 1], [2, 2], [33, 1], [1, 1], [17, 16], [30, 3], [1, 0]]
    if dim == 64:
        steps = [[130, 0], [1, 7], [1, 1], [2, 2], [65, 1], [1, 1], [64, 16], [63, 3], [3, 0]]
    assert [sum(s[r] for s in steps) for r in range(2)] == lens
    got = [torch.zeros(n, heads, vdim, dtype=torch.float64) for n in lens]
    dec = torch.tensor(decay, device=DEV)
    for ctx, who, starts, counts in _portions(ops, dtype, steps, slots=[3, 1]):
        x = torch.cat([rows[r][s:s + n] for r, s, n in zip(who, starts, counts)]).to(DEV)
        out = torch.empty(x.shape[0], vw, device=DEV)
        ops.lightning_attention(x, 3, 3 + qk, 3 + 2 * qk, heads, dim, vdim, dec, state, ctx, out)
        o = 0
        for r, s, n in zip(who, starts, counts):
            got[r][s:s + n] = out[o:o + n].double().cpu().reshape(n, heads, vdim)
            o += n
    for g, wnt in zip(got, want):
        assert rel_err(g, wnt) < 2e-5     # (the inputs are the same numbers in both precisions)
        assert rel_err(g[-1], wnt[-1]) < 2e-5
    assert state_all[0].abs().max() == 0 and state_all[2].abs().max() == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,k,n", [(3, 24, 40), (4, 64, 160), (1, 16, 32), (5, 40, 20), (2, 12, 10)])
@pytest.mark.parametrize("rows", [1, 7, 70])
def test_per_head_linear(ops, dtype, heads, k, n, rows):
    torch.manual_seed(rows + k)
    x = torch.randn(rows, heads, k + 8).to(dtype)
    w = (torch.randn(heads, n, k) * 0.3).to(dtype)
    want = torch.einsum("thk,hnk->thn", x[..., :k].double(), w.double())
    ctx = util.make_context(ops, dtype, [(0, rows)])
    for out_dtype in (dtype, torch.float32):
        out = torch.full((rows, heads, n + 4), 7.0, dtype=out_dtype, device=DEV)
        ops.per_head_linear(x.to(DEV), w.to(DEV), out, ctx, k, n)
        assert rel_err(out[..., :n], want) < (1e-5 if out_dtype == torch.float32 else 6e-3)
        assert (out[..., n:] == 7.0).all()     # columns beyond the product's are left alone


def _latent_case(ops, dtype, heads, rank, rd, page_size, lengths, new_rows, window=None, seed=0):
    """Requests of lengths[i] cached rows in shuffled pages, the last new_rows[i] of which are
    the step's rows. Returns (ctx, pool, table, q_abs, cached rows per request)."""
    g = torch.Generator().manual_seed(seed)
    Dk = rank + rd
    pages_each = [-(-n // page_size) for n in lengths]
    perm = torch.randperm(sum(pages_each) + 3, generator=g).tolist()
    pool = torch.full((sum(pages_each) + 3, page_size, Dk), float("nan"))
    table = torch.full((len(lengths), max(pages_each)), -1, dtype=torch.int32)
    cached, at = [], 0
    for i, n in enumerate(lengths):
        rows = (torch.randn(n, Dk, generator=g) * 0.7).to(dtype).float()
        for p in range(pages_each[i]):
            table[i, p] = perm[at]
            part = rows[p * page_size:(p + 1) * page_size]
            pool[perm[at], :part.shape[0]] = part
            at += 1
        cached.append(rows)
    ctx = util.make_context(ops, dtype, [(n - m, m) for n, m in zip(lengths, new_rows)])
    q = torch.randn(ctx.T, heads, Dk, generator=g)
    return ctx, pool, table, q, cached


def _plain_latent_rows(q, cached, lengths, new_rows, rank, scale, window, gate=None):
    out, r = [], 0
    for rows, n, m in zip(cached, lengths, new_rows):
        for pos in range(n - m, n):
            lo = 0 if not window else max(0, pos - window + 1)
            keys = rows[lo:pos + 1].double()
            s = torch.einsum("hd,jd->hj", q[r].double(), keys) * scale
            o = torch.softmax(s, -1) @ keys[:, :rank]
            if gate is not None:
                o = o * torch.sigmoid(gate[r].double())[:, None]
            out.append(o)
            r += 1
    return torch.stack(out)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,rank,rd,ps", [(3, 40, 8, 8), (4, 64, 32, 16), (1, 32, 16, 4), (2, 130, 6, 64)])
def test_latent_attention_rows(ops, dtype, heads, rank, rd, ps):
    """Prompt portions and single rows together, requests that end just before, at and just
    after the borders of pages and of the kernel's tiles of 64 keys, and a gate per head."""
    lengths = [1, ps, ps + 1, 63, 64, 65, 129, 200, 2 * ps - 1]
    new_rows = [1, 2, 1, 5, 1, 64, 1, 9, 1]
    ctx, pool, table, q, cached = _latent_case(ops, dtype, heads, rank, rd, ps, lengths, new_rows,
                                               seed=heads)
    gate_wide = torch.randn(ctx.T, heads + 5).to(dtype)
    want = _plain_latent_rows(q, cached, lengths, new_rows, rank, 0.2, None, gate_wide[:, 5:].float())
    out = torch.empty(ctx.T, heads * rank, dtype=dtype, device=DEV)
    ops.latent_attention(q.to(DEV), pool.to(dtype).to(DEV), table.to(DEV), ctx, heads, rank, rd, ps,
                         0.2, out, gate=gate_wide.to(DEV)[:, 5:])
    got = out.float().cpu().reshape(ctx.T, heads, rank)
    assert torch.isfinite(got).all()
    assert rel_err(got, want) < (1e-5 if dtype == torch.float32 else 6e-3)


@pytest.mark.parametrize("heads,rank,rd", [(16, 64, 16), (5, 200, 24)])
def test_latent_attention_whole_prompt_on_matrix_cores(ops, heads, rank, rd):
    """A prompt long enough that the bfloat16 kernel walks each block's keys in one piece
    (shorter steps cut the keys into chunks and merge), against the plain kernel and
    against the softmax written out."""
    n, ps = 1100, 16
    ctx, pool, table, q, cached = _latent_case(ops, torch.bfloat16, heads, rank, rd, ps, [n], [n], seed=rank)
    keys = cached[0].double()
    want = torch.zeros(n, heads, rank, dtype=torch.float64)
    mask = torch.tril(torch.ones(n, n, dtype=torch.bool))
    for h in range(heads):
        s = (q[:, h].double() @ keys.T * 0.3).masked_fill(~mask, float("-inf"))
        want[:, h] = torch.softmax(s, -1) @ keys[:, :rank]
    outs = []
    for plain in (False, True):
        ops.force_generic = plain
        try:
            out = torch.empty(n, heads * rank, dtype=torch.bfloat16, device=DEV)
            ops.latent_attention(q.to(DEV), pool.to(torch.bfloat16).to(DEV), table.to(DEV), ctx, heads,
                                 rank, rd, ps, 0.3, out)
        finally:
            ops.force_generic = False
        outs.append(out.float().cpu().reshape(n, heads, rank))
        assert rel_err(outs[-1], want) < 8e-3
    assert rel_err(outs[0][:3], want[:3]) < 8e-3 and rel_err(outs[0][-1], want[-1]) < 8e-3


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("where", [0, 1, 15, 16, 63, 64, 300, 498])
def test_latent_attention_finds_one_key(ops, dtype, where):
    """Among 500 keys one is made to match the query (its row is the query scaled up): the
    output is that key's latent, wherever it lies: far back, at the first positions, at
    a page's border."""
    heads, rank, rd, ps, n = 2, 32, 8, 16, 500
    ctx, pool, table, q, cached = _latent_case(ops, dtype, heads, rank, rd, ps, [n], [1], seed=where)
    q[0, 1] = q[0, 0]
    key = (q[0, 0] * 3).to(dtype).float()
    cached[0][where] = key
    pool[table[0, where // ps], where % ps] = key
    out = torch.empty(1, heads * rank, dtype=dtype, device=DEV)
    ops.latent_attention(q.to(DEV), pool.to(dtype).to(DEV), table.to(DEV), ctx, heads, rank, rd, ps,
                         1.0, out)
    got = out.float().cpu().reshape(heads, rank)
    want = _plain_latent_rows(q, cached, [n], [1], rank, 1.0, None)[0]
    assert rel_err(got, want) < (1e-5 if dtype == torch.float32 else 6e-3)
    assert rel_err(got[0], key[:rank]) < 0.02      # the one key has all the weight


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_attention_window_edges(ops, dtype):
    """The kernel's window (a parameter no present model sets): the key just inside counts,
    the one just outside does not, in a prompt portion and for single rows."""
    heads, rank, rd, ps, window = 2, 32, 8, 8, 20
    lengths, new_rows = [70, 41, 21, 20], [30, 1, 1, 1]
    ctx, pool, table, q, cached = _latent_case(ops, dtype, heads, rank, rd, ps, lengths, new_rows, seed=5)
    r = 0
    for i, (n, m) in enumerate(zip(lengths, new_rows)):   # a loud key just outside the last row's window
        pos = n - 1
        out_of = pos - window
        if out_of >= 0:
            loud = (q[r + m - 1, 0] * 4).to(dtype).float()
            cached[i][out_of] = loud
            pool[table[i, out_of // ps], out_of % ps] = loud
        r += m
    want = _plain_latent_rows(q, cached, lengths, new_rows, rank, 1.0, window)
    wrong = _plain_latent_rows(q, cached, lengths, new_rows, rank, 1.0, window + 1)
    out = torch.empty(ctx.T, heads * rank, dtype=dtype, device=DEV)
    ops.latent_attention(q.to(DEV), pool.to(dtype).to(DEV), table.to(DEV), ctx, heads, rank, rd, ps,
                         1.0, out, window=window)
    got = out.float().cpu().reshape(ctx.T, heads, rank)
    assert rel_err(got, want) < (1e-5 if dtype == torch.float32 else 6e-3)
    assert rel_err(wrong, want) > 0.1


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,rank,rd,turning", [(3, 24, 40, 8, 8), (2, 16, 32, 16, 8), (1, 8, 16, 4, 0)])
def test_latent_kv_write(ops, dtype, heads, dim, rank, rd, turning):
    from ninfer_amd.parts import Rotary
    torch.manual_seed(rank)
    ps = 4
    rot = {"base": 1000.0, "dims": turning, "scaling": {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}}
    ctx = util.make_context(ops, dtype, [(5, 6), (0, 3), (17, 1)])
    table = torch.tensor([[3, 1, 7, -1, -1], [0, -1, -1, -1, -1], [2, 4, 5, 6, 8]], dtype=torch.int32)
    down = torch.randn(ctx.T, rank + rd + heads).to(dtype)
    q = torch.randn(ctx.T, heads * (dim + rd)).to(dtype)
    norm_w = torch.randn(rank)
    pool = torch.zeros(9, ps, rank + rd, dtype=dtype, device=DEV)
    q_abs = torch.full((ctx.T, heads, rank + rd), 5.0, device=DEV)
    freq, mag = None, 1.0
    if turning:
        part = Rotary(turning, rot["base"], scaling=rot["scaling"])
        freq, mag = part.inv_freq().to(DEV), part.magnitude
    ops.latent_kv_write(down.to(DEV), q.to(DEV), q_abs, pool, table.to(DEV), ctx, heads, dim, rank, rd,
                        norm_w.to(DEV), 1e-5, freq, turning, mag, ps)
    pos = ctx.positions.cpu().tolist()
    seq = ctx.row_seq.cpu().tolist()
    d = down.double()
    c = plain_getodra.rms_unit(d[:, :rank], 1e-5) * norm_w.double()
    tol = 2e-6 if dtype == torch.float32 else 5e-3
    for t in range(ctx.T):
        def turned(v):   # the plain rotation counts positions from 0: give it the row at its place
            pad = torch.zeros(pos[t] + 1, *v.shape, dtype=torch.float64)
            pad[pos[t]] = v
            return plain_getodra.turn(pad, rot if turning else None)[pos[t]]
        row = pool[table[seq[t], pos[t] // ps], pos[t] % ps].double().cpu()
        assert rel_err(row[:rank], c[t]) < tol
        assert rel_err(row[rank:], turned(d[t, rank:rank + rd])) < tol
        qr = q[t].double().reshape(heads, dim + rd)[:, dim:]
        assert rel_err(q_abs[t, :, rank:].cpu(), turned(qr)) < tol
        assert (q_abs[t, :, :rank] == 5.0).all()


# ---- whole models ----------------------------------------------------------------------------

PROMPT_LENGTHS = [70, 1, 23, 97, 40, 64]


@pytest.fixture(scope="module", params=list(getodra_cases.CASES))
def case(request, tmp_path_factory):
    import ninfer_amd
    name = request.param
    make, seed = getodra_cases.CASES[name]
    raw = make()
    out = {"name": name, "cfg": raw, "dirs": {}, "ref": {}, "reqs": {}, "noise": {}}
    for i, n in enumerate(PROMPT_LENGTHS):
        out["reqs"][f"r{i}"] = util.random_tokens(n, raw["vocab"], 50 + i)
    for dtype in ("float32", "bfloat16"):
        d = str(tmp_path_factory.mktemp(f"getodra_{name}_{dtype}"))
        ninfer_amd.write_random_model(d, raw, seed, dtype=dtype, std=STD)
        out["dirs"][dtype] = d
        cfg, w = util.read_folder(d)
        out["ref"][dtype] = {k: plain_getodra.forward(w, cfg, v) for k, v in out["reqs"].items()}
        out.setdefault("noise", {})[dtype] = {k: noise_of(cfg, w, v, out["ref"][dtype][k])
                                              for k, v in out["reqs"].items()}
    return out


def make_runner(case, dtype, page_size=8, num_pages=40, seqs=4, **more):
    from ninfer_amd import EngineOptions, load_model
    opt = EngineOptions(dtype=dtype, max_context=case["cfg"]["max_positions"], num_sequences=seqs,
                        page_size=page_size, num_pages=num_pages, check_pages=True,
                        poison_freed_pages=True, **more)
    return load_model(case["dirs"][dtype], opt)


def row_errors(got, ref):
    """Per row: the error over the vocabulary (its mean taken off), against the size of the logits."""
    d = (got - ref).double()
    return (d - d.mean(-1, keepdim=True)).pow(2).mean(-1).sqrt() / ref.double().std()


def noise_of(cfg, w, toks, ref):
    """How far the plain implementation's logits move when every weight is disturbed by one
    part in 2^9 (what rounding to bfloat16 does to a number): median, ninth decile and
    largest of the rows' errors. Norms on small sublayer outputs and sharp softmaxes make
    some rows of some of these small models move by tens of percent, so the bounds of the
    comparisons below are taken from the model at hand, not fixed."""
    g = torch.Generator().manual_seed(len(toks))
    w2 = {k: v * (1 + torch.randn(v.shape, generator=g) * 2.0 ** -9) for k, v in w.items()}
    e = row_errors(plain_getodra.forward(w2, cfg, toks), ref)
    return e.median().item(), e.kthvalue(max(1, int(0.9 * len(e)))).values.item(), e.max().item()


def check_logits(case, dtype, got, what):
    for rid, g in got.items():
        ref = case["ref"][dtype][rid]
        who = f"{case['name']} {rid} {what}"
        assert g.shape == ref.shape, who
        assert torch.isfinite(g).all(), f"{who}: not finite"
        err = row_errors(g, ref)
        n50, n90, nmax = case["noise"][dtype][rid]
        # bfloat16 rounds activations as well as weights: three times the disturbance's effect;
        # 32-bit rounding is 2^-15 of bfloat16's, in every sum of the model: eight to sixteen times
        f50, f90, fmax, floor = (3, 3, 3, 0.03) if dtype == "bfloat16" else \
            (8 * 2.0 ** -15, 8 * 2.0 ** -15, 16 * 2.0 ** -15, 3e-6)
        e50 = err.median().item()
        e90 = err.kthvalue(max(1, int(0.9 * len(err)))).values.item()
        if len(err) >= 20:   # (deciles of a handful of rows say little)
            assert e50 <= max(f50 * n50, floor), f"{who}: median row error {e50:.2e} (disturbance {n50:.2e})"
            assert e90 <= max(f90 * n90, floor), f"{who}: ninth decile {e90:.2e} (disturbance {n90:.2e})"
        assert err.max().item() <= max(fmax * nmax, 4 * floor), \
            f"{who}: row {err.argmax()} is off by {err.max():.2e} (disturbance {nmax:.2e})"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_tail_portions(case, dtype):
    runner = make_runner(case, dtype)
    for rid, toks in case["reqs"].items():
        for what, sched in (("whole", util.schedule_whole(rid, toks)),
                            ("tail", util.schedule_tail(rid, toks, 48)),
                            ("portions", util.schedule_portions(rid, toks, seed=len(toks)))):
            if what == "tail" and len(toks) == 1:
                continue   # (nothing to decode)
            check_logits(case, dtype, util.run_schedule(runner, sched), what)
    runner.cache.check()
    assert all(g.allocator.in_use == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cut_does_not_matter_in_32_bit(case, dtype):
    """Every way of cutting a request gives the same logits: to the bit in 32-bit (all
    kernels of that path sum in an order that depends on the row alone)."""
    if dtype != "float32":
        pytest.skip("the bfloat16 kernels may sum portions in another order")
    runner = make_runner(case, dtype)
    toks = case["reqs"]["r3"]
    whole = util.run_schedule(runner, util.schedule_whole("a", toks))["a"]
    for sched in (util.schedule_tail("a", toks, 40), util.schedule_portions("a", toks, seed=3)):
        assert torch.equal(util.run_schedule(runner, sched)["a"], whole)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_reuse_pages_and_slots(case, dtype):
    """Up to four live requests, prompt portions beside single tokens, in a pool so small
    that pages are used again (freed pages are filled with NaN), then schedules drawn at
    random; every request's logits equal those of the request alone."""
    runner = make_runner(case, dtype, page_size=8, num_pages=34)
    reqs = dict(case["reqs"])
    reqs.update({k + "again": v for k, v in case["reqs"].items()})
    ref = case["ref"][dtype]
    case["ref"][dtype] = {**ref, **{k + "again": v for k, v in ref.items()}}
    noise = case["noise"][dtype]
    case["noise"][dtype] = {**noise, **{k + "again": v for k, v in noise.items()}}
    try:
        check_logits(case, dtype, util.run_schedule(runner, util.schedule_mixed(reqs, seed=1)), "mixed")
        for seed in (2, 3):
            steps = util.schedule_random(reqs, seed)
            got = util.run_schedule(runner, steps)
            wanted = {}
            for entries, _ in steps:   # the random schedule asks for some rows only
                for rid, toks, want in entries:
                    wanted.setdefault(rid, [0, []])
                    wanted[rid][1] += [wanted[rid][0] + w for w in want]
                    wanted[rid][0] += len(toks)
            full = case["ref"][dtype]
            case["ref"][dtype] = {rid: full[rid][rows] for rid, (_, rows) in wanted.items() if rows}
            check_logits(case, dtype, got, f"random {seed}")
            case["ref"][dtype] = full
    finally:
        case["ref"][dtype] = ref
        case["noise"][dtype] = noise
    assert runner.cache.pages_reused() > 0 or not runner.cache.groups
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32"])
def test_a_slot_used_again_starts_empty(case, dtype):
    """One state slot: every request gets the slot the last one left, with the lightning
    state and the convolutions' inputs of that request still in it unless they are cleared."""
    runner = make_runner(case, dtype, seqs=1)
    for rid in ("r3", "r0", "r2"):
        got = util.run_schedule(runner, util.schedule_tail(rid, case["reqs"][rid], 5))
        check_logits(case, dtype, got, "slot used again")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(case, dtype):
    """A few tokens of prompt, then more than a hundred single steps: across pages, across the
    attention kernel's tiles of 64 keys, with the lightning state carried all the way."""
    if case["name"] == "ones" and dtype == "bfloat16":
        pytest.skip("covered by the other two")
    import ninfer_amd
    n = min(150, case["cfg"]["max_positions"])
    toks = util.random_tokens(n, case["cfg"]["vocab"], 9)
    cfg, w = util.read_folder(case["dirs"][dtype])
    ref = plain_getodra.forward(w, cfg, toks)
    runner = make_runner(case, dtype)
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
    second is captured, the rest are replays): two requests decoded side by side for dozens of
    steps, every replay against the plain implementation."""
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


@pytest.mark.parametrize("kind", ["lightning", "latent_attention"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_models_of_one_kind_of_layer(kind, dtype, tmp_path):
    """A model with lightning layers alone holds no pages at all, one with latent attention
    alone no lightning state; widths and sizes that are no multiple of 8."""
    import ninfer_amd
    from ninfer_amd import EngineOptions, load_model
    raw = getodra_cases.config_odd()
    raw["width"], raw["vocab"] = 52, 90
    keep = [l for l in raw["layers"] if l["type"] == kind and "weights_of" not in l]
    again = dict(keep[0], weights_of=0)
    raw["layers"] = [keep[0], again]
    if kind == "latent_attention":
        raw["layers"][0]["mixer"].update(dim=14, rot_dim=6, kv_rank=23, vdim=9)
        raw["layers"][0]["mixer"]["rot"]["dims"] = 6
        raw["layers"][1] = dict(raw["layers"][0], weights_of=0)
    d = str(tmp_path)
    ninfer_amd.write_random_model(d, raw, 3, dtype=dtype, std=STD)
    cfg, w = util.read_folder(d)
    toks = util.random_tokens(45, raw["vocab"], 8)
    ref = plain_getodra.forward(w, cfg, toks)
    runner = load_model(d, EngineOptions(dtype=dtype, max_context=raw["max_positions"], num_sequences=2,
                                         page_size=8, num_pages=12, check_pages=True))
    assert bool(runner.cache.groups) == (kind == "latent_attention")
    case = {"name": kind, "ref": {dtype: {"x": ref}}, "noise": {dtype: {"x": noise_of(cfg, w, toks, ref)}}}
    for sched in (util.schedule_whole("x", toks), util.schedule_tail("x", toks, 20),
                  util.schedule_portions("x", toks, seed=1)):
        check_logits(case, dtype, util.run_schedule(runner, sched), "one kind of layer")


def test_greedy_generation_through_the_scheduler(case):
    """The framework's own entry point: prompts of unequal length generated greedily by the
    scheduler (admission, portions under a token budget, batched decoding, sampling kernel),
    token for token what the plain implementation chooses."""
    from ninfer_amd import Ninfer, SamplingParams
    cfg, w = util.read_folder(case["dirs"]["float32"])
    prompts = [util.random_tokens(n, cfg["vocab"], 70 + n) for n in (19, 3, 41)]
    new = 12
    want = []
    for p in prompts:
        toks = list(p)
        for _ in range(new):
            logits = plain_getodra.forward(w, cfg, toks)[-1]
            top = torch.topk(logits, 2).values
            assert top[0] - top[1] > 1e-3, "the plain choice is too close to call"
            toks.append(int(logits.argmax()))
        want.append(toks[len(p):])
    eng = Ninfer(case["dirs"]["float32"], max_context=None, prefill_chunk=16, num_sequences=2,
                 dtype="float32", page_size=8, num_pages=30)
    assert eng.max_context == cfg["max_positions"]
    assert eng.state_bytes_per_request > 0
    got = eng.generate(prompts, SamplingParams.greedy(new), stop_ids=[])
    eng.close()
    assert got == want


def test_trace_replay_program(case, tmp_path):
    """bin/trace_run on a Getodra folder: a mixed schedule as JSON lines, the logits files
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
