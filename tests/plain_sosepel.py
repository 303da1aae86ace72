"""Sosepel, plain and slow: one function per mechanism, whole sequences in 64-bit, no cache,
no batches. What the engine's parts and kernels are compared with; it shares no code with them.

Notation: n tokens, width w; rms(y) = y / sqrt(mean(y^2) + eps).
"""
import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def rms(y: torch.Tensor, eps: float) -> torch.Tensor:
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)


def pair_rows(tokens: List[int], buckets: int, mul_prev: int, mul_cur: int) -> List[int]:
    """Row of the pair table for every token: the hash of (previous, current); the extra last
    row for the first token."""
    rows = [buckets]
    for prev, cur in zip(tokens[:-1], tokens[1:]):
        rows.append((prev * mul_prev + cur * mul_cur) % buckets)
    return rows


def embed(w: Dict[str, torch.Tensor], cfg: dict, tokens: List[int]) -> torch.Tensor:
    e = cfg["embedding"]
    x = w["embed"][torch.tensor(tokens)].to(F) * e.get("scale", 1.0)
    b = e.get("bigram")
    if b:
        x = x + w["bigram"][torch.tensor(pair_rows(tokens, b["buckets"], b["mul_prev"], b["mul_cur"]))].to(F)
    return x


def query_temperature(n: int, q_temp: Optional[dict]) -> torch.Tensor:
    if not q_temp:
        return torch.ones(n, dtype=F)
    return torch.tensor([1.0 + q_temp["coef"] * math.log((p + 1) // q_temp["every"] + 1) for p in range(n)],
                        dtype=F)


def map_weight(lq1, lk1, lq2, lk2, diff: float) -> float:
    return math.exp(float(lq1.to(F) @ lk1.to(F))) - math.exp(float(lq2.to(F) @ lk2.to(F))) + diff


def differential_attention(q, k, v, m: dict, lam: float, eps: float) -> torch.Tensor:
    """q [n, H, 2, d], k [n, G, 2, d], v [n, G, vd] -> [n, H, vd]."""
    n, H = q.shape[0], q.shape[1]
    G = k.shape[1]
    q = q * query_temperature(n, m.get("q_temp"))[:, None, None, None]
    seen = torch.ones(n, n, dtype=torch.bool).tril()
    cap = m.get("softcap")
    out = torch.empty(n, H, v.shape[-1], dtype=F)
    for h in range(H):
        g = h // (H // G)
        maps = []
        for i in range(2):
            s = q[:, h, i] @ k[:, g, i].T * m["scale"]
            if cap:
                s = cap * torch.tanh(s / cap)
            s = s.masked_fill(~seen, -math.inf)
            maps.append(torch.softmax(s, -1) @ v[:, g])
        out[:, h] = rms(maps[0] - lam * maps[1], eps) * (1.0 - m["diff"])
    return out


def mixer(w, p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    n = h.shape[0]
    H, G, d, vd = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m["vdim"]
    q = (h @ w[p + "q"].to(F).T).view(n, H, 2, d)
    k = (h @ w[p + "k"].to(F).T).view(n, G, 2, d)
    v = (h @ w[p + "v"].to(F).T).view(n, G, vd)
    lam = map_weight(w[p + "lq1"], w[p + "lk1"], w[p + "lq2"], w[p + "lk2"], m["diff"])
    return differential_attention(q, k, v, m, lam, eps).reshape(n, H * vd) @ w[p + "o"].to(F).T


def dense_ff(w, p: str, h: torch.Tensor) -> torch.Tensor:
    return torch.relu(h @ w[p + "up"].to(F).T) ** 2 @ w[p + "down"].to(F).T


def gated_expert(w, p: str, h: torch.Tensor) -> torch.Tensor:
    a = h @ w[p + "gate"].to(F).T
    return (a * torch.sigmoid(a) * (h @ w[p + "up"].to(F).T)) @ w[p + "down"].to(F).T


def route(scores: torch.Tensor, r: dict):
    """scores [n, E] -> (chosen [n, top], weights [n, top], margin [n]): the best `keep` groups
    by the sum of their two largest scores, the `top` largest scores among their experts,
    weights divided by their sum. margin: how far, relative to the scores, the closest call of
    the choice was (between the last group kept and the first left out, and between the last
    expert chosen and the first left out)."""
    n, E = scores.shape
    top = r["top"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    count, keep = groups["count"], groups.get("keep", groups["count"])
    per = E // count
    margin = torch.full((n,), math.inf, dtype=F)
    allowed = torch.ones(n, E, dtype=torch.bool)
    if keep < count:
        gs = scores.view(n, count, per).topk(min(2, per), -1).values.sum(-1)
        order = gs.sort(dim=-1, descending=True, stable=True)
        allowed = torch.zeros(n, count, dtype=torch.bool)
        allowed.scatter_(1, order.indices[:, :keep], True)
        allowed = allowed[:, :, None].expand(n, count, per).reshape(n, E)
        margin = (order.values[:, keep - 1] - order.values[:, keep]) / order.values[:, keep - 1]
    cand = scores.masked_fill(~allowed, -1.0)
    order = cand.sort(dim=-1, descending=True, stable=True)
    chosen, val = order.indices[:, :top], order.values[:, :top]
    if top < int(allowed[0].sum()):
        margin = torch.minimum(margin, (val[:, -1] - order.values[:, top]) / val[:, -1])
    return chosen, val / (val.sum(-1, keepdim=True) + 1e-20), margin


def sparse_ff(w, p: str, c: dict, h: torch.Tensor, margins: Optional[list] = None) -> torch.Tensor:
    scores = torch.sigmoid(h @ w[p + "router"].to(F).T)
    chosen, weights, margin = route(scores, c["router"])
    if margins is not None:
        margins.append(margin)
    out = torch.zeros_like(h)
    for e in range(c["router"]["experts"]):
        rows, col = (chosen == e).nonzero(as_tuple=True)
        if len(rows):
            out[rows] += weights[rows, col, None] * gated_expert(w, f"{p}e{e}.", h[rows])
    if c.get("shared"):
        out = out + torch.sigmoid(h @ w[p + "shared.sg"].to(F).T) * gated_expert(w, p + "shared.", h)
    return out


def layer_order(cfg: dict):
    """(layer, does a pass of the loop begin here) for every run of a layer."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    runs = [(i, False) for i in range(loop["start"])]
    for _ in range(loop["times"]):
        runs += [(i, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, False) for i in range(loop["stop"], n)]


def forward(w: Dict[str, torch.Tensor], cfg: dict, tokens: List[int], streams: Optional[list] = None,
            margins: Optional[list] = None) -> torch.Tensor:
    """Logits [n, vocab]. `streams` receives the residual stream after every layer run,
    `margins` the routing margins [n] of every sparse layer run."""
    eps = cfg["norm"]["eps"]
    x0 = embed(w, cfg, tokens)
    x = x0
    for i, enters in layer_order(cfg):
        layer, p = cfg["layers"][i], f"l{i}."
        if enters:
            x = torch.cat([x, x0], -1) @ w["loop.in"].to(F).T
        h = rms(x, eps) * w[p + "norm1"].to(F)
        y = mixer(w, p + "mix.", layer["mixer"], eps, h) * w[p + "ls1"].to(F)
        c = layer.get("mlp")
        if c:
            f = dense_ff(w, p + "mlp.", h) if c.get("kind", "dense") == "dense" \
                else sparse_ff(w, p + "mlp.", c, h, margins)
            y = y + f * w[p + "ls2"].to(F)
        x = x + y
        if streams is not None:
            streams.append(x)
    logits = (rms(x, eps) * w["final.norm"].to(F)) @ w["embed"].to(F).T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits
