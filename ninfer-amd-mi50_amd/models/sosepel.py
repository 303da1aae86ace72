"""Sosepel put together from parts, layer by layer from its configuration.

x = embed[token] scale + pairs[hash(previous token, token)]; every layer is a parallel block,
x += s1 mixer(norm(x)) + s2 ff(norm(x)), with differential attention as the mixer and, as the
feed-forward, none, a dense one with the square of relu, or routed experts (sigmoid scores,
a choice limited to the best groups by the sum of their two largest scores, weights
renormalised) beside a gated shared expert. Layers `loop.start` .. `loop.stop - 1` run
`loop.times` times in a row, each run with a cache of its own, and every pass begins with
x <- W_in [x ; embedding output]. logits = cap tanh(embed norm(x) / cap): the head is the
embedding table without its scale.
Tensor names: embed, bigram, loop.in, final.norm, and per layer l<i>.{norm1, ls1, ls2,
mix.{q, k, v, o, lq1, lk1, lq2, lk2}, mlp.{up, down} or mlp.{router, e<j>.{gate, up, down},
shared.{gate, up, down, sg}}}.
"""
from __future__ import annotations

from .. import parts  # noqa: F401  (registers the part factories by kind and name)
from ..config.sosepel import SosepelConfig
from ..parts.embedding import LMHead, TokenEmbedding
from ..registry import make_part, register_architecture
from .spec import LayerCall, ModelSpec

# fixed by the design: a group's score sums its two best experts; the renormalised weights'
# divisor gets this much added
GROUP_TOP = 2
RENORM_EPS = 1e-20


def build_sosepel(cfg: SosepelConfig) -> ModelSpec:
    w = cfg.width
    pairs = None
    if cfg.pairs is not None:
        pairs = {"tensor": "bigram", "buckets": cfg.pairs.buckets, "mul_prev": cfg.pairs.mul_prev,
                 "mul_cur": cfg.pairs.mul_cur}
    embedding = TokenEmbedding("embed", cfg.vocab, w, leaf="", scale=cfg.embedding_scale, pairs=pairs)
    blocks = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        m = layer.mixer
        mixer = make_part("mixer", "differential_attention", prefix=p + "mix.", hidden=w,
                          heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale,
                          diff=m.diff, eps=cfg.eps, softcap=m.softcap, temp_coef=m.temp_coef,
                          temp_every=m.temp_every)
        ff = None
        f = layer.mlp
        if f is not None and f.kind == "dense":
            ff = make_part("feed_forward", "mlp", prefix=p + "mlp.", hidden=w, inner=f.ff,
                           act="relu2", names=("up", "down"))
        elif f is not None:
            per_group = f.experts // f.groups
            ff = make_part(
                "feed_forward", "sparse_moe", prefix=p + "mlp.", hidden=w, experts=f.experts,
                top_k=f.top, inner=f.ff, renorm=True, shared_inner=f.shared_ff, act="silu",
                router={"score": "sigmoid", "n_group": f.groups, "topk_group": f.groups_kept,
                        "group_top": min(GROUP_TOP, per_group), "renorm_eps": RENORM_EPS},
                names={"router": "router", "router_leaf": "", "experts": "e",
                       "expert_leaves": ("gate", "up", "down"), "shared": "shared.",
                       "shared_gate": "shared.sg"})
        blocks.append(make_part(
            "block", "parallel", norm=make_part("norm", "rmsnorm", prefix=p + "norm1", size=w,
                                                eps=cfg.eps, leaf=""),
            mixer=mixer, feed_forward=ff, mixer_scale=p + "ls1", ff_scale=p + "ls2", size=w))
    joins = []
    if cfg.loop is not None:
        joins.append(make_part("input", "stream_reentry", tensor="loop.in", hidden=w))
    plan = [LayerCall(i, before=0 if enters else None) for i, enters in cfg.runs()]
    final_norm = make_part("norm", "rmsnorm", prefix="final.norm", size=w, eps=cfg.eps, leaf="")
    head = LMHead("embed", cfg.vocab, w, tied_to=embedding, leaf="", softcap=cfg.logit_softcap)
    return ModelSpec(embedding, blocks, final_norm, head, plan=plan, joins=joins)


register_architecture("Sosepel", SosepelConfig.from_dict, build_sosepel)
