"""Getodra put together from parts, layer by layer from its configuration.

x = embed[token] + pos[position]; per layer x += norm1(mixer(x + conv1(x))), then
x += norm2(ff(x + conv2(x))) with single-gain RMS norms on the sublayers' outputs; the
mixer is latent attention (rotated by scaled frequencies) or lightning attention; the
feed-forward is a gated product with the tanh form of GELU; logits = head(norm(x)). A
layer with `weights_of` runs another layer's parts once more, with a cache and state of
its own: the plan names that layer's block again.
Tensor names: embed, pos, head, final.norm, and per layer l<i>.{norm1, norm2, canon1,
canon2, mix.*, mlp.{gate, up, down}}.
"""
from __future__ import annotations

from .. import parts  # noqa: F401  (registers the part factories by kind and name)
from ..config.getodra import GetodraConfig
from ..parts.embedding import LMHead, TokenEmbedding
from ..registry import make_part, register_architecture
from .spec import LayerCall, ModelSpec


def build_getodra(cfg: GetodraConfig) -> ModelSpec:
    w = cfg.width
    embedding = TokenEmbedding("embed", cfg.vocab, w, positions=cfg.max_positions,
                               position_prefix="pos", leaf="")
    blocks, block_of, plan = [], {}, []
    for i, layer in enumerate(cfg.layers):
        owner = cfg.owner(i)
        if owner == i:
            p = f"l{i}."
            m = layer.mixer
            if layer.type == "latent_attention":
                if m.rot_dims:
                    s = m.rot_scaling
                    position = make_part(
                        "position", "rotary", rot_dim=m.rot_dims, theta=m.rot_base,
                        scaling=None if s is None else {
                            "factor": s.factor, "original": s.original, "fast": s.fast,
                            "slow": s.slow})
                else:
                    position = make_part("position", "none")
                mixer = make_part("mixer", "latent_attention", prefix=p + "mix.", hidden=w,
                                  heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim,
                                  kv_rank=m.kv_rank, scale=m.scale, eps=cfg.eps, position=position)
            else:
                mixer = make_part("mixer", "lightning", prefix=p + "mix.", hidden=w, heads=m.heads,
                                  dim=m.dim, vdim=m.vdim, decay=m.decay, eps=cfg.eps)
            ff = ff_norm = ff_input = None
            if layer.ff is not None:
                ff = make_part("feed_forward", "swiglu", prefix=p + "mlp.", hidden=w,
                               inner=layer.ff, act="gelu_pytorch_tanh",
                               names=("gate", "up", "down"))
                ff_norm = make_part("norm", "output_rmsnorm", tensor=p + "norm2", size=w, eps=cfg.eps)
                ff_input = make_part("input", "short_conv", tensor=p + "canon2", channels=w,
                                     taps=cfg.taps)
            block_of[i] = len(blocks)
            blocks.append(make_part(
                "block", "output_norm", mixer=mixer,
                mixer_norm=make_part("norm", "output_rmsnorm", tensor=p + "norm1", size=w, eps=cfg.eps),
                feed_forward=ff, ff_norm=ff_norm,
                mixer_input=make_part("input", "short_conv", tensor=p + "canon1", channels=w,
                                      taps=cfg.taps),
                ff_input=ff_input))
    for i in range(len(cfg.layers)):
        plan.append(LayerCall(block_of[cfg.owner(i)]))
    final_norm = make_part("norm", "rmsnorm", prefix="final.norm", size=w, eps=cfg.eps, leaf="",
                           single_gain=True)
    head = LMHead("head", cfg.vocab, w, leaf="")
    return ModelSpec(embedding, blocks, final_norm, head, plan=plan)


register_architecture("Getodra", GetodraConfig.from_dict, build_getodra)
