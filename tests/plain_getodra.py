"""A plain, slow implementation of the Getodra design in 64-bit floats, one function per
mechanism, written from the design's equations. It shares nothing with the engine: whole
sequences, no cache, no state, no kernels. The tests compare the engine with it."""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square over the last dimension (eps inside the root)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def input_conv(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """h + conv(h): conv(h)[t] = sum_j w[:, j] * h[t - taps + 1 + j], zeros before row 0."""
    n, taps = h.shape[0], w.shape[1]
    out = h.clone()
    for t in range(n):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * h[src]
    return out


def rotary_table(rot: dict):
    """(frequency of every pair, factor on cosine and sine)."""
    n, base = rot["dims"], rot["base"]
    freq = [base ** (-2.0 * i / n) for i in range(n // 2)]
    factor_on_trig = 1.0
    sc = rot.get("scaling")
    if sc:
        def place(turns):
            return n * math.log(sc["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(place(sc["fast"])), 0)
        hi = min(math.ceil(place(sc["slow"])), n - 1)
        for i in range(n // 2):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            freq[i] = freq[i] / sc["factor"] * ramp + freq[i] * (1.0 - ramp)
        factor_on_trig = 0.1 * math.log(sc["factor"]) + 1.0
    return torch.tensor(freq, dtype=F), factor_on_trig


def turn(v: torch.Tensor, rot: Optional[dict]) -> torch.Tensor:
    """v [T, ..., m]: the first rot['dims'] numbers of the last dimension turn, pair
    (i, i + dims/2) by position * frequency_i; the rest pass."""
    if not rot or not rot.get("dims"):
        return v
    n = rot["dims"]
    freq, mag = rotary_table(rot)
    pos = torch.arange(v.shape[0], dtype=F)
    ang = pos[:, None] * freq[None, :]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [n // 2]
    c, s = (torch.cos(ang) * mag).reshape(shape), (torch.sin(ang) * mag).reshape(shape)
    a, b = v[..., :n // 2], v[..., n // 2:n]
    out = v.clone()
    out[..., :n // 2] = a * c - b * s
    out[..., n // 2:n] = b * c + a * s
    return out


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                     probabilities: Optional[list] = None) -> torch.Tensor:
    n = h.shape[0]
    H, dim, rd, vd, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w[p + "q"].T).reshape(n, H, dim + rd)
    down = h @ w[p + "dkv"].T
    c = rms_unit(down[:, :R], eps) * w[p + "dkv.norm"]
    k_rot = turn(down[:, R:], m.get("rot"))
    q_rot = turn(q[..., dim:], m.get("rot"))
    keys = (c @ w[p + "uk"].T).reshape(n, H, dim)
    values = (c @ w[p + "uv"].T).reshape(n, H, vd)
    gate = torch.sigmoid(h @ w[p + "g"].T)
    out = torch.zeros(n, H, vd, dtype=F)
    for t in range(n):
        for hh in range(H):
            s = (keys[:t + 1, hh] @ q[t, hh, :dim] + k_rot[:t + 1] @ q_rot[t, hh]) * m["scale"]
            pr = torch.softmax(s, 0)
            if probabilities is not None:
                probabilities.append((t, hh, pr))
            out[t, hh] = (pr[:, None] * values[:t + 1, hh]).sum(0) * gate[t, hh]
    return out.reshape(n, H * vd) @ w[p + "o"].T


def lightning_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict,
                        eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, dim, vd = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + "q"].T).reshape(n, H, dim)
    k = silu(h @ w[p + "k"].T).reshape(n, H, dim)
    v = silu(h @ w[p + "v"].T).reshape(n, H, vd)
    out = torch.zeros(n, H, vd, dtype=F)
    for hh in range(H):
        S = torch.zeros(dim, vd, dtype=F)
        for t in range(n):
            S = m["decay"][hh] * S + torch.outer(k[t, hh], v[t, hh])
            out[t, hh] = S.T @ q[t, hh]
    o = rms_unit(out.reshape(n, H * vd), eps) * w[p + "norm"]
    return (o * torch.sigmoid(h @ w[p + "g"].T)) @ w[p + "o"].T


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def forward(w32: Dict[str, torch.Tensor], cfg: dict, tokens: List[int],
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [len(tokens), vocab] (32-bit) of one whole sequence."""
    w = {k: v.to(F) for k, v in w32.items()}
    eps = cfg["norm"]["eps"]
    n = len(tokens)
    x = w["embed"][torch.tensor(tokens)] + w["pos"][:n]
    for i, layer in enumerate(cfg["layers"]):
        j = i
        while cfg["layers"][j].get("weights_of") is not None:
            j = cfg["layers"][j]["weights_of"]
        p = f"l{j}."
        h = input_conv(x, w[p + "canon1"])
        mix = latent_attention if layer["type"] == "latent_attention" else lightning_attention
        x = x + rms_unit(mix(h, w, p + "mix.", layer["mixer"], eps), eps) * w[p + "norm1"]
        if layer.get("mlp") is not None:
            h = input_conv(x, w[p + "canon2"])
            x = x + rms_unit(dense_ff(h, w, p + "mlp."), eps) * w[p + "norm2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms_unit(x, eps) * w["final.norm"]
    return (x @ w["head"].T).to(torch.float32)
