"""Plain, slow float64 implementation of the Mitunex design, one function per
mechanism, written from the design's equations. It shares no code with the
product path (no kllms_amd imports): tests compare the framework against it.

A model is a dict ``cfg`` in the checkpoint's config.json form plus a dict
``w`` of float64 tensors under the checkpoint's tensor names. Every function
works on one sequence, token by token or with explicit loops over positions.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F64 = torch.float64


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dim."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def rotate_pairs(v: torch.Tensor, p: int, base: float, dims: int) -> torch.Tensor:
    """Rotate the first ``dims`` entries of the last dim as pairs (2i, 2i+1)
    by the angle p * base^(-2i/dims); the rest passes unchanged."""
    out = v.clone()
    for i in range(dims // 2):
        a = p * base ** (-2.0 * i / dims)
        c, s = math.cos(a), math.sin(a)
        u, w = v[..., 2 * i], v[..., 2 * i + 1]
        out[..., 2 * i] = u * c - w * s
        out[..., 2 * i + 1] = w * c + u * s
    return out


def visible(i: int, window: Optional[int]) -> List[int]:
    """Positions that position i sees: j <= i, and i - j < window if there is one."""
    lo = 0 if not window else max(0, i - window + 1)
    return list(range(lo, i + 1))


def embed(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    rows = []
    for p, t in enumerate(tokens):
        rows.append(rms(w["embed"][t] + w["pos"][p], cfg["norm"]["eps"]) * w["embed.norm"])
    return torch.stack(rows)


def latent_attention(m: dict, eps: float, w: Dict[str, torch.Tensor], pre: str, h: torch.Tensor) -> torch.Tensor:
    """h [T, W] (the whole sequence from position 0) -> mixer output [T, W]."""
    T = h.shape[0]
    H, D, R, V, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    window = (m.get("mask") or {}).get("size")
    lat, krot, qs = [], [], []
    for p in range(T):
        q = (w[pre + "q"] @ h[p]).view(H, D + R)
        q = torch.cat([q[:, :D], rotate_pairs(q[:, D:], p, base, dims)], -1)
        qs.append(q)
        d = w[pre + "dkv"] @ h[p]
        lat.append(rms(d[:C], eps) * w[pre + "dkv.norm"])
        krot.append(rotate_pairs(d[C:], p, base, dims))
    kn = [(w[pre + "uk"] @ c).view(H, D) for c in lat]       # unrotated keys, per position
    vv = [(w[pre + "uv"] @ c).view(H, V) for c in lat]
    out = []
    for i in range(T):
        js = visible(i, window)
        heads = []
        gate = torch.sigmoid(w[pre + "g"] @ h[i])
        for hd in range(H):
            scores = torch.stack([(qs[i][hd, :D] @ kn[j][hd] + qs[i][hd, D:] @ krot[j]) * m["scale"] for j in js])
            pr = torch.softmax(scores, 0)
            heads.append((pr[:, None] * torch.stack([vv[j][hd] for j in js])).sum(0) * gate[hd])
        out.append(w[pre + "o"] @ torch.cat(heads))
    return torch.stack(out)


def dense_ff(w: Dict[str, torch.Tensor], pre: str, h: torch.Tensor) -> torch.Tensor:
    return torch.stack([w[pre + "down"] @ gelu_tanh(w[pre + "up"] @ x) for x in h])


def glu_expert(w: Dict[str, torch.Tensor], pre: str, x: torch.Tensor) -> torch.Tensor:
    return w[pre + "down"] @ (silu(w[pre + "gate"] @ x) * (w[pre + "up"] @ x))


def route(w_router: torch.Tensor, x: torch.Tensor, top: int):
    """Sigmoid scores; the ``top`` largest (ties to the lower index); weights =
    the chosen scores as they are."""
    s = torch.sigmoid(w_router @ x)
    order = sorted(range(s.numel()), key=lambda e: (-float(s[e]), e))[:top]
    return order, [s[e] for e in order]


def moe_ff(mlp: dict, w: Dict[str, torch.Tensor], pre: str, h: torch.Tensor) -> torch.Tensor:
    out = []
    for x in h:
        idx, wt = route(w[pre + "router"], x, mlp["router"]["top"])
        y = torch.zeros_like(x)
        for e, s in zip(idx, wt):
            y = y + glu_expert(w, f"{pre}e{e}.", s * x)      # the weight scales the expert's INPUT
        if mlp.get("shared"):
            y = y + torch.sigmoid(w[pre + "shared.sg"] @ x)[0] * glu_expert(w, pre + "shared.", x)
        out.append(y)
    return torch.stack(out)


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence; ``layers_out`` collects the
    residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = embed(cfg, w, tokens)
    for i, spec in enumerate(cfg["layers"]):
        src = spec.get("weights_of", i)
        pre = f"l{src}."
        assert spec["type"] == "latent_attention"
        x = x + rms(latent_attention(spec["mixer"], eps, w, pre + "mix.", x), eps) * w[pre + "norm1"]
        mlp = spec.get("mlp")
        if mlp:
            y = dense_ff(w, pre + "mlp.", x) if mlp["kind"] == "dense" else moe_ff(mlp, w, pre + "mlp.", x)
            x = x + rms(y, eps) * w[pre + "norm2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    z = (rms(x, eps) * w["final.norm"]) @ w["head"].T * cfg.get("logit_scale", 1.0)
    cap = cfg.get("logit_softcap")
    if cap:
        z = cap * torch.tanh(z / cap)
    return z


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Random float64 tensors (already rounded to bfloat16 values) under the
    checkpoint's names for a config in config.json form."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, std=None):
        return (torch.randn(o, i, generator=g, dtype=F64) * (std if std is not None else i ** -0.5)).bfloat16().double()

    def vec(n):
        return (1.0 + 0.2 * torch.randn(n, generator=g, dtype=F64)).bfloat16().double()

    w = {"embed": mat(cfg["vocab"], W, 1.0), "pos": mat(cfg.get("max_positions", 2048), W, 0.5),
         "embed.norm": vec(W), "final.norm": vec(W), "head": mat(cfg["vocab"], W)}
    for i, spec in enumerate(cfg["layers"]):
        if spec.get("weights_of", i) != i:
            continue
        m, pre = spec["mixer"], f"l{i}."
        H, D, R, V, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        w[pre + "norm1"] = vec(W)
        w[pre + "mix.q"] = mat(H * (D + R), W)
        w[pre + "mix.dkv"] = mat(C + R, W)
        w[pre + "mix.dkv.norm"] = vec(C)
        w[pre + "mix.uk"] = mat(H * D, C)
        w[pre + "mix.uv"] = mat(H * V, C)
        w[pre + "mix.g"] = mat(H, W)
        w[pre + "mix.o"] = mat(W, H * V)
        mlp = spec.get("mlp")
        if not mlp:
            continue
        w[pre + "norm2"] = vec(W)
        if mlp["kind"] == "dense":
            w[pre + "mlp.up"] = mat(mlp["ff"], W)
            w[pre + "mlp.down"] = mat(W, mlp["ff"])
            continue
        names = [f"e{e}" for e in range(mlp["router"]["experts"])]
        sizes = [mlp["expert"]["ff"]] * len(names)
        if mlp.get("shared"):
            names.append("shared")
            sizes.append(mlp["shared"]["ff"])
            w[pre + "mlp.shared.sg"] = mat(1, W)
        for n, ff in zip(names, sizes):
            w[f"{pre}mlp.{n}.gate"] = mat(ff, W)
            w[f"{pre}mlp.{n}.up"] = mat(ff, W)
            w[f"{pre}mlp.{n}.down"] = mat(W, ff)
        w[pre + "mlp.router"] = mat(mlp["router"]["experts"], W, 1.5 * W ** -0.5)
    return w
