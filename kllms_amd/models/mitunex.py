"""Mitunex: a decoder of post-normed layers
    x <- x + norm1(mixer(x));  x <- x + norm2(ff(x))
over an fp32 residual stream x; both sublayers read x itself, the RMS norm
sits on their output only. The embedding is the token row plus a learned
position row, RMS-normed. Every mixer is latent attention (one cached latent
row per token shared by all heads, a rotated key part beside it, sliding
window, per-head output gate); the feed-forward is a two-matrix gelu layer,
routed experts with sigmoid scores (weights on the experts' inputs, a gated
shared expert), or absent. The config lists the layers one by one; a layer
may name another layer whose weights it uses while keeping a cache of its
own. The logits are scaled and soft-capped: cap * tanh(scale * z / cap).
"""

from __future__ import annotations

import hashlib
import math
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from .. import ops
from ..engine.config import MitunexArchConfig, MitunexLayerSpec
from ..engine.kvcache import LayerCacheSpec, LayerState
from ..parallel.tp import ParallelContext
from .listed import ListedLayerLM
from .llama import ForwardBatch
from .mixers import ActFF, LatentAttention, RoutedExperts, _param


class MitunexLayer(nn.Module):
    def __init__(self, spec: MitunexLayerSpec, hidden: int, eps: float, dtype):
        super().__init__()
        self.norm1 = _param(hidden, dtype=torch.float32)
        self.mix = LatentAttention(spec.attention, hidden, eps, dtype)
        self.mlp = None
        self.norm2 = None
        if spec.mlp is not None:
            self.norm2 = _param(hidden, dtype=torch.float32)
            self.mlp = (ActFF(spec.mlp, hidden, dtype) if spec.mlp.kind == "dense"
                        else RoutedExperts(spec.mlp, hidden, dtype))

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        m = {pre + "norm1": self.norm1}
        m.update(self.mix.checkpoint_map(pre + "mix."))
        if self.mlp is not None:
            m[pre + "norm2"] = self.norm2
            m.update(self.mlp.checkpoint_map(pre + "mlp."))
        return m


class MitunexForCausalLM(ListedLayerLM):
    def __init__(self, cfg: MitunexArchConfig, ctx: Optional[ParallelContext] = None, dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        self.ctx = ctx or ParallelContext()
        assert self.ctx.world_size == 1, "the Mitunex family runs unsharded (tp_size must be 1)"
        self.dtype = dtype
        self.eps = cfg.rms_norm_eps
        W = cfg.hidden_size
        self.embed_tokens = nn.Embedding(cfg.vocab_size, W, dtype=dtype)
        self.embed_tokens.weight.requires_grad_(False)
        self.pos = _param(cfg.max_position_embeddings, W, dtype=dtype)
        self.embed_norm = _param(W, dtype=torch.float32)
        # modules exist for the layers that own weights; a layer run names its module
        self.layers = nn.ModuleDict({str(i): MitunexLayer(sp, W, self.eps, dtype)
                                     for i, sp in enumerate(cfg.layers) if sp.weights_of == i})
        self.runs: List[int] = [sp.weights_of for sp in cfg.layers]
        self.final_norm = _param(W, dtype=torch.float32)
        self.lm_head = nn.Linear(W, cfg.vocab_size, bias=False, dtype=dtype)
        self.lm_head.weight.requires_grad_(False)

    # --- cache layout ---------------------------------------------------------
    def cache_layout(self) -> List[LayerCacheSpec]:
        """One entry per listed layer: a layer that borrows weights still keeps
        its own latent cache."""
        return [self.layers[str(src)].mix.cache_spec() for src in self.runs]

    # --- weights ----------------------------------------------------------------
    def checkpoint_map(self) -> Dict[str, torch.Tensor]:
        m = {"embed": self.embed_tokens.weight, "pos": self.pos, "embed.norm": self.embed_norm,
             "final.norm": self.final_norm, "head": self.lm_head.weight}
        for i, layer in self.layers.items():
            m.update(layer.checkpoint_map(f"l{i}."))
        return m

    @torch.no_grad()
    def random_init_(self, seed: int = 0) -> None:
        """Deterministic random init, one generator per checkpoint name."""
        for name, dst in self.checkpoint_map().items():
            g = torch.Generator(device="cpu")
            g.manual_seed(int(hashlib.md5(f"{seed}/{name}".encode()).hexdigest()[:15], 16))
            leaf = name.split(".")[-1]
            if leaf in ("norm", "norm1", "norm2"):
                t = torch.ones(dst.shape)
            elif leaf == "embed":
                t = torch.randn(dst.shape, generator=g)
            elif leaf == "pos":
                t = torch.randn(dst.shape, generator=g) * 0.3
            else:
                t = torch.randn(dst.shape, generator=g) / math.sqrt(dst.shape[-1])
            dst.copy_(t.to(device=dst.device, dtype=dst.dtype))

    # --- forward ------------------------------------------------------------------
    def forward_hidden(self, input_ids: torch.Tensor, batch: ForwardBatch) -> torch.Tensor:
        assert batch.seg_start is not None, "this model takes segment batches"
        states: List[LayerState] = batch.kv_caches
        eps = self.eps
        exact = self.dtype == torch.float32
        x = ops.embed_rmsnorm(input_ids, self.embed_tokens.weight, self.embed_norm, eps, self.pos, batch.positions)
        # the sublayers read the stream itself: its fp32 rows in exact mode, else their cast
        if not self.runs:
            return ops.rmsnorm_cast(x, self.final_norm, eps, self.dtype)
        h = x if exact else x.to(self.dtype)
        last = len(self.runs) - 1
        for run, src in enumerate(self.runs):
            layer = self.layers[str(src)]
            a = layer.mix(h, batch, states[run])
            end = run == last and layer.mlp is None
            # x += norm1(a); the kernel also writes the next reader's input
            # (the cast stream, or the final norm after the last sublayer)
            h = ops.sandwich_residual(x, a, layer.norm1, eps, w_next=self.final_norm if end else None,
                                      out_dtype=self.dtype, cast=not exact and not end)
            if layer.mlp is not None:
                b = layer.mlp(x if h is None else h)
                end = run == last
                h = ops.sandwich_residual(x, b, layer.norm2, eps, w_next=self.final_norm if end else None,
                                          out_dtype=self.dtype, cast=not exact and not end)
            if self.trace_layers is not None:
                self.trace_layers.append(x.clone())
            if h is None:
                h = x
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        z = self.lm_head(hidden).float()
        ops.scale_softcap_(z, self.cfg.logit_scale, self.cfg.logit_softcap)
        return z
