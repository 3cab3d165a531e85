"""Pironex: a decoder over an fp32 stream x whose sublayers are layer-normed
before and after and read their input through a short causal convolution:
    x <- x + ln_b(sublayer(canon(ln_a(x))))        canon(h)_t = h_t + sum_j c[:, j] h_{t-K+1+j}
(ln = (v - mean) / sqrt(var + eps) * w, no bias). With X_0 the scaled
embedding and X_{i+1} the result of layer i, the stream that goes on after
layer i is sum_{j <= i+1} dwa_i[j] X_j. Mixers, listed layer by layer in the
config: sliding-window attention with pooled blocks before the window
(optionally on the cache of an earlier layer), mamba2, latent attention; the
feed-forward is a mixture of clamped-GLU experts with a gated shared expert,
or absent. The LM head is the embedding table without its scale.

Kernel plan of one layer: ln_canon (norm from the row statistics + input
convolution + cast) -> mixer -> ln_residual_mix (post-norm, residual add, row
statistics for the next norm; after the layer's last sublayer also the depth
average) and the same pair around the feed-forward.
"""

from __future__ import annotations

import hashlib
import math
from typing import Dict, List, Optional

import torch
import torch.nn as nn

from .. import ops
from ..engine.config import PironexArchConfig, PironexLayerSpec
from ..engine.kvcache import LayerCacheSpec, LayerState
from ..parallel.tp import ParallelContext
from .listed import ListedLayerLM
from .llama import ForwardBatch
from .mixers import LatentAttention, Mamba2Mixer, PoolWindowAttention, RoutedExperts, _param


class PironexLayer(nn.Module):
    def __init__(self, spec: PironexLayerSpec, index: int, hidden: int, eps: float, taps: int, dtype):
        super().__init__()
        self.kind = spec.type
        self.norm1 = _param(hidden, dtype=torch.float32)
        self.norm1b = _param(hidden, dtype=torch.float32)
        self.canon1 = _param(taps, hidden, dtype=torch.float32)       # taps-major
        self.dwa = _param(index + 2, dtype=torch.float32)
        if spec.type == "attention":
            self.mix = PoolWindowAttention(spec.attention, hidden, eps, dtype)
        elif spec.type == "mamba2":
            self.mix = Mamba2Mixer(spec.mamba2, hidden, eps, dtype)
        else:
            self.mix = LatentAttention(spec.latent, hidden, eps, dtype)
        self.mlp: Optional[RoutedExperts] = None
        if spec.mlp is not None:
            self.norm2 = _param(hidden, dtype=torch.float32)
            self.norm2b = _param(hidden, dtype=torch.float32)
            self.canon2 = _param(taps, hidden, dtype=torch.float32)
            self.mlp = RoutedExperts(spec.mlp, hidden, dtype)

    def cache_spec(self) -> LayerCacheSpec:
        sp = self.mix.cache_spec()
        taps, hidden = self.canon1.shape
        sp.canon = (2 if self.mlp is not None else 1, hidden, taps - 1)
        return sp

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        m = {pre + "norm1": self.norm1, pre + "norm1b": self.norm1b, pre + "canon1": self.canon1.t(),
             pre + "dwa": self.dwa}
        m.update(self.mix.checkpoint_map(pre + "mix."))
        if self.mlp is not None:
            m[pre + "norm2"] = self.norm2
            m[pre + "norm2b"] = self.norm2b
            m[pre + "canon2"] = self.canon2.t()
            m.update(self.mlp.checkpoint_map(pre + "mlp."))
        return m


class PironexForCausalLM(ListedLayerLM):
    def __init__(self, cfg: PironexArchConfig, ctx: Optional[ParallelContext] = None, dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        self.ctx = ctx or ParallelContext()
        assert self.ctx.world_size == 1, "the Pironex family runs unsharded (tp_size must be 1)"
        self.dtype = dtype
        self.eps = cfg.norm_eps
        W = cfg.hidden_size
        self.embed_tokens = nn.Embedding(cfg.vocab_size, W, dtype=dtype)
        self.embed_tokens.weight.requires_grad_(False)
        self.layers = nn.ModuleList([PironexLayer(sp, i, W, self.eps, cfg.canon_taps, dtype)
                                     for i, sp in enumerate(cfg.layers)])
        self.final_norm = _param(W, dtype=torch.float32)
        # the head is the embedding table itself
        self.lm_head = nn.Linear(W, cfg.vocab_size, bias=False, dtype=dtype)
        self.lm_head.weight = self.embed_tokens.weight

    # --- cache layout ---------------------------------------------------------
    def cache_layout(self) -> List[LayerCacheSpec]:
        return [layer.cache_spec() for layer in self.layers]

    # --- weights ----------------------------------------------------------------
    def checkpoint_map(self) -> Dict[str, torch.Tensor]:
        m = {"embed": self.embed_tokens.weight, "final.norm": self.final_norm}
        for i, layer in enumerate(self.layers):
            m.update(layer.checkpoint_map(f"l{i}."))
        return m

    @torch.no_grad()
    def random_init_(self, seed: int = 0) -> None:
        """Deterministic random init, one generator per checkpoint name:
        matrices ~ N(0, 1/in), norm weights 1, the depth average close to
        'the layer's own result', small convolutions and recurrence constants."""
        for name, dst in self.checkpoint_map().items():
            g = torch.Generator(device="cpu")
            g.manual_seed(int(hashlib.md5(f"{seed}/{name}".encode()).hexdigest()[:15], 16))
            leaf = name.split(".")[-1]
            parts = dst if isinstance(dst, (list, tuple)) else [dst]
            for part in parts:
                if leaf in ("norm", "norm1", "norm2", "norm1b", "norm2b"):
                    t = torch.ones(part.shape)
                elif leaf == "dwa":
                    t = torch.randn(part.shape, generator=g) * 0.05
                    t[-1] += 1.0
                elif leaf in ("canon1", "canon2"):
                    t = torch.randn(part.shape, generator=g) * 0.2
                elif leaf in ("A_log", "dt_bias", "D", "b"):
                    t = torch.randn(part.shape, generator=g) * 0.1
                elif leaf == "conv":
                    t = torch.randn(part.shape, generator=g) * 0.5
                elif leaf == "embed":
                    t = torch.randn(part.shape, generator=g)
                else:
                    t = torch.randn(part.shape, generator=g) / math.sqrt(part.shape[-1])
                part.copy_(t.to(device=part.device, dtype=part.dtype))

    # --- forward ------------------------------------------------------------------
    def forward_hidden(self, input_ids: torch.Tensor, batch: ForwardBatch) -> torch.Tensor:
        assert batch.seg_start is not None, "this model takes segment batches"
        states: List[LayerState] = batch.kv_caches
        eps = self.eps
        T, W = input_ids.numel(), self.cfg.hidden_size
        # X_0 .. X_L, the operands of the depth average
        streams = torch.empty((len(self.layers) + 1, T, W), dtype=torch.float32, device=input_ids.device)
        ops.embed_bigram(input_ids, self.embed_tokens.weight, None, self.cfg.embed_scale, 0, 0, 0, None,
                         batch.state_slots, batch.cu_seqlens, batch.seg_start, batch.token_seg, out=streams[0])
        x = streams[0]
        stats = ops.ln_residual_mix(x, None, None, eps, x)
        cur = torch.empty((T, W), dtype=torch.float32, device=x.device)
        seg = (batch.state_slots, batch.cu_seqlens, batch.seg_start, batch.token_seg)
        for i, layer in enumerate(self.layers):
            st = states[i]
            h = ops.ln_canon(x, stats, layer.norm1, layer.canon1, st.canon[:, 0], *seg, self.dtype)
            a = layer.mix(h, batch, st)
            if layer.mlp is None:
                stats = ops.ln_residual_mix(x, a, layer.norm1b, eps, cur, streams, i + 1, layer.dwa)
            else:
                stats = ops.ln_residual_mix(x, a, layer.norm1b, eps, cur)
                h = ops.ln_canon(cur, stats, layer.norm2, layer.canon2, st.canon[:, 1], *seg, self.dtype)
                b = layer.mlp(h)
                stats = ops.ln_residual_mix(cur, b, layer.norm2b, eps, cur, streams, i + 1, layer.dwa)
            x = cur
            if self.trace_layers is not None:
                self.trace_layers.append(x.clone())
        return ops.ln_canon(x, stats, self.final_norm, None, None, *seg, self.dtype)
