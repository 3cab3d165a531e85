"""Shared base of the models whose layers are listed one by one in the
checkpoint's config and that keep per-sequence state (recurrent matrices,
convolution or token-shift history) beside the paged attention cache. Such a
model runs "segment" batches only (ForwardBatch.seg_start etc.): prompt
portions, decoded tokens and mixes of both take the same path.

A subclass provides ``checkpoint_map()`` (checkpoint tensor name -> parameter
or slice of a fused parameter), ``cache_layout()`` (one LayerCacheSpec per
entry of the state cache), ``forward_hidden()`` and an ``lm_head``.
"""

from __future__ import annotations

from typing import Dict, Iterable, Optional, Tuple

import torch
import torch.nn as nn


class ListedLayerLM(nn.Module):
    # the engine keeps a recurrent-state slot per sequence and feeds segment
    # batches; prefix-block reuse is off (state cannot be rebuilt from blocks)
    stateful = True

    trace_layers: Optional[list] = None   # debugging: residual after each layer run

    def checkpoint_map(self) -> Dict[str, torch.Tensor]:
        raise NotImplementedError

    def _after_load(self) -> None:
        """Hook: fix up derived parameters once the tensors are in place."""

    @torch.no_grad()
    def load_named_tensors_(self, named: Iterable[Tuple[str, torch.Tensor]]) -> None:
        m = self.checkpoint_map()
        seen = set()
        for name, t in named:
            dst = m.get(name)
            if dst is None:
                raise RuntimeError(f"checkpoint tensor {name!r} has no place in this model")
            # a list: the checkpoint tensor's rows are dealt to several parameter slices in turn
            parts = dst if isinstance(dst, (list, tuple)) else [dst]
            shape = (sum(d.shape[0] for d in parts),) + tuple(parts[0].shape[1:])
            if shape != tuple(t.shape) or any(tuple(d.shape[1:]) != shape[1:] for d in parts):
                raise RuntimeError(f"{name}: checkpoint shape {tuple(t.shape)} != model {shape}")
            r = 0
            for d in parts:
                d.copy_(t[r:r + d.shape[0]].to(d.dtype))
                r += d.shape[0]
            seen.add(name)
        missing = sorted(set(m) - seen)
        if missing:
            raise RuntimeError(f"checkpoint left {len(missing)} tensors unassigned: {missing[:6]}")
        self._after_load()

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return self.lm_head(hidden).float()

    def forward_prefill(self, input_ids: torch.Tensor, batch) -> torch.Tensor:
        """Logits of the LAST row of each segment: [n_seg, V]."""
        hidden = self.forward_hidden(input_ids, batch)
        last_idx = (batch.cu_seqlens[1:] - 1).long()
        return self.compute_logits(hidden[last_idx])

    def forward_decode(self, input_ids: torch.Tensor, batch) -> torch.Tensor:
        return self.compute_logits(self.forward_hidden(input_ids, batch))

    def to_device(self, device):
        self.to(device)
        return self
