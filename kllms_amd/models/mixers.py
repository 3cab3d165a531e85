"""Sequence mixers and feed-forward blocks with their constants as
parameters: block-local softmax attention over the paged cache, decayed
linear attention, the gated delta rule with per-channel decay and short
convolutions, the clamped GLU; windowed attention with kept first tokens and
a sink, the wkv and mlstm recurrences, routed experts; latent attention and
the two-matrix gelu feed-forward. Each runs on "segment" batches
(ForwardBatch.seg_start / state_slots / token_seg): any mix of prompt
portions and single decoded tokens, attention keys found through the block
table and recurrent state carried in per-sequence slots.

GEMMs go through F.linear (hipBLASLt / rocBLAS); everything between them is a
kllms_amd.ops kernel. Activations are the model dtype (bf16 when serving,
fp32 in exact mode); norm weights, recurrence constants, attention weights
and recurrent state are fp32 in both.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..engine.config import (ActFFSpec, BlockAttnSpec, ChannelDeltaSpec, DecayLinearAttnSpec, GluSpec,
                             LatentAttnSpec, Mamba2Spec, MaskedAttnSpec, MlstmSpec, ParallelMixerSpec,
                             PoolWindowAttnSpec, RotarySpec, RoutedExpertsSpec, WkvSpec)
from ..engine.kvcache import LayerCacheSpec, LayerState


def _param(*shape, dtype) -> nn.Parameter:
    return nn.Parameter(torch.empty(*shape, dtype=dtype), requires_grad=False)


def rotary_inv_freq(rot: RotarySpec) -> torch.Tensor:
    """fp32 [dims/2] frequencies base^(-2i/dims), with the banded rescale:
    wavelengths shorter than original/high keep their frequency, longer than
    original/low are slowed by ``factor``, the band between blends the two
    linearly in original/wavelength."""
    n = rot.dims // 2
    f = [float(rot.base) ** (-2.0 * i / rot.dims) for i in range(n)]
    sc = rot.scaling
    if sc:
        fac, lo, hi, orig = (float(sc[k]) for k in ("factor", "low", "high", "original"))
        out = []
        for fi in f:
            wl = 2.0 * math.pi / fi
            if wl < orig / hi:
                out.append(fi)
            elif wl > orig / lo:
                out.append(fi / fac)
            else:
                s = (orig / wl - lo) / (hi - lo)
                out.append((1.0 - s) * fi / fac + s * fi)
        f = out
    return torch.tensor(f, dtype=torch.float64).to(torch.float32)


class FusedInput(nn.Module):
    """Several projections of the same input as ONE GEMM: the checkpoint's
    separate [out_i, in] matrices are stacked along the output dim (optionally
    with a bias that is zero where a part has none). ``parts`` keeps each
    name's column range; ``split`` returns row views of the result. Every
    part starts at a multiple of 8 columns and the total width is one too
    (zero rows in between), so the views stay 16-byte aligned for the
    kernels' vector loads whatever the part sizes are."""

    ALIGN = 8

    def __init__(self, in_features: int, parts: List[Tuple[str, int]], dtype, bias_parts=()):
        super().__init__()
        self.parts: Dict[str, Tuple[int, int]] = {}
        off = 0
        for name, n in parts:
            self.parts[name] = (off, n)
            off = (off + n + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        self.weight = nn.Parameter(torch.zeros(off, in_features, dtype=dtype), requires_grad=False)
        self.bias = nn.Parameter(torch.zeros(off, dtype=dtype), requires_grad=False) if bias_parts else None
        self.bias_parts = tuple(bias_parts)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(x, self.weight, self.bias)

    def split(self, y: torch.Tensor, name: str) -> torch.Tensor:
        off, n = self.parts[name]
        return y[:, off:off + n]

    def slot(self, name: str) -> torch.Tensor:
        off, n = self.parts[name]
        return self.weight[off:off + n]

    def bias_slot(self, name: str) -> torch.Tensor:
        off, n = self.parts[name]
        return self.bias[off:off + n]


class BlockLocalAttention(nn.Module):
    """GQA softmax attention whose causal mask is cut into aligned blocks of
    ``mask_size`` positions (counted from the start of the sequence), rotary on
    the first ``rot.dims`` dims (interleaved pairs), values optionally taken
    from the un-rotated keys, per-head sigmoid output gate. Projections are
    owned by the enclosing mixer (they share its fused input GEMM)."""

    def __init__(self, spec: BlockAttnSpec, hidden: int, dtype):
        super().__init__()
        assert spec.heads % spec.kv_heads == 0
        if spec.values_from_keys:
            assert spec.vdim == spec.dim, "values taken from keys need vdim == dim"
        self.spec = spec
        self.o_proj = _param(hidden, spec.heads * spec.vdim, dtype=dtype)
        self.register_buffer("inv_freq", rotary_inv_freq(spec.rot), persistent=False)

    def cache_spec(self) -> Tuple[int, int, int]:
        return (self.spec.kv_heads, self.spec.dim, self.spec.vdim)

    # pieces shorter than this stay on the paged kernel
    MIN_DENSE_ROWS = 32

    def _dense_plan(self, q: torch.Tensor, batch):
        """Split the step's rows between the dense MFMA prefill kernel and the
        paged kernel. A run of rows whose whole visible block lies inside this
        step (it starts at a block boundary of the mask, or at position 0 for
        a plain causal mask) is a 'piece': plain causal attention over fresh
        rows. Rows that continue a block begun in an earlier step, and short
        pieces, read their keys through the block table instead. Returns
        (tile groups, row_map or None), or None when nothing goes dense."""
        sp = self.spec
        if (batch.host_segs is None or not q.is_cuda or q.dtype != torch.bfloat16
                or sp.dim != 128 or sp.vdim != 128 or ops._force_torch()
                or q.stride(0) % 8 or q.data_ptr() % 16):      # the dense kernel loads 16 bytes at a time
            return None
        key = ("blocklocal", sp.mask_size)
        if key in batch.plans:
            return batch.plans[key]
        M = sp.mask_size
        pieces, paged = [], []
        row0 = 0
        for start, n in batch.host_segs:
            r = 0
            if M > 0 and start % M:
                r = min(n, M - start % M)
            elif M == 0 and start > 0:
                r = n
            paged.extend(range(row0, row0 + r))
            while r < n:
                L = min(M, n - r) if M > 0 else n - r
                if L >= self.MIN_DENSE_ROWS:
                    pieces.append((row0 + r, L))
                else:
                    paged.extend(range(row0 + r, row0 + r + L))
                r += L
            row0 += n
        plan = None
        if pieces:
            row_map = torch.tensor(paged, dtype=torch.int32, device=q.device) if paged else None
            plan = (ops.dense_tile_groups(pieces, q.device), row_map)
        batch.plans[key] = plan
        return plan

    def forward(self, q, k, v, gate, batch, st: LayerState) -> torch.Tensor:
        sp = self.spec
        T = q.shape[0]
        q = q.unflatten(1, (sp.heads, sp.dim))
        k = k.unflatten(1, (sp.kv_heads, sp.dim))
        if v is not None:
            v = v.unflatten(1, (sp.kv_heads, sp.vdim))
        plan = self._dense_plan(q, batch)
        if plan is None:
            ops.rope_pairs_store(q, k, v, batch.positions, self.inv_freq, st.k, st.v, batch.slot_mapping)
            att = ops.attn_blocklocal_paged(q, st.k, st.v, batch.block_tables, batch.token_seg,
                                            batch.positions, sp.scale, sp.mask_size, gate)
        else:
            (gs, gq, gl), row_map = plan
            fresh = torch.empty((T, 2, sp.kv_heads, sp.dim), dtype=q.dtype, device=q.device)
            ops.rope_pairs_store(q, k, v, batch.positions, self.inv_freq, st.k, st.v, batch.slot_mapping,
                                 kv_fresh=fresh)
            att = torch.empty((T, sp.heads, sp.vdim), dtype=q.dtype, device=q.device)
            ops.attn_varlen_mfma(att, q, fresh[:, 0], fresh[:, 1], gs, gq, gl, sp.scale)
            if row_map is not None:
                ops.attn_blocklocal_paged(q, st.k, st.v, batch.block_tables, batch.token_seg, batch.positions,
                                          sp.scale, sp.mask_size, None, row_map=row_map, out=att)
            if gate is not None:
                ops.head_gate(att, gate)
        return F.linear(att.reshape(T, -1), self.o_proj)


class DecayLinearAttention(nn.Module):
    """S <- decay_h S + k v^T, o = S^T q with silu on q, k, v; the heads'
    outputs are RMS-normed together, gated by sigmoid(g) and projected."""

    def __init__(self, spec: DecayLinearAttnSpec, hidden: int, eps: float, dtype):
        super().__init__()
        assert len(spec.decay) == spec.heads
        self.spec = spec
        self.eps = eps
        self.norm = _param(spec.heads * spec.vdim, dtype=torch.float32)
        self.o_proj = _param(hidden, spec.heads * spec.vdim, dtype=dtype)
        self.register_buffer("decay", torch.tensor(spec.decay, dtype=torch.float64).to(torch.float32),
                             persistent=False)

    def cache_spec(self) -> Tuple[int, int, int]:
        return (self.spec.heads, self.spec.dim, self.spec.vdim)

    def forward(self, q, k, v, gate, batch, st: LayerState) -> torch.Tensor:
        sp = self.spec
        o = ops.linear_attn_decay(q.unflatten(1, (sp.heads, sp.dim)), k.unflatten(1, (sp.heads, sp.dim)),
                                  v.unflatten(1, (sp.heads, sp.vdim)), self.decay, st.rec,
                                  batch.state_slots, batch.cu_seqlens, batch.seg_start)
        y = ops.gated_rmsnorm(o.view(o.shape[0], 1, -1), self.norm, gate, self.eps, self.o_proj.dtype)
        return F.linear(y, self.o_proj)


class ParallelMixer(nn.Module):
    """Block-local softmax attention and decayed linear attention side by
    side on the same input. Returns both branch outputs with their merge
    weights; the caller's fused epilogue forms
    (rms(left) w_left + rms(right) w_right) / 2."""

    def __init__(self, spec: ParallelMixerSpec, hidden: int, eps: float, dtype):
        super().__init__()
        le, ri = spec.left, spec.right
        parts = [("left.q", le.heads * le.dim), ("left.k", le.kv_heads * le.dim)]
        if not le.values_from_keys:
            parts.append(("left.v", le.kv_heads * le.vdim))
        parts += [("right.q", ri.heads * ri.dim), ("right.k", ri.heads * ri.dim),
                  ("right.v", ri.heads * ri.vdim), ("right.g", ri.heads * ri.vdim)]
        if le.head_gate:
            parts.append(("left.g", le.heads))          # odd-sized part last: the others stay aligned
        self.inp = FusedInput(hidden, parts, dtype, bias_parts=("left.q", "left.k") if le.qk_bias else ())
        self.left = BlockLocalAttention(le, hidden, dtype)
        self.right = DecayLinearAttention(ri, hidden, eps, dtype)
        self.left_out = _param(hidden, dtype=torch.float32)
        self.right_out = _param(hidden, dtype=torch.float32)

    def cache_spec(self) -> LayerCacheSpec:
        return LayerCacheSpec(kv=self.left.cache_spec(), rec=self.right.cache_spec())

    def forward(self, h: torch.Tensor, batch, st: LayerState):
        y = self.inp(h)
        s = self.inp.split
        le = self.left.spec
        left = self.left(s(y, "left.q"), s(y, "left.k"),
                         None if le.values_from_keys else s(y, "left.v"),
                         s(y, "left.g") if le.head_gate else None, batch, st)
        right = self.right(s(y, "right.q"), s(y, "right.k"), s(y, "right.v"), s(y, "right.g"), batch, st)
        return left, right

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        m = {pre + n: self.inp.slot(n) for n in self.inp.parts}
        for n in self.inp.bias_parts:
            m[pre + n + ".b"] = self.inp.bias_slot(n)
        m[pre + "left.o"] = self.left.o_proj
        m[pre + "right.o"] = self.right.o_proj
        m[pre + "right.norm"] = self.right.norm
        m[pre + "left.out"] = self.left_out
        m[pre + "right.out"] = self.right_out
        return m


class ChannelDeltaMixer(nn.Module):
    """Gated delta rule with one decay per head and key channel:
        g = exp(-exp(A_h) softplus(W_a2 W_a1 h + dt));  S <- g (.) S
        u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
    q/k/v pass a short causal convolution + silu; q, k are unit-normalised;
    each head's o is RMS-normed, gated by sigmoid(W_g2 W_g1 h) and projected."""

    def __init__(self, spec: ChannelDeltaSpec, hidden: int, eps: float, dtype):
        super().__init__()
        assert spec.heads % spec.kv_heads == 0
        self.spec = spec
        self.eps = eps
        self.gd, self.hv = spec.kv_heads * spec.dim, spec.heads * spec.vdim
        self.inp = FusedInput(hidden, [("q", self.gd), ("k", self.gd), ("v", self.hv),
                                       ("a1", spec.decay_rank), ("g1", spec.gate_rank), ("b", spec.heads)], dtype)
        # the convolution runs over the fused projection's q|k|v column range as it
        # is laid out (alignment gaps included: zero taps there); weights are
        # taps-major [K, C] (the checkpoint's [C, K] transposed: the kernels read 8
        # channels of one tap at a time)
        p = self.inp.parts
        self.oq, self.ok, self.ov = p["q"][0], p["k"][0], p["v"][0]
        self.cp = self.ov + self.hv
        self.conv = nn.Parameter(torch.zeros(spec.conv, self.cp, dtype=torch.float32), requires_grad=False)
        self.a2 = _param(spec.heads * spec.dim, spec.decay_rank, dtype=dtype)
        self.g2 = _param(self.hv, spec.gate_rank, dtype=dtype)
        self.dt_bias = _param(spec.heads * spec.dim, dtype=torch.float32)
        self.A_log = _param(spec.heads, dtype=torch.float32)
        self.norm = _param(spec.vdim, dtype=torch.float32)
        self.o_proj = _param(hidden, self.hv, dtype=dtype)

    def cache_spec(self) -> LayerCacheSpec:
        sp = self.spec
        return LayerCacheSpec(rec=(sp.heads, sp.dim, sp.vdim), conv=(self.cp, sp.conv - 1))

    def forward(self, h: torch.Tensor, batch, st: LayerState) -> torch.Tensor:
        sp = self.spec
        y = self.inp(h)
        s = self.inp.split
        qkv = ops.causal_conv_silu(y[:, :self.cp], self.conv, st.conv, batch.state_slots, batch.cu_seqlens,
                                   batch.seg_start, batch.token_seg)
        a = F.linear(s(y, "a1"), self.a2)
        gate = F.linear(s(y, "g1"), self.g2)
        o = ops.gated_delta_rule(
            qkv[:, self.oq:self.oq + self.gd].unflatten(1, (sp.kv_heads, sp.dim)),
            qkv[:, self.ok:self.ok + self.gd].unflatten(1, (sp.kv_heads, sp.dim)),
            qkv[:, self.ov:self.ov + self.hv].unflatten(1, (sp.heads, sp.vdim)),
            s(y, "b"), a, self.dt_bias, self.A_log, st.rec, batch.state_slots, batch.cu_seqlens,
            batch.seg_start)
        r = ops.gated_rmsnorm(o, self.norm, gate, self.eps, self.o_proj.dtype)
        return F.linear(r, self.o_proj)

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        m = {pre + n: self.inp.slot(n) for n in self.inp.parts}
        ct = self.conv.t()
        m[pre + "q.conv"] = ct[self.oq:self.oq + self.gd]
        m[pre + "k.conv"] = ct[self.ok:self.ok + self.gd]
        m[pre + "v.conv"] = ct[self.ov:self.ov + self.hv]
        for n in ("a2", "g2", "dt_bias", "A_log", "norm"):
            m[pre + n] = getattr(self, n)
        m[pre + "o"] = self.o_proj
        return m


class ClampedGLU(nn.Module):
    """y = W_down [ g sigmoid(alpha g) (u + 1) ], g = min(W_gate h, limit),
    u = clamp(W_up h, -limit, limit); gate and up share one GEMM."""

    def __init__(self, spec: GluSpec, hidden: int, dtype):
        super().__init__()
        self.spec = spec
        self.inp = FusedInput(hidden, [("gate", spec.ff), ("up", spec.ff)], dtype)
        self.down = _param(hidden, spec.ff, dtype=dtype)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        y = self.inp(h)
        act = ops.clamped_glu(self.inp.split(y, "gate"), self.inp.split(y, "up"),
                              self.spec.limit, self.spec.alpha)
        return F.linear(act, self.down)

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        return {pre + "gate": self.inp.slot("gate"), pre + "up": self.inp.slot("up"), pre + "down": self.down}


class WindowSinkAttention(nn.Module):
    """GQA softmax attention over the paged cache with a sliding window that
    also keeps the first tokens, a sink term in the denominator, an RMS norm on
    every q and k head, no rotation, and an elementwise sigmoid gate on the
    concatenated heads. q, k, v and the gate share one input GEMM."""

    def __init__(self, spec: MaskedAttnSpec, hidden: int, eps: float, dtype):
        super().__init__()
        assert spec.heads % spec.kv_heads == 0
        self.spec = spec
        self.eps = eps
        self.inp = FusedInput(hidden, [("q", spec.heads * spec.dim), ("k", spec.kv_heads * spec.dim),
                                       ("v", spec.kv_heads * spec.vdim), ("g", spec.heads * spec.vdim)], dtype)
        self.q_norm = _param(spec.dim, dtype=torch.float32)
        self.k_norm = _param(spec.dim, dtype=torch.float32)
        self.o_proj = _param(hidden, spec.heads * spec.vdim, dtype=dtype)

    def cache_spec(self) -> LayerCacheSpec:
        sp = self.spec
        return LayerCacheSpec(kv=(sp.kv_heads, sp.dim, sp.vdim))

    def forward(self, h: torch.Tensor, batch, st: LayerState) -> torch.Tensor:
        sp = self.spec
        T = h.shape[0]
        y = self.inp(h)
        s = self.inp.split
        q = s(y, "q").unflatten(1, (sp.heads, sp.dim))
        k = s(y, "k").unflatten(1, (sp.kv_heads, sp.dim))
        v = s(y, "v").unflatten(1, (sp.kv_heads, sp.vdim))
        ops.qk_norm_store(q, k, v, self.q_norm, self.k_norm, self.eps, st.k, st.v, batch.slot_mapping)
        att = ops.attn_window_sink(q, st, batch, sp, s(y, "g"))
        return F.linear(att.reshape(T, -1), self.o_proj)

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        m = {pre + n: self.inp.slot(n) for n in self.inp.parts}
        m[pre + "q.norm"] = self.q_norm
        m[pre + "k.norm"] = self.k_norm
        m[pre + "o"] = self.o_proj
        return m


class LatentAttention(nn.Module):
    """Softmax attention over one shared latent row per token. The input's
    down-projection gives the latent c (RMS-normed, kv_rank wide) and one
    rotated key part shared by the heads; only [c | rotated part] is cached
    (one paged row per token). Per head the key is [W_uk c | rotated part] and
    the value W_uv c, so with q = [q_n | q_r]
        score_j = (q_n . W_uk c_j + q_r . kr_j) scale = ((W_uk^T q_n) . c_j + q_r . kr_j) scale
        out     = W_uv sum_j p_j c_j
    and the attention proper runs in the latent space for all heads against
    the same cached rows: W_uk is applied to the queries before it (one
    batched product over the heads) and W_uv to its result. Sliding causal
    window, per-head sigmoid output gate; q, the down-projection and the gate
    share one input GEMM."""

    def __init__(self, spec: LatentAttnSpec, hidden: int, eps: float, dtype):
        super().__init__()
        assert spec.rot.dims == spec.rot_dim and spec.rot_dim % 2 == 0
        self.spec = spec
        self.eps = eps
        H, D, R, V, C = spec.heads, spec.dim, spec.rot_dim, spec.vdim, spec.kv_rank
        parts = [("q", H * (D + R)), ("dkv", C + R)]
        if spec.head_gate:
            parts.append(("g", H))
        self.inp = FusedInput(hidden, parts, dtype)
        self.dkv_norm = _param(C, dtype=torch.float32)
        self.uk = _param(H, D, C, dtype=dtype)
        self.uv = _param(H, V, C, dtype=dtype)
        self.o_proj = _param(hidden, H * V, dtype=dtype)
        self.register_buffer("inv_freq", rotary_inv_freq(spec.rot), persistent=False)

    def cache_spec(self) -> LayerCacheSpec:
        sp = self.spec
        return LayerCacheSpec(kv=(1, sp.kv_rank + sp.rot_dim, 0))

    def forward(self, h: torch.Tensor, batch, st: LayerState) -> torch.Tensor:
        sp = self.spec
        T = h.shape[0]
        H, D, R, V = sp.heads, sp.dim, sp.rot_dim, sp.vdim
        y = self.inp(h)
        s = self.inp.split
        q = s(y, "q").unflatten(1, (H, D + R))
        ops.latent_kv_store(q, s(y, "dkv"), self.dkv_norm, self.eps, batch.positions, self.inv_freq, st.k,
                            batch.slot_mapping, D)
        q_abs = torch.bmm(q[:, :, :D].transpose(0, 1), self.uk)                   # [H, T, C]
        # a step of single decoded tokens: one row per workgroup, a row's keys shared out over the chip
        single = batch.mode == "decode" or (batch.host_segs is not None
                                            and all(n == 1 for _, n in batch.host_segs))
        lat = ops.attn_latent_paged(q_abs.transpose(0, 1), q, st.k, batch.block_tables, batch.token_seg,
                                    batch.positions, sp.scale, sp.mask_size,
                                    s(y, "g") if sp.head_gate else None, D,
                                    tile_rows=1 if single else 0)                 # [T, H, C]
        att = torch.empty((T, H * V), dtype=y.dtype, device=y.device)
        torch.bmm(lat.transpose(0, 1), self.uv.transpose(1, 2), out=att.view(T, H, V).transpose(0, 1))
        return F.linear(att, self.o_proj)

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        m = {pre + n: self.inp.slot(n) for n in self.inp.parts}
        m[pre + "dkv.norm"] = self.dkv_norm
        m[pre + "uk"] = self.uk.view(-1, self.spec.kv_rank)
        m[pre + "uv"] = self.uv.view(-1, self.spec.kv_rank)
        m[pre + "o"] = self.o_proj
        return m


class PoolWindowAttention(nn.Module):
    """GQA softmax attention over the paged cache: a sliding window of
    ``mask_size`` tokens and, before it, one pooled key / value per aligned
    run of ``pool`` tokens that the window has left behind entirely (the fp32
    means of the run's cached keys and values, kept in a pooled cache that is
    filled whenever a step completes a run). q and k are RMS-normed over the
    whole projection, then rotated (entry i with i + dims/2); scores are
    soft-capped. A layer with ``kv_from`` projects queries only and reads the
    keys and values another layer cached in this step; its pooled cache is
    its own (its run length may differ)."""

    def __init__(self, spec: PoolWindowAttnSpec, hidden: int, eps: float, dtype):
        super().__init__()
        assert spec.heads % spec.kv_heads == 0 and spec.rot.dims % 2 == 0 and spec.rot.dims <= spec.dim
        assert spec.rot.layout == "half" and not spec.rot.scaling
        self.spec = spec
        self.eps = eps
        self.own_kv = spec.kv_from is None
        parts = [("q", spec.heads * spec.dim)]
        if self.own_kv:
            parts += [("k", spec.kv_heads * spec.dim), ("v", spec.kv_heads * spec.vdim)]
        self.inp = FusedInput(hidden, parts, dtype)
        self.q_norm = _param(spec.heads * spec.dim, dtype=torch.float32)
        self.k_norm = _param(spec.kv_heads * spec.dim, dtype=torch.float32) if self.own_kv else None
        self.o_proj = _param(hidden, spec.heads * spec.vdim, dtype=dtype)
        self.register_buffer("inv_freq", rotary_inv_freq(spec.rot), persistent=False)

    def cache_spec(self) -> LayerCacheSpec:
        sp = self.spec
        kv = (sp.kv_heads, sp.dim, sp.vdim)
        return LayerCacheSpec(kv=kv if self.own_kv else None, kv_of=sp.kv_from,
                              pool=kv + (sp.pool,) if sp.pool > 0 and sp.mask_size > 0 else None)

    @staticmethod
    def _run_ends(batch, run: int) -> Optional[torch.Tensor]:
        """Rows of the step whose position ends a run (int32, possibly empty),
        when the step was built on the host; None = not known, look at every
        row. Most decode steps complete no run and skip the pooling launch."""
        if batch.host_segs is None or batch.plans is None:
            return None
        key = ("run_ends", run)
        if key not in batch.plans:
            rows, row0 = [], 0
            for start, n in batch.host_segs:
                first = (-(start + 1)) % run            # first offset with (start + offset + 1) % run == 0
                rows.extend(range(row0 + first, row0 + n, run))
                row0 += n
            batch.plans[key] = torch.tensor(rows, dtype=torch.int32, device=batch.positions.device)
        return batch.plans[key]

    def forward(self, h: torch.Tensor, batch, st: LayerState) -> torch.Tensor:
        sp = self.spec
        T = h.shape[0]
        y = self.inp(h)
        s = self.inp.split
        q = s(y, "q").unflatten(1, (sp.heads, sp.dim))
        k = v = None
        if self.own_kv:
            k = s(y, "k").unflatten(1, (sp.kv_heads, sp.dim))
            v = s(y, "v").unflatten(1, (sp.kv_heads, sp.vdim))
        ops.qk_fullnorm_rope_store(q, k, v, self.q_norm, self.k_norm, self.eps, batch.positions, self.inv_freq,
                                   st.k, st.v, batch.slot_mapping)
        run = sp.pool if st.pool_k is not None else 0
        if run:
            rows = self._run_ends(batch, run)
            if rows is None or rows.numel():
                ops.pool_kv_update(st.k, st.v, st.pool_k, st.pool_v, batch.block_tables, batch.token_seg,
                                   batch.positions, run, rows)
        att = ops.attn_window_pool_paged(q, st.k, st.v, st.pool_k, st.pool_v, batch.block_tables, batch.token_seg,
                                         batch.positions, sp.scale, sp.softcap, sp.mask_size, run)
        return F.linear(att.reshape(T, -1), self.o_proj)

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        m = {pre + n: self.inp.slot(n) for n in self.inp.parts}
        m[pre + "q.norm"] = self.q_norm
        if self.own_kv:
            m[pre + "k.norm"] = self.k_norm
        m[pre + "o"] = self.o_proj
        return m


class Mamba2Mixer(nn.Module):
    """State-space mixer. One input GEMM gives [z | x | B | C | dt]; x, B, C
    pass a short causal convolution (with bias) and silu together; per head h
    of group g, with d = softplus(dt + dt_bias) in fp32:
        S <- exp(-exp(A_h) d) S + d B_g x_h^T,   y_h = S^T C_g + D_h x_h
    then y * silu(z), RMS norm in ``norm_groups`` equal parts, norm weight,
    projection. State: S [H, N, P] fp32 and the convolution's last inputs."""

    def __init__(self, spec: Mamba2Spec, hidden: int, eps: float, dtype):
        super().__init__()
        assert spec.heads % spec.groups == 0 and (spec.heads * spec.vdim) % spec.norm_groups == 0
        self.spec = spec
        self.eps = eps
        self.inner = spec.heads * spec.vdim
        self.gn = spec.groups * spec.state
        self.ch = self.inner + 2 * self.gn
        self.inp = FusedInput(hidden, [("z", self.inner), ("xbc", self.ch), ("dt", spec.heads)], dtype)
        self.conv = nn.Parameter(torch.zeros(spec.conv, self.ch, dtype=torch.float32), requires_grad=False)
        self.conv_bias = _param(self.ch, dtype=torch.float32)
        self.dt_bias = _param(spec.heads, dtype=torch.float32)
        self.A_log = _param(spec.heads, dtype=torch.float32)
        self.D = _param(spec.heads, dtype=torch.float32)
        self.norm = _param(self.inner, dtype=torch.float32)
        self.o_proj = _param(hidden, self.inner, dtype=dtype)

    def cache_spec(self) -> LayerCacheSpec:
        sp = self.spec
        return LayerCacheSpec(rec=(sp.heads, sp.state, sp.vdim), conv=(self.ch, sp.conv - 1))

    def forward(self, h: torch.Tensor, batch, st: LayerState) -> torch.Tensor:
        sp = self.spec
        y = self.inp(h)
        s = self.inp.split
        xbc = ops.causal_conv_silu(s(y, "xbc"), self.conv, st.conv, batch.state_slots, batch.cu_seqlens,
                                   batch.seg_start, batch.token_seg, self.conv_bias)
        o = ops.ssd_recurrence(xbc[:, :self.inner].unflatten(1, (sp.heads, sp.vdim)),
                               xbc[:, self.inner:self.inner + self.gn].unflatten(1, (sp.groups, sp.state)),
                               xbc[:, self.inner + self.gn:].unflatten(1, (sp.groups, sp.state)),
                               s(y, "dt"), self.dt_bias, self.A_log, self.D, st.rec, batch.state_slots,
                               batch.cu_seqlens, batch.seg_start)
        r = ops.gate_group_rmsnorm(o.view(o.shape[0], sp.norm_groups, -1), self.norm, s(y, "z"), self.eps,
                                   self.o_proj.dtype)
        return F.linear(r, self.o_proj)

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        m = {pre + "in": [self.inp.slot("z"), self.inp.slot("xbc"), self.inp.slot("dt")]}
        m[pre + "conv"] = self.conv.t()
        m[pre + "conv.b"] = self.conv_bias
        for n in ("dt_bias", "A_log", "D", "norm"):
            m[pre + n] = getattr(self, n)
        m[pre + "o"] = self.o_proj
        return m


class ActFF(nn.Module):
    """y = W_down act(W_up h) with the tanh-form gelu."""

    def __init__(self, spec: ActFFSpec, hidden: int, dtype):
        super().__init__()
        self.spec = spec
        self.up = _param(spec.ff, hidden, dtype=dtype)
        self.down = _param(hidden, spec.ff, dtype=dtype)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(ops.gelu_tanh(F.linear(h, self.up)), self.down)

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        return {pre + "up": self.up, pre + "down": self.down}


class WkvMixer(nn.Module):
    """Time mixing with token shift. With h' the previous token's input, each
    of r, k, v, g, w reads h + (h' - h) mu_s; r, k, v are projections of their
    mixes, the gate is silu of its projection, the decay
        w = exp(-exp(W_2 tanh(W_1 mix_w) + w0))
    is per head and key channel and kept in fp32 from the mix on. Per head
        o = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T
    then every head's o is RMS-normed, scaled by the norm weight and the gate,
    and projected. State: S [H, D, D] fp32 and the previous input."""

    STREAMS = ("r", "k", "v", "g", "w")
    # the four projections run as one batched product for decode-sized steps
    # and as four plain GEMMs for prompt portions
    BATCHED_MAX_ROWS = 64

    def __init__(self, spec: WkvSpec, hidden: int, eps: float, dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.hidden = hidden
        hd = spec.heads * spec.dim
        self.mu = _param(len(self.STREAMS), hidden, dtype=torch.float32)
        self.rkvg = _param(4, hd, hidden, dtype=dtype)            # one batched GEMM for r, k, v, g
        self.w1 = _param(spec.decay_rank, hidden, dtype=torch.float32)
        self.w2 = _param(hd, spec.decay_rank, dtype=torch.float32)
        self.w0 = _param(hd, dtype=torch.float32)
        self.u = _param(spec.heads, spec.dim, dtype=torch.float32)
        self.norm = _param(hd, dtype=torch.float32)
        self.o_proj = _param(hidden, hd, dtype=dtype)

    def cache_spec(self) -> LayerCacheSpec:
        sp = self.spec
        return LayerCacheSpec(rec=(sp.heads, sp.dim, sp.dim), shift=self.hidden)

    def forward(self, h: torch.Tensor, batch, st: LayerState) -> torch.Tensor:
        sp = self.spec
        mixes, mix_w = ops.token_shift_mix(h, self.mu, st.shift, batch.state_slots, batch.cu_seqlens,
                                           batch.seg_start, batch.token_seg, 4)
        if h.shape[0] <= self.BATCHED_MAX_ROWS:
            y = torch.bmm(mixes, self.rkvg.transpose(1, 2))                   # [4, T, H*D], one launch
        else:
            y = [F.linear(mixes[i], self.rkvg[i]) for i in range(4)]
        d = F.linear(torch.tanh(F.linear(mix_w[0], self.w1)), self.w2)       # fp32 [T, H*D]
        hd = (sp.heads, sp.dim)
        o = ops.wkv_recurrence(y[0].unflatten(1, hd), y[1].unflatten(1, hd), y[2].unflatten(1, hd), d,
                               self.w0, self.u, st.rec, batch.state_slots, batch.cu_seqlens, batch.seg_start)
        r = ops.head_rmsnorm_gate(o, self.norm, y[3], self.eps, "silu", self.o_proj.dtype)
        return F.linear(r, self.o_proj)

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        m = {pre + "mu." + n: self.mu[i] for i, n in enumerate(self.STREAMS)}
        for i, n in enumerate(self.STREAMS[:4]):
            m[pre + n] = self.rkvg[i]
        for n in ("w1", "w2", "w0", "u", "norm"):
            m[pre + n] = getattr(self, n)
        m[pre + "o"] = self.o_proj
        return m


class MlstmMixer(nn.Module):
    """Matrix memory with a stabilised exponential input gate. Per head, with
    i = cap tanh(z_i / cap), f = logsigmoid(cap tanh(z_f / cap)) and a running
    maximum m (from 0):
        m' = max(f + m, i);  S <- e^(f+m-m') S + e^(i-m') k v^T;  n likewise with k
        o = S^T q / (max(|n . q|, e^-m') + 1e-6),  q scaled by D^-1/2
    then RMS norm per head, norm weight, sigmoid gate, projection. The gate
    pre-activations come from an fp32 GEMM of their own. State per head:
    [D+1, V+1] fp32 — S, n as one more column, m in the extra row."""

    def __init__(self, spec: MlstmSpec, hidden: int, eps: float, dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        hv = spec.heads * spec.vdim
        self.inp = FusedInput(hidden, [("q", spec.heads * spec.dim), ("k", spec.heads * spec.dim),
                                       ("v", hv), ("g", hv)], dtype)
        self.gates = _param(2 * spec.heads, hidden, dtype=torch.float32)    # input rows, then forget rows
        self.gate_bias = _param(2 * spec.heads, dtype=torch.float32)
        self.norm = _param(hv, dtype=torch.float32)
        self.o_proj = _param(hidden, hv, dtype=dtype)

    def cache_spec(self) -> LayerCacheSpec:
        sp = self.spec
        return LayerCacheSpec(rec=(sp.heads, sp.dim + 1, sp.vdim + 1))

    def forward(self, h: torch.Tensor, batch, st: LayerState) -> torch.Tensor:
        sp = self.spec
        y = self.inp(h)
        s = self.inp.split
        z = F.linear(h.float(), self.gates)
        r = ops.mlstm_mix_out(s(y, "q").unflatten(1, (sp.heads, sp.dim)),
                              s(y, "k").unflatten(1, (sp.heads, sp.dim)),
                              s(y, "v").unflatten(1, (sp.heads, sp.vdim)), z, self.gate_bias, sp.gate_cap,
                              st.rec, batch.state_slots, batch.cu_seqlens, batch.seg_start, self.norm, s(y, "g"),
                              self.eps, self.o_proj.dtype)
        return F.linear(r, self.o_proj)

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        H = self.spec.heads
        m = {pre + n: self.inp.slot(n) for n in self.inp.parts}
        m[pre + "i"], m[pre + "f"] = self.gates[:H], self.gates[H:]
        m[pre + "i.b"], m[pre + "f.b"] = self.gate_bias[:H], self.gate_bias[H:]
        m[pre + "norm"] = self.norm
        m[pre + "o"] = self.o_proj
        return m


class RoutedExperts(nn.Module):
    """Mixture of GLU experts (silu(gate) * up, or the clamped form with
    limits of their own for the routed and the shared expert). The router runs in fp32: scores are the
    softmax over all outputs or the sigmoid of each; the choice is made on
    score (+ correction) within the best groups of neighbouring experts; the
    chosen scores, renormalised or as they are, weigh the experts — their
    outputs, or (``weight_on = "input"``) their inputs: expert(w h). The last
    ``identity`` router outputs stand for experts that return their input and
    have no weights. An optional shared expert runs for every row and is
    added times sigmoid of one more projection of the row.

    Few rows (decode): every expert runs on every row as two batched GEMMs
    (the weights stream from memory once either way, and shapes do not depend
    on the routing). More rows: rows are sorted by expert and each expert runs
    on its slice. Both end in one weighted gather that sums a row's choices in
    a fixed order, so a row's result does not depend on the batch around it.

    The batched form stays with small row counts: on the GPU a batched product
    of 8 x 512 rows against the experts of a 2048-wide layer ended in an
    illegal address inside the run, while the per-expert products of the
    sorted form ran the same rows cleanly."""

    # every expert runs on every row for steps of at most this many rows, and
    # at most this many (expert, row) pairs
    DENSE_MAX_ROWS = 64
    DENSE_MAX_PAIRS = 512

    def __init__(self, spec: RoutedExpertsSpec, hidden: int, dtype):
        super().__init__()
        self.spec = spec
        n = spec.experts + spec.identity
        assert n % spec.group_count == 0 and 1 <= spec.group_keep <= spec.group_count
        assert spec.top <= n // spec.group_count * spec.group_keep
        assert not (spec.weight_on == "input" and spec.identity), "identity experts take their weight on the output"
        self.router = _param(n, hidden, dtype=torch.float32)
        self.correction = _param(n, dtype=torch.float32) if spec.correction else None
        self.w_gate_up = _param(spec.experts, 2 * spec.ff, hidden, dtype=dtype)
        self.w_down = _param(spec.experts, hidden, spec.ff, dtype=dtype)
        self.shared_inp = self.shared_down = None
        if spec.shared is not None:
            sff = spec.shared.ff
            self.shared_inp = FusedInput(hidden, [("gate", sff), ("up", sff), ("sg", 1)], dtype)
            self.shared_down = _param(hidden, sff, dtype=dtype)

    def _act(self, gate: torch.Tensor, up: torch.Tensor, limit: Optional[float] = None) -> torch.Tensor:
        sp = self.spec
        if sp.act == "clamped":
            return ops.gated_act(gate, up, sp.limit if limit is None else limit, sp.alpha, 1.0)
        return ops.silu_glu(gate, up)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        sp = self.spec
        T, W = h.shape
        E, top = sp.experts, sp.top
        on_input = sp.weight_on == "input"
        dense = T <= self.DENSE_MAX_ROWS and E * T <= self.DENSE_MAX_PAIRS
        idx, w, rowidx = ops.moe_route_rows(h, self.router, self.correction, top, sp.group_count, sp.group_keep,
                                            E, dense, sp.score, sp.renormalize)
        if dense:
            if on_input:
                # expert e reads w[t, e] h[t] where it was chosen (zero rows elsewhere; they are never read back)
                xin = ops.moe_spread_rows(h, idx, w, E)
            else:
                xin = h.unsqueeze(0).expand(E, T, W)
            gu = torch.bmm(xin, self.w_gate_up.transpose(1, 2)).view(E * T, 2 * sp.ff)
            act = self._act(gu[:, :sp.ff], gu[:, sp.ff:]).view(E, T, sp.ff)
            rows = torch.bmm(act, self.w_down.transpose(1, 2)).view(E * T, W)
        else:
            flat = idx.reshape(-1).long().clamp(max=E)                # identity experts sort last
            order = torch.argsort(flat, stable=True)
            counts = torch.bincount(flat, minlength=E + 1)[:E].tolist()   # one host sync per call
            n_real = sum(counts)
            if on_input:
                xs = ops.scale_rows(h, (order[:n_real] // top).int(), w.reshape(-1)[order[:n_real]])
            else:
                xs = h[(order[:n_real] // top)]
            rows = torch.empty((max(n_real, 1), W), dtype=h.dtype, device=h.device)
            s0 = 0
            for e, c in enumerate(counts):
                if c:
                    gu = F.linear(xs[s0:s0 + c], self.w_gate_up[e])
                    rows[s0:s0 + c] = F.linear(self._act(gu[:, :sp.ff], gu[:, sp.ff:]), self.w_down[e])
                    s0 += c
            pos = torch.empty(T * top, dtype=torch.int32, device=h.device)
            pos[order] = torch.arange(T * top, dtype=torch.int32, device=h.device)
            rowidx = torch.where(idx < E, pos.view(T, top), torch.full_like(idx, -1))
        extra = gate = None
        if self.shared_inp is not None:
            ys = self.shared_inp(h)
            ss = self.shared_inp.split
            extra = F.linear(self._act(ss(ys, "gate"), ss(ys, "up"), sp.shared.limit), self.shared_down)
            gate = ss(ys, "sg")[:, 0]
        return ops.moe_combine(rows, h, rowidx, None if on_input else w, h.dtype, extra, gate)

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        ff = self.spec.ff
        m = {pre + "router": self.router}
        if self.correction is not None:
            m[pre + "correction"] = self.correction
        for e in range(self.spec.experts):
            m[f"{pre}e{e}.gate"] = self.w_gate_up[e, :ff]
            m[f"{pre}e{e}.up"] = self.w_gate_up[e, ff:]
            m[f"{pre}e{e}.down"] = self.w_down[e]
        if self.shared_inp is not None:
            for n in ("gate", "up", "sg"):
                m[f"{pre}shared.{n}"] = self.shared_inp.slot(n)
            m[pre + "shared.down"] = self.shared_down
        return m
