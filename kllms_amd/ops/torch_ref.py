"""Pure-PyTorch reference implementations of every engine op.

These are the numerics oracles for the HIP/CDNA4 kernels (tests compare the
kernels against these in fp32) and the CPU execution path for GPU-less test
environments. On a GPU box the dispatch layer (ops/__init__.py) routes to the
HIP kernels and refuses to fall back silently.

Conventions:
- q/k/v activations: [tokens, heads, head_dim]
- paged KV cache: [num_blocks, kv_heads, block_size, head_dim]
- cos/sin cache: [max_pos, head_dim] with cos in [:, :D/2], sin in [:, D/2:]
- logits: [batch, vocab]
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch


# --- normalization ------------------------------------------------------------

def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    norm = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (norm * weight.float()).to(x.dtype)


def fused_add_rmsnorm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
) -> Tuple[torch.Tensor, torch.Tensor]:
    """residual' = x + residual; y = rmsnorm(residual')."""
    new_residual = (x.float() + residual.float()).to(x.dtype)
    return rmsnorm(new_residual, weight, eps), new_residual


# --- rotary embedding ---------------------------------------------------------

def build_cos_sin_cache(head_dim: int, max_pos: int, theta: float, device,
                        dtype=torch.float32, rope_scaling=None) -> torch.Tensor:
    half = head_dim // 2
    inv_freq = 1.0 / (theta ** (torch.arange(0, half, dtype=torch.float64, device=device) / half))
    if rope_scaling:
        rt = rope_scaling.get("rope_type") or rope_scaling.get("type")
        if rt == "llama3":
            # Llama-3.1 frequency-banded NTK scaling: low-frequency bands
            # (wavelength > old context) are divided by `factor`; high-
            # frequency bands are untouched; the band between interpolates.
            import math as _math

            factor = float(rope_scaling.get("factor", 8.0))
            lo_f = float(rope_scaling.get("low_freq_factor", 1.0))
            hi_f = float(rope_scaling.get("high_freq_factor", 4.0))
            old_ctx = float(rope_scaling.get("original_max_position_embeddings", 8192))
            wavelen = 2 * _math.pi / inv_freq
            lo_wl = old_ctx / lo_f
            hi_wl = old_ctx / hi_f
            smooth = ((old_ctx / wavelen - lo_f) / (hi_f - lo_f)).clamp(0.0, 1.0)
            scaled = (1 - smooth) * inv_freq / factor + smooth * inv_freq
            inv_freq = torch.where(wavelen > lo_wl, inv_freq / factor,
                                   torch.where(wavelen < hi_wl, inv_freq, scaled))
        elif rt == "linear":
            inv_freq = inv_freq / float(rope_scaling.get("factor", 1.0))
        # unknown types: serve unscaled rather than failing (documented)
    t = torch.arange(max_pos, dtype=torch.float64, device=device)
    freqs = torch.outer(t, inv_freq)
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1).to(dtype)


def rope_inplace(
    q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor
) -> None:
    """Llama-style (rotate-half over contiguous halves) rotary embedding,
    applied in place to q [T, H, D] and k [T, KVH, D]."""
    D = q.shape[-1]
    half = D // 2
    cs = cos_sin[positions]  # [T, D]
    cos = cs[:, :half].unsqueeze(1).float()  # [T, 1, half]
    sin = cs[:, half:].unsqueeze(1).float()
    for t in (q, k):
        tf = t.float()
        x1 = tf[..., :half]
        x2 = tf[..., half:]
        t[..., :half] = (x1 * cos - x2 * sin).to(t.dtype)
        t[..., half:] = (x2 * cos + x1 * sin).to(t.dtype)


# --- activations --------------------------------------------------------------

def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return (torch.nn.functional.silu(gate.float()) * up.float()).to(gate.dtype)


# --- paged KV cache -----------------------------------------------------------

def store_kv(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    k_scale=None,
    v_scale=None,
) -> None:
    """Scatter new K/V ([T, KVH, D]) into the paged caches at flat slots.

    A flat slot s addresses (block = s // block_size, offset = s % block_size).
    fp8 caches with k_scale/v_scale ([NB, KVH, BS] fp32): each (token, head)
    row is quantized with its OWN scale s = max(amax(|row|)/448, 1e-8), the
    scale written alongside — outlier rows no longer saturate e4m3.
    """
    num_blocks, kv_heads, block_size, head_dim = k_cache.shape
    blk = slot_mapping // block_size
    off = slot_mapping % block_size
    if k_scale is not None:
        sk = (k.float().abs().amax(-1) / 448.0).clamp_(min=1e-8)  # [T, KVH]
        sv = (v.float().abs().amax(-1) / 448.0).clamp_(min=1e-8)
        k_scale[blk, :, off] = sk
        v_scale[blk, :, off] = sv
        k_cache[blk, :, off, :] = (k.float() / sk.unsqueeze(-1)).to(k_cache.dtype)
        v_cache[blk, :, off, :] = (v.float() / sv.unsqueeze(-1)).to(v_cache.dtype)
        return
    k_cache[blk, :, off, :] = k.to(k_cache.dtype)
    v_cache[blk, :, off, :] = v.to(v_cache.dtype)


# --- attention ----------------------------------------------------------------

def attn_prefill_varlen(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,
    scale: float,
) -> torch.Tensor:
    """Causal varlen attention over packed sequences.

    q: [T, H, D]; k/v: [T, KVH, D] (GQA: H % KVH == 0). Returns [T, H, D].
    """
    T, H, D = q.shape
    KVH = k.shape[1]
    rep = H // KVH
    out = torch.empty_like(q)
    cu = cu_seqlens.tolist()
    for i in range(len(cu) - 1):
        s, e = cu[i], cu[i + 1]
        qi = q[s:e].float().permute(1, 0, 2)  # [H, L, D]
        ki = k[s:e].float().repeat_interleave(rep, dim=1).permute(1, 0, 2)
        vi = v[s:e].float().repeat_interleave(rep, dim=1).permute(1, 0, 2)
        o = torch.nn.functional.scaled_dot_product_attention(
            qi, ki, vi, is_causal=True, scale=scale
        )
        out[s:e] = o.permute(1, 0, 2).to(q.dtype)
    return out


def attn_decode_paged(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    context_lens: torch.Tensor,
    scale: float,
    k_scale=None,
    v_scale=None,
) -> torch.Tensor:
    """Single-token decode attention against the paged KV cache.

    q: [B, H, D]; caches [num_blocks, KVH, block_size, D];
    block_tables: [B, max_blocks] int32; context_lens: [B] (length INCLUDING
    the token being decoded, whose K/V are already stored). k_scale/v_scale
    ([NB, KVH, BS] fp32, fp8 caches only): per-row dequant multipliers.
    """
    B, H, D = q.shape
    _, KVH, BS, _ = k_cache.shape
    rep = H // KVH
    out = torch.empty_like(q)
    for b in range(B):
        L = int(context_lens[b])
        nblk = (L + BS - 1) // BS
        blocks = block_tables[b, :nblk].long()
        kk = k_cache[blocks].permute(1, 0, 2, 3).reshape(KVH, nblk * BS, D)[:, :L].float()
        vv = v_cache[blocks].permute(1, 0, 2, 3).reshape(KVH, nblk * BS, D)[:, :L].float()
        if k_scale is not None:
            kk = kk * k_scale[blocks].permute(1, 0, 2).reshape(KVH, nblk * BS)[:, :L, None]
            vv = vv * v_scale[blocks].permute(1, 0, 2).reshape(KVH, nblk * BS)[:, :L, None]
        qb = q[b].float()  # [H, D]
        # per-head GQA mapping without materializing repeats
        for h in range(H):
            g = h // rep
            s = (qb[h] @ kk[g].T) * scale  # [L]
            p = torch.softmax(s, dim=-1)
            out[b, h] = (p @ vv[g]).to(q.dtype)
    return out


# --- sampling -----------------------------------------------------------------

def _stream_generator(seed: int, step: int, device) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed((seed * 0x9E3779B97F4A7C15 + step * 0xBF58476D1CE4E5B9) % (2**63))
    return g


def sample(
    logits: torch.Tensor,
    temperatures: torch.Tensor,
    top_ps: torch.Tensor,
    top_ks: torch.Tensor,
    seeds: torch.Tensor,
    steps: torch.Tensor,
    mask: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Fused sampling reference.

    - mask: optional [B, ceil(V/32)] uint32 bitmask of ALLOWED tokens
      (constrained decoding); disallowed logits become -inf.
    - temperature == 0 -> greedy.
    - top_k <= 0 means no top-k; top_p >= 1 means no top-p.
    - Returns (token_ids [B], logprobs [B]) where logprob is the
      log-softmax of the MASKED, UNtempered distribution at the chosen token
      (OpenAI-style model logprob).
    """
    B, V = logits.shape
    lf = logits.float().clone()
    if mask is not None:
        bit = torch.arange(V, device=logits.device)
        allowed = (mask[:, bit // 32] >> (bit % 32).to(torch.int64)) & 1
        lf = torch.where(allowed.bool(), lf, torch.full_like(lf, float("-inf")))
    base_logprobs = torch.log_softmax(lf, dim=-1)

    tokens = torch.empty(B, dtype=torch.long, device=logits.device)
    for b in range(B):
        temp = float(temperatures[b])
        row = lf[b]
        if temp == 0.0:
            tokens[b] = torch.argmax(row)
            continue
        scaled = row / temp
        k = int(top_ks[b])
        p = float(top_ps[b])
        probs = torch.softmax(scaled, dim=-1)
        if k > 0 and k < V:
            kth = torch.topk(probs, k).values[-1]
            probs = torch.where(probs >= kth, probs, torch.zeros_like(probs))
        if p < 1.0:
            sorted_probs, sorted_idx = torch.sort(probs, descending=True)
            cumsum = torch.cumsum(sorted_probs, dim=-1)
            # keep the smallest prefix with mass >= top_p (first token always kept)
            cut = (cumsum - sorted_probs) >= p
            sorted_probs = torch.where(cut, torch.zeros_like(sorted_probs), sorted_probs)
            probs = torch.zeros_like(probs).scatter(0, sorted_idx, sorted_probs)
        probs = probs / probs.sum()
        g = _stream_generator(int(seeds[b]), int(steps[b]), logits.device)
        u = torch.rand(V, generator=g).to(logits.device)
        # Gumbel-max over the truncated renormalized distribution
        e = (-torch.log(u.clamp_min(1e-20))).clamp_min(1e-20)  # Exp(1)
        gumbel = -torch.log(e)
        masked_logp = torch.where(probs > 0, torch.log(probs), torch.full_like(probs, float("-inf")))
        tokens[b] = torch.argmax(masked_logp + gumbel)

    logprobs = base_logprobs[torch.arange(B, device=logits.device), tokens]
    return tokens, logprobs


# --- listed-layer hybrid family: fp32 residual stream, block-local attention,
# --- recurrent mixers ---------------------------------------------------------
#
# Batch convention shared by these ops ("segments"): the step's tokens are
# packed [T, ...]; segment b covers rows cu_seqlens[b]..cu_seqlens[b+1] and
# continues sequence b at position seg_start[b] (0 = a fresh sequence, whose
# recurrent state is taken as zero whatever its slot holds). A decode step is
# the case of all segments having one row.

def embed_rmsnorm(ids: torch.Tensor, table: torch.Tensor, weight: torch.Tensor, eps: float,
                  pos_table: Optional[torch.Tensor] = None, positions: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp32 residual stream: rmsnorm(table[ids] (+ pos_table[positions])) * weight."""
    x = table[ids].float()
    if pos_table is not None:
        x = x + pos_table[positions].float()
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight.float()


def rmsnorm_cast(x: torch.Tensor, weight: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).to(out_dtype)


def sandwich_residual(x, a, w_post, eps, b=None, wa=None, wb=None, w_next=None, out_dtype=None, cast=False):
    """x (fp32, in place) += rmsnorm(y) * w_post, where y = a, or with a second
    branch y = (rmsnorm(a) * wa + rmsnorm(b) * wb) / 2. Returns
    rmsnorm(x) * w_next cast to out_dtype (the next sublayer's input); with
    w_next None: x itself cast to out_dtype if ``cast``, else None."""
    def n(t):
        t = t.float()
        return t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + eps)

    y = a.float()
    if b is not None:
        y = 0.5 * (n(a) * wa.float() + n(b) * wb.float())
    x.add_(n(y) * w_post.float())
    if w_next is None:
        return x.to(out_dtype) if cast else None
    return (n(x) * w_next.float()).to(out_dtype)


def rope_pairs_store(q, k, v, positions, inv_freq, k_cache, v_cache, slot_mapping) -> None:
    """Interleaved-pair rotary embedding on the first 2*len(inv_freq) dims of
    q [T,H,D] and k [T,G,D] (q in place), angle = position * inv_freq in fp32;
    the ROTATED k goes to k_cache and v (or, when v is None, the UN-rotated k)
    to v_cache at the flat slots. Caches: [NB, G, BS, D]."""
    R = inv_freq.numel()
    ang = positions.to(torch.float32)[:, None] * inv_freq.float()[None, :]   # [T, R]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]

    def rot(t):
        tf = t.float()
        u, w = tf[..., 0:2 * R:2], tf[..., 1:2 * R:2]
        out = tf.clone()
        out[..., 0:2 * R:2] = u * cos - w * sin
        out[..., 1:2 * R:2] = w * cos + u * sin
        return out

    BS = k_cache.shape[2]
    blk, off = slot_mapping // BS, slot_mapping % BS
    vals = k if v is None else v
    v_cache[blk, :, off, :] = vals.to(v_cache.dtype)
    k_cache[blk, :, off, :] = rot(k).to(k_cache.dtype)
    q.copy_(rot(q).to(q.dtype))


def attn_blocklocal_paged(q, k_cache, v_cache, block_tables, token_seg, positions, scale,
                          mask_size, gate=None, out_dtype=None) -> torch.Tensor:
    """Softmax attention of packed query rows against the paged cache. Row t
    (segment token_seg[t], position p) sees keys lo..p of its own sequence,
    lo = floor(p / mask_size) * mask_size (0 when mask_size == 0). ``gate``
    [T, H] (logits): each head's output is scaled by its sigmoid."""
    T, H, D = q.shape
    _, G, BS, Dv = v_cache.shape
    rep = H // G
    out = torch.empty(T, H, Dv, dtype=out_dtype or q.dtype, device=q.device)
    pos = positions.tolist()
    seg = token_seg.tolist()
    for t in range(T):
        p = pos[t]
        lo = (p // mask_size) * mask_size if mask_size > 0 else 0
        idx = torch.arange(lo, p + 1, device=q.device)
        blocks = block_tables[seg[t]].long()[idx // BS]
        kk = k_cache[blocks, :, idx % BS, :].float()          # [n, G, D]
        vv = v_cache[blocks, :, idx % BS, :].float()
        qt = q[t].float().view(G, rep, D)
        s = torch.einsum("grd,ngd->grn", qt, kk) * scale
        pr = torch.softmax(s, dim=-1)
        o = torch.einsum("grn,ngd->grd", pr, vv).reshape(H, Dv)
        if gate is not None:
            o = o * torch.sigmoid(gate[t].float())[:, None]
        out[t] = o.to(out.dtype)
    return out


def linear_attn_decay(q, k, v, decay, state, state_slots, cu_seqlens, seg_start) -> torch.Tensor:
    """Decayed linear attention over segments. q,k [T,H,D], v [T,H,V] are the
    raw projections (silu is applied here); decay [H] fp32;
    state [slots,H,D,V] fp32 is read (unless seg_start == 0) and written back.
    Returns o [T,H,V] fp32 with o_t = S_t^T q_t, S_t = decay S_{t-1} + k_t v_t^T."""
    T, H, _ = q.shape
    qf = torch.nn.functional.silu(q.float())
    kf = torch.nn.functional.silu(k.float())
    vf = torch.nn.functional.silu(v.float())
    o = torch.empty(T, H, v.shape[-1], dtype=torch.float32, device=q.device)
    cu, st, sl = cu_seqlens.tolist(), seg_start.tolist(), state_slots.tolist()
    d = decay.float().view(H, 1, 1)
    for b in range(len(sl)):
        S = state[sl[b]].clone() if st[b] > 0 else torch.zeros_like(state[sl[b]])
        for t in range(cu[b], cu[b + 1]):
            S = d * S + kf[t].unsqueeze(-1) * vf[t].unsqueeze(-2)
            o[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[sl[b]] = S
    return o


def gated_rmsnorm(o, weight, gate, eps, out_dtype) -> torch.Tensor:
    """o [T, n_groups, S] fp32: each group is divided by its root mean square,
    times weight [S], times sigmoid(gate) ([T, n_groups*S] logits).
    Returns [T, n_groups*S]."""
    T, Gn, S = o.shape
    of = o.float()
    y = of * torch.rsqrt(of.pow(2).mean(-1, keepdim=True) + eps) * weight.float()
    return (y.reshape(T, Gn * S) * torch.sigmoid(gate.float())).to(out_dtype)


def causal_conv_silu(x, w, conv_state, state_slots, cu_seqlens, seg_start, bias=None) -> torch.Tensor:
    """Per-channel causal convolution over time (+ bias [C]) + silu. x [T,C];
    w [K,C] taps-major (last row = current token); conv_state [slots, K-1, C]
    holds each sequence's last K-1 inputs (oldest first) and is updated."""
    T, C = x.shape
    K = w.shape[0]
    y = torch.empty(T, C, dtype=x.dtype, device=x.device)
    cu, st, sl = cu_seqlens.tolist(), seg_start.tolist(), state_slots.tolist()
    wf = w.float()
    for b in range(len(sl)):
        s, e = cu[b], cu[b + 1]
        hist = conv_state[sl[b]].float() if st[b] > 0 else torch.zeros(K - 1, C, device=x.device)
        ext = torch.cat([hist, x[s:e].float()], 0)           # [K-1+L, C]
        acc = torch.zeros(e - s, C, device=x.device)
        if bias is not None:
            acc += bias.float()
        for j in range(K):
            acc += ext[j:j + (e - s)] * wf[j]
        y[s:e] = torch.nn.functional.silu(acc).to(x.dtype)
        if K > 1:
            conv_state[sl[b]] = ext[ext.shape[0] - (K - 1):].to(conv_state.dtype)
    return y


def gated_delta_rule(q, k, v, beta_logit, a, dt_bias, a_log, state, state_slots, cu_seqlens,
                     seg_start) -> torch.Tensor:
    """Gated delta rule with a decay per head and key channel.
    q,k [T,G,D], v [T,H,V] (already convolved + silu); beta_logit [T,H];
    a [T,H*D] decay pre-activation (dt_bias [H*D] added here); a_log [H];
    state [slots,H,D,V] fp32. Per head: S <- g*S (rows), u = beta (v - S^T k),
    S <- S + k u^T, o = S^T q. q,k are unit-normalized (eps 1e-6 inside the
    root) and q scaled by D^-1/2. Returns o [T,H,V] fp32."""
    T, G, D = q.shape
    H, V = v.shape[1], v.shape[2]
    rep = H // G
    qf, kf, vf = q.float(), k.float(), v.float()
    qf = qf * torch.rsqrt(qf.pow(2).sum(-1, keepdim=True) + 1e-6) * (D ** -0.5)
    kf = kf * torch.rsqrt(kf.pow(2).sum(-1, keepdim=True) + 1e-6)
    qf = qf.repeat_interleave(rep, dim=1)
    kf = kf.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(beta_logit.float())
    sp = torch.nn.functional.softplus(a.float() + dt_bias.float()).view(T, H, D)
    g = torch.exp(-torch.exp(a_log.float()).view(1, H, 1) * sp)
    o = torch.empty(T, H, V, dtype=torch.float32, device=q.device)
    cu, st, sl = cu_seqlens.tolist(), seg_start.tolist(), state_slots.tolist()
    for b in range(len(sl)):
        S = state[sl[b]].clone() if st[b] > 0 else torch.zeros_like(state[sl[b]])
        for t in range(cu[b], cu[b + 1]):
            S = S * g[t].unsqueeze(-1)
            pred = torch.einsum("hdv,hd->hv", S, kf[t])
            u = beta[t].unsqueeze(-1) * (vf[t] - pred)
            S = S + kf[t].unsqueeze(-1) * u.unsqueeze(-2)
            o[t] = torch.einsum("hdv,hd->hv", S, qf[t])
        state[sl[b]] = S
    return o


def clamped_glu(gate, up, limit: float, alpha: float) -> torch.Tensor:
    g = gate.float().clamp(max=limit)
    u = up.float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gate.dtype)


# --- parallel-layer family: grouped norm, hashed bigram embedding, windowed
# attention with a sink, wkv and mlstm recurrences, routed experts ------------

def embed_bigram(ids, table, bigram, scale, mul_prev, mul_cur, buckets, tok_state, state_slots,
                 cu_seqlens, seg_start) -> torch.Tensor:
    """fp32 rows table[id] * scale + bigram[(prev * mul_prev + id * mul_cur) % buckets];
    a sequence's first token takes row ``buckets``. The previous token of a
    segment's first row comes from tok_state [slots] (int32), which is then set
    to the segment's last id."""
    x = table[ids].float() * scale
    if bigram is None:
        return x
    cu, st, sl = cu_seqlens.tolist(), seg_start.tolist(), state_slots.tolist()
    prev = torch.empty_like(ids)
    first = torch.zeros_like(ids, dtype=torch.bool)
    for b in range(len(sl)):
        s, e = cu[b], cu[b + 1]
        if e == s:
            continue
        prev[s + 1:e] = ids[s:e - 1]
        if st[b] == 0:
            prev[s] = 0
            first[s] = True
        else:
            prev[s] = tok_state[sl[b]].long()
        tok_state[sl[b]] = ids[e - 1].to(tok_state.dtype)
    row = (prev * mul_prev + ids * mul_cur) % buckets
    row = torch.where(first, torch.full_like(row, buckets), row)
    return x + bigram[row].float()


def group_norm_pair(x, a, b, w1, w2, groups, eps, out_dtype):
    """x (fp32, in place) += a + b (either may be None); returns
    (gnorm(x) * w1, gnorm(x) * w2) in out_dtype, where gnorm divides each of
    ``groups`` equal runs of the row by its own root mean square. w2 None ->
    second result None."""
    if a is not None:
        x.add_(a.float() if b is None else a.float() + b.float())
    T, W = x.shape
    xg = x.view(T, groups, W // groups)
    n = (xg * torch.rsqrt(xg.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, W)
    h1 = (n * w1.float()).to(out_dtype)
    h2 = (n * w2.float()).to(out_dtype) if w2 is not None else None
    return h1, h2


def cast_concat(x, x0, a, b, out_dtype):
    """x (fp32, in place) += a + b (either may be None); returns [x | x0] in
    out_dtype, [T, 2W]."""
    if a is not None:
        x.add_(a.float() if b is None else a.float() + b.float())
    return torch.cat([x, x0], -1).to(out_dtype)


def qk_norm_store(q, k, v, wq, wk, eps, k_cache, v_cache, slot_mapping) -> None:
    """RMS norm over the head dim of q [T,H,D] (in place) and k [T,G,D] with
    weights wq / wk [D]; the normed k and v go to the paged caches."""
    def n(t, w):
        tf = t.float()
        return tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + eps) * w.float()

    BS = k_cache.shape[2]
    blk, off = slot_mapping // BS, slot_mapping % BS
    k_cache[blk, :, off, :] = n(k, wk).to(k_cache.dtype)
    v_cache[blk, :, off, :] = v.to(v_cache.dtype)
    q.copy_(n(q, wq).to(q.dtype))


def attn_masked_paged(q, k_cache, v_cache, block_tables, token_seg, positions, scale, mask_kind,
                      mask_size, keep_first, sink, gate=None, out_dtype=None) -> torch.Tensor:
    """Softmax attention of packed query rows against the paged cache. Row t
    at position p sees key j <= p of its own sequence when
      mask_kind 0 (aligned blocks): floor(j / mask_size) == floor(p / mask_size)
      mask_kind 1 (sliding window): p - j < mask_size or j < keep_first
    (mask_size 0 = plain causal). ``sink``: one more term exp(0) in the
    denominator. ``gate`` logits [T, H] (per head) or [T, H*Dv] (per element)."""
    T, H, D = q.shape
    _, G, BS, Dv = v_cache.shape
    rep = H // G
    out = torch.empty(T, H, Dv, dtype=out_dtype or q.dtype, device=q.device)
    pos = positions.tolist()
    seg = token_seg.tolist()
    for t in range(T):
        p = pos[t]
        if mask_size <= 0:
            idx = torch.arange(0, p + 1, device=q.device)
        elif mask_kind == 0:
            idx = torch.arange((p // mask_size) * mask_size, p + 1, device=q.device)
        else:
            lo = max(0, p - mask_size + 1)
            idx = torch.cat([torch.arange(0, min(keep_first, lo), device=q.device),
                             torch.arange(lo, p + 1, device=q.device)])
        blocks = block_tables[seg[t]].long()[idx // BS]
        kk = k_cache[blocks, :, idx % BS, :].float()
        vv = v_cache[blocks, :, idx % BS, :].float()
        qt = q[t].float().view(G, rep, D)
        s = torch.einsum("grd,ngd->grn", qt, kk) * scale
        if sink:
            mx = s.max(-1, keepdim=True).values.clamp(min=0.0)
            e = torch.exp(s - mx)
            pr = e / (e.sum(-1, keepdim=True) + torch.exp(-mx))
        else:
            pr = torch.softmax(s, dim=-1)
        o = torch.einsum("grn,ngd->grd", pr, vv).reshape(H, Dv)
        if gate is not None:
            gt = torch.sigmoid(gate[t].float())
            o = o * (gt[:, None] if gt.numel() == H else gt.view(H, Dv))
        out[t] = o.to(out.dtype)
    return out


def token_shift_mix(h, mu, shift_state, state_slots, cu_seqlens, seg_start, n_act, out_dtype):
    """Mixes of each row with its predecessor: out[s] = h + (h_prev - h) * mu[s]
    for the rows of mu [n, W]. The predecessor of a segment's first row is
    shift_state[slot] (zeros for a fresh sequence); shift_state is set to the
    segment's last row. Returns ([n_act, T, W] in out_dtype, [n - n_act, T, W]
    fp32): the last mixes feed fp32 paths."""
    T, W = h.shape
    hf = h.float()
    prev = torch.zeros_like(hf)
    cu, st, sl = cu_seqlens.tolist(), seg_start.tolist(), state_slots.tolist()
    for b in range(len(sl)):
        s, e = cu[b], cu[b + 1]
        if e == s:
            continue
        prev[s + 1:e] = hf[s:e - 1]
        if st[b] > 0:
            prev[s] = shift_state[sl[b]].float()
        shift_state[sl[b]] = h[e - 1].to(shift_state.dtype)
    mixes = hf[None] + (prev - hf)[None] * mu.float()[:, None, :]
    return mixes[:n_act].to(out_dtype), mixes[n_act:].contiguous()


def wkv_recurrence(r, k, v, d, w0, u, state, state_slots, cu_seqlens, seg_start) -> torch.Tensor:
    """r, k, v [T,H,D|V]; d [T, H*D] fp32 decay pre-activation (w0 [H*D] is
    added here), w = exp(-exp(d + w0)); u [H, D] bonus; state [slots,H,D,V]
    fp32. Per head o_t = (S + diag(u) k v^T)^T r, then S <- diag(w) S + k v^T.
    Returns o [T,H,V] fp32."""
    T, H, D = r.shape
    V = v.shape[2]
    rf, kf, vf = r.float(), k.float(), v.float()
    w = torch.exp(-torch.exp(d.float() + w0.float())).view(T, H, D)
    uf = u.float()
    o = torch.empty(T, H, V, dtype=torch.float32, device=r.device)
    cu, st, sl = cu_seqlens.tolist(), seg_start.tolist(), state_slots.tolist()
    for b in range(len(sl)):
        S = state[sl[b]].clone() if st[b] > 0 else torch.zeros_like(state[sl[b]])
        for t in range(cu[b], cu[b + 1]):
            kv = kf[t].unsqueeze(-1) * vf[t].unsqueeze(-2)
            o[t] = torch.einsum("hdv,hd->hv", S + uf.unsqueeze(-1) * kv, rf[t])
            S = w[t].unsqueeze(-1) * S + kv
        state[sl[b]] = S
    return o


def mlstm_recurrence(q, k, v, gates, gate_bias, cap, state, state_slots, cu_seqlens, seg_start):
    """q, k [T,H,D], v [T,H,V]; gates [T, 2H] fp32 (input | forget
    pre-activations, gate_bias [2H] added here). i = cap tanh(./cap),
    f = logsigmoid(cap tanh(./cap)); m_t = max(f + m, i), m starting at 0;
    S <- e^(f+m-m_t) S + e^(i-m_t) k v^T, n likewise with k alone;
    o = S^T q' / (max(|n . q'|, e^-m_t) + 1e-6), q' = q D^-1/2.
    state [slots, H, D+1, V+1] fp32: [:, :, :D, :V] = S, [:, :, :D, V] = n,
    [:, :, D, :] = m. Returns o [T,H,V] fp32."""
    T, H, D = q.shape
    V = v.shape[2]
    qf, kf, vf = q.float() * (D ** -0.5), k.float(), v.float()
    g = gates.float() + gate_bias.float()
    ig = cap * torch.tanh(g[:, :H] / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh(g[:, H:] / cap))
    o = torch.empty(T, H, V, dtype=torch.float32, device=q.device)
    cu, st, sl = cu_seqlens.tolist(), seg_start.tolist(), state_slots.tolist()
    ones = torch.ones(H, 1, dtype=torch.float32, device=q.device)
    for b in range(len(sl)):
        if st[b] > 0:
            S = state[sl[b], :, :D, :].clone()             # [H, D, V+1], last column = n
            m = state[sl[b], :, D, 0].clone()
        else:
            S = torch.zeros(H, D, V + 1, dtype=torch.float32, device=q.device)
            m = torch.zeros(H, dtype=torch.float32, device=q.device)
        for t in range(cu[b], cu[b + 1]):
            m_new = torch.maximum(fg[t] + m, ig[t])
            fa, fi = torch.exp(fg[t] + m - m_new), torch.exp(ig[t] - m_new)
            ve = torch.cat([vf[t], ones], -1)
            S = fa.view(H, 1, 1) * S + fi.view(H, 1, 1) * kf[t].unsqueeze(-1) * ve.unsqueeze(-2)
            m = m_new
            oe = torch.einsum("hdv,hd->hv", S, qf[t])
            den = torch.maximum(oe[:, V].abs(), torch.exp(-m)) + 1e-6
            o[t] = oe[:, :V] / den[:, None]
        state[sl[b], :, :D, :] = S
        state[sl[b], :, D, :] = m[:, None]
    return o


def head_rmsnorm_gate(o, weight, gate, eps, gate_act, out_dtype) -> torch.Tensor:
    """o [T,H,S] fp32: each head is divided by its root mean square, the
    concatenation is scaled by weight [H*S] and by the gate ([T, H*S]):
    gate_act 'sigmoid' or 'silu' applied to the gate's logits."""
    T, H, S = o.shape
    y = (o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, H * S) * weight.float()
    gf = gate.float()
    gf = torch.sigmoid(gf) if gate_act == "sigmoid" else torch.nn.functional.silu(gf)
    return (y * gf).to(out_dtype)


def gated_act(gate, up, limit: float, alpha: float, up_bias: float) -> torch.Tensor:
    """min(g, limit) * sigmoid(alpha * min(g, limit)) * (clamp(u, +-limit) + up_bias);
    limit = inf, alpha = 1, up_bias = 0 is silu(g) * u."""
    g = gate.float().clamp(max=limit)
    u = up.float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + up_bias)).to(gate.dtype)


def moe_route(z, correction, top, group_count, group_keep, score="softmax", renormalize=True):
    """z [T, N] fp32 router logits. Scores s = softmax(z) over the outputs, or
    sigmoid(z) of each; the choice is made on c = s + correction (None = no
    correction) among the experts of the ``group_keep`` groups (of
    ``group_count`` equal runs of neighbours) whose largest c is largest;
    ties go to the lower index. Returns (idx [T, top] int32, w [T, top] fp32
    = chosen s, divided by (their sum + 1e-20) if ``renormalize``)."""
    T, N = z.shape
    s = torch.softmax(z.float(), -1) if score == "softmax" else torch.sigmoid(z.float())
    c = s + correction.float() if correction is not None else s
    per = N // group_count
    gs = c.view(T, group_count, per).max(-1).values
    # stable descending order = ties to the lower index
    gord = torch.sort(gs, dim=-1, descending=True, stable=True).indices[:, :group_keep]
    gmask = torch.zeros(T, group_count, dtype=torch.bool, device=z.device)
    gmask.scatter_(1, gord, True)
    cm = torch.where(gmask.repeat_interleave(per, dim=1), c, torch.full_like(c, float("-inf")))
    idx = torch.sort(cm, dim=-1, descending=True, stable=True).indices[:, :top]
    w = s.gather(1, idx)
    if renormalize:
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
    return idx.to(torch.int32), w


def moe_combine(rows, h, rowidx, w, out_dtype, extra=None, extra_gate=None) -> torch.Tensor:
    """out[t] = sum_j w[t, j] * (rows[rowidx[t, j]] if rowidx >= 0 else h[t]),
    summed in the order j = 0, 1, ... in fp32 (w None = all ones); then
    + sigmoid(extra_gate[t]) * extra[t] when given. rows [R, W], h [T, W]."""
    T, top = rowidx.shape
    out = torch.zeros(T, h.shape[1], dtype=torch.float32, device=h.device)
    hf = h.float()
    for j in range(top):
        ri = rowidx[:, j].long()
        src = torch.where((ri >= 0)[:, None], rows[ri.clamp(min=0)].float(), hf)
        out += src if w is None else w[:, j:j + 1].float() * src
    if extra is not None:
        out += torch.sigmoid(extra_gate.float()).reshape(T, 1) * extra.float()
    return out.to(out_dtype)


def scale_rows(h, src_row, scale) -> torch.Tensor:
    """out[i] = h[src_row[i]] * scale[i] (product in fp32), in h's dtype."""
    return (h[src_row.long()].float() * scale.float()[:, None]).to(h.dtype)


def moe_spread_rows(h, idx, w, experts: int) -> torch.Tensor:
    """[experts, T, W]: expert e's input rows in the all-experts form of
    input-weighted experts, w[t, j] * h[t] where e is row t's j-th choice and
    zero rows elsewhere."""
    T = h.shape[0]
    wsel = torch.zeros((T, experts), dtype=torch.float32, device=h.device).scatter_(1, idx.long(), w.float())
    return (h.float()[None] * wsel.t()[:, :, None]).to(h.dtype)


def gelu_tanh(x) -> torch.Tensor:
    """0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))) in fp32, in x's dtype."""
    z = x.float()
    return (0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))).to(x.dtype)


def scale_softcap_(z, scale: float, cap: float) -> None:
    """fp32 logits in place: z <- z * scale, then cap * tanh(z / cap) if cap > 0."""
    z.mul_(scale)
    if cap > 0:
        z.copy_(cap * torch.tanh(z / cap))


def latent_kv_store(q, dkv, w_norm, eps, positions, inv_freq, cache, slot_mapping, nope_dim) -> None:
    """Latent-attention step input. q [T, H, nope_dim + R]: the last R entries
    of every head are rotated in place (interleaved pairs, angle = position *
    inv_freq[i], fp32). dkv [T, C + R]: the first C entries are RMS-normed
    (weight w_norm [C]) -> the latent; the last R rotated -> the shared key
    part. cache [NB, 1, BS, C + R] takes the row [latent | rotated part] at
    the token's flat slot."""
    T, H, _ = q.shape
    R2 = inv_freq.numel()
    R = 2 * R2
    C = dkv.shape[1] - R
    BS = cache.shape[2]
    ang = positions.float()[:, None] * inv_freq.float()[None, :]
    cos, sin = torch.cos(ang), torch.sin(ang)

    def rot(x):                        # [..., R] with leading dim T
        xf = x.float()
        u, v = xf[..., 0::2], xf[..., 1::2]
        shp = (T,) + (1,) * (xf.dim() - 2) + (R2,)
        c, s_ = cos.view(shp), sin.view(shp)
        out = torch.empty_like(xf)
        out[..., 0::2] = u * c - v * s_
        out[..., 1::2] = v * c + u * s_
        return out

    q[:, :, nope_dim:] = rot(q[:, :, nope_dim:]).to(q.dtype)
    d = dkv[:, :C].float()
    lat = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w_norm.float()
    row = torch.cat([lat, rot(dkv[:, C:])], -1).to(cache.dtype)
    sl = slot_mapping.long()
    cache[sl // BS, 0, sl % BS] = row


def attn_latent_paged(q_abs, q, cache, block_tables, token_seg, positions, scale, mask_size, gate,
                      nope_dim, out_dtype=None) -> torch.Tensor:
    """Latent attention in its absorbed form. q_abs [T, H, C]: the unrotated
    query parts already multiplied into the latent space; q [T, H, nope_dim +
    R]: its last R entries are the rotated query parts. cache [NB, 1, BS,
    C + R] rows [latent | rotated key part]. Row t at position p sees keys j
    of its own sequence with 0 <= p - j < mask_size (0 = all j <= p):
      score = (q_abs . latent_j + q_rot . krot_j) * scale,  softmax in fp32,
      out[t, h] = sum_j weight_j latent_j   (times sigmoid(gate[t, h]))."""
    T, H, C = q_abs.shape
    BS = cache.shape[2]
    out = torch.empty(T, H, C, dtype=out_dtype or q.dtype, device=q.device)
    pos, seg = positions.tolist(), token_seg.tolist()
    for t in range(T):
        p = pos[t]
        lo = max(0, p - mask_size + 1) if mask_size > 0 else 0
        idx = torch.arange(lo, p + 1, device=q.device)
        rows = cache[block_tables[seg[t]].long()[idx // BS], 0, idx % BS].float()        # [n, C+R]
        s = (q_abs[t].float() @ rows[:, :C].T + q[t, :, nope_dim:].float() @ rows[:, C:].T) * scale
        o = torch.softmax(s, -1) @ rows[:, :C]
        if gate is not None:
            o = o * torch.sigmoid(gate[t].float())[:, None]
        out[t] = o.to(out.dtype)
    return out


# --- layer-normed sublayers with an input convolution and a depth-weighted
# stream; whole-projection q/k norm with half-split rotation; pooled blocks
# before a sliding window; the mamba2 recurrence -----------------------------------

def _ln_stats(y: torch.Tensor, eps: float) -> torch.Tensor:
    mu = y.mean(-1)
    var = (y - mu[:, None]).pow(2).mean(-1)
    return torch.stack([mu, torch.rsqrt(var + eps)], -1)


def ln_residual_mix(x_in, a, w_post, eps, x_out, streams=None, n_prev=0, dwa=None) -> torch.Tensor:
    """y = x_in + layernorm(a) * w_post (y = x_in when a is None; layernorm
    subtracts the mean and divides by sqrt(variance + eps), fp32). With
    ``streams`` [L, T, W]: y is kept as streams[n_prev] and replaced by
    sum_{j <= n_prev} dwa[j] * streams[j] (summed in that order). y goes to
    x_out (fp32, may be x_in); returns its per-row (mean, 1/sqrt(var + eps))
    as [T, 2] fp32, for the norm that reads the stream next."""
    y = x_in.float()
    if a is not None:
        af = a.float()
        st = _ln_stats(af, eps)
        y = y + (af - st[:, :1]) * st[:, 1:] * w_post.float()
    if streams is not None:
        streams[n_prev].copy_(y)
        y = torch.zeros_like(y)
        for j in range(n_prev + 1):
            y = y + dwa[j].float() * streams[j]
    x_out.copy_(y)
    return _ln_stats(y, eps)


def ln_canon(x, stats, w_norm, canon_w, hist, state_slots, cu_seqlens, seg_start, out_dtype) -> torch.Tensor:
    """h = (x - mean) * rstd * w_norm per row (stats [T, 2] from
    ln_residual_mix); returns h_t + sum_j canon_w[j] * h_{t-K+1+j} in
    out_dtype (canon_w [K, W] taps-major, last row = the current token; None:
    h itself). Rows before a segment come from hist [slots, K-1, W] fp32
    (oldest first; zeros for a fresh sequence), which then takes the
    sequence's last K-1 rows of h."""
    h = (x.float() - stats[:, :1]) * stats[:, 1:] * w_norm.float()
    if canon_w is None:
        return h.to(out_dtype)
    K = canon_w.shape[0]
    out = torch.empty_like(h)
    cu, st, sl = cu_seqlens.tolist(), seg_start.tolist(), state_slots.tolist()
    wf = canon_w.float()
    for b in range(len(sl)):
        s, e = cu[b], cu[b + 1]
        if e == s:
            continue
        old = hist[sl[b]].float() if st[b] > 0 else torch.zeros(K - 1, h.shape[1], device=h.device)
        ext = torch.cat([old, h[s:e]], 0)
        acc = h[s:e].clone()
        for j in range(K):
            acc += ext[j:j + (e - s)] * wf[j]
        out[s:e] = acc
        if K > 1:
            hist[sl[b]] = ext[ext.shape[0] - (K - 1):]
    return out.to(out_dtype)


def qk_fullnorm_rope_store(q, k, v, wq, wk, eps, positions, inv_freq, k_cache, v_cache, slot_mapping) -> None:
    """RMS norm over the whole projection of q [T, H, D] (weight wq [H*D]; in
    place) and k [T, G, D] (wk [G*D]), then rotation of the first
    2*len(inv_freq) entries of every head with entry i paired with
    i + len(inv_freq) (angle = position * inv_freq[i], fp32). The normed,
    rotated k and v go to the paged caches. k None: only q (a layer that
    reads another layer's cache)."""
    T = q.shape[0]
    R = inv_freq.numel()
    ang = positions.to(torch.float32)[:, None] * inv_freq.float()[None, :]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]

    def norm_rot(t, w):
        n, d = t.shape[1], t.shape[2]
        tf = t.float().reshape(T, n * d)
        tf = tf * torch.rsqrt(tf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        tf = tf.view(T, n, d)
        if R:
            out = tf.clone()
            u, x2 = tf[..., :R], tf[..., R:2 * R]
            out[..., :R] = u * cos - x2 * sin
            out[..., R:2 * R] = x2 * cos + u * sin
            tf = out
        return tf

    if k is not None:
        BS = k_cache.shape[2]
        blk, off = slot_mapping // BS, slot_mapping % BS
        k_cache[blk, :, off, :] = norm_rot(k, wk).to(k_cache.dtype)
        v_cache[blk, :, off, :] = v.to(v_cache.dtype)
    q.copy_(norm_rot(q, wq).to(q.dtype))


def pool_entry(b: int, run: int, BS: int):
    """(page index within the sequence, offset within the page's pooled
    entries) of pooled run b: the page of the run's last token, counted from
    the first run that ends in that page."""
    pg = ((b + 1) * run - 1) // BS
    return pg, b - (pg * BS) // run


def pool_kv_update(k_cache, v_cache, pool_k, pool_v, block_tables, token_seg, positions, run: int,
                   row_map=None) -> None:
    """For every row (of row_map, or of the step) whose position ends an
    aligned run of ``run`` positions: the fp32 means of the run's cached keys
    and values go to pool_k / pool_v [NB, G, ceil(BS / run), D|Dv]."""
    BS = k_cache.shape[2]
    pos, seg = positions.tolist(), token_seg.tolist()
    for t in (range(len(pos)) if row_map is None else row_map.tolist()):
        p = pos[t]
        if (p + 1) % run:
            continue
        b = p // run
        bt = block_tables[seg[t]].long()
        idx = torch.arange(b * run, (b + 1) * run, device=k_cache.device)
        pg, off = pool_entry(b, run, BS)
        pool_k[bt[pg], :, off, :] = k_cache[bt[idx // BS], :, idx % BS, :].float().mean(0)
        pool_v[bt[pg], :, off, :] = v_cache[bt[idx // BS], :, idx % BS, :].float().mean(0)


def attn_window_pool_paged(q, k_cache, v_cache, pool_k, pool_v, block_tables, token_seg, positions, scale,
                           softcap, mask_size, run, out_dtype=None) -> torch.Tensor:
    """Softmax attention of packed query rows against the paged cache. Row t
    at position p sees keys j of its own sequence with 0 <= p - j < mask_size
    (0 = all j <= p) and, when run > 0, the pooled entry of every aligned run
    of ``run`` positions that ends at or before p - mask_size. Scores are
    q . k * scale, soft-capped as cap * tanh(s / cap) when softcap > 0; one
    softmax over entries and tokens."""
    T, H, D = q.shape
    _, G, BS, Dv = v_cache.shape
    rep = H // G
    out = torch.empty(T, H, Dv, dtype=out_dtype or q.dtype, device=q.device)
    pos, seg = positions.tolist(), token_seg.tolist()
    for t in range(T):
        p = pos[t]
        lo = max(0, p - mask_size + 1) if mask_size > 0 else 0
        idx = torch.arange(lo, p + 1, device=q.device)
        bt = block_tables[seg[t]].long()
        kk = k_cache[bt[idx // BS], :, idx % BS, :].float()
        vv = v_cache[bt[idx // BS], :, idx % BS, :].float()
        nb = lo // run if run > 0 else 0
        if nb:
            ent = [pool_entry(b, run, BS) for b in range(nb)]
            pg = bt[torch.tensor([e[0] for e in ent], device=q.device)]
            off = torch.tensor([e[1] for e in ent], device=q.device)
            kk = torch.cat([pool_k[pg, :, off, :].float(), kk], 0)
            vv = torch.cat([pool_v[pg, :, off, :].float(), vv], 0)
        s = torch.einsum("grd,ngd->grn", q[t].float().view(G, rep, D), kk) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        o = torch.einsum("grn,ngd->grd", torch.softmax(s, dim=-1), vv).reshape(H, Dv)
        out[t] = o.to(out.dtype)
    return out


def ssd_recurrence(x, B, C, dt, dt_bias, a_log, skip, state, state_slots, cu_seqlens, seg_start) -> torch.Tensor:
    """State-space recurrence with a scalar decay per head and token.
    x [T, H, V], B and C [T, G, N] (already convolved + silu), dt [T, H] raw;
    per head h of group g: d = softplus(dt + dt_bias), S <- exp(-exp(a_log) d) S
    + d B x^T, o = S^T C + skip x. state [slots, H, N, V] fp32 is read (unless
    seg_start == 0) and written back. Everything in fp32; returns o [T, H, V]."""
    T, H, V = x.shape
    G = B.shape[1]
    rep = H // G
    xf = x.float()
    Bf = B.float().repeat_interleave(rep, dim=1)
    Cf = C.float().repeat_interleave(rep, dim=1)
    d = torch.nn.functional.softplus(dt.float() + dt_bias.float(), threshold=20.0)
    dec = torch.exp(-torch.exp(a_log.float()) * d)
    o = torch.empty(T, H, V, dtype=torch.float32, device=x.device)
    cu, st, sl = cu_seqlens.tolist(), seg_start.tolist(), state_slots.tolist()
    for b in range(len(sl)):
        S = state[sl[b]].clone() if st[b] > 0 else torch.zeros_like(state[sl[b]])
        for t in range(cu[b], cu[b + 1]):
            S = dec[t].view(H, 1, 1) * S + (d[t].view(H, 1) * Bf[t]).unsqueeze(-1) * xf[t].unsqueeze(-2)
            o[t] = torch.einsum("hnv,hn->hv", S, Cf[t]) + skip.float().view(H, 1) * xf[t]
        state[sl[b]] = S
    return o


def gate_group_rmsnorm(o, weight, gate, eps, out_dtype) -> torch.Tensor:
    """o [T, n_groups, S] fp32 times silu(gate) ([T, n_groups*S] logits), then
    each group divided by its root mean square, times weight [n_groups*S]."""
    T, Gn, S = o.shape
    y = o.float() * torch.nn.functional.silu(gate.float()).view(T, Gn, S)
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps)
    return (y.reshape(T, Gn * S) * weight.float()).to(out_dtype)
