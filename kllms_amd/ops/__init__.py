"""Op dispatch: HIP/CDNA4 kernels on GPU, torch reference on CPU.

Policy: on a GPU (`tensor.is_cuda`, which on
PyTorch-ROCm means an AMD GPU) the hand-written gfx950 HIP kernels in
``kllms_amd._C`` are the ONLY path — if the extension is missing the op
RAISES instead of silently falling back to eager PyTorch. On CPU the pure
torch reference implementations (torch_ref.py) run, which is what the
GPU-less CI environment uses.

Set ``KLLMS_AMD_FORCE_TORCH_OPS=1`` to force the torch path on GPU (used only
by numerics tests to produce the oracle on-device).
"""

from __future__ import annotations

import os
from typing import Optional, Tuple

import torch

from . import torch_ref

_C = None
_C_err: Optional[str] = None
try:
    from kllms_amd import _C  # type: ignore[no-redef]  # built by setup.py build_ext --inplace
except Exception as e:  # pragma: no cover - import-time probe
    _C = None
    _C_err = str(e)


def hip_available() -> bool:
    return _C is not None


def _force_torch() -> bool:
    return os.environ.get("KLLMS_AMD_FORCE_TORCH_OPS", "0") == "1"


def _hip_or_raise():
    if _C is None:
        raise RuntimeError(
            "kllms_amd HIP extension (kllms_amd/_C*.so) is not built but a GPU "
            "tensor was passed. Build it with `python setup.py build_ext --inplace` "
            f"(PYTORCH_ROCM_ARCH=gfx950). Import error: {_C_err}"
        )
    return _C


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    if x.is_cuda and not _force_torch():
        out = torch.empty_like(x)
        _hip_or_raise().rmsnorm(out, x, weight, eps)
        return out
    return torch_ref.rmsnorm(x, weight, eps)


def fused_add_rmsnorm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
) -> Tuple[torch.Tensor, torch.Tensor]:
    if x.is_cuda and not _force_torch():
        # in-place: residual += x; x_out = rmsnorm(residual)
        out = torch.empty_like(x)
        _hip_or_raise().fused_add_rmsnorm(out, x, residual, weight, eps)
        return out, residual
    return torch_ref.fused_add_rmsnorm(x, residual, weight, eps)


def rope_inplace(q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor, cos_sin: torch.Tensor) -> None:
    if q.is_cuda and not _force_torch():
        _hip_or_raise().rope_inplace(q, k, positions, cos_sin)
        return
    torch_ref.rope_inplace(q, k, positions, cos_sin)


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    if gate.is_cuda and not _force_torch():
        out = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
        _hip_or_raise().silu_mul(out, gate, up)
        return out
    return torch_ref.silu_mul(gate, up)


def store_kv(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    k_scale: Optional[torch.Tensor] = None,
    v_scale: Optional[torch.Tensor] = None,
) -> None:
    """k_scale/v_scale: [NB, KVH, BS] fp32 per-row dequant scales, REQUIRED
    when the caches are fp8 (written here: s = amax(|row|)/448), None for bf16."""
    if k.is_cuda and not _force_torch():
        none = torch.empty(0, dtype=torch.float32, device=k.device)
        _hip_or_raise().store_kv(
            k, v, k_cache, v_cache, slot_mapping,
            k_scale if k_scale is not None else none,
            v_scale if v_scale is not None else none)
        return
    torch_ref.store_kv(k, v, k_cache, v_cache, slot_mapping, k_scale, v_scale)


def _prefill_tiles(cu_seqlens: torch.Tensor, device) -> tuple:
    """Grouped q-tile metadata for the MFMA prefill kernel: 32-row q-tiles of
    each sequence packed 8 per workgroup (the 8 waves share the K/V LDS
    staging); idle wave slots padded with -1. One host round-trip per prefill
    batch (once per generate() call)."""
    NW = 8
    cu = cu_seqlens.cpu().tolist()
    grp_start, grp_len, grp_qpos0 = [], [], []
    for i in range(len(cu) - 1):
        s, e = cu[i], cu[i + 1]
        L = e - s
        tiles = list(range(0, L, 32))
        for g0 in range(0, len(tiles), NW):
            grp_start.append(s)
            grp_len.append(L)
            grp = tiles[g0 : g0 + NW]
            grp_qpos0.extend(grp + [-1] * (NW - len(grp)))
    t = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    return t(grp_start), t(grp_qpos0), t(grp_len)


def attn_prefill_varlen(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_seqlens: torch.Tensor, scale: float
) -> torch.Tensor:
    if q.is_cuda and not _force_torch():
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        gs, gq, gl = _prefill_tiles(cu_seqlens, q.device)
        _hip_or_raise().attn_prefill(out, q, k, v, gs, gq, gl, scale)
        return out
    return torch_ref.attn_prefill_varlen(q, k, v, cu_seqlens, scale)


def attn_decode_paged(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    context_lens: torch.Tensor,
    scale: float,
    k_scale: Optional[torch.Tensor] = None,
    v_scale: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    if q.is_cuda and not _force_torch():
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
        none = torch.empty(0, dtype=torch.float32, device=q.device)
        _hip_or_raise().attn_decode_paged(
            out, q, k_cache, v_cache, block_tables, context_lens, scale,
            k_scale if k_scale is not None else none,
            v_scale if v_scale is not None else none)
        return out
    return torch_ref.attn_decode_paged(q, k_cache, v_cache, block_tables, context_lens, scale,
                                       k_scale, v_scale)


def sample(
    logits: torch.Tensor,
    temperatures: torch.Tensor,
    top_ps: torch.Tensor,
    top_ks: torch.Tensor,
    seeds: torch.Tensor,
    steps: torch.Tensor,
    mask: Optional[torch.Tensor] = None,
    dbg: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    if logits.is_cuda and not _force_torch():
        B = logits.shape[0]
        tokens = torch.empty(B, dtype=torch.long, device=logits.device)
        logprobs = torch.empty(B, dtype=torch.float32, device=logits.device)
        _hip_or_raise().sample(
            tokens, logprobs, logits, temperatures, top_ps, top_ks, seeds, steps,
            mask if mask is not None else torch.empty(0, dtype=torch.int32, device=logits.device),
            dbg if dbg is not None else torch.empty(0, dtype=torch.float32, device=logits.device),
        )
        return tokens, logprobs
    return torch_ref.sample(logits, temperatures, top_ps, top_ks, seeds, steps, mask)


def moe_gateup(
    act: torch.Tensor,
    x: torch.Tensor,
    w_gate_up: torch.Tensor,
    sorted_ids: torch.Tensor,
    pad_offsets: torch.Tensor,
    zeros: torch.Tensor,
) -> None:
    """Grouped MoE gate/up GEMM + fused silu*mul into `act` (sorted-by-expert
    row space). GPU-only (Mixtral prefill hot path); the CPU path keeps the
    per-expert torch loop in models/mixtral.py."""
    _hip_or_raise().moe_gateup(act, x, w_gate_up, sorted_ids, pad_offsets, zeros)


def moe_down(
    y: torch.Tensor,
    act: torch.Tensor,
    w_down: torch.Tensor,
    pad_offsets: torch.Tensor,
) -> None:
    """Grouped MoE down GEMM in sorted-row space (see moe_gateup)."""
    _hip_or_raise().moe_down(y, act, w_down, pad_offsets)


def levenshtein_pairs(
    chars: torch.Tensor,
    lens: torch.Tensor,
    pair_i: torch.Tensor,
    pair_j: torch.Tensor,
) -> torch.Tensor:
    """Batched Myers bit-parallel edit distance over packed [N, 64] uint8
    normalized strings; returns int32 distances per (i, j) pair. GPU-only —
    the CPU consensus path keeps the pure-python DP (utils/text.py)."""
    return _hip_or_raise().levenshtein_pairs(chars, lens, pair_i, pair_j)


# --- sequence-mixer family (kllms_amd._C_seq) -----------------------------------
# fp32 residual stream, block-local paged attention, recurrent mixers. The
# extension is separate from _C so that a model of this family compiles only
# its own kernels in a checkout where nothing is built yet.

_SEQ = None


def _seq():
    global _SEQ
    if _SEQ is None:
        from . import jit

        _SEQ = jit.load("_C_seq")
    return _SEQ


def seq_hip_loaded() -> bool:
    return _SEQ is not None


def _gpu(t: torch.Tensor) -> bool:
    return t.is_cuda and not _force_torch()


def _none(ref: torch.Tensor, dtype=None) -> torch.Tensor:
    return torch.empty(0, dtype=dtype or ref.dtype, device=ref.device)


def embed_rmsnorm(ids, table, weight, eps, pos_table=None, positions=None):
    """fp32 rms(table[ids] (+ pos_table[positions])) * weight."""
    if _gpu(table):
        out = torch.empty((ids.numel(), table.shape[1]), dtype=torch.float32, device=table.device)
        has = pos_table is not None
        _seq().embed_rmsnorm(out, ids, table, weight, eps, pos_table if has else _none(table),
                             positions if has else _none(table, torch.long))
        return out
    return torch_ref.embed_rmsnorm(ids, table, weight, eps, pos_table, positions)


def rmsnorm_cast(x, weight, eps, out_dtype):
    if _gpu(x):
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _seq().rmsnorm_cast(out, x, weight, eps)
        return out
    return torch_ref.rmsnorm_cast(x, weight, eps, out_dtype)


def sandwich_residual(x, a, w_post, eps, b=None, wa=None, wb=None, w_next=None, out_dtype=None, cast=False):
    """x (fp32 residual, in place) += rms(y) * w_post with y = a, or
    y = (rms(a) wa + rms(b) wb) / 2; returns rms(x) * w_next in a's dtype.
    With w_next None: the new x in a's dtype if ``cast`` (the input of a
    sublayer that reads the stream itself), else None."""
    if _gpu(x):
        want = w_next is not None or cast
        out = torch.empty(a.shape, dtype=a.dtype, device=a.device) if want else _none(a)
        f = _none(x, torch.float32)
        _seq().sandwich_residual(
            x, a, b if b is not None else _none(a), wa if b is not None else f, wb if b is not None else f,
            w_post, w_next if w_next is not None else f, out, eps)
        return out if want else None
    return torch_ref.sandwich_residual(x, a, w_post, eps, b, wa, wb, w_next, out_dtype or a.dtype, cast)


def rope_pairs_store(q, k, v, positions, inv_freq, k_cache, v_cache, slot_mapping, kv_fresh=None) -> None:
    """kv_fresh (GPU only, optional): [T, 2, G, D] buffer that also receives
    this step's rotated keys ([:, 0]) and values ([:, 1]) packed, for the
    dense prefill kernel."""
    if _gpu(q):
        _seq().rope_pairs_store(q, k, v if v is not None else _none(q), positions, inv_freq,
                                k_cache, v_cache, slot_mapping,
                                kv_fresh if kv_fresh is not None else _none(q))
        return
    torch_ref.rope_pairs_store(q, k, v, positions, inv_freq, k_cache, v_cache, slot_mapping)


def attn_masked_paged(q, k_cache, v_cache, block_tables, token_seg, positions, scale, mask_kind, mask_size,
                      keep_first=0, sink=False, gate=None, row_map=None, out=None):
    """Paged softmax attention with a block-local (mask_kind 0) or sliding
    window + kept first tokens (mask_kind 1) causal mask, optional sink term,
    gate per head [T, H] or per element [T, H*Dv]. row_map / out (GPU only):
    serve just the listed rows, writing into an existing [T, H, Dv] tensor
    whose other rows another kernel fills."""
    if _gpu(q):
        if out is None:
            out = torch.empty((q.shape[0], q.shape[1], v_cache.shape[3]), dtype=q.dtype, device=q.device)
        _seq().attn_masked_paged(out, q, k_cache, v_cache, block_tables, token_seg, positions,
                                 gate if gate is not None else _none(q), scale, int(mask_kind), int(mask_size),
                                 int(keep_first), bool(sink),
                                 row_map if row_map is not None else _none(q, torch.int32),
                                 _none(q, torch.float32), _none(q, torch.float32), 0, 0.0,
                                 _none(q, torch.float32), _none(q, torch.float32))
        return out
    assert row_map is None and out is None
    return torch_ref.attn_masked_paged(q, k_cache, v_cache, block_tables, token_seg, positions, scale,
                                       mask_kind, mask_size, keep_first, sink, gate)


def attn_blocklocal_paged(q, k_cache, v_cache, block_tables, token_seg, positions, scale, mask_size,
                          gate=None, row_map=None, out=None):
    """Block-local mask, no sink, per-head gate: a case of attn_masked_paged."""
    if _gpu(q):
        return attn_masked_paged(q, k_cache, v_cache, block_tables, token_seg, positions, scale, 0, mask_size,
                                 0, False, gate, row_map, out)
    assert row_map is None and out is None
    return torch_ref.attn_blocklocal_paged(q, k_cache, v_cache, block_tables, token_seg, positions,
                                           scale, mask_size, gate)


def attn_varlen_mfma(out, q, k, v, grp_start, grp_qpos0, grp_len, scale) -> None:
    """Dense causal MFMA attention over packed pieces (bf16, head size 128;
    GPU only): each piece attends within itself. Tile groups come from
    dense_tile_groups()."""
    _seq().attn_varlen_mfma(out, q, k, v, grp_start, grp_qpos0, grp_len, scale)


def dense_tile_groups(pieces, device):
    """Host metadata for attn_varlen_mfma: pieces = [(first row, length)];
    32-row q-tiles of each piece, 8 per workgroup (idle wave slots = -1)."""
    NW = 8
    gs, gl, gq = [], [], []
    for row0, L in pieces:
        tiles = list(range(0, L, 32))
        for g0 in range(0, len(tiles), NW):
            grp = tiles[g0:g0 + NW]
            gs.append(row0)
            gl.append(L)
            gq.extend(grp + [-1] * (NW - len(grp)))
    t = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    return t(gs), t(gq), t(gl)


def head_gate(out, gate) -> None:
    """out[t, h, :] *= sigmoid(gate[t, h]) in place."""
    if _gpu(out):
        _seq().head_gate(out, gate)
        return
    out.mul_(torch.sigmoid(gate.float()).unsqueeze(-1).to(out.dtype))


def linear_attn_decay(q, k, v, decay, state, state_slots, cu_seqlens, seg_start):
    if _gpu(q):
        o = torch.empty((q.shape[0], q.shape[1], v.shape[2]), dtype=torch.float32, device=q.device)
        _seq().linear_attn_decay(o, q, k, v, decay, state, state_slots, cu_seqlens, seg_start)
        return o
    return torch_ref.linear_attn_decay(q, k, v, decay, state, state_slots, cu_seqlens, seg_start)


def gated_rmsnorm(o, weight, gate, eps, out_dtype):
    if _gpu(o):
        out = torch.empty((o.shape[0], o.shape[1] * o.shape[2]), dtype=out_dtype, device=o.device)
        _seq().gated_rmsnorm(out, o, weight, gate, eps, False)
        return out
    return torch_ref.gated_rmsnorm(o, weight, gate, eps, out_dtype)


def causal_conv_silu(x, w, conv_state, state_slots, cu_seqlens, seg_start, token_seg, bias=None):
    if _gpu(x):
        y = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _seq().causal_conv_silu(y, x, w, conv_state, state_slots, cu_seqlens, seg_start, token_seg,
                                bias if bias is not None else _none(x, torch.float32))
        return y
    return torch_ref.causal_conv_silu(x, w, conv_state, state_slots, cu_seqlens, seg_start, bias)


def gated_delta_rule(q, k, v, beta_logit, a, dt_bias, a_log, state, state_slots, cu_seqlens, seg_start):
    if _gpu(q):
        o = torch.empty((v.shape[0], v.shape[1], v.shape[2]), dtype=torch.float32, device=q.device)
        _seq().gated_delta_rule(o, q, k, v, beta_logit, a, dt_bias, a_log, state, state_slots,
                                cu_seqlens, seg_start)
        return o
    return torch_ref.gated_delta_rule(q, k, v, beta_logit, a, dt_bias, a_log, state, state_slots,
                                      cu_seqlens, seg_start)


def gated_act(gate, up, limit: float, alpha: float, up_bias: float):
    """min(g, limit) sigmoid(alpha min(g, limit)) (clamp(u, +-limit) + up_bias)."""
    if _gpu(gate):
        out = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
        _seq().gated_act(out, gate, up, limit, alpha, up_bias)
        return out
    return torch_ref.gated_act(gate, up, limit, alpha, up_bias)


def clamped_glu(gate, up, limit: float, alpha: float):
    if _gpu(gate):
        return gated_act(gate, up, limit, alpha, 1.0)
    return torch_ref.clamped_glu(gate, up, limit, alpha)


def silu_glu(gate, up):
    """silu(gate) * up in the activation dtype (bf16 or fp32)."""
    return gated_act(gate, up, float("inf"), 1.0, 0.0)


def embed_bigram(ids, table, bigram, scale, mul_prev, mul_cur, buckets, tok_state, state_slots, cu_seqlens,
                 seg_start, token_seg, out=None):
    """fp32 rows table[id] * scale (+ the hashed bigram row); ``out``: an
    existing contiguous [T, W] fp32 tensor to fill."""
    if _gpu(table):
        if out is None:
            out = torch.empty((ids.numel(), table.shape[1]), dtype=torch.float32, device=table.device)
        has = bigram is not None
        _seq().embed_bigram(out, ids, table, bigram if has else _none(table), float(scale), int(mul_prev),
                            int(mul_cur), int(buckets), tok_state if has else _none(table, torch.int32),
                            state_slots, cu_seqlens, seg_start, token_seg)
        return out
    x = torch_ref.embed_bigram(ids, table, bigram, scale, mul_prev, mul_cur, buckets, tok_state,
                               state_slots, cu_seqlens, seg_start)
    return x if out is None else out.copy_(x)


def group_norm_pair(x, a, b, w1, w2, groups, eps, out_dtype):
    """x (fp32 residual, in place) += a + b; returns the grouped RMS norm of x
    under two weights (the second may be None)."""
    if _gpu(x):
        h1 = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        h2 = torch.empty(x.shape, dtype=out_dtype, device=x.device) if w2 is not None else None
        f = _none(x, torch.float32)
        e = _none(x, out_dtype)
        _seq().group_norm_pair(x, a if a is not None else e, b if b is not None else e, w1,
                               w2 if w2 is not None else f, h1, h2 if h2 is not None else e, int(groups), eps)
        return h1, h2
    return torch_ref.group_norm_pair(x, a, b, w1, w2, groups, eps, out_dtype)


def cast_concat(x, x0, a, b, out_dtype):
    """x (fp32 residual, in place) += a + b; returns [x | x0] in out_dtype."""
    if _gpu(x):
        out = torch.empty((x.shape[0], 2 * x.shape[1]), dtype=out_dtype, device=x.device)
        e = _none(x, out_dtype)
        _seq().cast_concat(out, x, x0, a if a is not None else e, b if b is not None else e)
        return out
    return torch_ref.cast_concat(x, x0, a, b, out_dtype)


def qk_norm_store(q, k, v, wq, wk, eps, k_cache, v_cache, slot_mapping) -> None:
    if _gpu(q):
        _seq().qk_norm_store(q, k, v, wq, wk, eps, k_cache, v_cache, slot_mapping)
        return
    torch_ref.qk_norm_store(q, k, v, wq, wk, eps, k_cache, v_cache, slot_mapping)


def token_shift_mix(h, mu, shift_state, state_slots, cu_seqlens, seg_start, token_seg, n_act):
    """([n_act, T, W] in h's dtype, [n - n_act, T, W] fp32) mixes of each row
    with its predecessor; carries the last row in shift_state."""
    if _gpu(h):
        T, W = h.shape
        n = mu.shape[0]
        act = torch.empty((n_act, T, W), dtype=h.dtype, device=h.device)
        f32 = torch.empty((n - n_act, T, W), dtype=torch.float32, device=h.device)
        _seq().token_shift_mix(act, f32, h, mu, shift_state, state_slots, cu_seqlens, seg_start, token_seg)
        return act, f32
    return torch_ref.token_shift_mix(h, mu, shift_state, state_slots, cu_seqlens, seg_start, n_act, h.dtype)


def wkv_recurrence(r, k, v, d, w0, u, state, state_slots, cu_seqlens, seg_start):
    if _gpu(r):
        o = torch.empty((r.shape[0], r.shape[1], v.shape[2]), dtype=torch.float32, device=r.device)
        _seq().wkv_recurrence(o, r, k, v, d, w0, u, state, state_slots, cu_seqlens, seg_start)
        return o
    return torch_ref.wkv_recurrence(r, k, v, d, w0, u, state, state_slots, cu_seqlens, seg_start)


def mlstm_recurrence(q, k, v, gates, gate_bias, cap, state, state_slots, cu_seqlens, seg_start):
    if _gpu(q):
        o = torch.empty((q.shape[0], q.shape[1], v.shape[2]), dtype=torch.float32, device=q.device)
        e = _none(q, torch.float32)
        _seq().mlstm_recurrence(o, q, k, v, gates, gate_bias, float(cap), state, state_slots, cu_seqlens,
                                seg_start, e, e)
        return o
    return torch_ref.mlstm_recurrence(q, k, v, gates, gate_bias, cap, state, state_slots, cu_seqlens,
                                      seg_start)


def mlstm_mix_out(q, k, v, gates, gate_bias, cap, state, state_slots, cu_seqlens, seg_start, weight, gate, eps,
                  out_dtype):
    """mlstm_recurrence followed by head_rmsnorm_gate(sigmoid); on the GPU the
    read-out's division happens inside the norm kernel."""
    if _gpu(q):
        T, H, V = q.shape[0], q.shape[1], v.shape[2]
        oe = torch.empty((T, H, V + 1), dtype=torch.float32, device=q.device)
        mt = torch.empty((T, H), dtype=torch.float32, device=q.device)
        _seq().mlstm_recurrence(_none(q, torch.float32), q, k, v, gates, gate_bias, float(cap), state, state_slots,
                                cu_seqlens, seg_start, oe, mt)
        out = torch.empty((T, H * V), dtype=out_dtype, device=q.device)
        _seq().head_rmsnorm_gate(out, oe, weight, gate, eps, 0, mt)
        return out
    o = torch_ref.mlstm_recurrence(q, k, v, gates, gate_bias, cap, state, state_slots, cu_seqlens, seg_start)
    return torch_ref.head_rmsnorm_gate(o, weight, gate, eps, "sigmoid", out_dtype)


def head_rmsnorm_gate(o, weight, gate, eps, gate_act, out_dtype):
    if _gpu(o):
        out = torch.empty((o.shape[0], o.shape[1] * o.shape[2]), dtype=out_dtype, device=o.device)
        _seq().head_rmsnorm_gate(out, o, weight, gate, eps, 0 if gate_act == "sigmoid" else 1,
                                 _none(o, torch.float32))
        return out
    return torch_ref.head_rmsnorm_gate(o, weight, gate, eps, gate_act, out_dtype)


def moe_route(z, correction, top, group_count, group_keep, score="softmax", renormalize=True):
    """Routing from fp32 logits z [T, N]: (idx [T, top] int32, w [T, top] fp32)."""
    if _gpu(z):
        idx = torch.empty((z.shape[0], top), dtype=torch.int32, device=z.device)
        w = torch.empty((z.shape[0], top), dtype=torch.float32, device=z.device)
        _seq().moe_route(idx, w, _none(z, torch.int32), z, _none(z),
                         correction if correction is not None else _none(z), int(top), int(group_count),
                         int(group_keep), 0, 0 if score == "softmax" else 1, bool(renormalize))
        return idx, w
    return torch_ref.moe_route(z, correction, top, group_count, group_keep, score, renormalize)


def moe_route_rows(h, router, correction, top, group_count, group_keep, experts, all_experts_form,
                   score="softmax", renormalize=True):
    """Router GEMV in fp32 + routing in one kernel. Returns (idx, w, rowidx);
    rowidx [T, top] (only when all_experts_form) addresses rows of the
    all-experts output [experts * T, W]: choice * T + row, -1 = identity."""
    T = h.shape[0]
    if _gpu(h):
        idx = torch.empty((T, top), dtype=torch.int32, device=h.device)
        w = torch.empty((T, top), dtype=torch.float32, device=h.device)
        rowidx = torch.empty((T, top), dtype=torch.int32, device=h.device) if all_experts_form else None
        _seq().moe_route(idx, w, rowidx if rowidx is not None else _none(h, torch.int32), h, router,
                         correction if correction is not None else _none(router),
                         int(top), int(group_count), int(group_keep), int(experts),
                         0 if score == "softmax" else 1, bool(renormalize))
        return idx, w, rowidx
    z = torch.nn.functional.linear(h.float(), router)
    idx, w = torch_ref.moe_route(z, correction, top, group_count, group_keep, score, renormalize)
    rowidx = None
    if all_experts_form:
        t_idx = torch.arange(T, dtype=torch.int32, device=h.device).unsqueeze(1)
        rowidx = torch.where(idx < experts, idx * T + t_idx, torch.full_like(idx, -1))
    return idx, w, rowidx


def moe_combine(rows, h, rowidx, w, out_dtype, extra=None, extra_gate=None):
    """Fixed-order sum of each row's chosen expert rows, weighted by w (None =
    unweighted), plus sigmoid(extra_gate[t]) * extra[t] when given
    (extra_gate: a [T] view, any stride)."""
    if _gpu(h):
        out = torch.empty(h.shape, dtype=out_dtype, device=h.device)
        _seq().moe_combine(out, rows, h, rowidx, w if w is not None else _none(h, torch.float32),
                           extra if extra is not None else _none(h),
                           extra_gate if extra is not None else _none(h))
        return out
    return torch_ref.moe_combine(rows, h, rowidx, w, out_dtype, extra, extra_gate)


def scale_rows(h, src_row, scale):
    """out[i] = h[src_row[i]] * scale[i]: expert inputs that carry their
    routing weight. src_row int32 [n], scale fp32 [n]."""
    if _gpu(h):
        out = torch.empty((src_row.numel(), h.shape[1]), dtype=h.dtype, device=h.device)
        _seq().scale_rows(out, h, src_row, scale)
        return out
    return torch_ref.scale_rows(h, src_row, scale)


def moe_spread_rows(h, idx, w, experts: int):
    """[experts, T, W] inputs of the all-experts form when the routing weight
    sits on the expert's input: w[t, j] * h[t] for row t's j-th choice, zero
    rows for the experts a row did not choose."""
    if _gpu(h):
        out = torch.empty((experts, h.shape[0], h.shape[1]), dtype=h.dtype, device=h.device)
        _seq().moe_spread_rows(out, h, idx, w)
        return out
    return torch_ref.moe_spread_rows(h, idx, w, experts)


def gelu_tanh(x):
    """Tanh-form gelu of a [T, C] row view, in x's dtype."""
    if _gpu(x):
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
        _seq().gelu_tanh(out, x)
        return out
    return torch_ref.gelu_tanh(x)


def scale_softcap_(z, scale: float, cap: float) -> None:
    """fp32 logits in place: z * scale, then cap * tanh(. / cap) if cap > 0."""
    if _gpu(z):
        _seq().scale_softcap(z, float(scale), float(cap))
        return
    torch_ref.scale_softcap_(z, scale, cap)


def latent_kv_store(q, dkv, w_norm, eps, positions, inv_freq, cache, slot_mapping, nope_dim) -> None:
    """Rotates the rotated part of every query head in place; norms the
    latent, rotates the shared key part and stores [latent | key part] into
    the paged latent cache."""
    if _gpu(q):
        _seq().latent_kv_store(q, dkv, w_norm, eps, positions, inv_freq, cache, slot_mapping, int(nope_dim))
        return
    torch_ref.latent_kv_store(q, dkv, w_norm, eps, positions, inv_freq, cache, slot_mapping, nope_dim)


def attn_latent_paged(q_abs, q, cache, block_tables, token_seg, positions, scale, mask_size, gate, nope_dim,
                      tile_rows: int = 0, use_mfma: bool = True, key_splits: int = 0):
    """Sliding-window softmax attention over the paged latent cache in the
    absorbed form (one shared key/value row per token for all heads):
    returns the heads' weighted latent sums [T, H, C], gated per head.
    GPU: bf16 rows go through the matrix-unit kernel when the sizes fit it
    (``tile_rows`` = query rows per workgroup, 0 = as many as fit 32 (row,
    head) columns; 1 suits steps of single decoded tokens), fp32 rows and
    other sizes through the plain kernel. ``key_splits`` (with tile_rows 1):
    workgroups that share one row's keys, merged by a second kernel; 0 = as
    many as fill the chip for this step (few rows, long windows), -1 = none."""
    if _gpu(q):
        T, H, C = q.shape[0], q.shape[1], q_abs.shape[2]
        out = torch.empty((T, H, C), dtype=q.dtype, device=q.device)
        ns = 1
        if tile_rows == 1 and use_mfma and q.dtype == torch.bfloat16 and key_splits >= 0:
            # an upper bound of a row's 32-key tiles, from the window or the block table's width
            reach = mask_size if mask_size > 0 else block_tables.shape[1] * cache.shape[2]
            reach = min(reach, block_tables.shape[1] * cache.shape[2])
            tiles = max(1, (reach + 31) // 32)
            groups = T * ((H + 31) // 32)
            # about four tiles per workgroup, and no more workgroups than two per compute unit
            ns = key_splits or max(1, min((tiles + 3) // 4, 512 // max(1, groups)))
            ns = max(1, min(ns, tiles, 64))
        f = torch.float32
        part_o = torch.empty((T, H, ns, C), dtype=f, device=q.device) if ns > 1 else _none(q, f)
        part_ml = torch.empty((T, H, ns, 2), dtype=f, device=q.device) if ns > 1 else _none(q, f)
        _seq().attn_latent_paged(out, q_abs, q, cache, block_tables, token_seg, positions,
                                 gate if gate is not None else _none(q), float(scale), int(mask_size),
                                 int(nope_dim), int(tile_rows), bool(use_mfma), part_o, part_ml)
        return out
    return torch_ref.attn_latent_paged(q_abs, q, cache, block_tables, token_seg, positions, scale, mask_size,
                                       gate, nope_dim)


def attn_window_sink(q, st, batch, spec, gate):
    """Windowed attention with kept first tokens and a sink for one step's
    rows, keys through the block table (prompt portions, decoded tokens and
    mixes alike)."""
    return attn_masked_paged(q, st.k, st.v, batch.block_tables, batch.token_seg, batch.positions, spec.scale,
                             1, spec.mask_size, spec.keep_first, spec.sink, gate)


def ln_residual_mix(x_in, a, w_post, eps, x_out, streams=None, n_prev=0, dwa=None):
    """x_out = x_in + layernorm(a) * w_post (a None: x_in itself); with
    ``streams`` [L, T, W] the sum is kept as streams[n_prev] and x_out becomes
    sum_{j <= n_prev} dwa[j] * streams[j]. Returns the (mean, rstd) of every
    row of x_out, [T, 2] fp32 — what the next layer norm of the stream needs."""
    if _gpu(x_in):
        stats = torch.empty((x_in.shape[0], 2), dtype=torch.float32, device=x_in.device)
        f = _none(x_in, torch.float32)
        has = streams is not None
        _seq().ln_residual_mix(x_out, x_in, a if a is not None else f, w_post if a is not None else f, stats,
                               streams if has else f, dwa if has else f, int(n_prev), eps)
        return stats
    return torch_ref.ln_residual_mix(x_in, a, w_post, eps, x_out, streams, n_prev, dwa)


def ln_canon(x, stats, w_norm, canon_w, hist, state_slots, cu_seqlens, seg_start, token_seg, out_dtype):
    """Layer norm of the fp32 stream from its row statistics, times w_norm,
    plus the short causal convolution of that normed row with its
    predecessors (canon_w [K, W] taps-major; None = norm only); the
    sequence's last K-1 normed rows are carried in hist [slots, K-1, W] fp32."""
    if _gpu(x):
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        f = _none(x, torch.float32)
        has = canon_w is not None
        i = _none(x, torch.int32)
        _seq().ln_canon(out, x, stats, w_norm, canon_w if has else f, hist if has else f,
                        state_slots if has else i, cu_seqlens if has else i, seg_start if has else i,
                        token_seg if has else i)
        return out
    return torch_ref.ln_canon(x, stats, w_norm, canon_w, hist, state_slots, cu_seqlens, seg_start, out_dtype)


def qk_fullnorm_rope_store(q, k, v, wq, wk, eps, positions, inv_freq, k_cache, v_cache, slot_mapping) -> None:
    """Whole-projection RMS norm of q (in place) and k, half-split rotation of
    the first 2 * len(inv_freq) entries of every head, normed rotated k and v
    into the paged caches. k None: q only."""
    if _gpu(q):
        e = _none(q)
        has = k is not None
        _seq().qk_fullnorm_rope_store(q, k if has else e, v if has else e, wq,
                                      wk if has else _none(q, torch.float32), eps, positions, inv_freq,
                                      k_cache if has else e, v_cache if has else e,
                                      slot_mapping if has else _none(q, torch.long))
        return
    torch_ref.qk_fullnorm_rope_store(q, k, v, wq, wk, eps, positions, inv_freq, k_cache, v_cache, slot_mapping)


def pool_kv_update(k_cache, v_cache, pool_k, pool_v, block_tables, token_seg, positions, run: int,
                   row_map=None) -> None:
    """Means of the cached keys / values of every aligned run of ``run``
    positions that one of this step's rows completes, into the fp32 pooled
    caches. ``row_map`` (int32): the rows to look at, when the caller knows
    which rows end a run; None = every row."""
    if _gpu(k_cache):
        _seq().pool_kv_update(k_cache, v_cache, pool_k, pool_v, block_tables, token_seg, positions, int(run),
                              row_map if row_map is not None else _none(k_cache, torch.int32))
        return
    torch_ref.pool_kv_update(k_cache, v_cache, pool_k, pool_v, block_tables, token_seg, positions, run, row_map)


def attn_window_pool_paged(q, k_cache, v_cache, pool_k, pool_v, block_tables, token_seg, positions, scale,
                           softcap, mask_size, run, key_splits: int = 0):
    """Sliding-window attention over the paged cache with the pooled entries
    of the runs that lie wholly before the window, soft-capped scores; prompt
    portions, decoded tokens and mixes alike. ``key_splits`` (GPU): workgroups
    that share one (row, head)'s keys, merged by a second kernel; 0 = as many
    as fill the chip for this step (few rows, long windows), 1 = none."""
    if _gpu(q):
        out = torch.empty((q.shape[0], q.shape[1], v_cache.shape[3]), dtype=q.dtype, device=q.device)
        f = _none(q, torch.float32)
        has = run > 0
        # steps of few rows: a (row, head)'s key tiles are shared out over several workgroups.
        # An upper bound of the visible keys, from the mask or the block table's width
        T, H = q.shape[0], q.shape[1]
        ctx = block_tables.shape[1] * k_cache.shape[2]
        reach = min(ctx, mask_size + (ctx // run if has else 0)) if mask_size > 0 else ctx
        tiles = (reach + 63) // 64
        ns = key_splits or max(1, min((tiles + 3) // 4, 512 // max(1, T * H), 64))
        part_o = torch.empty((T, H, ns, v_cache.shape[3]), dtype=torch.float32, device=q.device) if ns > 1 else f
        part_ml = torch.empty((T, H, ns, 2), dtype=torch.float32, device=q.device) if ns > 1 else f
        _seq().attn_masked_paged(out, q, k_cache, v_cache, block_tables, token_seg, positions, _none(q),
                                 scale, 2, int(mask_size), 0, False, _none(q, torch.int32),
                                 pool_k if has else f, pool_v if has else f, int(run), float(softcap),
                                 part_o, part_ml)
        return out
    return torch_ref.attn_window_pool_paged(q, k_cache, v_cache, pool_k, pool_v, block_tables, token_seg,
                                            positions, scale, softcap, mask_size, run)


def ssd_recurrence(x, B, C, dt, dt_bias, a_log, skip, state, state_slots, cu_seqlens, seg_start):
    """S <- exp(-exp(a_log) d) S + d B x^T, o = S^T C + skip x with
    d = softplus(dt + dt_bias) per head and token; o [T, H, V] fp32."""
    if _gpu(x):
        o = torch.empty((x.shape[0], x.shape[1], x.shape[2]), dtype=torch.float32, device=x.device)
        _seq().ssd_recurrence(o, x, B, C, dt, dt_bias, a_log, skip, state, state_slots, cu_seqlens, seg_start)
        return o
    return torch_ref.ssd_recurrence(x, B, C, dt, dt_bias, a_log, skip, state, state_slots, cu_seqlens, seg_start)


def gate_group_rmsnorm(o, weight, gate, eps, out_dtype):
    """(o * silu(gate)) RMS-normed in groups, times weight: o [T, groups, S] fp32."""
    if _gpu(o):
        out = torch.empty((o.shape[0], o.shape[1] * o.shape[2]), dtype=out_dtype, device=o.device)
        _seq().gated_rmsnorm(out, o, weight, gate, eps, True)
        return out
    return torch_ref.gate_group_rmsnorm(o, weight, gate, eps, out_dtype)
