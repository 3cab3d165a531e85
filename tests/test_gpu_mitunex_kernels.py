"""HIP kernels of the Mitunex family (kllms_amd._C_seq) against the plain
PyTorch reference of the same op (ops/torch_ref.py), in fp32 and bf16, on
sizes that are not multiples of the wave, vector or matrix-tile sizes."""

import pytest
import torch

from kllms_amd import ops
from kllms_amd.ops import torch_ref

pytestmark = pytest.mark.gpu

DEV = "cuda"
DTYPES = [torch.float32, torch.bfloat16]


def close(a, b, dtype, scale=1.0):
    rt, at = (2e-5, 2e-5) if dtype == torch.float32 else (2e-2, 2e-2)
    torch.testing.assert_close(a.float(), b.float(), rtol=rt * scale, atol=at * scale)


def rnd(*shape, dtype=torch.float32, std=1.0, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * std).to(DEV).to(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [72, 256, 1000])
def test_embed_with_position_rows(dtype, W):
    V, P, T = 50, 37, 9
    table, pos = rnd(V, W, dtype=dtype), rnd(P, W, dtype=dtype, seed=1, std=0.3)
    w = rnd(W, seed=2) * 0.1 + 1
    ids = torch.randint(0, V, (T,), device=DEV)
    positions = torch.randint(0, P, (T,), device=DEV)
    close(ops.embed_rmsnorm(ids, table, w, 1e-6, pos, positions),
          torch_ref.embed_rmsnorm(ids, table, w, 1e-6, pos, positions), torch.float32)
    close(ops.embed_rmsnorm(ids, table, w, 1e-6), torch_ref.embed_rmsnorm(ids, table, w, 1e-6), torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [36, 320, 2048])
def test_post_norm_residual_with_stream_cast(dtype, W):
    T = 5
    x = rnd(T, W, std=3.0)
    a = rnd(T, W, dtype=dtype, seed=1)
    wp, wn = rnd(W, seed=3) * 0.1 + 1, rnd(W, seed=4) * 0.1 + 1
    for w_next, cast in [(None, True), (None, False), (wn, False)]:
        x1, x2 = x.clone(), x.clone()
        h1 = ops.sandwich_residual(x1, a, wp, 1e-6, w_next=w_next, out_dtype=dtype, cast=cast)
        h2 = torch_ref.sandwich_residual(x2, a, wp, 1e-6, w_next=w_next, out_dtype=dtype, cast=cast)
        close(x1, x2, torch.float32)
        assert (h1 is None) == (h2 is None)
        if h1 is not None:
            assert h1.dtype == dtype
            close(h1, h2, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cols,stride", [(40, 40), (37, 48), (1024, 2056)])
def test_gelu_tanh(dtype, cols, stride):
    buf = rnd(6, stride, dtype=dtype, std=2.0)
    x = buf[:, :cols]
    close(ops.gelu_tanh(x), torch_ref.gelu_tanh(x), dtype)


def test_scale_softcap():
    z = rnd(5, 77, std=20.0)
    for scale, cap in [(2.0, 15.0), (0.5, 0.0)]:
        a, b = z.clone(), z.clone()
        ops.scale_softcap_(a, scale, cap)
        torch_ref.scale_softcap_(b, scale, cap)
        close(a, b, torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [44, 512])
def test_scale_rows(dtype, W):
    h = rnd(7, W, dtype=dtype)
    src = torch.tensor([3, 3, 0, 6, 1], dtype=torch.int32, device=DEV)
    sc = torch.tensor([0.5, 0.0, 1.0, 0.9, 0.123], device=DEV)
    close(ops.scale_rows(h, src, sc), torch_ref.scale_rows(h, src, sc), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_spread_rows_for_the_all_experts_form(dtype):
    T, W, E, top = 9, 52, 5, 2
    h = rnd(T, W, dtype=dtype)
    idx = torch.stack([torch.randperm(E, generator=torch.Generator().manual_seed(i))[:top] for i in range(T)])
    idx = idx.to(torch.int32).to(DEV)
    w = torch.rand(T, top, device=DEV) + 0.05
    close(ops.moe_spread_rows(h, idx, w, E), torch_ref.moe_spread_rows(h, idx, w, E), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("score,renorm,corr", [("sigmoid", False, False), ("sigmoid", True, True),
                                               ("softmax", True, True), ("softmax", False, False)])
def test_router_variants(dtype, score, renorm, corr):
    T, W, N, top = 11, 72, 12, 3
    h = rnd(T, W, dtype=dtype)
    router = rnd(N, W, seed=1) * 0.3
    c = rnd(N, seed=2) * 0.01 if corr else None
    idx, w, rowidx = ops.moe_route_rows(h, router, c, top, 1, 1, N, True, score, renorm)
    z = torch.nn.functional.linear(h.float(), router)
    ridx, rw = torch_ref.moe_route(z, c, top, 1, 1, score, renorm)
    assert torch.equal(idx, ridx)
    close(w, rw, torch.float32, scale=10)
    assert torch.equal(rowidx, ridx * T + torch.arange(T, device=DEV, dtype=torch.int32)[:, None])
    idx2, w2 = ops.moe_route(z, c, top, 1, 1, score, renorm)
    assert torch.equal(idx2, ridx)
    close(w2, rw, torch.float32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [88, 52, 2048])
def test_combine_unweighted_with_gated_extra(dtype, W):
    T, top, R = 6, 2, 9
    rows, h, extra = rnd(R, W, dtype=dtype), rnd(T, W, dtype=dtype, seed=1), rnd(T, W, dtype=dtype, seed=2)
    rowidx = torch.randint(0, R, (T, top), device=DEV, dtype=torch.int32)
    w = torch.rand(T, top, device=DEV)
    gate = rnd(T, 8, dtype=dtype, seed=3)[:, 0]                  # strided [T] view
    for ww, ex, g in [(None, extra, gate), (w, extra, gate), (None, None, None), (w, None, None)]:
        close(ops.moe_combine(rows, h, rowidx, ww, dtype, ex, g),
              torch_ref.moe_combine(rows, h, rowidx, ww, dtype, ex, g), dtype)


def _latent_case(dtype, H, D, R, C, BS, lens, starts, seed=0):
    """Random packed step: segments of `lens` rows continuing sequences that
    already hold `starts` tokens; their caches are filled with random rows."""
    L = C + R
    NB = sum((s + n + BS - 1) // BS for s, n in zip(starts, lens)) + 2
    cache = rnd(NB, 1, BS, L, dtype=dtype, seed=seed)
    perm = torch.randperm(NB, generator=torch.Generator().manual_seed(seed)).tolist()
    width = max((s + n + BS - 1) // BS for s, n in zip(starts, lens))
    bt = torch.zeros(len(lens), width, dtype=torch.int32)
    pos, tseg, slots = [], [], []
    k = 0
    for b, (s, n) in enumerate(zip(starts, lens)):
        nb = (s + n + BS - 1) // BS
        blocks = perm[k:k + nb]
        k += nb
        bt[b, :nb] = torch.tensor(blocks, dtype=torch.int32)
        for p in range(s, s + n):
            pos.append(p)
            tseg.append(b)
            slots.append(blocks[p // BS] * BS + p % BS)
    T = len(pos)
    dev = lambda x, dt: torch.tensor(x, dtype=dt, device=DEV)
    return dict(cache=cache, bt=bt.to(DEV), pos=dev(pos, torch.long), tseg=dev(tseg, torch.int32),
                slots=dev(slots, torch.long), T=T,
                q=rnd(T, H * (D + R) + 8, dtype=dtype, seed=seed + 1)[:, :H * (D + R)].unflatten(1, (H, D + R)),
                q_abs=rnd(H, T, C, dtype=dtype, seed=seed + 2).transpose(0, 1),
                gate=rnd(T, H, dtype=dtype, seed=seed + 3))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,R,C", [(4, 16, 8, 32), (3, 20, 6, 44), (16, 128, 64, 512), (5, 8, 2, 24)])
def test_latent_kv_store(dtype, H, D, R, C):
    c = _latent_case(dtype, H, D, R, C, 16, [5, 1, 9], [0, 37, 14])
    dkv = rnd(c["T"], C + R + 8, dtype=dtype, seed=5)[:, :C + R]
    w = rnd(C, seed=6) * 0.1 + 1
    inv = (10000.0 ** (-torch.arange(R // 2, dtype=torch.float64) * 2 / R)).float().to(DEV)
    q1, q2 = c["q"].clone(), c["q"].clone()
    k1, k2 = c["cache"].clone(), c["cache"].clone()
    ops.latent_kv_store(q1, dkv, w, 1e-6, c["pos"], inv, k1, c["slots"], D)
    torch_ref.latent_kv_store(q2, dkv, w, 1e-6, c["pos"], inv, k2, c["slots"], D)
    close(q1, q2, dtype)
    close(k1, k2, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,D,R,C", [(4, 16, 8, 32), (3, 20, 6, 44), (16, 32, 64, 512), (6, 8, 2, 24),
                                     (40, 8, 8, 16), (1, 8, 4, 96)])
@pytest.mark.parametrize("mask", [0, 7, 37])
def test_latent_attention_kernels(dtype, H, D, R, C, mask):
    """Prompt portions that start anywhere, single decoded rows and a mix of
    both in one launch; the matrix-unit kernel (bf16) with both row tilings
    and the plain kernel against the reference."""
    c = _latent_case(dtype, H, D, R, C, 16, [33, 1, 2, 1, 70], [0, 52, 15, 0, 45], seed=H + C)
    ref = torch_ref.attn_latent_paged(c["q_abs"], c["q"], c["cache"], c["bt"], c["tseg"], c["pos"], 0.17, mask,
                                      c["gate"], D)
    for kw in [dict(use_mfma=False), dict(tile_rows=0), dict(tile_rows=1, key_splits=-1), dict(tile_rows=1),
               dict(tile_rows=1, key_splits=3), dict(tile_rows=1, key_splits=50)]:
        out = ops.attn_latent_paged(c["q_abs"], c["q"], c["cache"], c["bt"], c["tseg"], c["pos"], 0.17, mask,
                                    c["gate"], D, **kw)
        close(out, ref, dtype)
    out = ops.attn_latent_paged(c["q_abs"], c["q"], c["cache"], c["bt"], c["tseg"], c["pos"], 0.17, mask, None, D)
    ref = torch_ref.attn_latent_paged(c["q_abs"], c["q"], c["cache"], c["bt"], c["tseg"], c["pos"], 0.17, mask,
                                      None, D)
    close(out, ref, dtype)


def test_latent_attention_keeps_small_weights():
    """One key dominates, the others carry weights around 1e-3 with large
    values: the output shows whether the small weights keep their precision
    on the way into the matrix unit."""
    H, D, R, C = 4, 16, 8, 64
    c = _latent_case(torch.bfloat16, H, D, R, C, 16, [1], [99], seed=3)
    c["cache"][..., :C] = torch.where(torch.rand_like(c["cache"][..., :C].float()) < 0.5, 1.0, 1.0078125).to(torch.bfloat16)
    out = ops.attn_latent_paged(c["q_abs"], c["q"], c["cache"], c["bt"], c["tseg"], c["pos"], 0.3, 0, None, D)
    ref = torch_ref.attn_latent_paged(c["q_abs"].float(), c["q"].float(), c["cache"].float(), c["bt"], c["tseg"],
                                      c["pos"], 0.3, 0, None, D)
    # values lie in [1, 1.0078]: a weight vector that sums to 1 within 1e-4 keeps the output there too
    torch.testing.assert_close(out.float(), ref, rtol=0, atol=4e-3)
    assert float(out.float().min()) >= 1.0 - 1e-6 and float(out.float().max()) <= 1.0078125 + 1e-6
