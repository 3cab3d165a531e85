"""HIP kernels of the Pironex family (kllms_amd._C_seq) against the plain
PyTorch reference of the same op (ops/torch_ref.py), in fp32 and bf16, on
sizes that are and are not multiples of the vector width, with segments that
start a sequence, continue one, and are shorter than the convolutions."""

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


def i32(x):
    return torch.tensor(x, dtype=torch.int32, device=DEV)


def segments(lengths, starts, slots):
    cu = [0]
    tseg = []
    for b, n in enumerate(lengths):
        cu.append(cu[-1] + n)
        tseg += [b] * n
    return i32(slots), i32(cu), i32(starts), i32(tseg)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [36, 256, 1000, 2048])
def test_post_norm_residual_depth_average_and_stats(dtype, W):
    T, L = 7, 4
    x = rnd(T, W, std=3.0) + 1.5
    a = rnd(T, W, dtype=dtype, seed=1) + 0.7
    wp = rnd(W, seed=3) * 0.1 + 1
    # statistics only
    s1 = ops.ln_residual_mix(x, None, None, 1e-6, x)
    s2 = torch_ref.ln_residual_mix(x.clone(), None, None, 1e-6, x.clone())
    close(s1, s2, torch.float32)
    # post-norm + add, in place and into another buffer
    for inplace in (True, False):
        xa, xb = x.clone(), x.clone()
        oa = xa if inplace else torch.empty_like(xa)
        ob = xb if inplace else torch.empty_like(xb)
        s1 = ops.ln_residual_mix(xa, a, wp, 1e-6, oa)
        s2 = torch_ref.ln_residual_mix(xb, a, wp, 1e-6, ob)
        close(oa, ob, torch.float32)
        close(s1, s2, torch.float32)
    # with the depth average: stream n takes the sum, the output their weighted sum
    for n_prev in (0, 1, L - 1):
        st1 = rnd(L, T, W, seed=5)
        st2 = st1.clone()
        dwa = rnd(n_prev + 1, seed=6)
        oa, ob = torch.empty_like(x), torch.empty_like(x)
        s1 = ops.ln_residual_mix(x, a, wp, 1e-6, oa, st1, n_prev, dwa)
        s2 = torch_ref.ln_residual_mix(x, a, wp, 1e-6, ob, st2, n_prev, dwa)
        close(st1, st2, torch.float32)
        close(oa, ob, torch.float32, scale=4)
        close(s1, s2, torch.float32, scale=4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W,K", [(40, 3), (37, 4), (256, 3), (512, 2), (64, 1), (24, 6)])
def test_norm_with_input_convolution(dtype, W, K):
    lengths, starts, slots = [5, 1, 2, 9, 1], [0, 7, 3, 0, 0], [2, 0, 4, 1, 3]
    sl, cu, st, tseg = segments(lengths, starts, slots)
    T = sum(lengths)
    x = rnd(T, W, std=2.0) + 0.3
    stats = torch_ref.ln_residual_mix(x.clone(), None, None, 1e-6, x.clone())
    w = rnd(W, seed=1) * 0.1 + 1
    cw = rnd(K, W, seed=2, std=0.5)
    state = rnd(6, 2, K - 1, W, seed=3)
    for which in (0, 1):
        h1, h2 = state.clone(), state.clone()
        y1 = ops.ln_canon(x, stats, w, cw, h1[:, which], sl, cu, st, tseg, dtype)
        y2 = torch_ref.ln_canon(x, stats, w, cw, h2[:, which], sl, cu, st, dtype)
        assert y1.dtype == dtype
        close(y1, y2, dtype)
        close(h1, h2, torch.float32)
        assert torch.equal(h1[:, 1 - which], state[:, 1 - which])
        assert torch.equal(h1[5], state[5])
    # the norm alone
    close(ops.ln_canon(x, stats, w, None, None, sl, cu, st, tseg, dtype),
          torch_ref.ln_canon(x, stats, w, None, None, sl, cu, st, dtype), dtype)


def paged(T_total, G, D, Dv, BS, dtype, n_seq, seed=0):
    """Caches of n_seq sequences of T_total tokens on shuffled pages."""
    per = (T_total + BS - 1) // BS
    NB = per * n_seq + 3
    perm = torch.randperm(NB, generator=torch.Generator().manual_seed(seed))[:per * n_seq]
    bt = perm.view(n_seq, per).to(torch.int32).to(DEV)
    kc = rnd(NB, G, BS, D, dtype=dtype, seed=seed + 1)
    vc = rnd(NB, G, BS, Dv, dtype=dtype, seed=seed + 2)
    return bt, kc, vc


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv,R", [(6, 3, 64, 48, 8), (4, 2, 16, 24, 4), (3, 1, 10, 7, 5), (2, 2, 8, 8, 0),
                                        (8, 2, 128, 128, 64)])
def test_whole_projection_norm_rotation_store(dtype, H, G, D, Dv, R):
    T, BS, NB = 11, 8, 9
    tot = H * D + G * D + G * Dv + 8
    y = rnd(T, tot, dtype=dtype)
    q0 = y[:, :H * D].unflatten(1, (H, D))
    k = y[:, H * D:H * D + G * D].unflatten(1, (G, D))
    v = y[:, H * D + G * D:H * D + G * D + G * Dv].unflatten(1, (G, Dv))
    wq, wk = rnd(H * D, seed=1) * 0.2 + 1, rnd(G * D, seed=2) * 0.2 + 1
    pos = torch.randint(0, 3000, (T,), device=DEV)
    inv = (100.0 ** (-torch.arange(R, dtype=torch.float64) / max(R, 1))).float().to(DEV)
    slots = torch.randperm(NB * BS)[:T].to(DEV)
    for own in (True, False):
        ya, yb = y.clone(), y.clone()
        qa = ya[:, :H * D].unflatten(1, (H, D))
        qb = yb[:, :H * D].unflatten(1, (H, D))
        kc1, vc1 = rnd(NB, G, BS, D, dtype=dtype, seed=3), rnd(NB, G, BS, Dv, dtype=dtype, seed=4)
        kc2, vc2 = kc1.clone(), vc1.clone()
        if own:
            ops.qk_fullnorm_rope_store(qa, k, v, wq, wk, 1e-6, pos, inv, kc1, vc1, slots)
            torch_ref.qk_fullnorm_rope_store(qb, k, v, wq, wk, 1e-6, pos, inv, kc2, vc2, slots)
        else:
            ops.qk_fullnorm_rope_store(qa, None, None, wq, None, 1e-6, pos, inv, None, None, None)
            torch_ref.qk_fullnorm_rope_store(qb, None, None, wq, None, 1e-6, pos, inv, None, None, None)
        close(qa, qb, dtype)
        close(kc1, kc2, dtype)
        assert torch.equal(vc1, vc2)
        assert torch.equal(ya[:, H * D:], y[:, H * D:])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("G,D,Dv,BS,run", [(3, 64, 48, 16, 12), (2, 16, 24, 8, 3), (1, 10, 7, 4, 9), (2, 8, 8, 16, 16),
                                           (2, 32, 32, 16, 40)])
def test_pooled_runs_update_and_attention(dtype, G, D, Dv, BS, run):
    n_seq, ctx = 3, 150
    H = 2 * G
    bt, kc, vc = paged(ctx, G, D, Dv, BS, dtype, n_seq, seed=run)
    PB = (BS + run - 1) // run
    NB = kc.shape[0]
    pk1 = torch.full((NB, G, PB, D), 7.0, device=DEV)
    pv1 = torch.full((NB, G, PB, Dv), -7.0, device=DEV)
    pk2, pv2 = pk1.clone(), pv1.clone()
    # a step that covers every position of every sequence: all runs are completed
    pos = torch.arange(ctx, device=DEV).repeat(n_seq)
    tseg = torch.arange(n_seq, device=DEV).repeat_interleave(ctx).int()
    ops.pool_kv_update(kc, vc, pk1, pv1, bt, tseg, pos, run)
    torch_ref.pool_kv_update(kc, vc, pk2, pv2, bt, tseg, pos, run)
    close(pk1, pk2, torch.float32, scale=8)
    close(pv1, pv2, torch.float32, scale=8)
    # the same through a list of the rows that end a run (in any order), and an untouched cache for other rows
    ends = [t for t in range(n_seq * ctx) if (t % ctx + 1) % run == 0]
    pk3, pv3 = torch.full_like(pk1, 7.0), torch.full_like(pv1, -7.0)
    ops.pool_kv_update(kc, vc, pk3, pv3, bt, tseg, pos, run, i32(ends[::-1]))
    assert torch.equal(pk3, pk1) and torch.equal(pv3, pv1)
    pk3.fill_(7.0)
    ops.pool_kv_update(kc, vc, pk3, pv3, bt, tseg, pos, run, i32([run - 1, run]))     # one row ends a run, one does not
    assert int((pk3 != 7.0).sum()) == G * D
    # attention rows: a portion in the middle, single rows, the first rows, edges of window and runs
    for size, cap in [(37, 0.0), (run, 5.0), (1, 0.0), (200, 3.0)]:
        rows = [(0, 0), (0, 1), (1, size - 1), (1, size), (2, size + run - 2), (2, size + run - 1), (2, size + run),
                (0, 149), (1, 100), (1, 101), (1, 102), (2, 3 * run + size - 1), (2, 3 * run + size)]
        rows = [(s, p) for s, p in rows if 0 <= p < ctx]
        ts = i32([s for s, _ in rows])
        ps = torch.tensor([p for _, p in rows], device=DEV)
        q = rnd(len(rows), H, D, dtype=dtype, seed=size, std=1.5)
        o2 = torch_ref.attn_window_pool_paged(q, kc, vc, pk2, pv2, bt, ts, ps, 0.3, cap, size, run)
        # one workgroup per (row, head), and the keys shared out over 2 and 5 (more shares than key tiles)
        for splits in (1, 0, 2, 5):
            o1 = ops.attn_window_pool_paged(q, kc, vc, pk1, pv1, bt, ts, ps, 0.3, cap, size, run, key_splits=splits)
            close(o1, o2, dtype)
        # without pooling the far tokens are simply gone
        o3 = ops.attn_window_pool_paged(q, kc, vc, None, None, bt, ts, ps, 0.3, cap, size, 0)
        o4 = torch_ref.attn_window_pool_paged(q, kc, vc, None, None, bt, ts, ps, 0.3, cap, size, 0)
        close(o3, o4, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,Dv", [(8, 2, 128, 128), (16, 2, 64, 32), (4, 2, 32, 64), (8, 8, 16, 16), (6, 2, 64, 64),
                                      (8, 1, 32, 256)])
def test_window_attention_with_grouped_queries(dtype, H, G, D, Dv):
    """1, 2, 3, 4 and 8 query heads per key/value head, key and value sizes
    from 16 to 256, with and without key shares."""
    BS, run, size, ctx, n_seq = 16, 5, 70, 300, 2
    bt, kc, vc = paged(ctx, G, D, Dv, BS, dtype, n_seq, seed=H)
    NB, PB = kc.shape[0], (BS + run - 1) // run
    pk, pv = torch.zeros(NB, G, PB, D, device=DEV), torch.zeros(NB, G, PB, Dv, device=DEV)
    pos = torch.arange(ctx, device=DEV).repeat(n_seq)
    tseg = torch.arange(n_seq, device=DEV).repeat_interleave(ctx).int()
    torch_ref.pool_kv_update(kc, vc, pk, pv, bt, tseg, pos, run)
    rows = [(0, 0), (1, 3), (0, 69), (0, 70), (1, 74), (1, 75), (0, 299), (1, 200), (1, 201), (1, 202), (0, 150)]
    ts = i32([s_ for s_, _ in rows])
    ps = torch.tensor([p_ for _, p_ in rows], device=DEV)
    q = rnd(len(rows), H, D, dtype=dtype, seed=3, std=1.2)
    want = torch_ref.attn_window_pool_paged(q, kc, vc, pk, pv, bt, ts, ps, 0.25, 8.0, size, run)
    for splits in (1, 0, 3):
        close(ops.attn_window_pool_paged(q, kc, vc, pk, pv, bt, ts, ps, 0.25, 8.0, size, run, key_splits=splits),
              want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("C,K,stride", [(40, 4, 48), (37, 3, 37), (480, 4, 488), (16, 1, 16)])
def test_causal_conv_with_bias(dtype, C, K, stride):
    lengths, starts, slots = [6, 1, 2, 1], [0, 5, 9, 0], [1, 3, 0, 2]
    sl, cu, st, tseg = segments(lengths, starts, slots)
    T = sum(lengths)
    x = rnd(T, stride, dtype=dtype)[:, :C]
    w = rnd(K, C, seed=1, std=0.5)
    bias = rnd(C, seed=2, std=0.5)
    s1 = rnd(4, K - 1, C, dtype=dtype, seed=3)
    s2 = s1.clone()
    y1 = ops.causal_conv_silu(x, w, s1, sl, cu, st, tseg, bias)
    y2 = torch_ref.causal_conv_silu(x, w, s2, sl, cu, st, bias)
    close(y1, y2, dtype)
    close(s1, s2, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,N,V", [(6, 2, 48, 48), (4, 4, 16, 24), (3, 1, 10, 7), (8, 2, 128, 64)])
def test_state_space_recurrence(dtype, H, G, N, V):
    lengths, starts, slots = [9, 1, 2, 1, 30], [0, 4, 7, 0, 0], [2, 0, 3, 1, 4]
    sl, cu, st, _ = segments(lengths, starts, slots)
    T = sum(lengths)
    tot = H * V + 2 * G * N + 8
    buf = rnd(T, tot, dtype=dtype, std=0.7)
    x = buf[:, :H * V].unflatten(1, (H, V))
    B = buf[:, H * V:H * V + G * N].unflatten(1, (G, N))
    C = buf[:, H * V + G * N:H * V + 2 * G * N].unflatten(1, (G, N))
    dt = rnd(T, H + 3, dtype=dtype, seed=1)[:, :H]
    dt_bias, a_log, skip = rnd(H, seed=2, std=0.5), rnd(H, seed=3) - 1.0, rnd(H, seed=4)
    s1 = rnd(5, H, N, V, seed=5)
    s2 = s1.clone()
    o1 = ops.ssd_recurrence(x, B, C, dt, dt_bias, a_log, skip, s1, sl, cu, st)
    o2 = torch_ref.ssd_recurrence(x, B, C, dt, dt_bias, a_log, skip, s2, sl, cu, st)
    close(o1, o2, torch.float32, scale=20)
    close(s1, s2, torch.float32, scale=20)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("groups,S", [(2, 144), (1, 50), (3, 7), (8, 512)])
def test_gate_before_group_norm(dtype, groups, S):
    T = 6
    o = rnd(T, groups, S, std=2.0)
    gate = rnd(T, groups * S + 8, dtype=dtype, seed=1)[:, :groups * S]
    w = rnd(groups * S, seed=2) * 0.2 + 1
    close(ops.gate_group_rmsnorm(o, w, gate, 1e-6, dtype), torch_ref.gate_group_rmsnorm(o, w, gate, 1e-6, dtype), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_into_a_given_buffer(dtype):
    V, W, T = 50, 72, 9
    table = rnd(V, W, dtype=dtype)
    ids = torch.randint(0, V, (T,), device=DEV)
    sl, cu, st, tseg = segments([T], [0], [0])
    streams = torch.zeros(3, T, W, device=DEV)
    ops.embed_bigram(ids, table, None, 0.5, 0, 0, 0, None, sl, cu, st, tseg, out=streams[0])
    close(streams[0], table[ids].float() * 0.5, torch.float32)
    assert float(streams[1:].abs().max()) == 0.0
