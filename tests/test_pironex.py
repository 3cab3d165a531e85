"""Pironex family on the CPU path (fp32) against the plain float64 oracle in
tests/pironex_oracle.py: every mechanism alone, then whole models through the
engine's segment step, page and slot reuse, and greedy generation through
generate() and the scheduler. Configurations are small and lopsided: head
counts that are not powers of two, value sizes that differ from key sizes,
windows and pooled runs that do not divide the page size, runs longer than a
page and longer than the window, one and several taps, layers without a
feed-forward, an attention layer that reads another layer's cache with a mask
of its own."""

import json
import os

import pytest
import torch

import pironex_oracle as O
from kllms_amd import ops
from kllms_amd.engine.config import EngineConfig, PironexArchConfig
from kllms_amd.engine.engine import GenRequest, LLMEngine
from kllms_amd.engine.kvcache import HybridStateCache
from kllms_amd.engine.sampling import SamplingParams
from kllms_amd.engine.scheduler import BatchScheduler
from kllms_amd.models.llama import ForwardBatch
from kllms_amd.models.mixers import LatentAttention, Mamba2Mixer, PoolWindowAttention, RoutedExperts

EPS = 1e-6


def att(heads=4, kv_heads=2, dim=10, vdim=7, size=9, pool=3, scale=0.4, softcap=6.0, rot=6, base=50.0, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if softcap:
        m["softcap"] = softcap
    if size:
        m["mask"] = {"size": size}
        if pool:
            m["mask"]["pool"] = pool
    if rot:
        m["rot"] = {"base": base, "dims": rot}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def mam(heads=4, vdim=6, state=5, groups=2, conv=4, norm_groups=2):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def lat(heads=3, dim=10, rot_dim=6, vdim=7, kv_rank=12, size=9, scale=0.3, base=100.0):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim}}
    if size:
        m["mask"] = {"size": size}
    return m


MLPS = {
    None: None,
    "moe": {"kind": "moe", "expert": {"ff": 12, "limit": 1.0}, "router": {"experts": 5, "top": 3},
            "shared": {"ff": 20, "limit": 0.6}},
    "moe_top1": {"kind": "moe", "expert": {"ff": 16, "limit": 0.8}, "router": {"experts": 7, "top": 1},
                 "shared": {"ff": 8, "limit": 2.0}},
    "moe_bare": {"kind": "moe", "expert": {"ff": 8, "limit": 1.5}, "router": {"experts": 3, "top": 3}},
}


def layer(kind, mixer, mlp="moe"):
    return {"type": kind, "mixer": mixer, "mlp": MLPS[mlp]}


def _cfg_a():
    layers = [layer("mamba2", mam()),
              layer("latent_attention", lat(), "moe_top1"),
              layer("attention", att()),
              layer("attention", att(size=5, pool=4, scale=0.7, softcap=0.0, kv_from=2), None),
              layer("mamba2", mam(heads=3, vdim=8, state=7, groups=1, conv=2, norm_groups=3), None),
              layer("attention", att(size=13, pool=0, scale=0.5, kv_from=2), "moe_bare")]
    return {"architecture": "Pironex", "vocab": 61, "width": 24, "norm": {"eps": EPS}, "embedding": {"scale": 0.5},
            "canon": {"taps": 3}, "layers": layers}


def _cfg_b():
    # attention first and read at once by the next layer; ungrouped heads; a run longer than the page and the
    # window; the whole head rotated; no soft cap; one tap; top 1; no shared expert; one norm group; no window
    layers = [layer("attention", att(heads=3, kv_heads=3, dim=4, vdim=5, size=6, pool=11, scale=0.9, softcap=0.0, rot=4),
                    "moe_top1"),
              layer("attention", att(heads=3, kv_heads=3, dim=4, vdim=5, size=3, pool=2, scale=0.6, rot=4, kv_from=0),
                    "moe_bare"),
              layer("latent_attention", lat(heads=1, dim=6, rot_dim=2, vdim=5, kv_rank=7, size=0, scale=0.7), None),
              layer("mamba2", mam(heads=2, vdim=9, state=3, groups=2, conv=1, norm_groups=1), "moe_bare"),
              layer("attention", att(heads=2, kv_heads=1, dim=6, vdim=3, size=0, pool=0, scale=0.5, rot=0), None)]
    return {"architecture": "Pironex", "vocab": 47, "width": 20, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
            "canon": {"taps": 1}, "layers": layers}


CFG_A, CFG_B = _cfg_a(), _cfg_b()


def write_model(tmp, cfg, seed=0):
    from safetensors.torch import save_file

    w = O.random_weights(cfg, seed)
    os.makedirs(tmp, exist_ok=True)
    save_file({k: v.bfloat16().contiguous() for k, v in w.items()}, os.path.join(tmp, "model.safetensors"))
    with open(os.path.join(tmp, "config.json"), "w") as f:
        json.dump(cfg, f)
    return w


def make_engine(path, blocks=64, slots=4, **kw):
    return LLMEngine(EngineConfig(model=str(path), dtype="float32", device="cpu", max_kv_blocks=blocks,
                                  max_state_slots=slots, use_hip_graphs=False, **kw))


@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    d = tmp_path_factory.mktemp("pir_a")
    w = write_model(str(d), CFG_A, seed=1)
    return CFG_A, w, make_engine(d, blocks=96, kv_block_size=4)


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    d = tmp_path_factory.mktemp("pir_b")
    w = write_model(str(d), CFG_B, seed=2)
    return CFG_B, w, make_engine(d, blocks=24, slots=3, kv_block_size=8)


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def check(got, want, atol=2e-4):
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=atol)


def rows(L, W, seed):
    return torch.randn(L, W, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


# --- mechanisms alone -----------------------------------------------------------

def seg_batch(cache, seqs, counts):
    pos, tseg, cu, slots, starts = [], [], [0], [], []
    for b, (seq, n) in enumerate(zip(seqs, counts)):
        starts.append(seq.num_tokens)
        pos += list(range(seq.num_tokens, seq.num_tokens + n))
        slots += cache.extend(seq, n)
        tseg += [b] * n
        cu.append(cu[-1] + n)
    width = max(len(s.blocks) for s in seqs)
    bt = torch.zeros(len(seqs), width, dtype=torch.int32)
    for b, s in enumerate(seqs):
        bt[b, :len(s.blocks)] = torch.tensor(s.blocks, dtype=torch.int32)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32)
    return ForwardBatch(mode="segments", positions=torch.tensor(pos), slot_mapping=torch.tensor(slots),
                        kv_caches=cache.layer_caches(), cu_seqlens=i32(cu), block_tables=bt,
                        seg_start=i32(starts), state_slots=i32([s.state_slot for s in seqs]), token_seg=i32(tseg),
                        host_segs=[(s, n) for s, n in zip(starts, counts)])


def dirty_cache(specs, page):
    """A cache whose pages and slots hold whatever their last owner left, and
    whose first pages and slot are taken."""
    cache = HybridStateCache(specs, page, 200, 3, "cpu", torch.float32)
    for st in cache.layers:
        for t in st.block_tensors() + st.slot_tensors():
            t.normal_()
    cache.slots.alloc()
    for _ in range(3):
        cache.allocator.alloc()
    return cache


def run_mixers(mods, h, cuts, page=4):
    """Feed h [L, W] through mixers that share one cache (entry i = mods[i])
    in portions; returns one output per mixer."""
    cache = dirty_cache([m.cache_spec() for m in mods], page)
    seq = cache.open_sequence()
    outs, at = [[] for _ in mods], 0
    for n in cuts:
        batch = seg_batch(cache, [seq], [n])
        for i, m in enumerate(mods):
            outs[i].append(m(h[at:at + n].float(), batch, cache.layer_caches()[i]))
        at += n
    return [torch.cat(o) for o in outs]


def load_module(mod, w, pre):
    for name, dst in mod.checkpoint_map(pre).items():
        parts = dst if isinstance(dst, (list, tuple)) else [dst]
        r = 0
        for d in parts:
            d.copy_(w[name][r:r + d.shape[0]].to(d.dtype))
            r += d.shape[0]


def arch_of(layers, width=24, taps=3):
    return PironexArchConfig.from_checkpoint_config(
        {"vocab": 8, "width": width, "norm": {"eps": EPS}, "canon": {"taps": taps}, "layers": layers})


def one_cfg(layers, width=24):
    return {"vocab": 8, "width": width, "norm": {"eps": EPS}, "embedding": {"scale": 1.0}, "canon": {"taps": 3},
            "layers": layers}


def attention_modules(layers, w, width=24):
    arch = arch_of(layers, width)
    mods = []
    for i, sp in enumerate(arch.layers):
        mod = PoolWindowAttention(sp.attention, width, EPS, torch.float32)
        load_module(mod, w, f"l{i}.mix.")
        mods.append(mod)
    return mods


CUTS = [[60], [70], [25] + [1] * 35, [2, 5, 16, 1, 2, 17, 3, 14], [9, 2, 10, 1, 38], [2] * 30]


@pytest.mark.parametrize("cuts", CUTS)
@pytest.mark.parametrize("size,pool", [(9, 3), (5, 4), (7, 7), (4, 0), (0, 0), (6, 10), (1, 1)])
def test_attention_window_and_pooled_runs(cuts, size, pool):
    """Windows and pooled runs that do not fit the 4-token pages, with a scale
    that makes single keys dominate the softmax: a window, a run or a page
    border that is one position off shows at once. Portions cut windows, runs
    and pages anywhere; a run may be completed by a later step than it began in."""
    lay = layer("attention", att(size=size, pool=pool, scale=2.0, softcap=9.0), None)
    w = O.random_weights(one_cfg([lay]), 3)
    (mod,) = attention_modules([lay], w)
    h = rows(sum(cuts), 24, 4)
    m = lay["mixer"]
    want = O.attention_mixer(w, "l0.mix.", m, h, EPS, O.attention_keys(w, "l0.mix.", m, h, EPS))
    check(run_mixers([mod], h, cuts)[0], want)


@pytest.mark.parametrize("cuts", [[50], [3, 1, 1, 20, 2, 23], [2] * 25])
def test_attention_on_another_layers_cache(cuts):
    """The reading layer has its own queries, window and run length; its
    pooled entries are means over the owner's cached keys and values."""
    a = layer("attention", att(size=9, pool=3, scale=1.5), None)
    b = layer("attention", att(size=4, pool=5, scale=2.0, softcap=0.0, kv_from=0), None)
    w = O.random_weights(one_cfg([a, b]), 5)
    mods = attention_modules([a, b], w)
    assert mods[1].k_norm is None and "l1.mix.k" not in w
    h = rows(sum(cuts), 24, 6)
    h2 = rows(sum(cuts), 24, 7)
    kv = O.attention_keys(w, "l0.mix.", a["mixer"], h, EPS)
    # the reader is fed other rows than the owner: only the owner's rows reach the cache
    cache = dirty_cache([m.cache_spec() for m in mods], 4)
    assert cache.layers[1].k is cache.layers[0].k and cache.layers[1].pool_k is not cache.layers[0].pool_k
    seq = cache.open_sequence()
    got0, got1, at = [], [], 0
    for n in cuts:
        batch = seg_batch(cache, [seq], [n])
        got0.append(mods[0](h[at:at + n].float(), batch, cache.layers[0]))
        got1.append(mods[1](h2[at:at + n].float(), batch, cache.layers[1]))
        at += n
    check(torch.cat(got0), O.attention_mixer(w, "l0.mix.", a["mixer"], h, EPS, kv))
    check(torch.cat(got1), O.attention_mixer(w, "l1.mix.", b["mixer"], h2, EPS, kv))


def test_oracle_visibility_is_what_the_comparison_rests_on():
    """In the oracle a token just inside the window changes the output and one
    just outside does not — unless its run is already pooled; a run is seen
    from the step at which its last token leaves the window."""
    size, pool = 9, 4
    assert O.visible(20, size, pool) == (list(range(12, 21)), [0, 1, 2])      # run 2 = 8..11 ends at 11 = 20 - 9
    assert O.visible(19, size, pool) == (list(range(11, 20)), [0, 1])         # tokens 8..10 of run 2: not seen at all
    assert O.visible(18, size, pool)[1] == [0, 1] and O.visible(8, size, pool) == (list(range(9)), [])
    assert O.visible(12, size, pool) == (list(range(4, 13)), [0]) and O.visible(11, size, pool)[1] == []
    lay = layer("attention", att(size=size, pool=pool, scale=2.0), None)
    w = O.random_weights(one_cfg([lay]), 3)
    m = lay["mixer"]
    a = rows(30, 24, 5)
    run = lambda x: O.attention_mixer(w, "l0.mix.", m, x, EPS, O.attention_keys(w, "l0.mix.", m, x, EPS))
    base = run(a)
    for i, j, seen in [(20, 12, True), (20, 11, True), (19, 10, False), (19, 11, True), (19, 7, True),
                       (18, 9, False), (18, 8, False), (18, 3, True), (11, 2, False), (12, 2, True), (0, 0, True)]:
        b = a.clone()
        b[j] += 1.0
        moved = float((run(b)[i] - base[i]).abs().max())
        assert (moved > 1e-6) == seen, (i, j, moved)


def test_far_token_reaches_the_output_only_through_its_run():
    """150 positions on 16-token pages; the key projection equals the first
    head's query projection and one far token repeats the last token's input,
    so its key matches the last query: inside a pooled run it still stands
    out among the entries, and the product path agrees with the oracle there."""
    lay = layer("attention", att(heads=2, kv_heads=1, dim=8, vdim=6, size=20, pool=6, scale=1.0, softcap=0.0, rot=0),
                None)
    w = O.random_weights(one_cfg([lay]), 8)
    w["l0.mix.k"], w["l0.mix.k.norm"] = w["l0.mix.q"][:8].clone(), w["l0.mix.q.norm"][:8].clone()
    (mod,) = attention_modules([lay], w)
    h = rows(150, 24, 9) * 0.3
    h[31] = h[149] * 6.0
    m = lay["mixer"]
    want = O.attention_mixer(w, "l0.mix.", m, h, EPS, O.attention_keys(w, "l0.mix.", m, h, EPS))
    other = h.clone()
    other[31] = rows(1, 24, 10)[0] * 0.3
    moved = O.attention_mixer(w, "l0.mix.", m, other, EPS, O.attention_keys(w, "l0.mix.", m, other, EPS))
    assert float((want[149] - moved[149]).abs().max()) > 1e-3
    for cuts in ([150], [100] + [1] * 50, [33, 2, 115]):
        check(run_mixers([mod], h, cuts, page=16)[0], want)


def test_rotation_pairs_entries_half_a_block_apart():
    v = torch.arange(1.0, 9.0, dtype=torch.float64)
    out = O.rotate(v, 3, 10.0, 4, "half")
    import math
    a0, a1 = 3.0, 3.0 * 10.0 ** -0.5
    assert abs(float(out[0]) - (1 * math.cos(a0) - 3 * math.sin(a0))) < 1e-12
    assert abs(float(out[2]) - (3 * math.cos(a0) + 1 * math.sin(a0))) < 1e-12
    assert abs(float(out[1]) - (2 * math.cos(a1) - 4 * math.sin(a1))) < 1e-12
    assert torch.equal(out[4:], v[4:])
    inv = torch.tensor([1.0, 10.0 ** -0.5])
    q = v.float().view(1, 1, 8).clone()
    ops.qk_fullnorm_rope_store(q, None, None, torch.ones(8), None, 0.0, torch.tensor([3]), inv, None, None, None)
    check(q.view(8) * float(torch.sqrt((v * v).mean())), out, atol=1e-5)


@pytest.mark.parametrize("cuts", [[60], [25] + [1] * 35, [2, 5, 16, 1, 2, 17, 3, 14], [2] * 30, [1] * 60])
@pytest.mark.parametrize("conv,groups,norm_groups", [(4, 2, 2), (2, 1, 4), (5, 4, 1), (1, 2, 2)])
def test_mamba2(cuts, conv, groups, norm_groups):
    lay = layer("mamba2", mam(conv=conv, groups=groups, norm_groups=norm_groups), None)
    w = O.random_weights(one_cfg([lay]), 11)
    mod = Mamba2Mixer(arch_of([lay]).layers[0].mamba2, 24, EPS, torch.float32)
    load_module(mod, w, "l0.mix.")
    h = rows(sum(cuts), 24, 12)
    check(run_mixers([mod], h, cuts)[0], O.mamba2_mixer(w, "l0.mix.", lay["mixer"], h, EPS), atol=5e-4)


def test_mamba2_state_carries_a_far_token():
    """With a slow decay the first token still moves the output 120 steps on;
    the carried state must hold it through prompt portions and decoding."""
    lay = layer("mamba2", mam(), None)
    w = O.random_weights(one_cfg([lay]), 13)
    w["l0.mix.A_log"] = torch.full((4,), -7.0, dtype=torch.float64)
    mod = Mamba2Mixer(arch_of([lay]).layers[0].mamba2, 24, EPS, torch.float32)
    load_module(mod, w, "l0.mix.")
    h = rows(121, 24, 14)
    want = O.mamba2_mixer(w, "l0.mix.", lay["mixer"], h, EPS)
    other = h.clone()
    other[0] = rows(1, 24, 15)[0]
    assert float((O.mamba2_mixer(w, "l0.mix.", lay["mixer"], other, EPS)[120] - want[120]).abs().max()) > 1e-3
    for cuts in ([121], [1] * 121, [60, 2, 59]):
        check(run_mixers([mod], h, cuts)[0], want, atol=5e-4)


@pytest.mark.parametrize("cuts", [[40], [15] + [1] * 25, [2] * 20])
@pytest.mark.parametrize("size", [9, 4, 0])
def test_latent_attention_without_gate(cuts, size):
    lay = layer("latent_attention", lat(size=size, scale=2.0), None)
    w = O.random_weights(one_cfg([lay]), 16)
    mod = LatentAttention(arch_of([lay]).layers[0].latent, 24, EPS, torch.float32)
    assert "g" not in mod.inp.parts
    load_module(mod, w, "l0.mix.")
    h = rows(sum(cuts), 24, 17)
    check(run_mixers([mod], h, cuts)[0], O.latent_mixer(w, "l0.mix.", lay["mixer"], h, EPS))


@pytest.mark.parametrize("T", [1, 7, 90])
@pytest.mark.parametrize("mlp", ["moe", "moe_top1", "moe_bare"])
def test_clamped_experts(mlp, T):
    """Both expert forms (all experts on few rows, sorted rows on many); the
    input is large enough that both clamps of the routed and of the shared
    expert (which has a limit of its own) are at work."""
    lay = layer("mamba2", mam(), mlp)
    w = O.random_weights(one_cfg([lay]), 18)
    spec = arch_of([lay]).layers[0].mlp
    assert spec.act == "clamped" and (spec.shared is None or spec.shared.limit != spec.limit)
    mod = RoutedExperts(spec, 24, torch.float32)
    load_module(mod, w, "l0.mlp.")
    h = rows(T, 24, 19) * 2.0
    g = h @ w["l0.mlp.e0.gate"].T
    if T > 1:
        assert float(g.max()) > spec.limit and float((h @ w["l0.mlp.e0.up"].T).min()) < -spec.limit
    check(mod(h.float()), O.moe(w, "l0.mlp.", lay["mlp"], h))


@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_norm_and_input_convolution_in_portions(taps):
    W = 24
    x = rows(30, W, 20) * 2 + 0.5
    wn = 1 + 0.2 * rows(1, W, 21)[0]
    c = 0.4 * rows(W, taps, 22)
    want = O.canon(O.layer_norm(x, wn, EPS), c)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32)
    for cuts in ([30], [1] * 30, [2, 1, 7, 1, 1, 18]):
        hist = torch.randn(3, 2, taps - 1, W)
        got, at = [], 0
        for n in cuts:
            xs = x[at:at + n].float()
            stats = ops.ln_residual_mix(xs, None, None, EPS, xs)
            got.append(ops.ln_canon(xs, stats, wn.float(), c.t().contiguous().float(), hist[:, 1], i32([2]),
                                    i32([0, n]), i32([at]), i32([0] * n), torch.float32))
            at += n
        check(torch.cat(got), want)


def test_post_norm_subtracts_the_mean():
    x = rows(4, 24, 23)
    a = rows(4, 24, 24) + 3.0
    wn = 1 + 0.2 * rows(1, 24, 25)[0]
    out = torch.empty(4, 24)
    ops.ln_residual_mix(x.float(), a.float(), wn.float(), EPS, out)
    check(out, x + O.layer_norm(a, wn, EPS))
    assert float((out.double() - (x + O.rms(a, EPS) * wn)).abs().max()) > 0.1


# --- whole models through the engine ------------------------------------------------

def run_cuts(eng, ids, cuts):
    seq = eng.open_sequence()
    outs, at = [], 0
    for n in cuts:
        outs.append(eng.step_segments([(seq, ids[at:at + n], list(range(n)))]))
        at += n
    eng.kv.free_sequence(seq)
    return torch.cat(outs)


def test_whole_prompt_and_first_tokens(model_a):
    cfg, w, eng = model_a
    ids = toks(45, cfg["vocab"], 20)
    want = O.forward(cfg, w, ids)
    check(run_cuts(eng, ids, [45]), want)
    check(run_cuts(eng, ids[:1], [1]), want[:1])
    check(run_cuts(eng, ids[:3], [1, 1, 1]), want[:3])


def test_cache_entries_and_stream_after_every_layer(model_a):
    cfg, w, eng = model_a
    L = eng.kv.layers
    assert L[3].k is L[2].k and L[5].v is L[2].v and L[3].shared_kv and not L[2].shared_kv
    assert L[2].pool_k.shape[2] == 2 and L[3].pool_k.shape[2] == 1 and L[5].pool_k is None     # 4-token pages
    assert L[0].canon.shape[1:] == (2, 2, 24) and L[3].canon.shape[1] == 1 and L[0].rec.shape[1:] == (4, 5, 6)
    assert L[1].k.shape[-1] == 12 + 6 and L[1].v.numel() == 0
    assert eng.model.lm_head.weight is eng.model.embed_tokens.weight
    ids = toks(14, cfg["vocab"], 21)
    _, layers = O.forward(cfg, w, ids, want_layers=True)
    eng.model.trace_layers = []
    try:
        run_cuts(eng, ids, [5, 9])
        got = eng.model.trace_layers
    finally:
        eng.model.trace_layers = None
    assert len(got) == 12
    for i, b in enumerate(layers):
        check(torch.cat([got[i], got[6 + i]]), b, atol=5e-4)


def test_prefill_then_decode_long(model_a):
    """Every window and several pooled runs pass over decoded tokens."""
    cfg, w, eng = model_a
    ids = toks(4 + 130, cfg["vocab"], 22)
    check(run_cuts(eng, ids, [4] + [1] * 130), O.forward(cfg, w, ids), atol=5e-4)


@pytest.mark.parametrize("cuts", [[2] * 20, [7, 2, 13, 1, 1, 16], [3, 9, 2, 2, 24], [39, 1]])
def test_portions(model_a, cuts):
    cfg, w, eng = model_a
    ids = toks(sum(cuts), cfg["vocab"], 23)
    check(run_cuts(eng, ids, cuts), O.forward(cfg, w, ids))


def test_mixed_batches_reuse_pages_and_slots(model_b):
    """Five unequal requests through three slots and a pool smaller than their
    sum (8-token pages): portions beside single tokens, requests that pause,
    slots and pages that change hands."""
    cfg, w, eng = model_b
    reqs = {n: toks(L, cfg["vocab"], 30 + i) for i, (n, L) in enumerate(
        [("a", 70), ("b", 9), ("c", 33), ("d", 2), ("e", 41)])}
    want = {n: O.forward(cfg, w, ids) for n, ids in reqs.items()}
    plan = [[("a", 30), ("b", 2)], [("a", 1), ("b", 6), ("c", 20)], [("c", 1), ("b", 1)],        # b ends
            [("a", 2), ("d", 2), ("c", 12)],                                                   # d, c end
            [("a", 37), ("e", 1)], [("e", 40)]]
    at = {n: 0 for n in reqs}
    live = {}
    for step in plan:
        entries = []
        for n, c in step:
            if n not in live:
                live[n] = eng.open_sequence()
            entries.append((live[n], reqs[n][at[n]:at[n] + c], list(range(c))))
        got = eng.step_segments(entries)
        r = 0
        for n, c in step:
            check(got[r:r + c], want[n][at[n]:at[n] + c])
            r += c
            at[n] += c
            if at[n] == len(reqs[n]):
                eng.kv.free_sequence(live.pop(n))
    assert not live and eng.kv.slots.num_free == 3 and eng.kv.allocator.num_free == eng.kv.num_blocks


def test_batch_rows_equal_rows_alone(model_a):
    cfg, w, eng = model_a
    a, b, c = toks(19, cfg["vocab"], 44), toks(3, cfg["vocab"], 45), toks(40, cfg["vocab"], 46)
    alone = [run_cuts(eng, x, [len(x)]) for x in (a, b, c)]
    seqs = [eng.open_sequence() for _ in range(3)]
    got = eng.step_segments([(s, x, list(range(len(x)))) for s, x in zip(seqs, (a, b, c))])
    for s in seqs:
        eng.kv.free_sequence(s)
    torch.testing.assert_close(got, torch.cat(alone), rtol=1e-5, atol=1e-5)


def test_used_pages_and_slots_are_not_inherited(model_a):
    cfg, w, eng = model_a
    a, b = toks(37, cfg["vocab"], 40), toks(21, cfg["vocab"], 41)
    s = eng.open_sequence()
    eng.step_segments([(s, a, [])])
    blocks, slot = list(s.blocks), s.state_slot
    eng.kv.free_sequence(s)
    s2 = eng.open_sequence()
    out = eng.step_segments([(s2, b, list(range(21)))])
    assert set(s2.blocks) & set(blocks) and s2.state_slot == slot
    check(out, O.forward(cfg, w, b))
    eng.kv.free_sequence(s2)


def test_second_configuration_in_portions(model_b):
    cfg, w, eng = model_b
    ids = toks(50, cfg["vocab"], 42)
    want = O.forward(cfg, w, ids)
    check(run_cuts(eng, ids, [50]), want)
    check(run_cuts(eng, ids, [3, 1, 1, 2, 23, 2, 18]), want)
    check(run_cuts(eng, ids, [10] + [1] * 40), want)


def oracle_greedy(cfg, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(O.forward(cfg, w, ids)[-1].argmax()))
    return ids[len(prompt):]


def test_greedy_generation_and_fork(model_a):
    """n = 2 forks the prompt's sequence: the tail page (with its pooled
    entries) and the slot (state-space matrix, both convolution histories)
    are copied, and both streams go on like the oracle."""
    cfg, w, eng = model_a
    p1, p2 = toks(21, cfg["vocab"], 50), toks(5, cfg["vocab"], 51)
    sp = lambda n: SamplingParams(temperature=0.0, max_tokens=n)
    outs = eng.generate([GenRequest(prompt_ids=p1, n=2, sampling=sp(7)), GenRequest(prompt_ids=p2, n=1, sampling=sp(9))])
    want1, want2 = oracle_greedy(cfg, w, p1, 7), oracle_greedy(cfg, w, p2, 9)
    assert [s.token_ids for s in outs[0].streams] == [want1, want1]
    assert outs[1].streams[0].token_ids == want2
    assert eng.kv.slots.num_free == eng.kv.slots.num_slots and eng.kv.allocator.num_free == eng.kv.num_blocks


def test_scheduler_chunked_prefill_and_merge(tmp_path):
    w = write_model(str(tmp_path), CFG_A, seed=1)
    eng = make_engine(tmp_path, blocks=128, slots=8, prefill_chunk_tokens=8, max_batch_size=4)
    sched = BatchScheduler(eng)
    try:
        p1, p2 = toks(29, CFG_A["vocab"], 52), toks(6, CFG_A["vocab"], 53)
        sp = lambda n: SamplingParams(temperature=0.0, max_tokens=n)
        f1 = sched.submit(GenRequest(prompt_ids=p1, n=1, sampling=sp(6)))
        f2 = sched.submit(GenRequest(prompt_ids=p2, n=2, sampling=sp(8)))
        o1, o2 = f1.result(timeout=120), f2.result(timeout=120)
    finally:
        sched.shutdown()
    assert o1.streams[0].token_ids == oracle_greedy(CFG_A, w, p1, 6)
    want2 = oracle_greedy(CFG_A, w, p2, 8)
    assert [s.token_ids for s in o2.streams] == [want2, want2]
    assert eng.kv.slots.num_free == eng.kv.slots.num_slots


def test_config_reader_takes_everything_from_the_file(tmp_path):
    write_model(str(tmp_path), CFG_B, seed=2)
    arch = EngineConfig(model=str(tmp_path)).resolve_arch()
    assert arch.arch == "pironex" and arch.vocab_size == 47 and arch.hidden_size == 20
    assert arch.norm_eps == 1e-5 and arch.canon_taps == 1 and arch.embed_scale == 1.0 and arch.tie_word_embeddings
    assert [l.type for l in arch.layers] == ["attention", "attention", "latent_attention", "mamba2", "attention"]
    a0, a1, a4 = arch.layers[0].attention, arch.layers[1].attention, arch.layers[4].attention
    assert (a0.heads, a0.kv_heads, a0.dim, a0.vdim, a0.mask_size, a0.pool, a0.scale, a0.softcap) == \
        (3, 3, 4, 5, 6, 11, 0.9, 0.0)
    assert a0.kv_from is None and a1.kv_from == 0 and (a1.mask_size, a1.pool, a1.softcap) == (3, 2, 6.0)
    assert a0.rot.dims == 4 and a0.rot.base == 50.0 and a0.rot.layout == "half" and a4.rot.dims == 0
    assert (a4.mask_size, a4.pool) == (0, 0)
    la = arch.layers[2].latent
    assert (la.heads, la.dim, la.rot_dim, la.vdim, la.kv_rank, la.mask_size, la.head_gate) == (1, 6, 2, 5, 7, 0, False)
    mm = arch.layers[3].mamba2
    assert (mm.heads, mm.vdim, mm.state, mm.groups, mm.conv, mm.norm_groups) == (2, 9, 3, 2, 1, 1)
    m0, m1 = arch.layers[0].mlp, arch.layers[1].mlp
    assert (m0.experts, m0.top, m0.ff, m0.limit, m0.shared.ff, m0.shared.limit) == (7, 1, 16, 0.8, 8, 2.0)
    assert m1.shared is None and m1.top == 3 and arch.layers[2].mlp is None
    assert m0.score == "softmax" and m0.renormalize and m0.weight_on == "output" and not m0.correction
    # a layer may read only an earlier attention layer that has keys and values of its own
    for src in (1, 2, 4):
        bad = json.loads(json.dumps(CFG_B))
        bad["layers"][4]["mixer"]["kv_from"] = src
        with pytest.raises(ValueError):
            PironexArchConfig.from_checkpoint_config(bad)


def test_presets_build_and_generate():
    eng = LLMEngine(EngineConfig(model="tiny-pironex", dtype="float32", device="cpu", max_kv_blocks=64,
                                 max_state_slots=4, use_hip_graphs=False))
    out = eng.generate([GenRequest(prompt_ids=toks(9, 512, 60), n=2, sampling=SamplingParams(temperature=0.0, max_tokens=5))])
    assert len(out[0].streams) == 2 and out[0].streams[0].token_ids == out[0].streams[1].token_ids


def test_trace_replay_cli(tmp_path):
    import subprocess
    import sys

    import numpy as np

    cfg = CFG_B
    mdir, out = tmp_path / "m", tmp_path / "out"
    w = write_model(str(mdir), cfg, seed=4)
    a, b = toks(20, cfg["vocab"], 61), toks(5, cfg["vocab"], 62)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:18], "want": [0, 17]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[18:19], "want": []},
                                     {"id": "b", "tokens": b, "want": [4]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[19:], "want": [0]}], "end": ["a"]}]
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "trace_run")
    r = subprocess.run([sys.executable, exe, "--model", str(mdir), "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "64", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    la, lb = O.forward(cfg, w, a), O.forward(cfg, w, b)
    rd = lambda n: torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, cfg["vocab"]).copy())
    check(rd(0), la[[0, 17]])
    check(rd(1), lb[[4]])
    check(rd(2), la[[19]])
