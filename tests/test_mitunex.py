"""Mitunex family on the CPU path (fp32) against the plain float64 oracle in
tests/mitunex_oracle.py: every mechanism alone, then whole models through the
engine's segment step, page and slot reuse, and greedy generation through
generate() and the scheduler. Configurations are small and lopsided: head
counts that are not powers of two, value sizes that differ from key sizes,
latent sizes that are no multiple of 8 or 16, routers with top 1 and top 3,
with and without a shared expert, layers without a feed-forward, layers that
borrow weights, with and without a window and a soft cap."""

import json
import os

import pytest
import torch

import mitunex_oracle as O
from kllms_amd import ops
from kllms_amd.engine.config import (ActFFSpec, EngineConfig, LatentAttnSpec, RotarySpec, RoutedExpertsSpec,
                                     SharedExpertSpec)
from kllms_amd.engine.engine import GenRequest, LLMEngine
from kllms_amd.engine.kvcache import HybridStateCache
from kllms_amd.engine.sampling import SamplingParams
from kllms_amd.engine.scheduler import BatchScheduler
from kllms_amd.models.llama import ForwardBatch
from kllms_amd.models.mixers import ActFF, LatentAttention, RoutedExperts

EPS = 1e-6


def mixer(heads=3, dim=10, rot_dim=6, vdim=7, kv_rank=12, size=9, scale=0.3, base=100.0):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot_dim}}
    if size:
        m["mask"] = {"size": size}
    return m


MLPS = {
    None: None,
    "dense": {"kind": "dense", "ff": 40},
    "moe": {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 5, "top": 3}, "shared": {"ff": 20}},
    "moe_top1": {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 7, "top": 1}, "shared": {"ff": 8}},
    "moe_bare": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 3, "top": 2}},
}


def layer(mlp="dense", weights_of=None, **kw):
    d = {"type": "latent_attention", "mixer": mixer(**kw), "mlp": MLPS[mlp]}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def shared(cfg_layers, i, j):
    """Layer entry that uses layer j's weights: the rest of the entry equals layer j's."""
    d = dict(cfg_layers[j])
    d["weights_of"] = j
    return d


def _cfg_a():
    layers = [layer("dense"), layer("moe", heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=16, size=5, scale=0.5)]
    layers += [shared(layers, 2, 1), shared(layers, 3, 1), layer(None, heads=5, dim=4, rot_dim=2, vdim=3, kv_rank=9, size=17)]
    return {"architecture": "Mitunex", "vocab": 61, "width": 24, "norm": {"eps": EPS}, "max_positions": 300,
            "logit_scale": 3.0, "logit_softcap": 4.0, "layers": layers}


def _cfg_b():
    # no window, no soft cap, one head, top 1, a router without a shared expert, the first layer shared
    layers = [layer("moe_top1", heads=1, dim=6, rot_dim=2, vdim=5, kv_rank=7, size=0, scale=0.7)]
    layers += [shared(layers, 1, 0), layer("moe_bare", heads=4, dim=2, rot_dim=8, vdim=2, kv_rank=3, size=64, scale=0.9),
               layer("dense", heads=2, dim=16, rot_dim=2, vdim=4, kv_rank=20, size=2)]
    return {"architecture": "Mitunex", "vocab": 47, "width": 20, "norm": {"eps": 1e-5}, "max_positions": 128,
            "logit_scale": 1.0, "layers": layers}


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
    d = tmp_path_factory.mktemp("mit_a")
    w = write_model(str(d), CFG_A, seed=1)
    return CFG_A, w, make_engine(d, blocks=96)


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    d = tmp_path_factory.mktemp("mit_b")
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


def run_mixer(mod, h, cuts, page=4):
    """Feed h [L, W] through a mixer in portions; its pages are not the first
    ones of the pool and were used before."""
    cache = HybridStateCache([mod.cache_spec()], page, 200, 3, "cpu", torch.float32)
    cache.layers[0].k.normal_()                       # a page holds whatever its last owner left
    cache.slots.alloc()
    for _ in range(3):
        cache.allocator.alloc()
    seq = cache.open_sequence()
    outs, at = [], 0
    for n in cuts:
        outs.append(mod(h[at:at + n].float(), seg_batch(cache, [seq], [n]), cache.layer_caches()[0]))
        at += n
    return torch.cat(outs)


def load_module(mod, w, pre):
    for name, dst in mod.checkpoint_map(pre).items():
        dst.copy_(w[name].to(dst.dtype))


def attn_module(m, width):
    spec = LatentAttnSpec(heads=m["heads"], dim=m["dim"], rot_dim=m["rot_dim"], vdim=m["vdim"], kv_rank=m["kv_rank"],
                          scale=m["scale"], mask_size=(m.get("mask") or {}).get("size", 0),
                          rot=RotarySpec(base=m["rot"]["base"], dims=m["rot"]["dims"]))
    return LatentAttention(spec, width, EPS, torch.float32)


def one_layer(lay, width=24, seed=3):
    return O.random_weights({"vocab": 8, "width": width, "max_positions": 4, "layers": [lay]}, seed)


CUTS = [[60], [70], [25] + [1] * 35, [2, 5, 16, 1, 2, 17, 3, 14], [9, 2, 10, 1, 38], [2] * 30]


@pytest.mark.parametrize("cuts", CUTS)
@pytest.mark.parametrize("size", [9, 4, 0])
def test_latent_attention_window_edges(cuts, size):
    """Window of 9 (4, none) on 4-token pages with a scale that makes single
    keys dominate the softmax: a window or a page border that is one position
    off shows at once. Portions cut the window and the pages anywhere."""
    lay = layer(size=size, scale=2.0)
    w = one_layer(lay)
    mod = attn_module(lay["mixer"], 24)
    load_module(mod, w, "l0.mix.")
    h = rows(sum(cuts), 24, 4)
    check(run_mixer(mod, h, cuts), O.latent_attention(lay["mixer"], EPS, w, "l0.mix.", h))


def test_oracle_window_is_what_the_comparison_rests_on():
    """In the oracle a key just inside the window changes the output and one
    just outside does not; position 0 sees only itself."""
    lay = layer(size=9, scale=2.0)
    w = one_layer(lay)
    m = lay["mixer"]
    a = rows(30, 24, 5)
    base = O.latent_attention(m, EPS, w, "l0.mix.", a)
    for i, j, seen in [(20, 12, True), (20, 11, False), (20, 20, True), (8, 0, True), (9, 0, False)]:
        b = a.clone()
        b[j] = rows(1, 24, 99)[0]
        assert (float((O.latent_attention(m, EPS, w, "l0.mix.", b)[i] - base[i]).abs().max()) > 1e-6) == seen, (i, j)
    # one token: softmax over itself, output = gate * W_o W_uv c
    h = a[:1]
    W = lambda n: w["l0.mix." + n]
    d = W("dkv") @ h[0]
    c = O.rms(d[:m["kv_rank"]], EPS) * W("dkv.norm")
    want = W("o") @ ((W("uv") @ c).view(m["heads"], m["vdim"]) * torch.sigmoid(W("g") @ h[0])[:, None]).reshape(-1)
    check(base[0], O.latent_attention(m, EPS, w, "l0.mix.", h)[0], atol=1e-9)
    check(O.latent_attention(m, EPS, w, "l0.mix.", h)[0], want, atol=1e-9)


def test_rotation_pairs_neighbours_and_leaves_the_rest():
    """The rotated part pairs entry 2i with 2i+1 at angle p * base^(-2i/dims);
    the unrotated query part and the latent do not depend on the position."""
    lay = layer(heads=2, dim=6, rot_dim=4, vdim=5, kv_rank=8, size=0, base=50.0)
    m = lay["mixer"]
    w = one_layer(lay)
    mod = attn_module(m, 24)
    load_module(mod, w, "l0.mix.")
    v = torch.tensor([1.0, 0.0, 0.0, 1.0], dtype=torch.float64)
    r = O.rotate_pairs(v, 3, 50.0, 4)
    import math
    f1 = 50.0 ** (-2.0 / 4)
    check(r, torch.tensor([math.cos(3), math.sin(3), -math.sin(3 * f1), math.cos(3 * f1)], dtype=torch.float64), atol=1e-12)
    # the product path at positions far from 0: a prompt of 150 tokens, compared at the end
    h = rows(150, 24, 8)
    check(run_mixer(mod, h, [140] + [1] * 10)[-10:], O.latent_attention(m, EPS, w, "l0.mix.", h)[-10:])


def test_far_key_within_the_window_dominates():
    """A key 100 tokens back whose latent matches the last query: scaled so
    that it takes nearly all the weight. A window that ends early, a wrong
    page or a wrong rotation of the shared key part loses it."""
    lay = layer(heads=2, dim=8, rot_dim=4, vdim=6, kv_rank=10, size=120, scale=1.0)
    m = lay["mixer"]
    w = one_layer(lay, seed=11)
    h = rows(130, 24, 12) * 0.2
    h[29] = h[129] * 6.0               # the same direction, much longer: its key stands out for the last query
    mod = attn_module(m, 24)
    load_module(mod, w, "l0.mix.")
    want = O.latent_attention(m, EPS, w, "l0.mix.", h)
    hh = h.clone()
    hh[29] = rows(1, 24, 13)[0] * 0.2
    assert float((O.latent_attention(m, EPS, w, "l0.mix.", hh)[129] - want[129]).abs().max()) > 1e-3
    for cuts in ([130], [100, 29, 1], [28, 2] + [1] * 100):
        check(run_mixer(mod, h, cuts, page=16)[-1], want[-1])


def test_gelu_feed_forward():
    w = one_layer(layer("dense"))
    mod = ActFF(ActFFSpec(ff=40), 24, torch.float32)
    load_module(mod, w, "l0.mlp.")
    h = rows(9, 24, 6) * 2.0
    check(mod(h.float()), O.dense_ff(w, "l0.mlp.", h))
    z = torch.tensor([-3.0, -0.5, 0.0, 0.7, 4.0], dtype=torch.float64)
    check(ops.gelu_tanh(z.float()), O.gelu_tanh(z), atol=1e-6)
    assert abs(float(O.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12


@pytest.mark.parametrize("name,T,sorted_form", [("moe", 7, False), ("moe", 90, True), ("moe_top1", 80, True),
                                                ("moe_top1", 5, False), ("moe_bare", 11, False),
                                                ("moe_bare", 70, True)])
def test_sigmoid_routed_experts(name, T, sorted_form):
    """Sigmoid scores, weights not renormalised and applied to the expert's
    input, gated shared expert; the all-experts form and the sorted form."""
    mlp = MLPS[name]
    w = one_layer(layer(name))
    sh = mlp.get("shared")
    spec = RoutedExpertsSpec(experts=mlp["router"]["experts"], top=mlp["router"]["top"], ff=mlp["expert"]["ff"],
                             score="sigmoid", renormalize=False, correction=False, weight_on="input",
                             shared=SharedExpertSpec(ff=sh["ff"]) if sh else None)
    mod = RoutedExperts(spec, 24, torch.float32)
    load_module(mod, w, "l0.mlp.")
    h = rows(T, 24, 7)
    dense = T <= mod.DENSE_MAX_ROWS and spec.experts * T <= mod.DENSE_MAX_PAIRS
    assert dense != sorted_form
    want = O.moe_ff(mlp, w, "l0.mlp.", h)
    check(mod(h.float()), want)
    # the weight sits on the input: scaling the output instead gives something else
    x = h[0]
    idx, wt = O.route(w["l0.mlp.router"], x, mlp["router"]["top"])
    other = sum(s * O.glu_expert(w, f"l0.mlp.e{e}.", x) for e, s in zip(idx, wt))
    mine = sum(O.glu_expert(w, f"l0.mlp.e{e}.", s * x) for e, s in zip(idx, wt))
    assert float((other - mine).abs().max()) > 1e-4
    assert all(0.0 < float(s) < 1.0 for s in wt) and sorted(wt, reverse=True) == wt


def test_embedding_adds_position_rows_before_the_norm(model_a):
    cfg, w, eng = model_a
    ids = toks(6, cfg["vocab"], 9)
    m = eng.model
    got = ops.embed_rmsnorm(torch.tensor(ids), m.embed_tokens.weight, m.embed_norm, EPS, m.pos,
                            torch.tensor([10, 11, 12, 13, 14, 15]))
    x = torch.stack([w["embed"][t] + w["pos"][10 + i] for i, t in enumerate(ids)])
    check(got, O.rms(x, EPS) * w["embed.norm"])


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
    assert float(want.abs().max()) <= cfg["logit_softcap"] and float(want.abs().max()) > 0.5 * cfg["logit_softcap"]
    check(run_cuts(eng, ids, [45]), want)
    check(run_cuts(eng, ids[:1], [1]), want[:1])
    check(run_cuts(eng, ids[:3], [1, 1, 1]), want[:3])


def test_layers_that_borrow_weights_keep_their_own_cache(model_a):
    cfg, w, eng = model_a
    assert len(eng.kv.layers) == 5 and len(eng.model.layers) == 3
    assert eng.kv.layers[1].k is not eng.kv.layers[2].k and eng.kv.layers[1].k.shape == eng.kv.layers[2].k.shape
    assert all(st.v.numel() == 0 for st in eng.kv.layers)          # only the latent rows are cached
    assert eng.kv.layers[1].k.shape[-1] == 16 + 4
    ids = toks(12, cfg["vocab"], 21)
    layers = []
    O.forward(cfg, w, ids, layers)
    eng.model.trace_layers = []
    try:
        run_cuts(eng, ids, [5, 7])
        got = eng.model.trace_layers
    finally:
        eng.model.trace_layers = None
    assert len(got) == 10
    for i, b in enumerate(layers):
        check(torch.cat([got[i], got[5 + i]]), b, atol=5e-4)


def test_prefill_then_decode_long(model_a):
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


def test_batch_rows_equal_rows_alone(model_b):
    cfg, w, eng = model_b
    a, b, c = toks(19, cfg["vocab"], 44), toks(3, cfg["vocab"], 45), toks(40, cfg["vocab"], 46)
    alone = [run_cuts(eng, x, [len(x)]) for x in (a, b, c)]
    seqs = [eng.open_sequence() for _ in range(3)]
    got = eng.step_segments([(s, x, list(range(len(x)))) for s, x in zip(seqs, (a, b, c))])
    for s in seqs:
        eng.kv.free_sequence(s)
    torch.testing.assert_close(got, torch.cat(alone), rtol=1e-5, atol=1e-5)


def test_a_used_page_is_not_inherited(model_b):
    cfg, w, eng = model_b
    a, b = toks(25, cfg["vocab"], 40), toks(11, cfg["vocab"], 41)
    s = eng.open_sequence()
    eng.step_segments([(s, a, [])])
    blocks = list(s.blocks)
    eng.kv.free_sequence(s)
    s2 = eng.open_sequence()
    out = eng.step_segments([(s2, b, list(range(11)))])
    assert set(s2.blocks) & set(blocks)
    check(out, O.forward(cfg, w, b))
    eng.kv.free_sequence(s2)


def test_second_configuration_in_portions(model_b):
    cfg, w, eng = model_b
    ids = toks(50, cfg["vocab"], 42)
    want = O.forward(cfg, w, ids)
    check(run_cuts(eng, ids, [50]), want)
    check(run_cuts(eng, ids, [3, 1, 1, 2, 23, 2, 18]), want)


def oracle_greedy(cfg, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(O.forward(cfg, w, ids)[-1].argmax()))
    return ids[len(prompt):]


def test_greedy_generation_and_fork(model_a):
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
    assert arch.arch == "mitunex" and arch.vocab_size == 47 and arch.hidden_size == 20
    assert arch.rms_norm_eps == 1e-5 and arch.max_position_embeddings == 128
    assert arch.logit_scale == 1.0 and arch.logit_softcap == 0.0
    assert [l.weights_of for l in arch.layers] == [0, 0, 2, 3]
    a0, a2 = arch.layers[0].attention, arch.layers[2].attention
    assert (a0.heads, a0.dim, a0.rot_dim, a0.vdim, a0.kv_rank, a0.mask_size, a0.scale) == (1, 6, 2, 5, 7, 0, 0.7)
    assert a2.mask_size == 64 and a2.rot.base == 100.0 and a2.rot.dims == 8
    m0, m2 = arch.layers[0].mlp, arch.layers[2].mlp
    assert (m0.experts, m0.top, m0.ff, m0.shared.ff) == (7, 1, 16, 8) and m2.shared is None and m2.top == 2
    assert m0.score == "sigmoid" and not m0.renormalize and m0.weight_on == "input"
    assert arch.layers[3].mlp.kind == "dense" and arch.layers[3].mlp.ff == 40
    # a layer may borrow only from a layer that has weights of its own
    bad = json.loads(json.dumps(CFG_B))
    bad["layers"][2]["weights_of"] = 1
    from kllms_amd.engine.config import MitunexArchConfig
    with pytest.raises(ValueError):
        MitunexArchConfig.from_checkpoint_config(bad)


def test_presets_build_and_generate():
    eng = LLMEngine(EngineConfig(model="tiny-mitunex", dtype="float32", device="cpu", max_kv_blocks=64,
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
