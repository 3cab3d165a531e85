"""Pironex family on the GPU: the engine with its HIP kernels (fp32 exact mode
and bf16 serving mode) against the float64 oracle, through mixed schedules
with page reuse, long decoding over the windows and pooled runs, and greedy
generation through generate() (which forks pages with pooled entries and
slots with convolution histories)."""

import pytest
import torch

import pironex_oracle as O
from kllms_amd import ops
from kllms_amd.engine.config import EngineConfig
from kllms_amd.engine.engine import GenRequest, LLMEngine
from kllms_amd.engine.sampling import SamplingParams
from test_pironex import CFG_A, CFG_B, oracle_greedy, toks, write_model
from test_zutalix import run_schedule

pytestmark = pytest.mark.gpu


def gpu_engine(path, dtype, **kw):
    return LLMEngine(EngineConfig(model=str(path), dtype=dtype, device="cuda", max_kv_blocks=96,
                                  max_state_slots=6, use_hip_graphs=False, **kw))


SCHED = [[("a", 16)], [("a", 3), ("b", 20)], [("a", 1), ("b", 1), ("c", 30)], [("a", 10), ("b", 2), ("c", 1)],
         [("a", 20), ("c", 6)], [("d", 2), ("e", 8)], [("d", 1), ("e", 1), ("f", 7)], [("d", 30), ("f", 1)],
         [("d", 8), ("f", 22)]]
LENS = {"a": 50, "b": 23, "c": 37, "d": 41, "e": 9, "f": 30}


@pytest.mark.parametrize("cfg,seed", [(CFG_A, 1), (CFG_B, 2)])
def test_fp32_mixed_schedule_matches_oracle(tmp_path, cfg, seed):
    w = write_model(str(tmp_path), cfg, seed=seed)
    eng = gpu_engine(tmp_path, "float32")
    prompts = {r: toks(n, cfg["vocab"], 10 + i) for i, (r, n) in enumerate(LENS.items())}
    got = run_schedule(eng, SCHED, prompts)
    assert ops.seq_hip_loaded()
    for r in LENS:
        torch.testing.assert_close(got[r].double().cpu(), O.forward(cfg, w, prompts[r]), rtol=1e-4, atol=3e-4)
    assert eng.kv.allocator.num_free == eng.kv.num_blocks


def test_fp32_long_decode_and_sorted_experts(tmp_path, monkeypatch):
    """150 single-token steps after a short prompt (every window and many
    pooled runs pass over decoded tokens), and whole portions with the
    experts' rows sorted by expert instead of every expert on every row."""
    cfg = CFG_A
    w = write_model(str(tmp_path), cfg, seed=1)
    eng = gpu_engine(tmp_path, "float32")
    p = toks(154, cfg["vocab"], 7)
    want = O.forward(cfg, w, p)
    got = run_schedule(eng, [[("x", 4)]] + [[("x", 1)]] * 150, {"x": p})["x"]
    torch.testing.assert_close(got.double().cpu(), want, rtol=1e-4, atol=5e-4)
    got = run_schedule(eng, [[("y", 154)]], {"y": p})["y"]
    torch.testing.assert_close(got.double().cpu(), want, rtol=1e-4, atol=5e-4)
    from kllms_amd.models.mixers import RoutedExperts

    monkeypatch.setattr(RoutedExperts, "DENSE_MAX_ROWS", 0)
    got = run_schedule(eng, [[("z", 100)], [("z", 1)], [("z", 53)]], {"z": p})["z"]
    torch.testing.assert_close(got.double().cpu(), want, rtol=1e-4, atol=5e-4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation(tmp_path, dtype):
    cfg = CFG_A
    w = write_model(str(tmp_path), cfg, seed=1)
    p1, p2 = toks(21, cfg["vocab"], 40), toks(5, cfg["vocab"], 41)
    sp = lambda n: SamplingParams(temperature=0.0, max_tokens=n)
    eng = gpu_engine(tmp_path, dtype, max_seq_len=256)
    out = eng.generate([GenRequest(prompt_ids=p1, n=2, sampling=sp(40)), GenRequest(prompt_ids=p2, n=1, sampling=sp(25))])
    assert out[0].streams[0].token_ids == out[0].streams[1].token_ids and len(out[1].streams[0].token_ids) == 25
    if dtype == "float32":
        assert out[0].streams[0].token_ids[:8] == oracle_greedy(cfg, w, p1, 8)
        assert out[1].streams[0].token_ids[:8] == oracle_greedy(cfg, w, p2, 8)
    assert eng.kv.allocator.num_free == eng.kv.num_blocks


@pytest.mark.parametrize("cfg,seed", [(CFG_A, 1), (CFG_B, 2)])
def test_bf16_close_to_oracle_and_cut_invariant(tmp_path, cfg, seed):
    """Serving mode: bf16 GEMMs and caches, fp32 stream, norms, scores and
    recurrent state; sizes that are no multiple of the kernels' vector width."""
    w = write_model(str(tmp_path), cfg, seed=seed)
    eng = gpu_engine(tmp_path, "bfloat16")
    p = toks(90, cfg["vocab"], 5)
    want = O.forward(cfg, w, p)
    whole = run_schedule(eng, [[("x", 90)]], {"x": p})["x"].double().cpu()
    cut = run_schedule(eng, [[("x", n)] for n in [2, 30, 1, 1, 17, 39]], {"x": p})["x"].double().cpu()
    single = run_schedule(eng, [[("x", 60)]] + [[("x", 1)]] * 30, {"x": p})["x"].double().cpu()
    scale = want.std()
    assert (whole - want).std() / scale < 0.08
    assert (cut - whole).std() / scale < 0.08
    assert (single - whole).std() / scale < 0.08


def test_preset_generates_on_gpu():
    eng = LLMEngine(EngineConfig(model="mid-pironex", device="cuda", max_kv_blocks=512, max_state_slots=16,
                                 use_hip_graphs=False, max_seq_len=1024))
    out = eng.generate([GenRequest(prompt_ids=list(range(1, 300)), n=3,
                                   sampling=SamplingParams(temperature=0.8, max_tokens=24, seed=3))])
    assert all(len(s.token_ids) > 0 for s in out[0].streams)
    assert eng.kv.allocator.num_free == eng.kv.num_blocks
