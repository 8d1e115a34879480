"""The Solopel stack through the engine (InferenceEngine.run_ragged / generate) against the plain whole-sequence
restatement in oracle/ref_solopel.py: whole prompts layer by layer, token-by-token decoding, portions down to two
tokens, mixed batches, pages and slots that are used again, long decoding, a far token, greedy generation through
the scheduler, a checkpoint directory through the registry and the trace runner.  fp32 runs are held to 1e-4 of the
logits' norm; bf16 runs to a few per cent (what rounding of the projections' operands costs)."""
import pytest
import torch

from oracle import ref_solopel as ref
from ragged_util import rel_err, run_in_portions
from solopel_util import config_a, config_b, config_c, make_engine, random_config

pytestmark = pytest.mark.gpu


def tokens_for(cfg, n, seed):
    return torch.randint(0, cfg.vocab_size, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def oracle_logits(eng, cfg, toks, residuals=None):
    weights = {name: eng.model.get(name) for name in eng.model.names()}
    return ref.forward(cfg.to_json(), weights, toks, residuals=residuals)


@pytest.mark.parametrize("make", [config_a, config_b, config_c])
def test_whole_prompt_layer_by_layer_fp32(make):
    cfg = make()
    eng = make_engine(cfg, torch.float32)
    toks = tokens_for(cfg, 150, 1)
    res, want_res = [], []
    got = eng.run_ragged([("a", toks, list(range(len(toks))))], residuals=res).double().cpu()
    want = oracle_logits(eng, cfg, toks, want_res)
    assert len(res) == len(want_res) == len(cfg.runs)
    for i, (r, w) in enumerate(zip(res, want_res)):
        assert rel_err(r.cpu(), w) < 2e-5, f"residual stream after layer run {i}"
    assert rel_err(got, want) < 1e-4
    assert bool((got.argmax(-1) == want.argmax(-1)).float().mean() > 0.98)
    eng.release("a")
    # the stream between layers travels with the sublayer output still to be added: without snapshots the same logits
    assert rel_err(run_in_portions(eng, "b", toks, [150]), got) < 1e-6


@pytest.mark.parametrize("make", [config_a, config_b, config_c])
def test_whole_prompt_and_decoding_bf16(make):
    cfg = make()
    eng = make_engine(cfg, torch.bfloat16)
    toks = tokens_for(cfg, 150, 2)
    want = oracle_logits(eng, cfg, toks)
    whole = run_in_portions(eng, "a", toks, [150])
    assert rel_err(whole, want) < 0.1          # eleven layer runs deep in one of the configurations
    cut = run_in_portions(eng, "b", toks, [100, 2, 17] + [1] * 31)
    assert rel_err(cut, want) < 0.1 and rel_err(cut, whole) < 0.06
    # the matrix-core attention against the one-workgroup-per-token form on the same pages
    eng.runner.tiled_attn = False
    assert rel_err(run_in_portions(eng, "c", toks, [150]), whole) < 0.02


@pytest.mark.parametrize("make", [config_a, config_b, config_c])
def test_portions_and_decoding_match_the_whole_prompt_fp32(make):
    cfg = make()
    eng = make_engine(cfg, torch.float32)
    toks = tokens_for(cfg, 200, 3)
    want = oracle_logits(eng, cfg, toks)
    for portions in ([200], [64, 64, 64, 8], [37, 64, 3, 2, 64, 30], [2] * 100, [150] + [1] * 50, [1] * 200):
        got = run_in_portions(eng, "p", toks, portions)
        assert rel_err(got, want) < 1e-4, portions[:6]


@pytest.mark.parametrize("seed", [0, 1, 2, 3, 5, 8, 13, 21, 34, 55])
def test_configurations_drawn_at_random(seed):
    cfg = random_config(seed)
    eng = make_engine(cfg, torch.float32, seed=seed)
    toks = tokens_for(cfg, 140, seed)
    want = oracle_logits(eng, cfg, toks)
    assert rel_err(run_in_portions(eng, "w", toks, [140]), want) < 1e-4
    assert rel_err(run_in_portions(eng, "p", toks, [70, 2, 5, 33] + [1] * 30), want) < 1e-4
    a, b = toks[:90], toks[90:]
    wb = oracle_logits(eng, cfg, b)
    out = eng.run_ragged([("a", a, list(range(90))), ("b", b, list(range(50)))]).double().cpu()
    assert rel_err(out[:90], want[:90]) < 1e-4 and rel_err(out[90:], wb) < 1e-4
    eng16 = make_engine(cfg, torch.bfloat16, seed=seed)
    whole = run_in_portions(eng16, "w", toks, [140])
    assert rel_err(whole, want) < 0.12
    assert rel_err(run_in_portions(eng16, "d", toks, [120] + [1] * 20), whole) < 0.12


def test_first_tokens_fp32():
    """Fewer tokens than the convolutions have taps: what lies before the sequence counts as zero, whatever the slot
    held before."""
    cfg = config_a()
    eng = make_engine(cfg, torch.float32)
    run_in_portions(eng, "dirt", tokens_for(cfg, 40, 99), [40])     # leaves its tails in slot 0
    toks = tokens_for(cfg, 6, 4)
    want = oracle_logits(eng, cfg, toks)
    for portions in ([6], [1] * 6, [2, 2, 2], [1, 5]):
        assert rel_err(run_in_portions(eng, "f", toks, portions), want) < 1e-4
    assert rel_err(run_in_portions(eng, "g", toks[:1], [1]), want[:1]) < 1e-4


def test_mixed_batch_equals_each_request_alone_fp32():
    cfg = config_a()
    eng = make_engine(cfg, torch.float32, pages=40)
    reqs = {"a": tokens_for(cfg, 130, 5), "b": tokens_for(cfg, 9, 6), "c": tokens_for(cfg, 70, 7), "d": tokens_for(cfg, 33, 8)}
    alone = {k: run_in_portions(eng, k + "!", t, [len(t)]) for k, t in reqs.items()}
    # portions of some beside single tokens of others, requests joining, pausing and leaving
    plan = [{"a": 64, "b": 2}, {"a": 3, "b": 1, "c": 70}, {"a": 1, "b": 1, "c": 0, "d": 2}, {"a": 62, "b": 5, "d": 31}]
    at = {k: 0 for k in reqs}
    got = {k: [] for k in reqs}
    for step in plan:
        entries = [(k, reqs[k][at[k]:at[k] + n], list(range(n))) for k, n in step.items() if n]
        out = eng.run_ragged(entries).double().cpu()
        o = 0
        for k, t, _ in entries:
            got[k].append(out[o:o + len(t)])
            o += len(t)
            at[k] += len(t)
            if at[k] == len(reqs[k]):
                eng.release(k)
    for k in reqs:
        assert at[k] == len(reqs[k])
        assert rel_err(torch.cat(got[k]), alone[k]) < 2e-5, k


def test_pages_and_slots_used_again_fp32():
    cfg = config_a()
    eng = make_engine(cfg, torch.float32, pages=6, slots=2)           # 384 tokens, two live requests
    a, b, c = tokens_for(cfg, 190, 9), tokens_for(cfg, 180, 10), tokens_for(cfg, 120, 11)
    ref_c = run_in_portions(eng, "fresh", c, [len(c)])
    run_in_portions(eng, "a", a, [100, 90], release=False)
    run_in_portions(eng, "b", b, [180], release=False)
    assert eng.cache_manager.stats["free"] == 0 and eng.cache_manager.stats["slots_free"] == 0
    from micro_vllm_amd.core.state_cache import PoolExhausted
    with pytest.raises(PoolExhausted):
        eng.run_ragged([("c", c[:5], [])])
    eng.release("a")                                   # its pages hold a's keys, its slot the tails of a's convolutions
    got = run_in_portions(eng, "c", c, [1, 1, 5, 64, 49], release=False)
    assert rel_err(got, ref_c) < 2e-5
    eng.release("b")
    eng.release("c")
    assert eng.cache_manager.stats["free"] == 6 and eng.cache_manager.stats["slots_free"] == 2


@pytest.mark.parametrize("make", [config_a, config_b])
def test_long_decoding_fp32_and_captured_steps(make):
    """Three hundred single-token steps: page after page is opened, the convolutions' tails roll, and the steps run
    from the recorded graph (one row) - checked against the restatement and against uncaptured steps."""
    cfg = make()
    eng = make_engine(cfg, torch.float32, pages=12)
    toks = tokens_for(cfg, 320, 12)
    want = oracle_logits(eng, cfg, toks)
    got = run_in_portions(eng, "l", toks, [20] + [1] * 300)
    assert rel_err(got, want) < 2e-4
    assert rel_err(got[-50:], want[-50:]) < 2e-4
    eng.runner.use_graphs = False
    plain = run_in_portions(eng, "m", toks, [20] + [1] * 300)
    assert rel_err(got, plain) < 1e-5


def test_a_far_token_still_counts_fp32():
    """Both attentions are causal without a window: a token hundreds of positions back changes the last logits, and the
    engine follows the restatement there through portions and decoding."""
    cfg = config_a()
    eng = make_engine(cfg, torch.float32, pages=12)
    toks = tokens_for(cfg, 400, 13)
    other = list(toks)
    other[2] = (other[2] + 1) % cfg.vocab_size
    want, want2 = (oracle_logits(eng, cfg, t)[-1] for t in (toks, other))
    assert rel_err(want2, want) > 1e-4
    got = run_in_portions(eng, "x", toks, [64, 3, 200, 2] + [1] * 131)[-1]
    got2 = run_in_portions(eng, "y", other, [400])[-1]
    assert rel_err(got, want) < 1e-4 and rel_err(got2, want2) < 1e-4
    assert rel_err(got2 - got, want2 - want) < 0.1       # the far token's own contribution


def test_greedy_generation_through_the_scheduler():
    cfg = config_b()
    eng = make_engine(cfg, torch.float32, pages=16, rows=3, slots=3, step_tokens=48)
    prompts = [tokens_for(cfg, n, 20 + n) for n in (5, 70, 31, 2)]     # more requests than slots, prompts cut by the budget
    out = eng.generate([" ".join(map(str, p)) for p in prompts], max_tokens=12, temperature=0.0)
    assert len(out) == len(prompts)
    weights = {name: eng.model.get(name) for name in eng.model.names()}
    for p in prompts:
        ids = [int(t) for t in out[" ".join(map(str, p))].split()]
        assert ids[:len(p)] == list(p) and len(ids) == len(p) + 12
        # every generated token is the restatement's pick for the tokens before it (the sampler reads
        # bf16 logits: a runner-up within one bf16 step of the best may win a tie)
        logits = ref.forward(cfg.to_json(), weights, ids[:-1])
        for i in range(len(p) - 1, len(ids) - 1):
            best = logits[i].max().item()
            assert logits[i, ids[i + 1]].item() >= best - 2.0 ** -7 * abs(best) - 1e-3, (len(p), i)
    st = eng.cache_manager.stats
    assert st["free"] == st["total"] and st["slots_free"] == 3


def test_checkpoint_directory_and_trace_replay(tmp_path):
    """config.json + model.safetensors -> registry -> engine; the trace runner replays steps on it."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    from safetensors.torch import save_file
    from micro_vllm_amd.models.solopel import random_weights
    cfg = config_a()
    weights = random_weights(cfg, 3)
    os.makedirs(tmp_path / "m")
    save_file(weights, str(tmp_path / "m" / "model.safetensors"))
    (tmp_path / "m" / "config.json").write_text(json.dumps(cfg.to_json()))
    toks = tokens_for(cfg, 90, 14)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": toks[:50], "want": [0, 49]}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": toks[50:52], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "q", "tokens": toks[52:], "want": [37]}, {"id": "r", "tokens": toks[:3], "want": [2]}],
              "end": ["q", "r"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dtype, tol in (("float32", 1e-4), ("bfloat16", 0.1)):
        out = tmp_path / ("o" + dtype)
        p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(tmp_path / "m"), "--dtype",
                            dtype, "--out", str(out), "--max-tokens", "192"],
                           input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
        want = ref.forward(cfg.to_json(), weights, toks)
        s0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1))
        s2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1))
        assert not os.path.exists(out / "1.f32")
        assert rel_err(s0, want[[0, 49]]) < tol and rel_err(s2, torch.stack([want[89], want[2]])) < tol
