"""Host-side parts of the Nesisun design (no GPU): configuration reader, tensor table, registry and checkpoint
loading, cache layout, the token before each token in a step's plan, and the plain restatement's own consistency
(what is visible behind a window with kept first positions, the sink, rotation of adjacent pairs, the hashed pair
table, a router whose correction moves the choice but not the weights)."""
import json
import math
import os

import pytest
import torch

from oracle import ref_nesisun as ref
from nesisun_util import config_a, config_b, random_config


def test_config_reader_and_tensor_table(mv):
    from micro_vllm_amd.models.nesisun import NesisunConfig, tensor_shapes
    cfg = config_a()
    again = NesisunConfig.from_json(json.loads(json.dumps(cfg.to_json())))
    assert (again.vocab_size, again.width, again.eps, again.embed_scale) == (331, 176, 1e-5, 2.5)
    assert (again.pair_buckets, again.pair_mul_prev, again.pair_mul_cur) == (97, 31, 7)
    assert [i for i, _ in again.layer_runs()] == [0, 1, 2, 0, 1] and again.num_hidden_layers == 5
    assert [ref.weights_layer(cfg.to_json(), i) for i in range(5)] == [0, 1, 2, 0, 1]
    shapes = tensor_shapes(again)
    assert shapes["bigram"] == (98, 176) and shapes["embed"] == (331, 176) and shapes["final.norm"] == (176,)
    assert shapes["l0.mix.q"] == (6 * 40, 176) and shapes["l0.mix.k"] == (2 * 40, 176) and shapes["l0.mix.k.b"] == (80,)
    assert shapes["l0.mix.sink"] == (6,) and shapes["l0.mix.o"] == (176, 240) and "l0.mix.v" not in shapes
    assert shapes["l0.mlp.gate"] == (150, 176) and shapes["l0.mlp.down"] == (176, 150)
    assert shapes["l1.mlp.router"] == (5 + 2, 176) and shapes["l1.mlp.correction"] == (7,)
    assert shapes["l1.mlp.e4.up"] == (48, 176) and "l1.mlp.e5.up" not in shapes      # pass-through experts have no tensors
    assert "l2.mlp.gate" not in shapes and "l2.mlp.router" not in shapes and "l2.norm2" not in shapes
    assert not any(n.startswith(("l3.", "l4.")) for n in shapes)                    # borrowed weights
    for spoil in (lambda d: d["layers"][0].update(type="conv"), lambda d: d["layers"][0]["mlp"].update(kind="glu"),
                  lambda d: d["layers"][0]["mixer"].update(vdim=48), lambda d: d["layers"][0]["mixer"].update(kv_heads=4),
                  lambda d: d["layers"][0]["mixer"]["rot"].update(dims=42), lambda d: d["layers"][3].update(weights_of=4),
                  lambda d: d["layers"][1]["mlp"]["router"].update(top=8)):
        bad = json.loads(json.dumps(cfg.to_json()))
        spoil(bad)
        with pytest.raises(ValueError):
            NesisunConfig.from_json(bad)
    for seed in range(20):
        c = random_config(seed)
        assert NesisunConfig.from_json(json.loads(json.dumps(c.to_json()))).to_json() == c.to_json()


def test_registry_loads_a_checkpoint_directory(mv, tmp_path):
    from safetensors.torch import save_file
    from micro_vllm_amd.core.model_loader import load_model
    from micro_vllm_amd.models.nesisun import random_weights
    cfg = config_a()
    w = random_weights(cfg, 1)
    save_file(w, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_json()))
    model, tok = load_model(str(tmp_path))
    assert model.family == "ragged" and model.config.architecture == "Nesisun" and model.config.width == 176
    assert torch.equal(model.get("l1.mlp.correction"), w["l1.mlp.correction"]) and model.get("bigram").dtype == torch.bfloat16
    assert tok.encode("3 17 330") == [3, 17, 330]
    os.remove(tmp_path / "model.safetensors")
    del w["l0.mix.sink"]
    save_file(w, str(tmp_path / "model.safetensors"))
    with pytest.raises(KeyError):
        load_model(str(tmp_path))


def test_cache_layout_gives_every_layer_run_its_own_pages(mv):
    """A run on borrowed weights still has pages of its own; a page row holds the rotated key and, as the value, the
    key as projected; nothing is kept in state slots."""
    from micro_vllm_amd.core.layer.ragged_runner import RaggedRunner
    cfg = config_a()
    runner = RaggedRunner.__new__(RaggedRunner)
    runner.cfg, runner.width, runner.runs = cfg, cfg.width, cfg.layer_runs()
    kv, state = runner.cache_layout()
    assert sorted(kv) == [0, 1, 2, 3, 4] and state == {}
    assert kv[0] == kv[3] == (2, 40, 40) and kv[1] == kv[4] == (1, 24, 24) and kv[2] == (3, 56, 56)


def test_step_plan_carries_the_token_before_each_token(mv):
    from micro_vllm_amd.core.state_cache import HybridCacheManager
    c = HybridCacheManager(6, 64, 2, {0: (1, 8, 8)}, {}, dtype=torch.float32, device="cpu", max_tokens=256, max_rows=3,
                           max_step_tokens=300)

    def step(rows):
        c.reserve([(s, len(t)) for s, t in rows])
        st = c.plan(rows)
        c.advance([(s, len(t)) for s, t in rows])
        return st.tok_prev.tolist()

    assert step([("a", [5, 6, 7]), ("b", [9])]) == [-1, 5, 6, -1]
    assert step([("b", [4]), ("a", [8, 2])]) == [9, 7, 8]
    assert step([("a", [3])]) == [2]                       # b pauses for a step
    assert step([("b", [1, 1])]) == [4, 1]
    c.free("a")
    assert step([("c", [11, 12])]) == [-1, 11]             # a's slot and pages, none of its history
    # a plan that is never advanced (the step failed) leaves the sequence where it was
    c.reserve([("b", 1)])
    c.plan([("b", [77])])
    c.reserve([("b", 1)])
    st = c.plan([("b", [78])])
    assert st.tok_prev.tolist() == [1]
    # tokens in rows short enough to stay outside the chunk table (the attention's per-token form serves them)
    c.free("b")
    c.free("c")
    c.reserve([("x", 40), ("y", 3)])
    assert c.plan([("x", [1] * 40), ("y", [2] * 3)]).short_tokens == 3
    c.advance([("x", 40), ("y", 3)])
    c.reserve([("x", 20)])
    assert c.plan([("x", [1] * 20)]).short_tokens == 0


def test_restatement_visibility_sink_and_values():
    assert [j for j in range(10) if ref.visible(9, j, 3, 2)] == [0, 1, 7, 8, 9]
    assert [j for j in range(10) if ref.visible(3, j, 3, 2)] == [0, 1, 2, 3]
    assert [j for j in range(10) if ref.visible(9, j, 3, 0)] == [7, 8, 9]
    assert [j for j in range(10) if ref.visible(9, j, 100, 0)] == list(range(10))
    g = torch.Generator().manual_seed(1)
    q = torch.randn(12, 4, 6, generator=g, dtype=torch.float64)
    k, v = (torch.randn(12, 2, 6, generator=g, dtype=torch.float64) for _ in range(2))
    gone = torch.full((4,), -1e9, dtype=torch.float64)
    full = ref.sink_attention(q, k, v, 0.5, 100, 0, gone)
    assert torch.allclose(full[0], v[0, [0, 0, 1, 1]])                     # the first token sees itself only; head -> kv head
    for i in range(12):
        w = torch.softmax(k[:i + 1, 1] @ q[i, 2] * 0.5, dim=0)
        assert torch.allclose(full[i, 2], w @ v[:i + 1, 1])
    one = ref.sink_attention(q, k, v, 0.5, 1, 0, gone)
    assert torch.allclose(one, v[:, [0, 0, 1, 1]])                         # a window of one token
    kept = ref.sink_attention(q, k, v, 0.5, 1, 12, gone)
    assert torch.allclose(kept, full)                                      # everything kept = causal
    # a sink of s takes exp(s) / (sum + exp(s)) of the weight and gives nothing back
    sink = torch.tensor([0.0, 2.0, -1.0, 5.0], dtype=torch.float64)
    sunk = ref.sink_attention(q, k, v, 0.5, 4, 1, sink)
    plain = ref.sink_attention(q, k, v, 0.5, 4, 1, gone)
    for h in range(4):
        js = [j for j in range(12) if ref.visible(11, j, 4, 1)]
        tot = torch.exp(k[js, h // 2] @ q[11, h] * 0.5).sum()
        assert torch.allclose(sunk[11, h], plain[11, h] * tot / (tot + math.exp(float(sink[h]))))


def test_restatement_rotation_pairs_and_hashed_table():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 3, 12, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 7, 100, 1000])
    y = ref.rotate_adjacent(x, pos, 8, 1e4)
    assert torch.allclose(y[0], x[0]) and torch.allclose(y[..., 8:], x[..., 8:]) and torch.allclose(y.norm(dim=-1), x.norm(dim=-1))
    # the pair (2i, 2i+1) turns by pos * base^(-2i/dims): the first pair by `pos` radians
    assert torch.allclose(y[1, 0, 0], x[1, 0, 0] * math.cos(1.0) - x[1, 0, 1] * math.sin(1.0))
    assert torch.allclose(y[1, 0, 3], x[1, 0, 3] * math.cos(1e4 ** -0.25) + x[1, 0, 2] * math.sin(1e4 ** -0.25))
    a, b = ref.rotate_adjacent(x[:1].expand(5, 3, 12), pos, 8, 1e4), ref.rotate_adjacent(x[1:2].expand(5, 3, 12), pos + 3, 8, 1e4)
    d = (a * b).sum(-1)
    assert torch.allclose(d, d[:1].expand_as(d))                           # scores depend on the distance only
    embed, table = torch.randn(50, 4, generator=g, dtype=torch.float64), torch.randn(12, 4, generator=g, dtype=torch.float64)
    out = ref.pair_embedding([7, 3, 3, 49], embed, table, 2.0, 11, 5, 3)
    assert torch.allclose(out[0], embed[7] * 2 + table[11])
    assert torch.allclose(out[1], embed[3] * 2 + table[(7 * 5 + 3 * 3) % 11]) and torch.allclose(out[3], embed[49] * 2 + table[(3 * 5 + 49 * 3) % 11])


def test_restatement_router_correction_moves_the_choice_only():
    g = torch.Generator().manual_seed(3)
    W_, ff, E, n_id = 16, 8, 3, 2
    W = {"router": torch.randn(E + n_id, W_, generator=g, dtype=torch.float64), "correction": torch.zeros(E + n_id, dtype=torch.float64)}
    for e in range(E):
        W[f"e{e}.gate"], W[f"e{e}.up"] = (torch.randn(ff, W_, generator=g, dtype=torch.float64) for _ in range(2))
        W[f"e{e}.down"] = torch.randn(W_, ff, generator=g, dtype=torch.float64)
    mlp = {"expert": {"ff": ff, "limit": 1.0}, "router": {"experts": E, "identity": n_id, "top": 2, "scale": 3.0}}
    h = torch.randn(6, W_, generator=g, dtype=torch.float64)
    s = torch.softmax(h @ W["router"].T, dim=-1)
    # all the weight on the two pass-through outputs: the layer returns scale * h whatever the scores are
    W["correction"] = torch.tensor([-9.0, -9.0, -9.0, 9.0, 9.0], dtype=torch.float64)
    assert torch.allclose(ref.routed_with_identity(h, W, "", mlp), 3.0 * h)
    # one expert and one pass-through output forced: weights are the scores of those two, renormalised
    W["correction"] = torch.tensor([9.0, -9.0, -9.0, -9.0, 9.0], dtype=torch.float64)
    want = torch.stack([3.0 * (s[t, 0] * ref.clamped_expert(h[t:t + 1], W["e0.gate"], W["e0.up"], W["e0.down"], 1.0)[0]
                               + s[t, 4] * h[t]) / (s[t, 0] + s[t, 4]) for t in range(6)])
    assert torch.allclose(ref.routed_with_identity(h, W, "", mlp), want)
    # the clamp: a gate far above the limit acts as the limit, an `up` far below -limit as -limit
    big = ref.clamped_expert(torch.ones(1, 2, dtype=torch.float64), torch.tensor([[50.0, 50.0]], dtype=torch.float64),
                             torch.tensor([[-50.0, -50.0]], dtype=torch.float64), torch.ones(1, 1, dtype=torch.float64), 2.0)
    assert torch.allclose(big, torch.tensor([[2.0 / (1 + math.exp(-1.702 * 2.0)) * (-2.0 + 1.0)]], dtype=torch.float64))
