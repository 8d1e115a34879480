"""Host-side parts of the Solopel design (no GPU): configuration reader, the looped span's plan of layer runs, tensor
table, registry and checkpoint loading, cache layout, and the plain restatement's own consistency (the convolution's
zero past, the two-map attention against one softmax, a soft cap that saturates, the router's unnormalised sigmoid
weights on the expert's input, the loop's input projection)."""
import json
import math
import os

import pytest
import torch

from oracle import ref_solopel as ref
from solopel_util import config_a, config_b, config_c, random_config


def test_config_reader_run_plan_and_tensor_table(mv):
    from micro_vllm_amd.models.solopel import SolopelConfig, tensor_shapes
    cfg = config_a()
    again = SolopelConfig.from_json(json.loads(json.dumps(cfg.to_json())))
    assert (again.vocab_size, again.width, again.eps, again.taps, again.logit_scale) == (331, 176, 1e-5, 3, 0.7)
    assert again.runs == [0, 1, 2, 3, 1, 2, 3, 1, 2, 3, 4] and again.num_hidden_layers == 11
    # the run that opens each pass of the looped span carries the pass's number
    assert [t for _, t in again.run_plan()] == [-1, 0, -1, -1, 1, -1, -1, 2, -1, -1, -1]
    assert [t for _, t in config_c().run_plan()] == [0, -1] and [t for _, t in config_b().run_plan()] == [-1, -1, -1]
    shapes = tensor_shapes(again)
    assert shapes["embed"] == (331, 176) and "head" not in shapes and shapes["final.norm"] == (176,)
    assert shapes["loop.in"] == (176, 352) and shapes["loop.step"] == (3, 176)
    assert shapes["l0.canon1"] == (176, 3) and shapes["l0.rg1"] == (176, 176) and shapes["l0.rg2.b"] == (176,)
    assert shapes["l0.mix.q"] == (6 * 2 * 24, 176) and shapes["l0.mix.k"] == (2 * 2 * 24, 176) and shapes["l0.mix.v"] == (80, 176)
    assert shapes["l0.mix.q.conv"] == (288, 3) and shapes["l0.mix.v.conv"] == (80, 3) and shapes["l0.mix.g"] == (6, 176)
    assert shapes["l0.mix.lq1"] == (24,) and shapes["l0.mix.o"] == (176, 240)
    assert shapes["l1.mix.q"] == (120, 176) and shapes["l1.mix.dkv"] == (72, 176) and shapes["l1.mix.dkv.norm"] == (72,)
    assert shapes["l1.mix.uk"] == (120, 72) and shapes["l1.mix.uv"] == (72, 72) and shapes["l1.mix.o"] == (176, 72)
    assert shapes["l1.mlp.router"] == (5, 176) and shapes["l1.mlp.e4.down"] == (176, 48) and shapes["l1.mlp.shared.up"] == (56, 176)
    assert "l2.mlp.shared.up" not in shapes and shapes["l2.mlp.e6.gate"] == (40, 176)
    assert "l3.norm2" not in shapes and "l3.rg2" not in shapes and "l3.mlp.up" not in shapes
    assert shapes["l4.mlp.up"] == (100, 176) and "l4.mlp.gate" not in shapes
    b = tensor_shapes(config_b())
    assert "loop.in" not in b and "l0.mix.q.conv" not in b and b["l2.mix.k.conv"] == (64, 1) and b["l0.canon1"] == (128, 1)
    assert "l0.canon1" not in tensor_shapes(config_c())
    for spoil in (lambda d: d["layers"][0].update(type="conv"), lambda d: d["layers"][0]["mlp"].update(kind="glu"),
                  lambda d: d["layers"][0]["mixer"].update(kv_heads=4), lambda d: d["loop"].update(stop=9),
                  lambda d: d["loop"].update(times=0), lambda d: d["loop"].update(start=4, stop=3)):
        bad = json.loads(json.dumps(cfg.to_json()))
        spoil(bad)
        with pytest.raises(ValueError):
            SolopelConfig.from_json(bad)
    empty = json.loads(json.dumps(cfg.to_json()))
    empty["loop"].update(start=2, stop=2)                       # an empty span: no pass, no loop tensors
    e = SolopelConfig.from_json(empty)
    assert e.runs == [0, 1, 2, 3, 4] and "loop.in" not in tensor_shapes(e)
    for seed in range(20):
        c = random_config(seed)
        assert SolopelConfig.from_json(json.loads(json.dumps(c.to_json()))).to_json() == c.to_json()


def test_registry_loads_a_checkpoint_directory(mv, tmp_path):
    from safetensors.torch import save_file
    from micro_vllm_amd.core.model_loader import load_model
    from micro_vllm_amd.models.solopel import random_weights
    cfg = config_a()
    w = random_weights(cfg, 1)
    save_file(w, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_json()))
    model, tok = load_model(str(tmp_path))
    assert model.family == "ragged" and model.config.architecture == "Solopel" and model.config.width == 176
    assert torch.equal(model.get("l0.mix.lq1"), w["l0.mix.lq1"]) and model.get("loop.step").dtype == torch.bfloat16
    assert tok.encode("3 17 330") == [3, 17, 330]
    os.remove(tmp_path / "model.safetensors")
    del w["l2.rg2.b"]
    save_file(w, str(tmp_path / "model.safetensors"))
    with pytest.raises(KeyError):
        load_model(str(tmp_path))


def test_cache_layout_gives_every_layer_run_its_own_pages_and_tails(mv):
    """A pass of the looped span has pages and convolution tails of its own; a latent layer keeps one vector per
    token that serves as key and value, a differential layer both maps' keys side by side."""
    from micro_vllm_amd.core.layer.ragged_runner import RaggedRunner
    cfg = config_a()
    runner = RaggedRunner.__new__(RaggedRunner)
    runner.cfg, runner.width, runner.runs = cfg, cfg.width, cfg.layer_runs()
    kv, state = runner.cache_layout()
    assert sorted(kv) == list(range(11)) and sorted(state) == list(range(11))
    assert kv[0] == (2, 48, 40) and kv[1] == kv[4] == kv[7] == (1, 72, 0) and kv[2] == kv[5] == (1, 32, 72)
    assert kv[3] == (1, 130, 0) and kv[10] == (1, 33, 0)
    assert all(s["canon"] == (2, 176) for s in state.values())
    assert state[0]["qkv"] == (2, 288 + 96 + 80) and state[2]["qkv"] == (4, 128 + 32 + 72) and "qkv" not in state[1]
    cfg = config_b()
    runner.cfg, runner.width, runner.runs = cfg, cfg.width, cfg.layer_runs()
    kv, state = runner.cache_layout()
    assert state[0] == {"canon": (0, 128)} and "qkv" not in state[2]       # one tap: nothing is carried
    cfg = config_c()
    runner.cfg, runner.width, runner.runs = cfg, cfg.width, cfg.layer_runs()
    assert runner.cache_layout()[1] == {0: {"qkv": (3, 256 + 128 + 128)}, 1: {}}


def test_restatement_convolution_and_attention():
    g = torch.Generator().manual_seed(0)
    u, w = torch.randn(9, 5, generator=g, dtype=torch.float64), torch.randn(5, 4, generator=g, dtype=torch.float64)
    y = ref.causal_conv(u, w)
    assert torch.allclose(y[0], w[:, 3] * u[0]) and torch.allclose(y[2], w[:, 3] * u[2] + w[:, 2] * u[1] + w[:, 1] * u[0])
    assert torch.allclose(ref.causal_conv(u, w)[:6], ref.causal_conv(u[:6], w))            # causal
    # lambda = 0 and no cap: the first map alone, an ordinary softmax attention, unit-normed
    T, H, G, d, dv = 7, 4, 2, 6, 5
    q, k = torch.randn(T, H, 2, d, generator=g, dtype=torch.float64), torch.randn(T, G, 2, d, generator=g, dtype=torch.float64)
    v = torch.randn(T, G, dv, generator=g, dtype=torch.float64)
    out = ref.difference_attention(q, k, v, None, 0.4, 0.0, 0.0, 0.0, 0.0)
    for h in range(H):
        s = (k[:, h // 2, 0] @ q[-1, h, 0]) * 0.4
        a = torch.softmax(s, 0) @ v[:, h // 2]
        assert torch.allclose(out[-1, h], a / a.pow(2).mean().sqrt())
    # equal maps and lambda = 1 cancel: only eps is left under the root
    q[:, :, 1], k[:, :, 1] = q[:, :, 0], k[:, :, 0]
    assert ref.difference_attention(q, k, v, None, 0.4, 0.0, 1.0, 0.2, 1e-6).abs().max().item() < 1e-9
    # a saturated cap: all visible keys weigh the same
    out = ref.difference_attention(q * 1e4, k.abs() + 1, v, None, 1.0, 1e-3, 0.0, 0.0, 0.0)
    q_pos = (q[:, :, 0] * 1e4)
    for h in range(H):
        signs = torch.sign(k[:, h // 2, 0].abs().add(1) @ q_pos[-1, h])
        if bool((signs > 0).all()):
            a = v[:, h // 2].mean(0)
            assert torch.allclose(out[-1, h], a / a.pow(2).mean().sqrt(), atol=1e-6)
    W = {"lq1": torch.full((3,), 0.5, dtype=torch.float64), "lk1": torch.full((3,), 2.0, dtype=torch.float64),
         "lq2": torch.zeros(3, dtype=torch.float64), "lk2": torch.ones(3, dtype=torch.float64)}
    assert abs(ref.difference_lambda(W, "", 0.25) - (math.exp(3.0) - 1.0 + 0.25)) < 1e-12


def test_restatement_router_and_loop():
    g = torch.Generator().manual_seed(1)
    n, ff, E = 6, 4, 3
    W = {"router": torch.tensor([[9.0] + [0.0] * 5, [0.0, 9.0] + [0.0] * 4, [0.0] * 6], dtype=torch.float64)}
    for e in range(E):
        for name, shape in (("gate", (ff, n)), ("up", (ff, n)), ("down", (n, ff))):
            W[f"e{e}.{name}"] = torch.randn(shape, generator=g, dtype=torch.float64)
    h = torch.zeros(2, n, dtype=torch.float64)
    h[0, 0], h[0, 1], h[1, 1] = 0.3, 0.2, -0.5                  # token 0: experts 0, 1; token 1: experts 0 and 2 tie at 0 -> 0
    out = ref.routed_ff(h, W, "", {"router": {"experts": E, "top": 2}})
    s = torch.sigmoid(h @ W["router"].T)
    want0 = ref.silu_expert((s[0, 0] * h[0])[None], W, "e0.")[0] + ref.silu_expert((s[0, 1] * h[0])[None], W, "e1.")[0]
    want1 = ref.silu_expert((0.5 * h[1])[None], W, "e0.")[0] + ref.silu_expert((0.5 * h[1])[None], W, "e2.")[0]
    assert torch.allclose(out[0], want0) and torch.allclose(out[1], want1)
    assert abs(float(s[0, 0] + s[0, 1]) - 1.0) > 0.3           # the weights are not renormalised
    # the stack: a looped span of one layer twice equals the two passes written out by hand
    from micro_vllm_amd.models.solopel import random_weights
    cfg = config_c()
    cfg.loop = {"start": 1, "stop": 2, "times": 2}
    Wt = {k: v.double() for k, v in random_weights(cfg, 2).items()}
    toks = [5, 9, 1, 0, 7]
    res = []
    logits = ref.forward(cfg.to_json(), Wt, toks, residuals=res)
    assert len(res) == 3
    x0 = Wt["embed"][toks]
    x = ref.layer_forward(x0, Wt, 0, cfg.layers[0], cfg.eps)
    assert torch.allclose(res[0], x)
    for t in range(2):
        x = torch.cat([x, x0], -1) @ Wt["loop.in"].T + Wt["loop.step"][t]
        x = ref.layer_forward(x, Wt, 1, cfg.layers[1], cfg.eps)
        assert torch.allclose(res[1 + t], x)
    assert torch.allclose(logits, ref.offset_norm(x, Wt["final.norm"], cfg.eps) @ Wt["embed"].T * 2.0)
    # a prefix's logits do not depend on what follows
    assert torch.allclose(ref.forward(cfg.to_json(), Wt, toks[:3]), logits[:3])
