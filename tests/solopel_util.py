"""Small Solopel configurations for the tests (none with the proportions of a real checkpoint) and an engine builder;
the helpers that feed a request in portions are those of ragged_util."""
import torch

from micro_vllm_amd.models.solopel import SolopelConfig, build_random_model


def latent(heads=3, dim=40, vdim=24, rank=72, scale=0.2):
    return {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale}


def differential(heads=6, kv_heads=2, dim=24, vdim=40, conv=3, diff=0.4, scale=0.25, softcap=8.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff, "scale": scale}
    if conv:
        m["conv"] = conv
    if softcap:
        m["softcap"] = softcap
    return m


def dense(ff=150):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=48, shared=56):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def config_a():
    """Odd sizes everywhere: a layer before and one after the looped span, three passes, three taps in front of the
    mixers and two or five behind the attention's projections, grouped key/value heads, two experts used, a routed
    layer without a shared expert, a layer without feed-forward, a soft cap that scores do reach."""
    return SolopelConfig(vocab_size=331, width=176, eps=1e-5, taps=3, logit_scale=0.7,
                         loop={"start": 1, "stop": 4, "times": 3}, layers=[
        layer("attention", differential(), dense()),
        layer("latent_attention", latent(), moe()),
        layer("attention", differential(heads=4, kv_heads=1, dim=16, vdim=72, conv=5, diff=0.15, scale=0.6, softcap=3.0),
              moe(experts=7, top=3, ff=40, shared=0)),
        layer("latent_attention", latent(heads=2, dim=56, vdim=56, rank=130, scale=0.13), None),
        layer("latent_attention", latent(heads=5, dim=16, vdim=48, rank=33, scale=0.3), dense(100)),
    ])


def config_b():
    """Values that other configurations keep apart made equal, one or absent: as many key/value heads as query heads,
    one expert used, a single expert, one tap, no convolution behind the projections, no soft cap, no loop, unit logit
    scale; widths the wave-tile projections and the matrix-core attention take (so the bf16 run uses both)."""
    return SolopelConfig(vocab_size=256, width=128, eps=1e-6, taps=1, logit_scale=1.0, loop=None, layers=[
        layer("attention", differential(heads=2, kv_heads=2, dim=64, vdim=64, conv=0, diff=0.25, scale=0.125, softcap=0),
              moe(experts=4, top=1, ff=64, shared=64)),
        layer("latent_attention", latent(heads=2, dim=64, vdim=64, rank=64, scale=0.125), dense(128)),
        layer("attention", differential(heads=4, kv_heads=1, dim=32, vdim=64, conv=1, diff=0.5, scale=0.2, softcap=30.0),
              moe(experts=1, top=1, ff=64, shared=0)),
    ])


def config_c():
    """The whole stack looped once, no convolution in front of the mixers at all, the matrix-core attention's widest
    shape."""
    return SolopelConfig(vocab_size=200, width=128, eps=1e-6, taps=0, logit_scale=2.0,
                         loop={"start": 0, "stop": 2, "times": 1}, layers=[
        layer("attention", differential(heads=2, kv_heads=1, dim=64, vdim=128, conv=4, diff=0.25, scale=0.125, softcap=15.0),
              dense(128)),
        layer("latent_attention", latent(heads=4, dim=32, vdim=32, rank=128, scale=0.18), moe(experts=3, top=3, ff=64, shared=64)),
    ])


def random_config(seed):
    """A configuration drawn at random: layer order, the looped span and its passes, head counts and widths (among
    them the shapes the matrix-core attention and the wave-tile projections take and ones they do not), taps from none
    to 5, with and without soft cap, dense, routed (with and without a shared expert) and absent feed-forwards."""
    import random
    rng = random.Random(seed)
    layers = []
    n = rng.randint(2, 5)
    for i in range(n):
        kind = rng.choice(["dense", "moe", "moe", None])
        if kind == "dense":
            mlp = dense(rng.choice([64, 150, 256]))
        elif kind == "moe":
            E = rng.choice([1, 2, 4, 9, 20])
            mlp = moe(E, rng.randint(1, min(E, 4)), rng.choice([16, 40, 64, 96]), rng.choice([0, 24, 64]))
        else:
            mlp = None
        if rng.random() < 0.5:
            layers.append(layer("latent_attention", latent(rng.choice([1, 2, 4, 5]), rng.choice([8, 24, 32, 64, 128]),
                                                            rng.choice([8, 24, 32, 64, 128]), rng.choice([16, 33, 64, 128, 200]),
                                                            rng.choice([0.1, 0.2, 0.5])), mlp))
        else:
            kv = rng.choice([1, 2, 3])
            dim, vdim = rng.choice([(8, 8), (24, 40), (32, 32), (32, 64), (64, 64), (64, 128), (56, 72), (128, 128), (40, 200)])
            layers.append(layer("attention", differential(kv * rng.choice([1, 2, 4]), kv, dim, vdim, rng.choice([0, 1, 2, 4, 5]),
                                                          rng.choice([0.1, 0.3, 0.8]), rng.choice([0.1, dim ** -0.5, 0.5]),
                                                          rng.choice([0, 2.0, 20.0, 50.0])), mlp))
    loop = None
    if rng.random() < 0.75:
        a = rng.randint(0, n - 1)
        loop = {"start": a, "stop": rng.randint(a + 1, n), "times": rng.randint(1, 3)}
    return SolopelConfig(vocab_size=rng.choice([97, 256, 331, 1000]), width=rng.choice([48, 100, 192, 256]), layers=layers,
                         eps=rng.choice([1e-5, 1e-6]), taps=rng.choice([0, 1, 2, 4, 5]),
                         logit_scale=rng.choice([0.5, 1.0, 3.0]), loop=loop)


def make_engine(cfg, dtype=torch.float32, seed=0, pages=24, slots=4, rows=4, step_tokens=512, max_tokens=512, model=None):
    from micro_vllm_amd.core.engine import InferenceEngine
    return InferenceEngine(model=model or build_random_model(cfg, seed), max_batch_size=rows,
                           max_prefill_tokens=step_tokens, n_blocks=pages, max_tokens=max_tokens, state_slots=slots,
                           dtype=dtype)
