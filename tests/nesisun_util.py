"""Small Nesisun configurations for the tests (none with the proportions of a real checkpoint) and an engine
builder; the helpers that feed a request in portions are those of ragged_util."""
import torch

from micro_vllm_amd.models.nesisun import NesisunConfig, build_random_model


def attention(heads=6, kv_heads=2, dim=40, rot=24, base=5000.0, window=37, keep=5, scale=0.2):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": window, "keep_first": keep},
            "rot": {"base": base, "dims": rot}, "scale": scale}


def dense(ff=150):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, identity=2, top=3, ff=48, limit=1.2, scale=1.7):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "identity": identity, "top": top, "scale": scale}}


def layer(mixer, mlp, weights_of=None):
    d = {"type": "attention", "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def config_a():
    """Odd sizes everywhere, every layer its own attention shape: rotation over a part of the head, a window cut
    inside a page, a few kept positions, a layer without feed-forward, two layers on borrowed weights."""
    a0, a1 = attention(), attention(heads=4, kv_heads=1, dim=24, rot=8, base=300.0, window=70, keep=66, scale=0.3)
    return NesisunConfig(vocab_size=331, width=176, eps=1e-5, embed_scale=2.5, pair_buckets=97, pair_mul_prev=31,
                         pair_mul_cur=7, layers=[
        layer(a0, dense()),
        layer(a1, moe()),
        layer(attention(heads=3, kv_heads=3, dim=56, rot=56, window=3, keep=1, scale=0.13), None),
        layer(a0, dense(), weights_of=0),
        layer(a1, moe(), weights_of=1),
    ])


def config_b():
    """Values that other configurations keep apart made equal, one or nothing: as many key/value heads as query
    heads, nothing kept behind the window, a window of exactly one page, no rotation in one layer, one expert used,
    no pass-through expert, unit scales, one bucket; widths the wave-tile projections and the matrix-core attention
    take (so the bf16 run uses both)."""
    return NesisunConfig(vocab_size=256, width=128, eps=1e-6, embed_scale=1.0, pair_buckets=1, pair_mul_prev=1,
                         pair_mul_cur=1, layers=[
        layer(attention(heads=2, kv_heads=2, dim=64, rot=64, base=100.0, window=64, keep=0, scale=0.125), dense(128)),
        layer(attention(heads=4, kv_heads=1, dim=32, rot=0, window=200, keep=64, scale=0.25),
              moe(experts=4, identity=0, top=1, ff=64, limit=0.5, scale=1.0)),
        layer(attention(heads=1, kv_heads=1, dim=128, rot=2, window=1, keep=2, scale=0.1),
              moe(experts=1, identity=1, top=2, ff=64, limit=9.0, scale=0.5)),
    ])


def random_config(seed):
    """A configuration drawn at random: layer order, borrowed weights, head counts and widths (among them the shapes
    the matrix-core attention takes and ones it does not), windows from 1 to beyond the prompt, kept positions from
    none to beyond the window, rotation over none / part / all of a head, dense, routed (with and without
    pass-through experts) and absent feed-forwards."""
    import random
    rng = random.Random(seed)
    layers = []
    for i in range(rng.randint(2, 5)):
        own = [k for k in range(i) if "weights_of" not in layers[k]]
        if own and rng.random() < 0.3:
            j = rng.choice(own)
            layers.append(dict(layers[j], weights_of=j))
            continue
        kv = rng.choice([1, 2, 3])
        dim = rng.choice([8, 24, 32, 40, 64, 96, 128])
        mixer = attention(heads=kv * rng.choice([1, 2, 4]), kv_heads=kv, dim=dim,
                          rot=rng.choice([r for r in (0, 2, 8, 16, dim) if r <= dim]), base=rng.choice([100.0, 1e4, 1e6]),
                          window=rng.choice([1, 2, 17, 64, 65, 100, 300]), keep=rng.choice([0, 1, 3, 20, 64, 70, 200]),
                          scale=rng.choice([0.1, dim ** -0.5, 0.5]))
        kind = rng.choice(["dense", "moe", "moe", None])
        if kind == "dense":
            mlp = dense(rng.choice([64, 150, 256]))
        elif kind == "moe":
            E, n_id = rng.choice([1, 2, 4, 9, 20]), rng.choice([0, 1, 3])
            mlp = moe(E, n_id, rng.randint(1, min(E + n_id, 4)), rng.choice([16, 40, 64, 96]), rng.choice([0.7, 2.0, 7.0]),
                      rng.choice([1.0, 2.5]))
        else:
            mlp = None
        layers.append(layer(mixer, mlp))
    return NesisunConfig(vocab_size=rng.choice([97, 256, 331, 1000]), width=rng.choice([48, 100, 192, 256]), layers=layers,
                         embed_scale=rng.choice([1.0, 4.0]), pair_buckets=rng.choice([1, 13, 1009, 100003]),
                         pair_mul_prev=rng.choice([1, 29, 1000003]), pair_mul_cur=rng.choice([0, 1, 31]),
                         eps=rng.choice([1e-5, 1e-6]))


def make_engine(cfg, dtype=torch.float32, seed=0, pages=24, slots=4, rows=4, step_tokens=512, max_tokens=512, model=None):
    from micro_vllm_amd.core.engine import InferenceEngine
    return InferenceEngine(model=model or build_random_model(cfg, seed), max_batch_size=rows,
                           max_prefill_tokens=step_tokens, n_blocks=pages, max_tokens=max_tokens, state_slots=slots,
                           dtype=dtype)
