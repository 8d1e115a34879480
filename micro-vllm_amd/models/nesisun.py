"""Nesisun: a decoder-only stack of PARALLEL layers listed one by one in config.json.

  embedding     embed[token] * scale plus a row of a hashed table chosen by (previous token, token):
                row (prev * mul_prev + token * mul_cur) mod buckets, the table's extra last row for a
                sequence's first token.  The previous token is part of what a sequence carries between steps.
  layer         x += mixer(n(x)) + ff(n(x)): ONE RMS norm (plain weight) whose output both sublayers read
  mixer         'attention': grouped-query softmax attention whose VALUES ARE THE KEYS before rotation (no value
                projection), biases on the query and key projections, rotation of adjacent pairs over the first
                rot.dims dimensions of a head, a sliding window that also keeps the sequence's first
                mask.keep_first positions, and a learned per-head sink that enters the softmax's denominator
                without a key or a value
  feed-forward  'dense': down(gelu_tanh(gate h) * (up h)); 'moe': clamped experts
                (g = min(gate h, limit), u = clamp(up h, +-limit), down(g sigmoid(1.702 g) (u + 1))) chosen by a
                softmax router with a selection-only correction per expert, weights renormalised over the chosen
                and scaled; the router's last `identity` outputs stand for experts that pass h through; or none
  weights_of    a layer may use an earlier layer's tensors with a cache of its own
The residual stream is fp32.

This module holds the configuration (every size and constant is read from config.json), the tensor names and a
random-weight builder for tests and benchmarks.  The compute path is core/layer/ragged_runner.py.
"""
import math
from dataclasses import dataclass, field
from typing import Dict, List

import torch

from .pagazen import PagazenModel

MIXERS = ("attention",)
FEED_FORWARDS = ("dense", "moe")
GATE_SLOPE = 1.702          # the experts' gate is g * sigmoid(GATE_SLOPE * g)
WEIGHT_SUM_FLOOR = 1e-20    # added to the sum the chosen experts' scores are divided by


@dataclass
class NesisunConfig:
    vocab_size: int
    width: int
    layers: List[dict]
    embed_scale: float = 1.0
    pair_buckets: int = 1
    pair_mul_prev: int = 1
    pair_mul_cur: int = 1
    eps: float = 1e-6
    name: str = "nesisun"
    architecture: str = "Nesisun"
    family: str = "ragged"
    raw: dict = field(default_factory=dict, repr=False)

    @property
    def hidden_size(self):
        return self.width

    @property
    def num_hidden_layers(self):
        return len(self.layers)

    @property
    def max_position_embeddings(self):
        return 1 << 20

    def weights_layer(self, i: int) -> int:
        """The layer whose tensors layer run i uses."""
        j = self.layers[i].get("weights_of")
        return i if j is None else int(j)

    def layer_runs(self):
        """[(index of the layer whose tensors the run uses, its description)] in running order."""
        return [(self.weights_layer(i), layer) for i, layer in enumerate(self.layers)]

    @classmethod
    def from_json(cls, d: dict, name: str = "nesisun") -> "NesisunConfig":
        layers = d["layers"]
        for i, layer in enumerate(layers):
            if layer["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
            m = layer["mixer"]
            H, G, dim, vdim = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
            if G <= 0 or H % G:
                raise ValueError(f"layer {i}: {H} query heads do not divide over {G} key/value heads")
            if vdim != dim:
                raise ValueError(f"layer {i}: the values are the keys, so vdim {vdim} must equal dim {dim}")
            rot = int(m["rot"]["dims"])
            if rot % 2 or not 0 <= rot <= dim:
                raise ValueError(f"layer {i}: rotation over {rot} of {dim} dimensions")
            if int(m["mask"]["size"]) < 1 or int(m["mask"].get("keep_first", 0)) < 0:
                raise ValueError(f"layer {i}: mask {m['mask']!r}")
            mlp = layer.get("mlp")
            if mlp is not None:
                if mlp.get("kind") not in FEED_FORWARDS:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                if mlp["kind"] == "moe":
                    r = mlp["router"]
                    if not 1 <= int(r["top"]) <= int(r["experts"]) + int(r.get("identity", 0)):
                        raise ValueError(f"layer {i}: top {r['top']} of {r['experts']} + {r.get('identity', 0)} experts")
            j = layer.get("weights_of")
            if j is not None and not (0 <= int(j) < len(layers) and layers[int(j)].get("weights_of") is None):
                raise ValueError(f"layer {i}: weights_of {j!r} does not name a layer with tensors of its own")
        emb = d.get("embedding", {})
        pair = emb["bigram"]
        return cls(vocab_size=int(d["vocab"]), width=int(d["width"]), layers=layers,
                   embed_scale=float(emb.get("scale", 1.0)), pair_buckets=int(pair["buckets"]),
                   pair_mul_prev=int(pair["mul_prev"]), pair_mul_cur=int(pair["mul_cur"]),
                   eps=float(d["norm"]["eps"]), name=name, raw=d)

    def to_json(self) -> dict:
        return {"architecture": self.architecture,
                "embedding": {"scale": self.embed_scale,
                              "bigram": {"buckets": self.pair_buckets, "mul_prev": self.pair_mul_prev,
                                         "mul_cur": self.pair_mul_cur}},
                "layers": self.layers, "norm": {"eps": self.eps}, "vocab": self.vocab_size, "width": self.width}


def tensor_shapes(cfg: NesisunConfig) -> Dict[str, tuple]:
    """Name -> shape of every tensor a checkpoint of this configuration holds."""
    W = cfg.width
    out = {"embed": (cfg.vocab_size, W), "bigram": (cfg.pair_buckets + 1, W), "final.norm": (W,),
           "head": (cfg.vocab_size, W)}
    for i, layer in enumerate(cfg.layers):
        if layer.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", layer["mixer"]
        H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        out.update({p + "norm1": (W,), p + "mix.q": (H * d, W), p + "mix.q.b": (H * d,), p + "mix.k": (G * d, W),
                    p + "mix.k.b": (G * d,), p + "mix.sink": (H,), p + "mix.o": (W, H * dv)})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        if mlp["kind"] == "dense":
            ff = int(mlp["ff"])
            out.update({p + "mlp.gate": (ff, W), p + "mlp.up": (ff, W), p + "mlp.down": (W, ff)})
        else:
            ff, r = int(mlp["expert"]["ff"]), mlp["router"]
            E, n_id = int(r["experts"]), int(r.get("identity", 0))
            for e in range(E):
                out.update({p + f"mlp.e{e}.gate": (ff, W), p + f"mlp.e{e}.up": (ff, W), p + f"mlp.e{e}.down": (W, ff)})
            out.update({p + "mlp.router": (E + n_id, W), p + "mlp.correction": (E + n_id,)})
    return out


class NesisunModel(PagazenModel):
    """Configuration plus a name -> tensor source (`get(name)`): a checkpoint's files or a dict."""


def random_weights(cfg: NesisunConfig, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors of the right shapes and sensible ranges (projections ~ 1/sqrt(fan-in), norm weights near
    one, sinks and biases of order one, router logits spread enough that the choice is no close call)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name in ("embed", "bigram"):
            t = torch.randn(shape, generator=g) / max(cfg.embed_scale, 1.0)
        elif name.endswith("mlp.router"):
            t = torch.randn(shape, generator=g) * 4.0 / math.sqrt(shape[1])
        elif name.endswith("mlp.correction"):
            t = torch.randn(shape, generator=g) * 0.05
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name.endswith(".sink"):
            t = torch.randn(shape, generator=g)
        elif name.endswith(".b"):
            t = torch.randn(shape, generator=g) * 0.3
        else:
            t = 1.0 + torch.randn(shape, generator=g) * 0.1
        out[name] = t.to(dtype)
    return out


def build_random_model(cfg: NesisunConfig, seed: int = 0) -> NesisunModel:
    return NesisunModel(cfg, random_weights(cfg, seed))


def bench_config(width: int, n_layers: int, vocab: int = 32000, ff_mult: int = 4, window: int = 1024,
                 keep_first: int = 64, experts: int = 8, top: int = 2, moe_every: int = 2) -> NesisunConfig:
    """A configuration with the proportions of a served model: 128-wide heads, one key/value head per four query
    heads, every `moe_every`-th layer routed (active feed-forward width ff_mult * width; 0: none), the others dense."""
    heads = max(1, width // 128)
    mixer = {"heads": heads, "kv_heads": max(1, heads // 4), "dim": 128, "vdim": 128,
             "mask": {"size": window, "keep_first": keep_first}, "rot": {"base": 10000.0, "dims": 128},
             "scale": 128 ** -0.5}
    eff = (ff_mult * width // top + 63) // 64 * 64
    moe = {"kind": "moe", "expert": {"ff": eff, "limit": 7.0},
           "router": {"experts": experts, "identity": 1, "top": top, "scale": 1.0}}
    dense = {"kind": "dense", "ff": ff_mult * width}
    layers = [{"type": "attention", "mixer": mixer, "mlp": moe if moe_every and i % moe_every == moe_every - 1 else dense}
              for i in range(n_layers)]
    return NesisunConfig(vocab_size=vocab, width=width, layers=layers, embed_scale=1.0, pair_buckets=65521,
                         pair_mul_prev=1000003, pair_mul_cur=31, eps=1e-5, name=f"nesisun-w{width}-l{n_layers}")
