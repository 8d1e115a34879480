"""Solopel: a decoder-only stack whose layers are listed one by one in config.json, with a span of them that may
run several times in a row on the same weights (`loop`), each pass with a cache and state of its own.

  embedding     a table row as it is; the same table is the output head, the logits times `logit_scale`
  loop          every pass starts from  W_in [x ; x0] + step_t  (x0 = the embedding, t = number of the pass)
  layer         pre-norm with gated residuals:  x += mixer(n + conv(n)) * sigmoid(R1 n + b1),  n = norm1(x);
                x += ff(n2) * sigmoid(R2 n2 + b2),  n2 = norm2(x).  The norm is an RMS norm with weight 1 + w; conv is
                a short causal convolution per channel over time in front of the mixer only (its last taps - 1 inputs
                are part of a sequence's state in every layer run)
  mixers        'latent_attention'   causal softmax attention without positions whose keys and values are expanded
                                     per head from ONE normed latent per token; only the latent is cached
                'attention'          differential attention: two softmax maps per head over the same values (grouped
                                     key/value heads, short convolutions behind the q, k and v projections, scores
                                     soft-capped), o = a1 - lambda a2, unit-RMS per head times (1 - diff), a sigmoid
                                     gate of one number per head
  feed-forward  dense GELU (tanh form); or routed SiLU-gated experts chosen by the largest sigmoid scores, the score
                scaling the expert's INPUT, plus a shared expert; or none
The residual stream is fp32.

This module holds the configuration (every size and constant is read from config.json), the tensor names and a
random-weight builder for tests and benchmarks.  The compute path is core/layer/ragged_runner.py.
"""
import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

from .pagazen import PagazenModel

MIXERS = ("latent_attention", "attention")


@dataclass
class SolopelConfig:
    vocab_size: int
    width: int
    layers: List[dict]
    eps: float = 1e-6
    taps: int = 0                        # taps of the convolution in front of every mixer (0: there is none)
    logit_scale: float = 1.0
    loop: Optional[dict] = None          # {"start", "stop", "times"}
    name: str = "solopel"
    architecture: str = "Solopel"
    family: str = "ragged"
    raw: dict = field(default_factory=dict, repr=False)

    @property
    def hidden_size(self):
        return self.width

    @property
    def num_hidden_layers(self):
        return len(self.runs)

    @property
    def max_position_embeddings(self):
        return 1 << 20

    @property
    def runs(self) -> List[int]:
        """The layer each layer RUN takes its tensors from, in running order."""
        return [i for i, _ in self.run_plan()]

    def run_plan(self):
        """[(layer, number of the loop pass that STARTS with this run, or -1)] in running order."""
        n = len(self.layers)
        if not self.looped:
            return [(i, -1) for i in range(n)]
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        plan = [(i, -1) for i in range(a)]
        for t in range(times):
            plan += [(i, t if i == a else -1) for i in range(a, b)]
        return plan + [(i, -1) for i in range(b, n)]

    @property
    def looped(self) -> bool:
        """Whether a span of at least one layer is looped (an empty span has no pass and needs no tensors)."""
        return bool(self.loop) and int(self.loop["start"]) < int(self.loop["stop"])

    def layer_runs(self):
        """[(index of the layer whose tensors the run uses, its description)] in running order."""
        return [(i, self.layers[i]) for i in self.runs]

    @classmethod
    def from_json(cls, d: dict, name: str = "solopel") -> "SolopelConfig":
        layers = d["layers"]
        for i, layer in enumerate(layers):
            if layer["type"] not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer type {layer['type']!r}")
            mlp = layer.get("mlp")
            if mlp is not None and mlp.get("kind") not in ("dense", "moe"):
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            m = layer["mixer"]
            if layer["type"] == "attention" and int(m["heads"]) % int(m["kv_heads"]):
                raise ValueError(f"layer {i}: {m['heads']} query heads over {m['kv_heads']} key/value heads")
        loop = d.get("loop")
        if loop:
            a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
            if not (0 <= a <= b <= len(layers)) or times < 1:
                raise ValueError(f"loop {loop!r} does not fit {len(layers)} layers")
        canon = d.get("canon")
        return cls(vocab_size=int(d["vocab"]), width=int(d["width"]), layers=layers, eps=float(d["norm"]["eps"]),
                   taps=int(canon["taps"]) if canon else 0, logit_scale=float(d.get("logit_scale", 1.0)), loop=loop,
                   name=name, raw=d)

    def to_json(self) -> dict:
        d = {"architecture": self.architecture, "layers": self.layers, "norm": {"eps": self.eps},
             "logit_scale": self.logit_scale, "vocab": self.vocab_size, "width": self.width}
        if self.taps:
            d["canon"] = {"taps": self.taps}
        if self.loop:
            d["loop"] = self.loop
        return d


def expert_shapes(prefix: str, ff: int, W: int) -> Dict[str, tuple]:
    return {prefix + "gate": (ff, W), prefix + "up": (ff, W), prefix + "down": (W, ff)}


def tensor_shapes(cfg: SolopelConfig) -> Dict[str, tuple]:
    """Name -> shape of every tensor a checkpoint of this configuration holds."""
    W = cfg.width
    out = {"embed": (cfg.vocab_size, W), "final.norm": (W,)}
    if cfg.looped:
        out.update({"loop.in": (W, 2 * W), "loop.step": (int(cfg.loop["times"]), W)})
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}.", layer["mixer"]
        H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
        out.update({p + "norm1": (W,), p + "rg1": (W, W), p + "rg1.b": (W,)})
        if cfg.taps:
            out[p + "canon1"] = (W, cfg.taps)
        if layer["type"] == "latent_attention":
            R = int(m["kv_rank"])
            out.update({p + "mix.q": (H * d, W), p + "mix.dkv": (R, W), p + "mix.dkv.norm": (R,),
                        p + "mix.uk": (H * d, R), p + "mix.uv": (H * dv, R), p + "mix.o": (W, H * dv)})
        else:
            G, taps = int(m["kv_heads"]), int(m.get("conv") or 0)
            out.update({p + "mix.q": (H * 2 * d, W), p + "mix.k": (G * 2 * d, W), p + "mix.v": (G * dv, W),
                        p + "mix.lq1": (d,), p + "mix.lk1": (d,), p + "mix.lq2": (d,), p + "mix.lk2": (d,),
                        p + "mix.g": (H, W), p + "mix.o": (W, H * dv)})
            if taps:
                out.update({p + "mix.q.conv": (H * 2 * d, taps), p + "mix.k.conv": (G * 2 * d, taps),
                            p + "mix.v.conv": (G * dv, taps)})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        out.update({p + "norm2": (W,), p + "rg2": (W, W), p + "rg2.b": (W,)})
        if mlp["kind"] == "dense":
            ff = int(mlp["ff"])
            out.update({p + "mlp.up": (ff, W), p + "mlp.down": (W, ff)})
        else:
            ff, E = int(mlp["expert"]["ff"]), int(mlp["router"]["experts"])
            out[p + "mlp.router"] = (E, W)
            for e in range(E):
                out.update(expert_shapes(p + f"mlp.e{e}.", ff, W))
            if mlp.get("shared"):
                out.update(expert_shapes(p + "mlp.shared.", int(mlp["shared"]["ff"]), W))
    return out


class SolopelModel(PagazenModel):
    """Configuration plus a name -> tensor source (`get(name)`): a checkpoint's files or a dict."""


def random_weights(cfg: SolopelConfig, seed: int = 0, dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    """Random tensors of the right shapes and sensible ranges (projections ~ 1/sqrt(fan-in), norm weights near zero -
    they are offsets from one -, convolution taps and biases of order one half, router logits spread enough that the
    choice of experts is no close call)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name == "embed":
            t = torch.randn(shape, generator=g)
        elif name == "loop.step":
            t = torch.randn(shape, generator=g) * 0.3
        elif name.endswith(".conv") or name.endswith("canon1"):
            t = torch.randn(shape, generator=g) * 0.5
        elif name.endswith("mlp.router"):
            t = torch.randn(shape, generator=g) * 4.0 / math.sqrt(shape[1])
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif name.endswith(".b"):
            t = torch.randn(shape, generator=g) * 0.5
        elif ".mix.l" in name:
            t = torch.randn(shape, generator=g) * 0.3
        else:
            t = torch.randn(shape, generator=g) * 0.1
        out[name] = t.to(dtype)
    return out


def build_random_model(cfg: SolopelConfig, seed: int = 0) -> SolopelModel:
    return SolopelModel(cfg, random_weights(cfg, seed))


def bench_config(width: int, n_layers: int, vocab: int = 32000, ff_mult: int = 4, every: int = 4, experts: int = 8,
                 top: int = 2, moe_every: int = 2, loop_times: int = 1) -> SolopelConfig:
    """A configuration with the proportions of a served model: 128-wide heads; every `every`-th layer a differential
    attention (one key/value head per four query heads, half-width maps so that a head's two maps cost what one
    128-wide map would), the others latent attention over a 512-wide latent; every `moe_every`-th layer routed
    (active feed-forward width ff_mult * width over top experts + a shared one; 0: none), the others dense."""
    heads = max(1, width // 128)
    eff = (ff_mult * width // (top + 1) + 63) // 64 * 64
    moe = {"kind": "moe", "expert": {"ff": eff}, "router": {"experts": experts, "top": top}, "shared": {"ff": eff}}
    dense = {"kind": "dense", "ff": ff_mult * width}
    layers = []
    for i in range(n_layers):
        mlp = moe if moe_every and i % moe_every == moe_every - 1 else dense
        if i % every == every - 1:
            mixer = {"heads": heads, "kv_heads": max(1, heads // 4), "dim": 64, "vdim": 128, "conv": 4, "diff": 0.2,
                     "scale": 64 ** -0.5, "softcap": 30.0}
            layers.append({"type": "attention", "mixer": mixer, "mlp": mlp})
        else:
            mixer = {"heads": heads, "dim": 128, "vdim": 128, "kv_rank": 512, "scale": 128 ** -0.5}
            layers.append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
    loop = {"start": 0, "stop": n_layers, "times": loop_times} if loop_times else None
    return SolopelConfig(vocab_size=vocab, width=width, layers=layers, eps=1e-6, taps=4, logit_scale=1.0, loop=loop,
                         name=f"solopel-w{width}-l{n_layers}")
