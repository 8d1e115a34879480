"""Step function of the "ragged" model family (models/registry.py): one forward over a step's tokens -
portions of prompts beside single decoded tokens, all rows in one set of launches - reading and
extending what each sequence holds in the HybridCacheManager.  Stands beside ModelPrefillRunner /
ModelGraphRunner, which serve the Llama-shaped family with padded batches.

Precision.  The residual stream, every norm, rotation, softmax, decay, gate of a recurrence and the
recurrent state are fp32.  Projections take their operand in the activation type (bf16, or fp32 when
the runner is built with dtype=float32 - then nothing at all is rounded to 16 bits) and leave fp32
accumulators; cached keys and values are of the activation type.

Per layer (Pagazen):
  mamba2    in-projection -> conv+SiLU over x|B|C (tail kept per slot) -> softplus step / decay ->
            outer-product scan (state per slot) -> SiLU(z) gate, grouped unit-RMS, weight -> out-projection
  parallel  left: fused q|k|v projection -> unit-RMS of q and k per head, k/v into the pages ->
            windowed softmax attention with distance penalty -> out-projection
            right: fused q|k|v|g projection -> rotate q,k (k scaled) -> fixed-decay scan ->
            unit-RMS per head, SiLU(g) gate -> out-projection
  then      x += unit_rms(sublayer output) * (1 + w)  (both mixers of a parallel layer enter one norm)
  mlp       up -> relu^2 -> down -> the same post-norm residual step

Per layer (Fagunex; norms are Dynamic Tanh, before and after each sublayer):
  every mixer reads  act( n + (n_prev - n) * shift ), n = norm1(x): norm and token shift in one launch, the
            last n of a row kept per slot
  hgrn2     fused q|f|v projection -> silu(q), f = lower + (1 - lower) sigmoid(f + b) -> gated scan with
            key 1 - f (state per slot) -> unit-RMS per head, weight -> out-projection
  latent attention (both kinds)  fused [dq|]dkv[|g] projection -> (kind 1: unit-RMS of the query latent ->
            up-projection; kind 2: q in the fused projection) -> latent normed and rotated key part into the
            page, q's rotated part rotated -> per-head product carrying q's unrotated part into the latent
            space -> attention over the cached latents (window / causal, sink or none) -> per-head value
            up-projection -> (sigmoid gate,) cast -> out-projection
  then      x += norm1b(mixer output)
  moe       (norm2 comes out of the launch that adds the mixer) -> router (fp32, top-k, softmax over the chosen,
            shared expert's sigmoid) -> (token, choice) pairs sorted by expert -> gate|up by segment -> SiLU-gate ->
            down by segment; shared expert gate|up -> SiLU-gate -> down; weighted sum, norm2b and the residual sum
            in one launch
  side      gate projection of x -> gelu_tanh * slice of the second embedding -> projection ->
            x += unit-RMS * weight

Per layer (Nesisun; both sublayers of a layer read ONE RMS norm and enter the stream together):
  embedding table row * scale + row of the pair-hashed table (the token before each token comes with the step), and
            the first layer's norm of it, in one launch
  attention ONE projection of h gives q | k (| gate | up of a dense feed-forward) -> biases, rotation of adjacent pairs,
            the rotated key into the key page and the key as projected into the value page (the values ARE the
            unrotated keys), and in the same launch the dense feed-forward's gelu_tanh(gate) * up -> softmax attention over the window and the kept first positions with a sink in the
            denominator, written beside the feed-forward's activations
  dense     its activations land next to the attention output; ONE projection over [attention | activations]
            with [W_o | W_down] gives mixer + feed-forward
  moe       router (fp32 softmax over all outputs, correction for the choice only, renormalised weights) -> pairs
            sorted by expert -> gate|up by segment -> clamped gate -> down by segment -> weighted sum, a choice of
            a pass-through expert adding h itself; W_o separately
  then      x += both, and the NEXT layer's norm of the new x, in one launch

Per layer (Solopel; pre-norm, every sublayer output passes a sigmoid gate computed from the sublayer's normed input):
  residual  x += y * sigmoid(g + b) of the sublayer before, and the norm (weight 1 + w) of the new x, in one launch:
            n in fp32 for the convolution and in the activation type for the gate projection R n
  canon     act( n + conv(n) ): a short causal convolution per channel in front of the mixer, its last inputs kept per slot
  latent attention  fused q|dkv projection -> the normed latent into the page, q in the activation type -> per-head
            product carrying q into the latent space -> causal attention over the cached latents -> per-head value
            up-projection -> cast -> out-projection
  differential attention  fused q|k|v|gate projection -> short convolution over q|k|v (inputs kept per slot), keys and
            values into the pages -> two softmax maps per head over the same values, their difference unit-normed and
            gated per head, in one launch -> out-projection
  dense     fused up|R2 projection -> gelu_tanh -> down
  moe       router (fp32, sigmoid scores, top-k) -> pairs sorted by expert -> gate|up by segment -> SiLU-gate of the
            products scaled by the pair's score (the score scales the expert's input) -> down by segment; shared
            expert's gate|up|R2 in one projection; plain sum
  loop      a pass of the looped span starts from W_in [x | x0] + step_t, x0 the embedding
"""
import logging
import math
from typing import Dict, List, Optional

import torch

from ...kernel import ragged_ops as ops
from ...models.nesisun import GATE_SLOPE, WEIGHT_SUM_FLOOR
from ...models.pagazen import mamba2_sizes
from ..state_cache import HybridCacheManager, RaggedStep

logger = logging.getLogger(__name__)


class RaggedRunner:
    PAGE = 64

    def __init__(self, model, device="cuda", dtype=torch.bfloat16, wave_tiles: bool = True,
                 chunked_scan: bool = True, graphs: bool = True, max_graph_rows: int = 64, tiled_attn: bool = True,
                 grouped_attn: bool = True):
        """`wave_tiles` / `chunked_scan` = False keep every projection on the plain any-shape kernel and
        every recurrence token by token, `tiled_attn` = False every token on the plain attention kernel (the
        forms the faster ones are checked against), `grouped_attn` = False the tokens of short rows on the
        one-workgroup-per-(token, head) attention instead of the one that shares reads among query heads.  `graphs`:
        steps in which every row brings one token (decoding) are captured once per row count into a
        hipGraph and replayed - some seventy launches become one."""
        assert dtype in (torch.bfloat16, torch.float32)
        self.chunked_scan, self.tiled_attn, self.grouped_attn = chunked_scan, tiled_attn, grouped_attn
        self.use_graphs, self.max_graph_rows = graphs, max_graph_rows
        self._graphs: Dict[int, tuple] = {}
        self._arena, self._arena_off, self._measured = None, 0, 0
        self.model, self.cfg, self.device, self.dtype = model, model.config, device, dtype
        self.wave_tiles = wave_tiles
        cfg = self.cfg
        self.vocab_size, self.width = cfg.vocab_size, cfg.width
        self.weight_bytes = 0
        self._w: Dict[int, dict] = {}
        # a layer RUN = (layer whose tensors it uses, its description); every run has a cache / state of its own
        self.runs = cfg.layer_runs()
        self.sandwich = cfg.architecture == "Fagunex"     # Dynamic Tanh before and after each sublayer
        self.parallel_prenorm = cfg.architecture == "Nesisun"   # one RMS norm feeds mixer and feed-forward alike
        self.gated_prenorm = cfg.architecture == "Solopel"      # pre-norm layers whose sublayer outputs pass a gate
        for wi, layer in self.runs:
            if wi not in self._w:
                self._w[wi] = self._prepare_layer(wi, layer)
        self.embed = self._act(model.get("embed"))
        if self.sandwich:
            self.final_norm = self._dyt_norm("final.norm")
            self.side_embed = self._act(model.get("side.embed")) if cfg.side_dim else None
        elif self.parallel_prenorm:
            self.final_norm = self._small(model.get("final.norm"))
            self.pair_embed = self._act(model.get("bigram"))
        elif self.gated_prenorm:
            self.final_norm = self._small(model.get("final.norm"))
            if cfg.looped:
                self.loop_in = self._linear(model.get("loop.in"))
                self.loop_step = self._small(model.get("loop.step"))
        else:
            self.final_norm = self._small(model.get("final.norm"))
        # Solopel's output head is its embedding table
        self.head = self._linear(model.get("embed" if self.gated_prenorm else "head"))

    # ------------------------------------------------------------------ weights
    def _act(self, t):
        return t.to(device=self.device, dtype=self.dtype).contiguous()

    def _small(self, t):
        return t.to(device=self.device, dtype=torch.float32).contiguous()

    def _linear(self, *parts):
        w = torch.cat([self._act(p) for p in parts], dim=0) if len(parts) > 1 else self._act(parts[0])
        lin = ops.AnyLinear(w, wave_tiles=self.wave_tiles)
        self.weight_bytes += lin.nbytes
        return lin

    def _dyt_norm(self, name):
        g = self.model.get
        return (self._small(g(name)), self._small(g(name + ".b")), self._small(g(name + ".alpha")).reshape(1))

    def _stacked(self, parts):
        """[E, n, k] in the activation type: the same projection of several experts or heads."""
        w = torch.stack([self._act(p) for p in parts], dim=0).contiguous()
        self.weight_bytes += w.numel() * w.element_size()
        return w

    def _prepare_layer(self, i: int, layer: dict) -> dict:
        if self.sandwich:
            return self._prepare_fagunex(i, layer)
        if self.parallel_prenorm:
            return self._prepare_nesisun(i, layer)
        if self.gated_prenorm:
            return self._prepare_solopel(i, layer)
        g, p, m = self.model.get, f"l{i}.", layer["mixer"]
        w = {"norm1": self._small(g(p + "norm1"))}
        if layer["type"] == "mamba2":
            w.update(sizes=mamba2_sizes(m), w_in=self._linear(g(p + "mix.in")), conv=self._small(g(p + "mix.conv")),
                     conv_b=self._small(g(p + "mix.conv.b")), dt_bias=self._small(g(p + "mix.dt_bias")),
                     a_log=self._small(g(p + "mix.A_log")), skip=self._small(g(p + "mix.D")),
                     norm=self._small(g(p + "mix.norm")), w_o=self._linear(g(p + "mix.o")))
        else:
            L, R = m["left"], m["right"]
            H = int(L["heads"])
            slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], dtype=torch.float64)
            rot = int(R["rot"]["dims"])
            inv_freq = float(R["rot"]["base"]) ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot)
            w.update(left_qkv=self._linear(g(p + "mix.left.q"), g(p + "mix.left.k"), g(p + "mix.left.v")),
                     left_o=self._linear(g(p + "mix.left.o")), slopes=self._small(slopes),
                     right_qkvg=self._linear(g(p + "mix.right.q"), g(p + "mix.right.k"), g(p + "mix.right.v"),
                                             g(p + "mix.right.g")),
                     right_o=self._linear(g(p + "mix.right.o")),
                     decay=self._small(torch.tensor([float(x) for x in R["decay"]], dtype=torch.float64)),
                     log_decay=self._small(torch.log(torch.tensor([float(x) for x in R["decay"]], dtype=torch.float64))),
                     inv_freq=inv_freq.to(self.device))
            assert len(R["decay"]) == int(R["heads"]), "one decay per retention head"
        if layer.get("mlp"):
            w.update(norm2=self._small(g(p + "norm2")), up=self._linear(g(p + "mlp.up")),
                     down=self._linear(g(p + "mlp.down")))
        return w

    def _prepare_fagunex(self, i: int, layer: dict) -> dict:
        g, p, m, cfg = self.model.get, f"l{i}.", layer["mixer"], self.cfg
        w = {"norm1": self._dyt_norm(p + "norm1"), "norm1b": self._dyt_norm(p + "norm1b"),
             "shift": self._small(g(p + "shift"))}
        H = int(m["heads"])
        if layer["type"] == "hgrn2":
            w.update(qfv=self._linear(g(p + "mix.q"), g(p + "mix.f"), g(p + "mix.v")), f_b=self._small(g(p + "mix.f.b")),
                     lower=self._small(g(p + "mix.lower")), norm=self._small(g(p + "mix.norm")),
                     w_o=self._linear(g(p + "mix.o")))
        else:
            d, r, dv, R = int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
            rot = int(m["rot"]["dims"]) if m.get("rot") else 0
            base = float(m["rot"]["base"]) if rot else 1.0
            inv_freq = base ** (-2.0 * torch.arange(max(rot // 2, 1), dtype=torch.float64) / max(rot, 1))
            if layer["type"] == "latent_attention":
                w.update(w_in=self._linear(g(p + "mix.dq"), g(p + "mix.dkv"), g(p + "mix.g")),
                         q_norm=self._small(g(p + "mix.dq.norm")), w_uq=self._linear(g(p + "mix.uq")),
                         sink=self._small(g(p + "mix.sink")))
            else:
                w.update(w_in=self._linear(g(p + "mix.q"), g(p + "mix.dkv")))
            # per head: q_abs = W_uk,h^T q (so the stacked weight is [H, R, d]), value = W_uv,h * latent sum ([H, dv, R])
            uk = g(p + "mix.uk").reshape(H, d, R).transpose(1, 2)
            uv = g(p + "mix.uv").reshape(H, dv, R)
            w.update(kv_norm=self._small(g(p + "mix.dkv.norm")), uk_t=self._stacked(list(uk)), uv=self._stacked(list(uv)),
                     w_o=self._linear(g(p + "mix.o")), inv_freq=inv_freq.to(self.device), rot=rot)
        mlp = layer.get("mlp")
        if mlp:
            E = int(mlp["router"]["experts"])
            w.update(norm2=self._dyt_norm(p + "norm2"), norm2b=self._dyt_norm(p + "norm2b"),
                     router=self._small(g(p + "mlp.router")),
                     e_gu=self._stacked([torch.cat([g(p + f"mlp.e{e}.gate"), g(p + f"mlp.e{e}.up")], dim=0) for e in range(E)]),
                     e_down=self._stacked([g(p + f"mlp.e{e}.down") for e in range(E)]))
            if mlp.get("shared"):
                w.update(s_gu=self._linear(g(p + "mlp.shared.gate"), g(p + "mlp.shared.up")),
                         s_down=self._linear(g(p + "mlp.shared.down")), s_gate=self._small(g(p + "mlp.shared.sg")).reshape(-1))
        if cfg.side_dim:
            w.update(side_gate=self._linear(g(p + "side.gate")), side_proj=self._linear(g(p + "side.proj")),
                     side_norm=self._small(g(p + "side.norm")), side_off=i * cfg.side_dim)
        return w

    def _prepare_nesisun(self, i: int, layer: dict) -> dict:
        g, p, m = self.model.get, f"l{i}.", layer["mixer"]
        rot = int(m["rot"]["dims"])
        inv_freq = float(m["rot"]["base"]) ** (-2.0 * torch.arange(max(rot // 2, 1), dtype=torch.float64) / max(rot, 1))
        w = {"norm1": self._small(g(p + "norm1")), "q_b": self._small(g(p + "mix.q.b")),
             "k_b": self._small(g(p + "mix.k.b")), "sink": self._small(g(p + "mix.sink")),
             "inv_freq": inv_freq.to(self.device)}
        mlp = layer.get("mlp")
        if mlp and mlp["kind"] == "dense":
            # both sublayers read the same h and their outputs are summed: one projection in (q | k | gate | up),
            # one out ([W_o | W_down] over [attention output | activations])
            w.update(w_in=self._linear(g(p + "mix.q"), g(p + "mix.k"), g(p + "mlp.gate"), g(p + "mlp.up")),
                     w_out=self._linear(torch.cat([g(p + "mix.o"), g(p + "mlp.down")], dim=1)))
        else:
            w.update(w_in=self._linear(g(p + "mix.q"), g(p + "mix.k")), w_out=self._linear(g(p + "mix.o")))
        if mlp and mlp["kind"] == "moe":
            E = int(mlp["router"]["experts"])
            w.update(router=self._small(g(p + "mlp.router")), correction=self._small(g(p + "mlp.correction")))
            if E:
                w.update(e_gu=self._stacked([torch.cat([g(p + f"mlp.e{e}.gate"), g(p + f"mlp.e{e}.up")], dim=0)
                                             for e in range(E)]),
                         e_down=self._stacked([g(p + f"mlp.e{e}.down") for e in range(E)]))
        return w

    def _prepare_solopel(self, i: int, layer: dict) -> dict:
        g, p, m, cfg, W = self.model.get, f"l{i}.", layer["mixer"], self.cfg, self.width
        w = {"norm1": self._small(g(p + "norm1")), "rg1": self._linear(g(p + "rg1")), "rg1_b": self._small(g(p + "rg1.b"))}
        if cfg.taps:
            w["canon"] = self._small(g(p + "canon1"))
        H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
        if layer["type"] == "latent_attention":
            R = int(m["kv_rank"])
            # per head: q_abs = W_uk,h^T q (so the stacked weight is [H, R, d]), value = W_uv,h * latent sum ([H, dv, R])
            uk = g(p + "mix.uk").reshape(H, d, R).transpose(1, 2)
            uv = g(p + "mix.uv").reshape(H, dv, R)
            w.update(w_in=self._linear(g(p + "mix.q"), g(p + "mix.dkv")), kv_norm=self._small(g(p + "mix.dkv.norm")),
                     uk_t=self._stacked(list(uk)), uv=self._stacked(list(uv)), w_o=self._linear(g(p + "mix.o")))
        else:
            G, taps = int(m["kv_heads"]), int(m.get("conv") or 0)
            C = H * 2 * d + G * 2 * d + G * dv
            # the per-head gate rides the q | k | v projection; zero rows fill its width up to what the wave-tile
            # projections take
            pad = (-(C + H)) % 16
            parts = [g(p + "mix.q"), g(p + "mix.k"), g(p + "mix.v"), g(p + "mix.g")]
            if pad:
                parts.append(torch.zeros(pad, W, dtype=parts[0].dtype))
            dot = lambda a, b: float((g(p + a).double() * g(p + b).double()).sum())   # noqa: E731
            diff = float(m["diff"])
            w.update(w_in=self._linear(*parts), w_o=self._linear(g(p + "mix.o")),
                     lam=math.exp(dot("mix.lq1", "mix.lk1")) - math.exp(dot("mix.lq2", "mix.lk2")) + diff,
                     conv=self._small(torch.cat([g(p + "mix.q.conv"), g(p + "mix.k.conv"), g(p + "mix.v.conv")], dim=0))
                     if taps else None)
        mlp = layer.get("mlp")
        if mlp:
            w.update(norm2=self._small(g(p + "norm2")), rg2_b=self._small(g(p + "rg2.b")))
            if mlp["kind"] == "dense":
                # the feed-forward and its output gate read the same normed vector: one projection
                w.update(up_rg=self._linear(g(p + "mlp.up"), g(p + "rg2")), down=self._linear(g(p + "mlp.down")))
            else:
                E = int(mlp["router"]["experts"])
                w.update(router=self._small(g(p + "mlp.router")),
                         e_gu=self._stacked([torch.cat([g(p + f"mlp.e{e}.gate"), g(p + f"mlp.e{e}.up")], dim=0)
                                             for e in range(E)]),
                         e_down=self._stacked([g(p + f"mlp.e{e}.down") for e in range(E)]))
                if mlp.get("shared"):
                    w.update(s_gu_rg=self._linear(g(p + "mlp.shared.gate"), g(p + "mlp.shared.up"), g(p + "rg2")),
                             s_down=self._linear(g(p + "mlp.shared.down")))
                else:
                    w.update(rg2=self._linear(g(p + "rg2")))
        return w

    # ------------------------------------------------------------------ cache geometry
    def cache_layout(self):
        """(kv_layers, state_layers) for HybridCacheManager: what every layer RUN keeps per sequence."""
        kv, state = {}, {}
        if self.cfg.architecture == "Solopel":
            for i, (_, layer) in enumerate(self.runs):
                m = layer["mixer"]
                state[i] = {"canon": (self.cfg.taps - 1, self.width)} if self.cfg.taps else {}
                if layer["type"] == "latent_attention":
                    kv[i] = (1, int(m["kv_rank"]), 0)          # one normed latent per token: key and value alike
                else:
                    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
                    kv[i] = (G, 2 * d, dv)                     # both maps' keys of a key/value head side by side
                    if int(m.get("conv") or 0) > 1:
                        state[i]["qkv"] = (int(m["conv"]) - 1, H * 2 * d + G * 2 * d + G * dv)
            return kv, state
        for i, (_, layer) in enumerate(self.runs):
            m = layer["mixer"]
            if layer["type"] == "mamba2":
                s = mamba2_sizes(m)
                state[i] = {"conv": (max(s["taps"] - 1, 0), s["conv_ch"]), "ssm": (s["heads"], s["n"], s["p"])}
            elif layer["type"] == "attention":
                kv[i] = (int(m["kv_heads"]), int(m["dim"]), int(m["dim"]))   # rotated key | the key as projected = value
            elif layer["type"] == "hgrn2":
                state[i] = {"shift": (self.width,), "gated": (int(m["heads"]), int(m["dim"]), int(m["vdim"]))}
            elif layer["type"] in ("latent_attention", "latent_attention_2"):
                kv[i] = (1, int(m["kv_rank"]) + int(m["rot_dim"]), 0)    # one latent + rotated key part per token
                state[i] = {"shift": (self.width,)}
            else:
                L, R = m["left"], m["right"]
                kv[i] = (int(L["kv_heads"]), int(L["dim"]), int(L["vdim"]))
                state[i] = {"ret": (int(R["heads"]), int(R["dim"]), int(R["vdim"]))}
        return kv, state

    def make_cache(self, n_pages: int, n_slots: int, max_tokens: int = 4096, max_rows: int = 32,
                   max_step_tokens: int = 8192) -> HybridCacheManager:
        kv, state = self.cache_layout()
        return HybridCacheManager(n_pages, self.PAGE, n_slots, kv, state, dtype=self.dtype, device=self.device,
                                  max_tokens=max_tokens, max_rows=max_rows, max_step_tokens=max_step_tokens)

    # ------------------------------------------------------------------ layers
    def _take(self, rows, cols, dtype):
        """A [rows, cols] buffer: from the arena of the step being captured or replayed (the same
        addresses every time), else a fresh allocation."""
        nbytes = (rows * cols * (4 if dtype == torch.float32 else 2) + 255) // 256 * 256
        self._measured += nbytes
        if self._arena is None:
            return torch.empty(rows, cols, dtype=dtype, device=self.device)
        assert self._arena_off + nbytes <= self._arena.numel(), "step arena too small"
        t = self._arena[self._arena_off:self._arena_off + nbytes].view(dtype)[:rows * cols].view(rows, cols)
        self._arena_off += nbytes
        return t

    def _f32buf(self, rows, cols):
        return self._take(rows, cols, torch.float32)

    def _actbuf(self, rows, cols):
        return self._take(rows, cols, self.dtype)

    def _mamba2(self, li, w, h, step: RaggedStep, cache: HybridCacheManager):
        s, T, eps = w["sizes"], step.tokens, self.cfg.eps
        inner, ch, H, N, P, G = s["inner"], s["conv_ch"], s["heads"], s["n"], s["p"], s["groups"]
        st = cache.states[li]
        proj = w["w_in"](h, self._f32buf(T, w["w_in"].n))     # [z | x B C | dt]
        xbc = self._f32buf(T, ch)
        ops.conv_silu(proj[:, inner:inner + ch], st["conv"], w["conv"], w["conv_b"], xbc, step)
        gain, decay, log_decay = self._f32buf(T, H), self._f32buf(T, H), self._f32buf(T, H)
        ops.softplus_decay(proj[:, inner + ch:inner + ch + H], w["dt_bias"], w["a_log"], gain, decay, log_decay)
        y = self._f32buf(T, inner)
        ops.scan_outer(q=xbc[:, inner + G * N:], k=xbc[:, inner:inner + G * N], v=xbc[:, :inner], decay=decay,
                       gain=gain, skip=w["skip"], state=st["ssm"], out=y, step=step, heads=H, n=N, p=P,
                       q_div=H // G, k_div=H // G, log_decay=log_decay, chunked=self.chunked_scan)
        u = self._actbuf(T, inner)
        ops.gated_group_norm(y, proj[:, :inner], w["norm"], u, groups=s["norm_groups"], gate_first=True, eps=eps)
        return w["w_o"](u, self._f32buf(T, self.width)), None

    def _parallel(self, li, w, m, h, step: RaggedStep, cache: HybridCacheManager):
        T, eps = step.tokens, self.cfg.eps
        L, R = m["left"], m["right"]
        H, G, d, dv = int(L["heads"]), int(L["kv_heads"]), int(L["dim"]), int(L["vdim"])
        qkv = w["left_qkv"](h, self._f32buf(T, w["left_qkv"].n))
        kc, vc = cache.k_caches[li], cache.v_caches[li]
        ops.qk_unitnorm_store(qkv, kc, vc, step, H, G, d, dv, eps)
        a = self._actbuf(T, H * dv)
        ops.window_attn(qkv, kc, vc, a, step, w["slopes"], H, G, d, dv, float(L["scale"]), int(L["mask"]["size"]),
                        tiled=self.tiled_attn)
        left = w["left_o"](a, self._f32buf(T, self.width))

        Hr, dr, dvr, rot = int(R["heads"]), int(R["dim"]), int(R["vdim"]), int(R["rot"]["dims"])
        qkvg = w["right_qkvg"](h, self._f32buf(T, w["right_qkvg"].n))
        q, k = qkvg[:, :Hr * dr], qkvg[:, Hr * dr:2 * Hr * dr]
        v, g = qkvg[:, 2 * Hr * dr:2 * Hr * dr + Hr * dvr], qkvg[:, 2 * Hr * dr + Hr * dvr:]
        ops.rotary_pairs_(q, w["inv_freq"], step.tok_pos, Hr, dr, rot, 1.0)
        ops.rotary_pairs_(k, w["inv_freq"], step.tok_pos, Hr, dr, rot, dr ** -0.5)
        o = self._f32buf(T, Hr * dvr)
        ops.scan_outer(q=q, k=k, v=v, decay=w["decay"], gain=None, skip=None, state=cache.states[li]["ret"], out=o,
                       step=step, heads=Hr, n=dr, p=dvr, log_decay=w["log_decay"], chunked=self.chunked_scan)
        u = self._actbuf(T, Hr * dvr)
        ops.gated_group_norm(o, g, None, u, groups=Hr, gate_first=False, eps=eps)
        return left, w["right_o"](u, self._f32buf(T, self.width))

    @torch.inference_mode()
    def forward(self, step: RaggedStep, cache: HybridCacheManager, want: Optional[torch.Tensor] = None,
                residuals: Optional[List[torch.Tensor]] = None, want_all: bool = False) -> torch.Tensor:
        """Run the step; returns fp32 logits [len(want), vocab] for the token indices in `want` (int32 on
        the device; None = every token; `want_all`: the caller knows that `want` lists every token in order).
        `residuals` receives a copy of the stream after every layer run (debugging and tests)."""
        if (self.use_graphs and residuals is None and step.tokens == step.rows <= self.max_graph_rows):
            return self._replay(step, cache, None if want_all else want)
        return self._run(step, cache, want, residuals)

    # ------------------------------------------------------------------ captured decoding steps
    def _replay(self, step: RaggedStep, cache: HybridCacheManager, want):
        B = step.rows
        key = (B, id(cache))
        if key not in self._graphs:
            try:
                self._graphs[key] = self._capture(step, cache)
            except Exception as e:   # the recording failed (nothing of it ran): this row count stays uncaptured
                logger.warning("decoding steps of %d rows are not captured: %r", B, e)
                self._graphs[key] = None
        entry = self._graphs[key]
        if entry is None:
            return self._run(step, cache, want, None)
        graph, logits = entry[0], entry[2]
        graph.replay()
        if want is None:
            return logits.clone()
        return logits.index_select(0, want.long())

    def _capture(self, step: RaggedStep, cache: HybridCacheManager):
        """One run of the step on a side stream with fresh allocations (it sizes the arena and lets the
        projections set up their per-stream workspaces), the recurrent state of the step's slots put back
        as it was, then the same launches recorded over an arena.  Everything a replay reads that
        changes from step to step - tokens, positions, slots, block table - lies in the cache manager's
        one device buffer; keys and values of the step are written again by the replay with the same
        contents."""
        import ctypes
        from ... import _native as nv
        from .model_graph import HipGraph
        B, slots = step.rows, list(step.slots)
        idx = torch.tensor(slots, dtype=torch.long, device=self.device)
        saved = [(t, t.index_select(0, idx)) for named in cache.states.values() for t in named.values()]
        all_rows = torch.arange(B, dtype=torch.int32, device=self.device)
        side = torch.cuda.Stream(device=self.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self._arena, self._measured = None, 0
            try:
                self._run(step, cache, all_rows, None)
            finally:   # whatever that run did to the slots' state is undone: the step itself is still to come
                for t, old in saved:
                    t.index_copy_(0, idx, old)
            arena = torch.empty(self._measured + 4096, dtype=torch.uint8, device=self.device)
            side.synchronize()
            self._arena, self._arena_off = arena, 0
            nv.check("mv_graph_begin_capture", nv.lib().mv_graph_begin_capture(side.cuda_stream))
            try:
                logits = self._run(step, cache, all_rows, None)
            finally:
                handle = ctypes.c_void_p()
                rc = nv.lib().mv_graph_end_capture(side.cuda_stream, ctypes.byref(handle))
                self._arena = None
            nv.check("mv_graph_end_capture", rc)
        torch.cuda.current_stream().wait_stream(side)
        logger.info("captured a decoding step of %d rows (%d KiB of intermediates)", B, arena.numel() >> 10)
        return HipGraph(handle), arena, logits, all_rows      # the arena and the row list stay alive with the graph

    def _run(self, step: RaggedStep, cache: HybridCacheManager, want, residuals) -> torch.Tensor:
        cfg, T = self.cfg, step.tokens
        if not self.gated_prenorm:       # that design's stack lays out its own streams
            x, h = self._f32buf(T, self.width), self._actbuf(T, self.width)
        if self.parallel_prenorm:
            ops.embed_pair(self.embed, self.pair_embed, step.ids, step.tok_prev, x, cfg.embed_scale, cfg.pair_buckets,
                           cfg.pair_mul_prev, cfg.pair_mul_cur, w=self._w[self.runs[0][0]]["norm1"], eps=cfg.eps, h=h)
            for li, (wi, layer) in enumerate(self.runs):
                y1, y2 = self._nesisun_layer(li, self._w[wi], layer, h, step, cache)
                # both sublayers enter the stream; the next layer's norm of the new x comes out of the same launch
                nxt = self._w[self.runs[li + 1][0]]["norm1"] if li + 1 < len(self.runs) else None
                ops.add_rmsnorm(x, y1, y2, w=nxt, eps=cfg.eps, h=None if nxt is None else h)
                if residuals is not None:
                    residuals.append(x.clone())
        elif self.gated_prenorm:
            x = self._solopel_stack(step, cache, residuals)
        elif self.sandwich:
            ops.embed_scaled(self.embed, step.ids, 1.0, x, h)
            for li, (wi, layer) in enumerate(self.runs):
                self._fagunex_layer(li, self._w[wi], layer, x, h, step, cache)
                if residuals is not None:
                    residuals.append(x.clone())
        else:
            ops.embed_scaled(self.embed, step.ids, cfg.embed_scale, x, h)
            for li, (wi, layer) in enumerate(self.runs):
                w, m = self._w[wi], layer["mixer"]
                if layer["type"] == "mamba2":
                    y1, y2 = self._mamba2(li, w, h, step, cache)
                    ops.postnorm_residual(y1, w["norm1"], cfg.eps, x, h)
                else:
                    y1, y2 = self._parallel(li, w, m, h, step, cache)
                    ops.postnorm_residual(y1, w["norm1"], cfg.eps, x, h, y2=y2, s1=float(m["left_scale"]),
                                          s2=float(m["right_scale"]))
                if layer.get("mlp"):
                    up = w["up"](h, self._f32buf(T, w["up"].n))
                    act = self._actbuf(T, up.shape[1])
                    ops.relu_squared(up, act)
                    ops.postnorm_residual(w["down"](act, self._f32buf(T, self.width)), w["norm2"], cfg.eps, x, h)
                if residuals is not None:
                    residuals.append(x.clone())
        rows = T if want is None else want.numel()
        normed = self._actbuf(rows, self.width)
        if rows == 0:
            return self._f32buf(0, self.vocab_size)
        if self.sandwich:
            ops.dyt_gather(x, want, self.final_norm, normed)
        elif self.parallel_prenorm:
            ops.rmsnorm_gather(x, want, self.final_norm, cfg.eps, normed)
        else:
            ops.offset_rmsnorm_gather(x, want, self.final_norm, cfg.eps, normed)
        logits = self.head(normed, self._f32buf(rows, self.vocab_size))
        if getattr(cfg, "logit_scale", 1.0) != 1.0:
            ops.scale_(logits, cfg.logit_scale)
        if getattr(cfg, "logit_softcap", None):
            ops.softcap_(logits, cfg.logit_softcap)
        return logits

    # ------------------------------------------------------------------ Nesisun layers
    def _nesisun_layer(self, li, w, layer, h, step: RaggedStep, cache: HybridCacheManager):
        """Mixer and feed-forward of one layer run on the normed input h: returns their outputs (fp32; the second
        is None where one projection has already summed them, or where there is no feed-forward)."""
        T, m, mlp = step.tokens, layer["mixer"], layer.get("mlp")
        H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
        dense = bool(mlp) and mlp["kind"] == "dense"
        ff = int(mlp["ff"]) if dense else 0
        proj = w["w_in"](h, self._f32buf(T, w["w_in"].n))          # [q | k (| gate | up)]
        qk = proj[:, :(H + G) * d]
        kc, vc = cache.k_caches[li], cache.v_caches[li]
        cat = self._actbuf(T, H * d + ff)                          # [attention output | activations]
        # gelu_tanh(gate) * up lands next to where the attention output will go.  In steps of few tokens it comes out of
        # the rotation's launch (a launch saved); in long ones it runs behind the attention, whose keys and values the
        # activations' traffic would otherwise push out of the caches
        act = (proj[:, (H + G) * d:], cat[:, H * d:], ops.GATE_GELU_TANH, 0.0, 1.0) if dense else None
        fuse_act = dense and T <= 64
        ops.qk_rotary_store(qk, w["q_b"], w["k_b"], kc, vc, w["inv_freq"], step, H, G, d, int(m["rot"]["dims"]),
                            adjacent=True, act=act if fuse_act else None)
        window, keep = int(m["mask"]["size"]), int(m["mask"].get("keep_first", 0))
        # tokens of short rows (decoding): the query heads of a key/value head share its reads, the keys are cut over
        # several workgroups and the pieces meet in `part`
        splits = ops.window_attn_splits(T, H, G, window, keep) if self.grouped_attn else 0
        part = self._f32buf(1, T * H * splits * (d + 2)) if splits else None
        ops.window_attn(qk, kc, vc, cat[:, :H * d], step, None, H, G, d, d, float(m["scale"]), window,
                        tiled=self.tiled_attn, keep_first=keep, sinks=w["sink"], part=part, splits=splits)
        if dense and not fuse_act:
            ops.gated_act(act[0], act[1], act[2])
        y1 = w["w_out"](cat, self._f32buf(T, self.width))
        if not mlp or dense:
            return y1, None
        return y1, self._routed_with_pass(w, mlp, h, T)

    def _routed_with_pass(self, w, mlp, h, T):
        r = mlp["router"]
        E, n_pass, top, ff = int(r["experts"]), int(r.get("identity", 0)), int(r["top"]), int(mlp["expert"]["ff"])
        ids = self._i32buf(T * top).view(T, top)
        wts = self._f32buf(T, top)
        ops.moe_route_scored(h, w["router"], w["correction"], ids, wts, float(r.get("scale", 1.0)), WEIGHT_SUM_FLOOR)
        seg, order, place = self._i32buf(E + n_pass + 1), self._i32buf(T * top), self._i32buf(T * top)
        ops.moe_plan(ids, seg, order, place, E + n_pass)
        down = self._f32buf(T * top, self.width)
        if E:
            gu = ops.linear_segments(h, w["e_gu"], self._f32buf(T * top, 2 * ff), seg[:E + 1], order, top, T)
            act = self._actbuf(T * top, ff)
            ops.gated_act(gu, act, ops.GATE_CLAMPED, float(mlp["expert"]["limit"]), GATE_SLOPE)
            ops.linear_segments(act, w["e_down"], down, seg[:E + 1], None, 1, T)
        y = self._f32buf(T, self.width)
        ops.moe_combine(down, place, wts, None, None, y, ids=ids.view(-1), first_pass=E, passed=h)
        return y

    # ------------------------------------------------------------------ Solopel layers
    def _solopel_stack(self, step: RaggedStep, cache: HybridCacheManager, residuals):
        """All layer runs on a fresh stream; returns it.  A sublayer's output enters the stream in the launch that
        forms the NEXT norm, so between layers it travels as `pend` = (y, gate logits, gate bias, replace)."""
        cfg, T, W = self.cfg, step.tokens, self.width
        plan = cfg.run_plan()
        x0, x, h = self._f32buf(T, W), self._f32buf(T, W), self._actbuf(T, W)
        ops.embed_scaled(self.embed, step.ids, 1.0, x0, h)
        if plan[0][1] < 0:
            ops.embed_scaled(self.embed, step.ids, 1.0, x, h)
        pend = None
        for li, ((wi, layer), (_, t_pass)) in enumerate(zip(self.runs, plan)):
            if t_pass >= 0:       # a pass of the looped span starts: x = W_in [x | x0] + step_t
                if pend is not None:
                    ops.gated_residual_norm(x, *pend)
                cat = self._actbuf(T, 2 * W)
                ops.cast_concat(x if li > 0 else x0, x0, cat)
                pend = (self.loop_in(cat, self._f32buf(T, W)), None, self.loop_step[t_pass], True)
            pend = self._solopel_layer(li, self._w[wi], layer, x, pend, step, cache)
            if residuals is not None:
                ops.gated_residual_norm(x, *pend)
                pend = None
                residuals.append(x.clone())
        if pend is not None:
            ops.gated_residual_norm(x, *pend)
        return x

    def _solopel_layer(self, li, w, layer, x, pend, step: RaggedStep, cache: HybridCacheManager):
        T, W, cfg, eps = step.tokens, self.width, self.cfg, self.cfg.eps
        y, g, b, replace = pend if pend is not None else (None, None, None, False)
        h = self._actbuf(T, W)
        # the convolution reads the norm in fp32; in fp32 runs that is h itself
        n32 = self._f32buf(T, W) if cfg.taps and self.dtype != torch.float32 else None
        ops.gated_residual_norm(x, y, g, b, replace, w=w["norm1"], eps=eps, offset=1.0, n32=n32, h=h)
        hc = h
        if cfg.taps:
            hc = self._actbuf(T, W)
            ops.conv_taps(h if n32 is None else n32, cache.states[li]["canon"], w["canon"], step, out_act=hc,
                          add_input=True)
        g1 = w["rg1"](h, self._f32buf(T, W))
        if layer["type"] == "latent_attention":
            y = self._solopel_latent(li, w, layer["mixer"], hc, step, cache)
        else:
            y = self._solopel_diff(li, w, layer["mixer"], hc, step, cache)
        mlp = layer.get("mlp")
        if not mlp:
            return y, g1, w["rg1_b"], False
        h2 = self._actbuf(T, W)
        ops.gated_residual_norm(x, y, g1, w["rg1_b"], w=w["norm2"], eps=eps, offset=1.0, h=h2)
        if mlp["kind"] == "dense":
            ff = int(mlp["ff"])
            proj = w["up_rg"](h2, self._f32buf(T, ff + W))            # [up | gate logits of the residual]
            act = self._actbuf(T, ff)
            ops.gelu_tanh(proj[:, :ff], act)
            return w["down"](act, self._f32buf(T, W)), proj[:, ff:], w["rg2_b"], False
        E, top, ff = int(mlp["router"]["experts"]), int(mlp["router"]["top"]), int(mlp["expert"]["ff"])
        ids = self._i32buf(T * top).view(T, top)
        wts = self._f32buf(T, top)
        ops.moe_route_sigmoid(h2, w["router"], ids, wts)
        seg, order, place = self._i32buf(E + 1), self._i32buf(T * top), self._i32buf(T * top)
        ops.moe_plan(ids, seg, order, place, E)
        # an expert reads score * h: its gate and up products are linear in h, so the score goes onto the products
        gu = ops.linear_segments(h2, w["e_gu"], self._f32buf(T * top, 2 * ff), seg, order, top, T)
        act = self._actbuf(T * top, ff)
        ops.gated_act_scaled(gu, act, ops.GATE_SILU, wts.view(-1), order)
        down = ops.linear_segments(act, w["e_down"], self._f32buf(T * top, W), seg, None, 1, T)
        s_out = None
        if mlp.get("shared"):
            sf = int(mlp["shared"]["ff"])
            proj = w["s_gu_rg"](h2, self._f32buf(T, 2 * sf + W))     # [gate | up | gate logits of the residual]
            s_act = self._actbuf(T, sf)
            ops.silu_mul(proj[:, :2 * sf], s_act)
            s_out, g2 = w["s_down"](s_act, self._f32buf(T, W)), proj[:, 2 * sf:]
        else:
            g2 = w["rg2"](h2, self._f32buf(T, W))
        y2 = self._f32buf(T, W)
        ops.moe_combine(down, place, None, s_out, None, y2)
        return y2, g2, w["rg2_b"], False

    def _solopel_latent(self, li, w, m, hc, step: RaggedStep, cache: HybridCacheManager):
        T, eps = step.tokens, self.cfg.eps
        H, d, dv, R = int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"])
        proj = w["w_in"](hc, self._f32buf(T, H * d + R))               # [q | dkv]
        pages = cache.k_caches[li]
        pages = pages.view(pages.shape[0], pages.shape[1], R)
        q_plain, q_abs = self._actbuf(T, H * d), self._f32buf(T, H * R)
        ops.latent_prep(proj[:, H * d:], w["kv_norm"], eps, pages, proj[:, :H * d], q_plain, q_abs, None, step, H, d, 0,
                        R, 0, interleaved=False)
        ops.linear_heads(q_plain, w["uk_t"], q_abs.view(T, H, R), H)
        lat = self._actbuf(T, H * R)
        ops.latent_attn(q_abs, pages, lat, step, None, H, R, 0, float(m["scale"]), 0, tiled=self.tiled_attn)
        val = self._f32buf(T, H * dv)
        ops.linear_heads(lat, w["uv"], val.view(T, H, dv), H)
        a = self._actbuf(T, H * dv)
        ops.sigmoid_gate(val, None, a)
        return w["w_o"](a, self._f32buf(T, self.width))

    def _solopel_diff(self, li, w, m, hc, step: RaggedStep, cache: HybridCacheManager):
        T = step.tokens
        H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        C = H * 2 * d + G * 2 * d + G * dv
        proj = w["w_in"](hc, self._f32buf(T, w["w_in"].n))             # [q | k | v | head gates (| zeros)]
        q = self._f32buf(T, H * 2 * d)
        kc, vc = cache.k_caches[li], cache.v_caches[li]
        ops.conv_qkv_store(proj, cache.states[li].get("qkv"), w["conv"], q, kc, vc, step)
        a = self._actbuf(T, H * dv)
        diff = float(m["diff"])
        ops.diff_attn(q, kc, vc, a, proj[:, C:C + H], step, H, G, d, dv, float(m["scale"]), float(m.get("softcap") or 0.0),
                      w["lam"], 1.0 - diff, self.cfg.eps, tiled=self.tiled_attn)
        return w["w_o"](a, self._f32buf(T, self.width))

    # ------------------------------------------------------------------ Fagunex layers
    def _i32buf(self, count):
        return self._take(1, count, torch.float32).view(torch.int32).view(-1)

    def _fagunex_layer(self, li, w, layer, x, h, step: RaggedStep, cache: HybridCacheManager):
        """One layer run on the stream x (fp32, updated in place); h is scratch of the activation type."""
        T, cfg = step.tokens, self.cfg
        ops.dyt_shift(x, w["norm1"], w["shift"], cache.states[li]["shift"], h, step)
        if layer["type"] == "hgrn2":
            y = self._hgrn2(li, w, layer["mixer"], h, step, cache)
        else:
            y = self._latent_attention(li, w, layer["mixer"], h, step, cache, layer["type"] == "latent_attention")
        mlp = layer.get("mlp")
        if mlp:
            # the norm after the mixer, the residual sum and the norm before the feed-forward in one launch; the
            # experts' weighted sum goes through the norm after the feed-forward straight into the stream
            ops.dyt_residual(y, w["norm1b"], x, h, next_norm=w["norm2"])
            self._moe(w, mlp, h, T, x, w["norm2b"], h if cfg.side_dim else None)
        else:
            # the copy of x in the activation type is what the side input's gate reads
            ops.dyt_residual(y, w["norm1b"], x, h if cfg.side_dim else None)
        if cfg.side_dim:
            a = w["side_gate"](h, self._f32buf(T, cfg.side_dim))
            g = self._actbuf(T, cfg.side_dim)
            ops.gelu_gate_rows(a, self.side_embed, w["side_off"], step.ids, g)
            ops.unitnorm_residual(w["side_proj"](g, self._f32buf(T, self.width)), w["side_norm"], cfg.eps, x)

    def _hgrn2(self, li, w, m, h, step: RaggedStep, cache: HybridCacheManager):
        T, H, n, p = step.tokens, int(m["heads"]), int(m["dim"]), int(m["vdim"])
        proj = w["qfv"](h, self._f32buf(T, w["qfv"].n))               # [q | f | v]
        q, f, v = proj[:, :H * n], proj[:, H * n:2 * H * n], proj[:, 2 * H * n:]
        ops.gate_lower_bound_(q, f, w["f_b"], w["lower"])
        o = self._f32buf(T, H * p)
        ops.scan_gated(q, f, v, cache.states[li]["gated"], o, step, H, n, p, chunked=self.chunked_scan)
        u = self._actbuf(T, H * p)
        ops.rmsnorm_rows(o, w["norm"], self.cfg.eps, u, per=H)
        return w["w_o"](u, self._f32buf(T, self.width))

    def _latent_attention(self, li, w, m, h, step: RaggedStep, cache: HybridCacheManager, first_kind: bool):
        T, eps = step.tokens, self.cfg.eps
        H, d, r, dv, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
        proj = w["w_in"](h, self._f32buf(T, w["w_in"].n))
        if first_kind:        # [dq | dkv | g]: queries through a normed latent
            Q = int(m["q_rank"])
            cq = self._actbuf(T, Q)
            ops.rmsnorm_rows(proj[:, :Q], w["q_norm"], eps, cq)
            q = w["w_uq"](cq, self._f32buf(T, H * (d + r)))
            dkv, gate = proj[:, Q:Q + R + r], proj[:, Q + R + r:]
            window, sink = int(m["mask"]["size"]), w["sink"]
        else:                 # [q | dkv]
            q, dkv, gate = proj[:, :H * (d + r)], proj[:, H * (d + r):], None
            window, sink = 0, None
        pages = cache.k_caches[li]
        pages = pages.view(pages.shape[0], pages.shape[1], R + r)
        q_plain, q_abs = self._actbuf(T, H * d), self._f32buf(T, H * (R + r))
        ops.latent_prep(dkv, w["kv_norm"], eps, pages, q, q_plain, q_abs, w["inv_freq"], step, H, d, r, R, w["rot"],
                        interleaved=first_kind)
        ops.linear_heads(q_plain, w["uk_t"], q_abs.view(T, H, R + r)[:, :, :R], H)
        lat = self._actbuf(T, H * R)
        ops.latent_attn(q_abs, pages, lat, step, sink, H, R, r, float(m["scale"]), window, tiled=self.tiled_attn)
        val = self._f32buf(T, H * dv)
        ops.linear_heads(lat, w["uv"], val.view(T, H, dv), H)
        a = self._actbuf(T, H * dv)
        ops.sigmoid_gate(val, gate, a)
        return w["w_o"](a, self._f32buf(T, self.width))

    def _moe(self, w, mlp, h, T, x, norm_after, h_out):
        E, top, ff = int(mlp["router"]["experts"]), int(mlp["router"]["top"]), int(mlp["expert"]["ff"])
        shared = mlp.get("shared")
        ids = self._i32buf(T * top).view(T, top)
        wts, sgate = self._f32buf(T, top), self._f32buf(1, T).view(-1)
        ops.moe_route(h, w["router"], w["s_gate"] if shared else None, ids, wts, sgate)
        seg, order, place = self._i32buf(E + 1), self._i32buf(T * top), self._i32buf(T * top)
        ops.moe_plan(ids, seg, order, place, E)
        gu = ops.linear_segments(h, w["e_gu"], self._f32buf(T * top, 2 * ff), seg, order, top, T)
        act = self._actbuf(T * top, ff)
        ops.silu_mul(gu, act)
        down = ops.linear_segments(act, w["e_down"], self._f32buf(T * top, self.width), seg, None, 1, T)
        s_out = None
        if shared:
            sf = int(shared["ff"])
            s_act = self._actbuf(T, sf)
            ops.silu_mul(w["s_gu"](h, self._f32buf(T, 2 * sf)), s_act)
            s_out = w["s_down"](s_act, self._f32buf(T, self.width))
        ops.moe_combine(down, place, wts, s_out, sgate, x, norm=norm_after, h=h_out)
