"""Plain, slow restatement of the Nesisun layer stack: one function per mechanism, whole sequences,
loops over tokens and heads.  Shares nothing with the product path; the tests compare the engine
against it.  Everything runs in `dtype` (float64 by default) on the CPU.

Weights come as a dict name -> tensor with the checkpoint's names ('l<i>.mix.q', ...), the
configuration as the parsed config.json dict.

Notation: every layer is PARALLEL, x <- x + mixer(n(x)) + ff(n(x)) with one RMS norm n (plain weight).
The mixer is softmax attention whose values are the keys before rotation, over a sliding window that
also keeps the sequence's first positions, with one extra term exp(sink_h) in the denominator.  The
token embedding is joined by a row of a hashed table indexed by (previous token, token).
"""
import math

import torch


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def pair_embedding(tokens, embed, table, scale, buckets, mul_prev, mul_cur):
    """embed[t] * scale + table[(prev * mul_prev + t * mul_cur) mod buckets]; a sequence's first token
    takes the table's extra last row (index `buckets`)."""
    rows = []
    for i, t in enumerate(tokens):
        r = buckets if i == 0 else (int(tokens[i - 1]) * mul_prev + int(t) * mul_cur) % buckets
        rows.append(embed[int(t)] * scale + table[r])
    return torch.stack(rows)


def rotate_adjacent(x, positions, dims, base):
    """x [T, H, d]: (x[2i], x[2i+1]) turned by angle pos * base^(-2i/dims) for i < dims/2; the rest pass."""
    out = x.clone()
    for i in range(dims // 2):
        ang = positions.to(x.dtype) * (base ** (-2.0 * i / dims))
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def visible(i, j, window, keep_first):
    return j <= i and (i - j < window or j < keep_first)


def sink_attention(q, k, v, scale, window, keep_first, sink):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads key/value head h // (H/G).
    weights_ij = exp(s_ij) / (sum over visible j of exp(s_ij) + exp(sink_h))."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            js = [j for j in range(i + 1) if visible(i, j, window, keep_first)]
            s = (k[js, g] @ q[i, h]) * scale
            m = max(float(s.max()), float(sink[h]))
            e = torch.exp(s - m)
            out[i, h] = (e / (e.sum() + math.exp(float(sink[h]) - m))) @ v[js, g]
    return out


def attention_mixer(h, W, p, m, positions=None):
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    T = h.shape[0]
    pos = torch.arange(T) if positions is None else positions
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, d)
    dims, base = int(m["rot"]["dims"]), float(m["rot"]["base"])
    a = sink_attention(rotate_adjacent(q, pos, dims, base), rotate_adjacent(k, pos, dims, base), k,
                       float(m["scale"]), int(m["mask"]["size"]), int(m["mask"]["keep_first"]), W[p + "sink"])
    return a.reshape(T, -1) @ W[p + "o"].T


def gated_gelu(h, gate, up, down):
    return (gelu_tanh(h @ gate.T) * (h @ up.T)) @ down.T


def clamped_expert(h, gate, up, down, limit):
    g = torch.clamp(h @ gate.T, max=limit)
    u = torch.clamp(h @ up.T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ down.T


def routed_with_identity(h, W, p, mlp):
    """softmax over ALL router outputs; the choice adds a per-expert correction, the weights do not;
    weights of the chosen are renormalised and scaled; the last `identity` outputs pass h through."""
    r = mlp["router"]
    E, n_id, top, scale = int(r["experts"]), int(r["identity"]), int(r["top"]), float(r["scale"])
    limit = float(mlp["expert"]["limit"])
    s = torch.softmax(h @ W[p + "router"].T, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        pick = s[t] + W[p + "correction"]
        order = sorted(range(E + n_id), key=lambda e: (-float(pick[e]), e))[:top]
        total = sum(float(s[t, e]) for e in order) + 1e-20
        for e in order:
            w = float(s[t, e]) / total * scale
            if e >= E:
                out[t] += w * h[t]
            else:
                out[t] += w * clamped_expert(h[t:t + 1], W[p + f"e{e}.gate"], W[p + f"e{e}.up"], W[p + f"e{e}.down"],
                                             limit)[0]
    return out


def weights_layer(config, i):
    j = config["layers"][i].get("weights_of")
    return i if j is None else int(j)


def forward(config, weights, tokens, dtype=torch.float64, residuals=None):
    """tokens: list of ids of ONE sequence from position 0 -> logits [T, vocab]."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    emb = config["embedding"]
    bg = emb["bigram"]
    x = pair_embedding(tokens, W["embed"], W["bigram"], float(emb["scale"]), int(bg["buckets"]), int(bg["mul_prev"]),
                       int(bg["mul_cur"]))
    for i, layer in enumerate(config["layers"]):
        p = f"l{weights_layer(config, i)}."
        h = rms_norm(x, W[p + "norm1"], eps)
        y = attention_mixer(h, W, p + "mix.", layer["mixer"])
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                y = y + gated_gelu(h, W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"])
            else:
                y = y + routed_with_identity(h, W, p + "mlp.", mlp)
        x = x + y
        if residuals is not None:
            residuals.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T
