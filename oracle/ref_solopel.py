"""Plain, slow restatement of the Solopel layer stack: one function per mechanism, whole sequences,
loops over tokens and heads.  Shares nothing with the product path; the tests compare the engine
against it.  Everything runs in `dtype` (float64 by default) on the CPU.

Weights come as a dict name -> tensor with the checkpoint's names ('l<i>.mix.q', ...), the
configuration as the parsed config.json dict.

Notation.  A layer is pre-norm with gated residuals:
    n1 = N1(x);  x <- x + M(n1 + C(n1)) * sigmoid(R1 n1 + b1)
    n2 = N2(x);  x <- x + F(n2) * sigmoid(R2 n2 + b2)
N = RMS norm with weight 1 + w; C = causal per-channel convolution over time (the mixer's input only);
M = the mixer ('latent_attention': causal softmax attention whose keys and values are expanded from one
normed latent per token; 'attention': two softmax maps per head over the same values, their difference
unit-normed and gated per head); F = dense GELU feed-forward, or routed SiLU-gated experts whose sigmoid
score scales the expert's INPUT, plus a shared expert; or nothing.  A span of layers may run several
times on the same weights; each pass starts from W_in [x ; x0] + step_t with x0 the embedding.
"""
import math

import torch


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    return rms_unit(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros before the start."""
    T, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def softmax_rows(s):
    e = torch.exp(s - s.max())
    return e / e.sum()


def latent_attention(q, c, uk, uv, scale):
    """q [T, H, d]; c [T, R] the normed latents; uk [H*d, R], uv [H*dv, R]: causal softmax per head over the keys
    uk_h c_j, values uv_h c_j."""
    T, H, d = q.shape
    k = (c @ uk.T).view(T, H, d)
    v = (c @ uv.T).view(T, H, -1)
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for hd in range(H):
        for i in range(T):
            s = (k[:i + 1, hd] @ q[i, hd]) * scale
            out[i, hd] = softmax_rows(s) @ v[:i + 1, hd]
    return out


def latent_mixer(h, W, p, m, eps):
    """Keys and values of every head come from ONE normed latent per token; no positions enter."""
    H, d = int(m["heads"]), int(m["dim"])
    T = h.shape[0]
    q = (h @ W[p + "q"].T).view(T, H, d)
    c = rms_unit(h @ W[p + "dkv"].T, eps) * W[p + "dkv.norm"]
    return latent_attention(q, c, W[p + "uk"], W[p + "uv"], float(m["scale"])).reshape(T, -1) @ W[p + "o"].T


def difference_attention(q, k, v, gate, scale, cap, lam, diff, eps):
    """q [T, H, 2, d], k [T, G, 2, d], v [T, G, dv], gate [T, H] (logits) or None: two causal softmax maps per head
    over the same values; o = a1 - lam a2, unit-normed over the head, times (1 - diff), times sigmoid(gate)."""
    T, H = q.shape[:2]
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            a = []
            for mp in range(2):
                s = (k[:i + 1, g, mp] @ q[i, hd, mp]) * scale
                if cap:
                    s = cap * torch.tanh(s / cap)
                a.append(softmax_rows(s) @ v[:i + 1, g])
            o = rms_unit(a[0] - lam * a[1], eps) * (1.0 - diff)
            out[i, hd] = o if gate is None else o * torch.sigmoid(gate[i, hd])
    return out


def difference_lambda(W, p, diff):
    return math.exp(float((W[p + "lq1"] * W[p + "lk1"]).sum())) - math.exp(float((W[p + "lq2"] * W[p + "lk2"]).sum())) + diff


def difference_mixer(h, W, p, m, eps):
    """Projections, a short causal convolution behind each of q, k, v, then the two-map attention."""
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    diff = float(m["diff"])

    def proj(name):
        u = h @ W[p + name].T
        return causal_conv(u, W[p + name + ".conv"]) if (p + name + ".conv") in W else u

    out = difference_attention(proj("q").view(T, H, 2, d), proj("k").view(T, G, 2, d), proj("v").view(T, G, dv),
                               h @ W[p + "g"].T, float(m["scale"]), float(m["softcap"]) if m.get("softcap") else 0.0,
                               difference_lambda(W, p, diff), diff, eps)
    return out.reshape(T, H * dv) @ W[p + "o"].T


def dense_ff(h, W, p):
    return gelu_tanh(h @ W[p + "up"].T) @ W[p + "down"].T


def silu_expert(h, W, p):
    a = h @ W[p + "gate"].T
    return (a * torch.sigmoid(a) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def routed_ff(h, W, p, mlp):
    """Scores = sigmoid of the router's outputs; the `top` largest are chosen (ties: the lower index); a chosen
    expert reads score * h; the shared expert reads h."""
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    s = torch.sigmoid(h @ W[p + "router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            out[t] += silu_expert((s[t, e] * h[t])[None], W, p + f"e{e}.")[0]
    if mlp.get("shared"):
        out = out + silu_expert(h, W, p + "shared.")
    return out


def layer_forward(x, W, i, layer, eps):
    p = f"l{i}."
    n1 = offset_norm(x, W[p + "norm1"], eps)
    u = n1 + causal_conv(n1, W[p + "canon1"]) if (p + "canon1") in W else n1
    if layer["type"] == "latent_attention":
        y = latent_mixer(u, W, p + "mix.", layer["mixer"], eps)
    elif layer["type"] == "attention":
        y = difference_mixer(u, W, p + "mix.", layer["mixer"], eps)
    else:
        raise ValueError(layer["type"])
    x = x + y * torch.sigmoid(n1 @ W[p + "rg1"].T + W[p + "rg1.b"])
    mlp = layer.get("mlp")
    if mlp is not None:
        n2 = offset_norm(x, W[p + "norm2"], eps)
        f = dense_ff(n2, W, p + "mlp.") if mlp["kind"] == "dense" else routed_ff(n2, W, p + "mlp.", mlp)
        x = x + f * torch.sigmoid(n2 @ W[p + "rg2"].T + W[p + "rg2.b"])
    return x


def forward(config, weights, tokens, dtype=torch.float64, residuals=None):
    """tokens: list of ids of ONE sequence from position 0 -> logits [T, vocab]."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    layers = config["layers"]
    x0 = W["embed"][torch.tensor(list(tokens), dtype=torch.long)]
    x = x0

    def run(span):
        nonlocal x
        for i in span:
            x = layer_forward(x, W, i, layers[i], eps)
            if residuals is not None:
                residuals.append(x.clone())

    loop = config.get("loop")
    if loop and int(loop["start"]) < int(loop["stop"]):
        a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
        run(range(a))
        for t in range(times):
            x = torch.cat([x, x0], dim=-1) @ W["loop.in"].T + W["loop.step"][t]
            run(range(a, b))
        run(range(b, len(layers)))
    else:
        run(range(len(layers)))
    return (offset_norm(x, W["final.norm"], eps) @ W["embed"].T) * float(config.get("logit_scale", 1.0))
