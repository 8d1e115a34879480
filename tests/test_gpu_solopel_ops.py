"""Each mechanism the Solopel stack adds to the ragged family alone: the HIP kernel against the plain restatement in
oracle/ref_solopel.py (fp64 on the CPU), on random inputs and on inputs built so that a fault shows (one key made
dominant on the last visible and the first invisible position, at page borders, far back among hundreds; scores far
beyond the soft cap; pages and slots dirtied before use; router scores that a softmax would weigh differently)."""
import math

import pytest
import torch

from oracle import ref_solopel as ref

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def ops():
    import micro_vllm_amd  # noqa: F401
    from micro_vllm_amd.kernel import ragged_ops
    return ragged_ops


def make_cache(kv=None, state=None, pages=16, slots=3, dtype=torch.float32, page=64, max_tokens=1024):
    from micro_vllm_amd.core.state_cache import HybridCacheManager
    return HybridCacheManager(pages, page, slots, kv or {}, state or {}, dtype=dtype, device=DEV, max_tokens=max_tokens,
                              max_rows=4, max_step_tokens=1024)


def step_of(cache, rows):
    cache.reserve([(sid, len(t)) for sid, t in rows])
    st = cache.plan(rows)
    cache.advance([(sid, len(t)) for sid, t in rows])
    return st


def feed(cache, plan, fn):
    """plan = [[(seq, count)]]: runs fn(step, {seq: (first position, count, first token of the step)}) per step."""
    at = {}
    for rows in plan:
        st = step_of(cache, [(k, [0] * c) for k, c in rows])
        where, o = {}, 0
        for k, c in rows:
            where[k] = (at.get(k, 0), c, o)
            at[k] = at.get(k, 0) + c
            o += c
        fn(st, where)


# ----------------------------------------------------------------------------------------------- row-wise steps
@pytest.mark.parametrize("f32", [False, True])
def test_gated_residual_norm(ops, f32):
    g = torch.Generator().manual_seed(1)
    dt = torch.float32 if f32 else torch.bfloat16
    tol = 1e-5 if f32 else 2e-2
    T, n, eps = 37, 203, 1e-5
    x0, y, gl = (torch.randn(T, n, generator=g) * 2 for _ in range(3))
    b, w = torch.randn(n, generator=g), 0.2 * torch.randn(n, generator=g)
    # operands may be column slices of wider buffers
    wide = torch.zeros(T, 2 * n + 3, device=DEV)
    wide[:, 3:3 + n] = gl.to(DEV)
    x, h, n32 = x0.to(DEV), torch.empty(T, n, dtype=dt, device=DEV), torch.empty(T, n, device=DEV)
    ops.gated_residual_norm(x, y.to(DEV), wide[:, 3:3 + n], b.to(DEV), w=w.to(DEV), eps=eps, offset=1.0, n32=n32, h=h)
    want_x = x0.double() + y.double() * torch.sigmoid(gl.double() + b.double())
    want_n = ref.offset_norm(want_x, w.double(), eps)
    assert (x.cpu().double() - want_x).abs().max().item() < 1e-5
    assert (n32.cpu().double() - want_n).abs().max().item() < 1e-5
    assert (h.float().cpu().double() - want_n).abs().max().item() < tol
    # the add alone (nothing normed), without a bias
    x = x0.to(DEV)
    ops.gated_residual_norm(x, y.to(DEV), gl.to(DEV), None)
    assert (x.cpu().double() - (x0.double() + y.double() * torch.sigmoid(gl.double()))).abs().max().item() < 1e-5
    # a pass of a looped span: the stream is replaced
    x = x0.to(DEV)
    ops.gated_residual_norm(x, y.to(DEV), None, b.to(DEV), True, w=w.to(DEV), eps=eps, offset=1.0, h=h)
    assert (x.cpu().double() - (y.double() + b.double())).abs().max().item() < 1e-6
    assert (h.float().cpu().double() - ref.offset_norm(y.double() + b.double(), w.double(), eps)).abs().max().item() < tol
    # the norm alone
    x = x0.to(DEV)
    ops.gated_residual_norm(x, w=w.to(DEV), eps=eps, offset=1.0, n32=n32)
    assert torch.equal(x.cpu(), x0) and (n32.cpu().double() - ref.offset_norm(x0.double(), w.double(), eps)).abs().max().item() < 1e-5


@pytest.mark.parametrize("f32", [False, True])
def test_cast_concat_gelu_scale(ops, f32):
    g = torch.Generator().manual_seed(2)
    dt = torch.float32 if f32 else torch.bfloat16
    T, n = 19, 150
    a, b = torch.randn(T, n, generator=g), torch.randn(T, n, generator=g)
    out = torch.empty(T, 2 * n, dtype=dt, device=DEV)
    ops.cast_concat(a.to(DEV), b.to(DEV), out)
    assert torch.equal(out.cpu(), torch.cat([a, b], dim=1).to(dt))
    v = torch.randn(T, n, generator=g) * 3
    o = torch.empty(T, n, dtype=dt, device=DEV)
    ops.gelu_tanh(v.to(DEV), o)
    assert (o.float().cpu().double() - ref.gelu_tanh(v.double())).abs().max().item() < (1e-5 if f32 else 5e-3 * v.abs().max().item())
    z = v.to(DEV).contiguous()
    ops.scale_(z, 0.3)
    assert (z.cpu() - v * 0.3).abs().max().item() < 1e-6


# ----------------------------------------------------------------------------------------------- convolutions
@pytest.mark.parametrize("taps", [1, 2, 4, 5])
@pytest.mark.parametrize("f32", [False, True])
def test_convolution_over_steps(ops, taps, f32):
    """Portions shorter and longer than the taps, single tokens, a sequence that takes over a slot whose tail is
    another sequence's: what lies before a sequence's start counts as zero."""
    g = torch.Generator().manual_seed(3 + taps)
    dt = torch.float32 if f32 else torch.bfloat16
    C = 70
    w = torch.randn(C, taps, generator=g)
    seqs = {k: torch.randn(n, C, generator=g) for k, n in (("a", 40), ("b", 9), ("c", 3))}
    cache = make_cache(kv={0: (1, 8, 8)}, state={0: {"tail": (taps - 1, C)}}, slots=2)
    cache.states[0]["tail"].fill_(7.0)        # whatever a slot held before
    got = {k: [] for k in seqs}

    def run(st, where):
        inp = torch.cat([seqs[k][p:p + c] for k, (p, c, _) in where.items()]).to(DEV)
        out32 = torch.empty(st.tokens, C, device=DEV)
        act = torch.empty(st.tokens, C, dtype=dt, device=DEV)
        ops.conv_taps(inp, cache.states[0]["tail"], w.to(DEV), st, out32=out32, out_act=act, add_input=True)
        assert (act.float() - out32).abs().max().item() < (1e-6 if f32 else 0.1)
        for k, (p, c, o) in where.items():
            got[k].append(out32[o:o + c].cpu().double())

    feed(cache, [[("a", 5), ("b", 1)], [("a", 1), ("b", 2)], [("a", 30), ("b", 1)], [("b", 5), ("a", 4)]], run)
    cache.free("b")
    feed(cache, [[("c", 1)], [("c", 2)]], run)   # takes b's slot
    for k, u in seqs.items():
        want = u.double() + ref.causal_conv(u.double(), w.double())
        assert (torch.cat(got[k]) - want).abs().max().item() < 1e-5, k
    # without the input added, fp32 only
    st = step_of(make_cache(kv={0: (1, 8, 8)}), [("z", [0] * 12)])
    out32 = torch.empty(12, C, device=DEV)
    ops.conv_taps(seqs["a"][:12].to(DEV), torch.zeros(3, max(taps - 1, 0), C, device=DEV), w.to(DEV), st, out32=out32)
    assert (out32.cpu().double() - ref.causal_conv(seqs["a"][:12].double(), w.double())).abs().max().item() < 1e-5


@pytest.mark.parametrize("taps", [0, 1, 3])
def test_convolution_of_queries_keys_values_into_pages(ops, taps):
    g = torch.Generator().manual_seed(11)
    H, G, d, dv = 3, 1, 8, 20
    cq, ck, cv = H * 2 * d, G * 2 * d, G * dv
    C = cq + ck + cv
    w = torch.randn(C, taps, generator=g) if taps else None
    u = torch.randn(150, C + 5, generator=g)             # the projection is wider than q | k | v
    cache = make_cache(kv={0: (G, 2 * d, dv)}, state={0: {"qkv": (max(taps - 1, 0), C)}})
    cache.k_caches[0].fill_(5.0)
    cache.v_caches[0].fill_(5.0)
    cache.states[0]["qkv"].fill_(3.0)
    qs, pages = [], None

    def run(st, where):
        nonlocal pages
        (p, c, _), = where.values()
        q = torch.empty(c, cq, device=DEV)
        ops.conv_qkv_store(u[p:p + c].to(DEV), cache.states[0]["qkv"], None if w is None else w.to(DEV), q,
                           cache.k_caches[0], cache.v_caches[0], st)
        qs.append(q.cpu().double())
        pages = st.block_table[0].cpu().tolist()

    feed(cache, [[("a", 2)], [("a", 1)], [("a", 70)], [("a", 77)]], run)
    x = u[:, :C].double()
    want = ref.causal_conv(x, w.double()) if taps else x
    assert (torch.cat(qs) - want[:, :cq]).abs().max().item() < 1e-5
    k = torch.cat([cache.k_caches[0][pg] for pg in pages[:3]]).view(-1, ck)[:150].cpu().double()
    v = torch.cat([cache.v_caches[0][pg] for pg in pages[:3]]).view(-1, cv)[:150].cpu().double()
    assert (k - want[:, cq:cq + ck]).abs().max().item() < 1e-5 and (v - want[:, cq + ck:]).abs().max().item() < 1e-5


# ----------------------------------------------------------------------------------------------- differential attention
def diff_case(ops, H, G, d, dv, dt, portions, q, k, v, gate, scale, cap, lam, diff, eps, tiled=True, pages=16):
    """q [T,H,2,d], k [T,G,2,d], v [T,G,dv] through pages dirtied before use, in the given portions."""
    T = q.shape[0]
    cache = make_cache(kv={0: (G, 2 * d, dv)}, dtype=dt, pages=pages)
    cache.k_caches[0].fill_(9.0)
    cache.v_caches[0].fill_(-9.0)
    qkv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1).float().to(DEV)
    outs = []

    def run(st, where):
        (p, c, _), = where.values()
        qq = torch.empty(c, H * 2 * d, device=DEV)
        ops.conv_qkv_store(qkv[p:p + c], None, None, qq, cache.k_caches[0], cache.v_caches[0], st)
        out = torch.empty(c, H * dv, dtype=dt, device=DEV)
        ops.diff_attn(qq, cache.k_caches[0], cache.v_caches[0], out, None if gate is None else gate[p:p + c].float().to(DEV),
                      st, H, G, d, dv, scale, cap, lam, 1.0 - diff, eps, tiled=tiled)
        outs.append(out.float().cpu().double())

    feed(cache, [[("a", c)] for c in portions], run)
    return torch.cat(outs).view(T, H, dv)


SHAPES = [(6, 2, 24, 40), (4, 2, 56, 72), (2, 1, 64, 64), (4, 1, 32, 64), (2, 2, 64, 128), (3, 3, 32, 32),
          (2, 1, 128, 128), (1, 1, 8, 200)]


@pytest.mark.parametrize("H,G,d,dv", SHAPES)
@pytest.mark.parametrize("f32", [False, True])
def test_differential_attention_whole_portions_decoded(ops, H, G, d, dv, f32):
    g = torch.Generator().manual_seed(H * 100 + d)
    dt = torch.float32 if f32 else torch.bfloat16
    T = 150
    q, k = torch.randn(T, H, 2, d, generator=g), torch.randn(T, G, 2, d, generator=g)
    v, gate = torch.randn(T, G, dv, generator=g), torch.randn(T, H, generator=g)
    if not f32:     # what the pages hold is what the restatement is given
        k, v = k.bfloat16().float(), v.bfloat16().float()
    scale, cap, lam, diff, eps = 0.3, 4.0, 0.45, 0.3, 1e-5
    want = ref.difference_attention(q.double(), k.double(), v.double(), gate.double(), scale, cap, lam, diff, eps)
    tol = 2e-5 if f32 else 2e-2      # bf16: q is rounded for the matrix cores, the output to the activation type
    for portions in ([150], [70, 2, 30, 17] + [1] * 31, [1] * 20 + [130]):
        got = diff_case(ops, H, G, d, dv, dt, portions, q, k, v, gate, scale, cap, lam, diff, eps)
        assert (got - want).abs().max().item() < tol * max(1.0, want.abs().max().item()), portions[:4]
    plain = diff_case(ops, H, G, d, dv, dt, [150], q, k, v, gate, scale, cap, lam, diff, eps, tiled=False)
    assert (plain - want).abs().max().item() < tol * max(1.0, want.abs().max().item())
    # no cap, no gate
    want = ref.difference_attention(q.double(), k.double(), v.double(), None, scale, 0.0, lam, diff, eps)
    got = diff_case(ops, H, G, d, dv, dt, [100, 50], q, k, v, None, scale, 0.0, lam, diff, eps)
    assert (got - want).abs().max().item() < tol * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("H,G,d,dv", [(2, 1, 24, 40), (2, 1, 64, 64)])
@pytest.mark.parametrize("f32", [False, True])
def test_differential_attention_one_key_stands_out(ops, H, G, d, dv, f32):
    """Each map of the last queries is made to look at ONE key: the first token of the sequence far back, the last
    key of a page, the first of the next, the query's own position (the last visible one); a dominant key one
    position AFTER a query must not be seen by it.  The two maps look at different keys, so their difference is the
    difference of two known value rows."""
    g = torch.Generator().manual_seed(17)
    dt = torch.float32 if f32 else torch.bfloat16
    T = 330
    q, k = torch.randn(T, H, 2, d, generator=g) * 0.1, torch.randn(T, G, 2, d, generator=g) * 0.1
    v = torch.randn(T, G, dv, generator=g).bfloat16().float()
    e1, e2 = torch.zeros(d), torch.zeros(d)
    e1[0], e2[1] = 1.0, 1.0
    targets = {300: (0, 63), 301: (64, 255), 302: (256, 302), 303: (303, 127), 329: (128, 0)}
    for j in {t for pair in targets.values() for t in pair}:
        k[j, :, 0] = 30.0 * e1 * (1 + j % 3)          # map 1 keys live on axis 0, map 2 keys on axis 1
        k[j, :, 1] = 30.0 * e2 * (1 + j % 3)
    k[304, :, 0] = 500.0 * e1                         # just after query 303: invisible to it
    k = k.bfloat16().float()
    scale, lam, diff, eps = 1.0, 0.5, 0.2, 1e-6
    for i, (j1, j2) in targets.items():
        q[i] = 0.0
        # a query that looks along -axis at everything except its target: subtract the others' pull by making the
        # target's score the largest by far
        q[i, :, 0] = e1 * 0.0
        q[i, :, 1] = e2 * 0.0
    # a direct construction: per query, scores are 30 (1 + j % 3) q0 on the marked keys; to single one key out, give it
    # a key of its own direction
    for n, (i, (j1, j2)) in enumerate(targets.items()):
        a1, a2 = torch.zeros(d), torch.zeros(d)
        a1[2 + 2 * n], a2[3 + 2 * n] = 1.0, 1.0
        k[j1, :, 0] = k[j1, :, 0] + 40.0 * a1
        k[j2, :, 1] = k[j2, :, 1] + 40.0 * a2
        q[i, :, 0], q[i, :, 1] = a1, a2
    k = k.bfloat16().float()
    want = ref.difference_attention(q.double(), k.double(), v.double(), None, scale, 0.0, lam, diff, eps)
    for i, (j1, j2) in targets.items():     # the construction does what it says
        o = v[j1, 0].double() - lam * v[j2, 0].double()
        assert (want[i, 0] - ref.rms_unit(o, eps) * (1 - diff)).abs().max().item() < 1e-6
    tol = 2e-5 if f32 else 2e-2
    for portions in ([330], [300, 1, 1, 1, 1, 26], [64, 64, 64, 64, 64, 10], [299, 2, 3, 26]):
        got = diff_case(ops, H, G, d, dv, dt, portions, q, k, v, None, scale, 0.0, lam, diff, eps)
        assert (got[290:] - want[290:]).abs().max().item() < tol * want.abs().max().item(), portions
    plain = diff_case(ops, H, G, d, dv, dt, [330], q, k, v, None, scale, 0.0, lam, diff, eps, tiled=False)
    assert (plain[290:] - want[290:]).abs().max().item() < tol * want.abs().max().item()


@pytest.mark.parametrize("f32", [False, True])
def test_soft_cap_flattens_large_scores(ops, f32):
    """Scores ten times the cap: every key weighs nearly the same, where uncapped scores would pick one."""
    g = torch.Generator().manual_seed(19)
    dt = torch.float32 if f32 else torch.bfloat16
    H, G, d, dv, T = 2, 2, 64, 64, 100
    q, k = torch.randn(T, H, 2, d, generator=g) * 3, (torch.randn(T, G, 2, d, generator=g) * 3).bfloat16().float()
    v = torch.randn(T, G, dv, generator=g).bfloat16().float()
    want = ref.difference_attention(q.double(), k.double(), v.double(), None, 1.0, 2.0, 0.3, 0.1, 1e-6)
    raw = ref.difference_attention(q.double(), k.double(), v.double(), None, 1.0, 0.0, 0.3, 0.1, 1e-6)
    assert (want - raw).abs().max().item() > 0.5
    for portions in ([100], [60] + [1] * 40):
        got = diff_case(ops, H, G, d, dv, dt, portions, q, k, v, None, 1.0, 2.0, 0.3, 0.1, 1e-6)
        assert (got - want).abs().max().item() < (2e-5 if f32 else 3e-2) * want.abs().max().item()


# ----------------------------------------------------------------------------------------------- latent attention
@pytest.mark.parametrize("H,d,dv,R", [(3, 40, 24, 72), (2, 64, 64, 64), (4, 32, 48, 128), (1, 16, 16, 33), (2, 32, 40, 256),
                                      (1, 64, 32, 512)])
@pytest.mark.parametrize("f32", [False, True])
def test_latent_attention_without_positions(ops, H, d, dv, R, f32):
    """The product path's sequence (latent into the page, queries carried into the latent space per head, attention
    over the cached latents, values expanded per head) against keys and values formed per head; one latent far back
    and one at a page border made dominant for the last queries."""
    g = torch.Generator().manual_seed(23 + R)
    dt = torch.float32 if f32 else torch.bfloat16
    T, eps, scale = 200, 1e-5, 0.3
    q = torch.randn(T, H * d, generator=g)
    dkv = torch.randn(T, R, generator=g)
    wn = 1.0 + 0.1 * torch.randn(R, generator=g)
    uk, uv = (torch.randn(H * d, R, generator=g) / math.sqrt(R)).to(dt), (torch.randn(H * dv, R, generator=g) / math.sqrt(R)).to(dt)
    # queries 198 and 199 are aimed at the keys of tokens 1 and 64 (head 0)
    c = ref.rms_unit(dkv.double(), eps) * wn.double()
    for i, j in ((198, 1), (199, 64)):
        kj = (c[j] @ uk.double().T).view(H, d)
        q[i] = (kj * 40.0 / (kj.norm(dim=-1, keepdim=True) ** 2 * scale)).reshape(-1).float() * 1.0
    if not f32:
        q = q.bfloat16().float()
    cache = make_cache(kv={0: (1, R, 0)}, dtype=dt)
    cache.k_caches[0].fill_(6.0)
    pages = cache.k_caches[0].view(cache.k_caches[0].shape[0], 64, R)
    uk_t = uk.view(H, d, R).transpose(1, 2).contiguous().to(DEV)
    uv_s = uv.view(H, dv, R).contiguous().to(DEV)
    outs = []

    def run(st, where):
        (p, n, _), = where.values()
        q_plain, q_abs = torch.empty(n, H * d, dtype=dt, device=DEV), torch.empty(n, H * R, device=DEV)
        ops.latent_prep(dkv[p:p + n].to(DEV), wn.to(DEV), eps, pages, q[p:p + n].to(DEV), q_plain, q_abs, None, st, H, d, 0,
                        R, 0, interleaved=False)
        ops.linear_heads(q_plain, uk_t, q_abs.view(n, H, R), H)
        lat = torch.empty(n, H * R, dtype=dt, device=DEV)
        ops.latent_attn(q_abs, pages, lat, st, None, H, R, 0, scale, 0)
        val = torch.empty(n, H * dv, device=DEV)
        ops.linear_heads(lat, uv_s, val.view(n, H, dv), H)
        outs.append(val.cpu().double())

    want = ref.latent_attention(q.double().view(T, H, d), c, uk.double(), uv.double(), scale).reshape(T, -1)
    kj = (c[1] @ uk.double().T).view(H, d)[0]
    assert float((kj @ q[198].double().view(H, d)[0]) * scale) > 30.0
    for portions in ([200], [100, 2, 60] + [1] * 38, [198, 1, 1]):
        outs.clear()
        cache.free("a")
        feed(cache, [[("a", n)] for n in portions], run)
        got = torch.cat(outs)
        assert (got - want).abs().max().item() < (3e-5 if f32 else 4e-2) * want.abs().max().item(), portions[:3]


# ----------------------------------------------------------------------------------------------- routed experts
@pytest.mark.parametrize("f32", [False, True])
@pytest.mark.parametrize("E,top", [(5, 2), (1, 1), (16, 1), (9, 4)])
def test_sigmoid_router_and_scaled_experts(ops, f32, E, top):
    g = torch.Generator().manual_seed(29 + E)
    dt = torch.float32 if f32 else torch.bfloat16
    T, n, ff = 45, 96, 40
    h = torch.randn(T, n, generator=g).to(dt)
    W = {"router": (torch.randn(E, n, generator=g) * 4 / math.sqrt(n)).to(dt).float()}
    for e in range(E):
        W[f"e{e}.gate"], W[f"e{e}.up"] = (torch.randn(ff, n, generator=g) / math.sqrt(n)).to(dt), (torch.randn(ff, n, generator=g) / math.sqrt(n)).to(dt)
        W[f"e{e}.down"] = (torch.randn(n, ff, generator=g) / math.sqrt(ff)).to(dt)
    W["shared.gate"], W["shared.up"] = (torch.randn(ff, n, generator=g) / math.sqrt(n)).to(dt), (torch.randn(ff, n, generator=g) / math.sqrt(n)).to(dt)
    W["shared.down"] = (torch.randn(n, ff, generator=g) / math.sqrt(ff)).to(dt)
    mlp = {"router": {"experts": E, "top": top}, "shared": {"ff": ff}}
    want = ref.routed_ff(h.double(), {k: v.double() for k, v in W.items()}, "", mlp)
    hd = h.to(DEV)
    ids = torch.empty(T, top, dtype=torch.int32, device=DEV)
    wts = torch.empty(T, top, device=DEV)
    ops.moe_route_sigmoid(hd, W["router"].to(DEV), ids, wts)
    s = torch.sigmoid(h.double() @ W["router"].double().T)
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        assert ids[t].tolist() == order
        assert (wts[t].cpu().double() - s[t, order]).abs().max().item() < 1e-5
    seg, order_, place = (torch.empty(m, dtype=torch.int32, device=DEV) for m in (E + 1, T * top, T * top))
    ops.moe_plan(ids, seg, order_, place, E)
    e_gu = torch.stack([torch.cat([W[f"e{e}.gate"], W[f"e{e}.up"]]) for e in range(E)]).to(DEV)
    e_down = torch.stack([W[f"e{e}.down"] for e in range(E)]).to(DEV)
    gu = ops.linear_segments(hd, e_gu, torch.empty(T * top, 2 * ff, device=DEV), seg, order_, top, T)
    act = torch.empty(T * top, ff, dtype=dt, device=DEV)
    ops.gated_act_scaled(gu, act, ops.GATE_SILU, wts.view(-1), order_)
    down = ops.linear_segments(act, e_down, torch.empty(T * top, n, device=DEV), seg, None, 1, T)
    sgu = torch.cat([W["shared.gate"], W["shared.up"]]).to(DEV).float() if f32 else torch.cat([W["shared.gate"], W["shared.up"]]).to(DEV)
    s_lin = ops.AnyLinear(sgu, wave_tiles=False)
    s_act = torch.empty(T, ff, dtype=dt, device=DEV)
    ops.silu_mul(s_lin(hd), s_act)
    s_out = ops.AnyLinear(W["shared.down"].to(DEV), wave_tiles=False)(s_act)
    y = torch.empty(T, n, device=DEV)
    ops.moe_combine(down, place, None, s_out, None, y)
    assert (y.cpu().double() - want).abs().max().item() < (2e-5 if f32 else 4e-2) * max(1.0, want.abs().max().item())
