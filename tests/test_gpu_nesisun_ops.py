"""Each mechanism the Nesisun stack adds to the ragged family alone: the HIP kernel against the plain restatement
in oracle/ref_nesisun.py (fp64 on the CPU), on random inputs and on inputs built so that a fault shows (one key made
dominant just inside / just outside the window and the kept first positions, at page borders, far back among
hundreds; a sink that outweighs every key; pages dirtied before use; a correction that overturns the router's
choice)."""
import math

import pytest
import torch

from oracle import ref_nesisun as ref

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def ops():
    import micro_vllm_amd  # noqa: F401
    from micro_vllm_amd.kernel import ragged_ops
    return ragged_ops


def make_cache(kv=None, pages=16, slots=3, dtype=torch.float32, page=64, max_tokens=512):
    from micro_vllm_amd.core.state_cache import HybridCacheManager
    return HybridCacheManager(pages, page, slots, kv or {}, {}, dtype=dtype, device=DEV, max_tokens=max_tokens, max_rows=4,
                              max_step_tokens=1024)


def step_of(cache, rows):
    cache.reserve([(sid, len(t)) for sid, t in rows])
    st = cache.plan(rows)
    cache.advance([(sid, len(t)) for sid, t in rows])
    return st


# ----------------------------------------------------------------------------------------------- row-wise steps
@pytest.mark.parametrize("f32", [False, True])
@pytest.mark.parametrize("buckets,mul_prev,mul_cur", [(97, 31, 7), (1, 1, 1), (100003, 1000003, 0)])
def test_pair_hashed_embedding_over_steps(ops, f32, buckets, mul_prev, mul_cur):
    g = torch.Generator().manual_seed(5)
    dt = torch.float32 if f32 else torch.bfloat16
    V, n = 211, 70
    embed = torch.randn(V, n, generator=g).to(dt)
    table = torch.randn(buckets + 1, n, generator=g).to(dt)
    seqs = {"a": torch.randint(0, V, (40,), generator=g).tolist(), "b": torch.randint(0, V, (9,), generator=g).tolist(),
            "c": [V - 1, V - 1, 0]}
    cache = make_cache(kv={0: (1, 8, 8)})
    # portions of unequal length side by side, single tokens among them, a sequence that starts later
    plan = [[("a", 5), ("b", 1)], [("a", 1), ("b", 2), ("c", 3)], [("a", 30), ("b", 1)], [("b", 5), ("a", 4)]]
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    for rows in plan:
        st = step_of(cache, [(k, seqs[k][at[k]:at[k] + c]) for k, c in rows])
        x = torch.full((st.tokens, n), 9.0, device=DEV)
        ops.embed_pair(embed.to(DEV), table.to(DEV), st.ids, st.tok_prev, x, 2.5, buckets, mul_prev, mul_cur)
        o = 0
        for k, c in rows:
            got[k].append(x[o:o + c].cpu().double())
            o += c
            at[k] += c
    for k, toks in seqs.items():
        want = ref.pair_embedding(toks, embed.double(), table.double(), 2.5, buckets, mul_prev, mul_cur)
        assert (torch.cat(got[k]) - want).abs().max().item() < 1e-6, k
    # with the first layer's norm out of the same launch
    w = 1.0 + 0.2 * torch.randn(n, generator=g)
    ids = torch.tensor(seqs["a"], dtype=torch.int32, device=DEV)
    prev = torch.tensor([-1] + seqs["a"][:-1], dtype=torch.int32, device=DEV)
    x, h = torch.empty(40, n, device=DEV), torch.empty(40, n, dtype=dt, device=DEV)
    ops.embed_pair(embed.to(DEV), table.to(DEV), ids, prev, x, 2.5, buckets, mul_prev, mul_cur, w=w.to(DEV), eps=1e-5, h=h)
    want = ref.pair_embedding(seqs["a"], embed.double(), table.double(), 2.5, buckets, mul_prev, mul_cur)
    assert (x.cpu().double() - want).abs().max().item() < 1e-6
    assert (h.float().cpu().double() - ref.rms_norm(want, w.double(), 1e-5)).abs().max().item() < (1e-5 if f32 else 3e-2)
    # a sequence that ends gives its slot to the next one, which starts without a predecessor
    cache.free("c")
    st = step_of(cache, [("d", [7, 8])])
    x = torch.empty(2, n, device=DEV)
    ops.embed_pair(embed.to(DEV), table.to(DEV), st.ids, st.tok_prev, x, 2.5, buckets, mul_prev, mul_cur)
    assert (x.cpu().double() - ref.pair_embedding([7, 8], embed.double(), table.double(), 2.5, buckets, mul_prev, mul_cur)).abs().max().item() < 1e-6


def test_pair_hash_of_large_factors_matches_exact_integers(ops):
    """Multipliers near 2^31 and a bucket count near 2^24: the row index equals the exact integer hash.  A one-column
    fp32 table whose row j holds j mod 65536 reads the index back."""
    buckets, mul_prev, mul_cur = 16777213, 2147483629, 2147483587
    V = 50000
    table = (torch.arange(buckets + 1, dtype=torch.int32) % 65536).float().view(-1, 1).to(DEV)
    embed = torch.zeros(V, 1, device=DEV)
    ids = torch.tensor([49999, 1, 31337, 0, 49998], dtype=torch.int32, device=DEV)
    prev = torch.tensor([49998, 49999, 12345, -1, 49999], dtype=torch.int32, device=DEV)
    x = torch.empty(5, 1, device=DEV)
    ops.embed_pair(embed, table, ids, prev, x, 1.0, buckets, mul_prev, mul_cur)
    want = [buckets if p < 0 else (p * mul_prev + t * mul_cur) % buckets for p, t in zip(prev.tolist(), ids.tolist())]
    assert x.view(-1).cpu().tolist() == [float(w % 65536) for w in want]


@pytest.mark.parametrize("f32", [False, True])
def test_rowwise_steps(ops, f32):
    g = torch.Generator().manual_seed(7)
    dt = torch.float32 if f32 else torch.bfloat16
    tol = 1e-5 if f32 else 2e-2
    T, n, eps = 37, 203, 1e-5
    x0, y1, y2 = (torch.randn(T, n, generator=g) * 2 for _ in range(3))
    w = 1.0 + 0.2 * torch.randn(n, generator=g)
    # the two sublayers enter the stream, the next norm comes out; operands may be column slices of wider buffers
    wide = torch.zeros(T, 2 * n + 3, device=DEV)
    wide[:, 3:3 + n] = y1.to(DEV)
    x, h = x0.to(DEV), torch.empty(T, n, dtype=dt, device=DEV)
    ops.add_rmsnorm(x, wide[:, 3:3 + n], y2.to(DEV), w=w.to(DEV), eps=eps, h=h)
    want_x = x0.double() + (y1.double() + y2.double())
    assert (x.cpu().double() - want_x).abs().max().item() < 1e-5
    assert (h.float().cpu().double() - ref.rms_norm(want_x, w.double(), eps)).abs().max().item() < tol
    x = x0.to(DEV)
    ops.add_rmsnorm(x, y1.to(DEV))                                          # one sublayer, no norm (the last layer)
    assert (x.cpu().double() - (x0.double() + y1.double())).abs().max().item() < 1e-5
    x = x0.to(DEV)
    ops.add_rmsnorm(x, w=w.to(DEV), eps=eps, h=h)                           # the norm alone (after the embedding)
    assert torch.equal(x.cpu(), x0)
    assert (h.float().cpu().double() - ref.rms_norm(x0.double(), w.double(), eps)).abs().max().item() < tol
    # the final norm on chosen rows
    idx = torch.tensor([5, 0, 36, 5], dtype=torch.int32, device=DEV)
    out = torch.empty(4, n, dtype=dt, device=DEV)
    ops.rmsnorm_gather(x0.to(DEV), idx, w.to(DEV), eps, out)
    assert (out.float().cpu().double() - ref.rms_norm(x0.double()[[5, 0, 36, 5]], w.double(), eps)).abs().max().item() < tol
    # gated activations on [gate | up]
    ff = 150
    a = torch.randn(T, 2 * ff, generator=g) * 3
    gate, up = a[:, :ff].double(), a[:, ff:].double()
    act = torch.empty(T, ff, dtype=dt, device=DEV)

    def close(want):      # bf16: one rounding of the result
        err = (act.float().cpu().double() - want).abs()
        return bool((err <= (1e-5 if f32 else 2.0 ** -8 * want.abs() + 1e-6)).all())

    ops.gated_act(a.to(DEV), act, ops.GATE_GELU_TANH)
    assert close(ref.gelu_tanh(gate) * up)
    for limit in (0.7, 2.0, 50.0):
        ops.gated_act(a.to(DEV), act, ops.GATE_CLAMPED, limit, 1.702)
        gc, uc = gate.clamp(max=limit), up.clamp(-limit, limit)
        assert close(gc * torch.sigmoid(1.702 * gc) * (uc + 1))
    ops.gated_act(a.to(DEV), act, ops.GATE_SILU)
    assert close(torch.nn.functional.silu(gate) * up)


# ------------------------------------------------------------------------------------------------- attention
def attn_case(g, T, H, G, d):
    return (torch.randn(T, (H + G) * d, generator=g), torch.randn(H * d, generator=g) * 0.3,
            torch.randn(G * d, generator=g) * 0.3)


def attn_reference(qk, qb, kb, H, G, d, rot, base, scale, window, keep, sink):
    T = qk.shape[0]
    q = (qk[:, :H * d].double() + qb.double()).view(T, H, d)
    k = (qk[:, H * d:].double() + kb.double()).view(T, G, d)
    pos = torch.arange(T)
    s = torch.full((H,), -1e9, dtype=torch.float64) if sink is None else sink.double()
    return ref.sink_attention(ref.rotate_adjacent(q, pos, rot, base), ref.rotate_adjacent(k, pos, rot, base), k, scale,
                              window, keep, s)


def attn_run(ops, cache, sid, lo, hi, qk, qb, kb, H, G, d, rot, base, scale, window, keep, sink, dt, tiled=True, splits=0):
    """Tokens lo .. hi of sequence `sid` through bias / rotation / store and the attention kernel.  `splits` > 0: the
    tokens of short rows take the kernel that shares reads among the query heads of a key/value head, the keys cut
    into that many pieces (more pieces than there are tiles leave some of them empty)."""
    T = hi - lo
    st = step_of(cache, [(sid, [0] * T)])
    inv = (base ** (-2.0 * torch.arange(max(rot // 2, 1), dtype=torch.float64) / max(rot, 1))).to(DEV)
    wide = torch.zeros(T, (H + G) * d + 16, device=DEV)          # the projection's output carries more columns
    wide[:, :(H + G) * d] = qk[lo:hi].to(DEV)
    x = wide[:, :(H + G) * d]
    kc, vc = cache.k_caches[0], cache.v_caches[0]
    ops.qk_rotary_store(x, qb.to(DEV), kb.to(DEV), kc, vc, inv, st, H, G, d, rot)
    out = torch.empty(T, H * d + 8, dtype=dt, device=DEV)[:, :H * d]
    part = torch.full((T * H * splits * (d + 2),), float("nan"), device=DEV) if splits else None
    ops.window_attn(x, kc, vc, out, st, None, H, G, d, d, scale, window, tiled=tiled, keep_first=keep,
                    sinks=None if sink is None else sink.to(DEV), part=part, splits=splits)
    return out.float().cpu().double().view(T, H, d)


SHAPES = [
    # H, G, d, rot, window, keep
    (6, 2, 40, 24, 37, 5),        # odd sizes, rotation over a part of the head
    (4, 1, 24, 8, 70, 66),        # kept positions reach into the second page and nearly to the window
    (3, 3, 56, 56, 3, 1),         # as many key heads as query heads, a tiny window
    (2, 2, 64, 64, 64, 0),        # a shape the matrix-core kernel takes: window = page, nothing kept
    (4, 2, 32, 0, 100, 64),       # no rotation, a page of kept positions
    (2, 1, 128, 128, 75, 20),
    (4, 1, 96, 32, 20, 70),       # more kept positions than the window is long
    (2, 2, 256, 16, 50, 3),       # four value columns a lane
]


@pytest.mark.parametrize("f32", [False, True])
@pytest.mark.parametrize("H,G,d,rot,window,keep", SHAPES)
def test_attention_whole_portions_and_decoding(ops, f32, H, G, d, rot, window, keep):
    g = torch.Generator().manual_seed(H * 10 + d)
    dt = torch.float32 if f32 else torch.bfloat16
    T, scale, base = 200, 0.6 * d ** -0.5, 5000.0
    qk, qb, kb = attn_case(g, T, H, G, d)
    sink = torch.randn(H, generator=g) * 2
    want = attn_reference(qk, qb, kb, H, G, d, rot, base, scale, window, keep, sink)
    tol = 3e-5 if f32 else 4e-2
    args = (qk, qb, kb, H, G, d, rot, base, scale, window, keep, sink, dt)
    cache = make_cache(kv={0: (G, d, d)}, dtype=dt)
    cache.k_caches[0].fill_(50.0)                     # pages are not cleared: nothing unwritten may be read
    cache.v_caches[0].fill_(-50.0)
    whole = attn_run(ops, cache, "w", 0, T, *args)
    assert (whole - want).abs().max().item() < tol
    cache.free("w")
    if not f32:                                       # the plain kernel on the same prompt
        plain = attn_run(ops, cache, "n", 0, T, *args, tiled=False)
        assert (plain - want).abs().max().item() < tol
        cache.free("n")
    # portions cut inside a page, the window and the kept positions, down to two tokens, then token by token; the
    # pages are used again
    parts, at = [], 0
    for n in [61, 2, 3, 40, 2, 17, 50] + [1] * 25:
        parts.append(attn_run(ops, cache, "p", at, at + n, *args))
        at += n
    got = torch.cat(parts)
    assert at == T and (got - want).abs().max().item() < tol
    if f32:
        assert (got - whole).abs().max().item() < 1e-5
    cache.free("p")
    # the same portions with the short rows on the kernel that shares reads among query heads: uncut, cut in three,
    # and cut as the library would choose for a step of that many tokens
    for splits in (1, 3, None):
        parts, at = [], 0
        for n in [61, 2, 3, 40, 2, 17, 50] + [1] * 25:
            sp = splits or ops.window_attn_splits(n, H, G, window, keep)
            parts.append(attn_run(ops, cache, "g", at, at + n, *args, splits=sp))
            at += n
        got = torch.cat(parts)
        assert (got - want).abs().max().item() < tol, splits
        cache.free("g")
    # every row short (also the first portions), so that all of it runs there; and the whole prompt at once (fp32, or
    # with the matrix-core kernel switched off)
    parts = [attn_run(ops, cache, "s", at, min(at + 16, T), *args, splits=2) for at in range(0, T, 16)]
    assert (torch.cat(parts) - want).abs().max().item() < tol
    cache.free("s")
    assert (attn_run(ops, cache, "a", 0, T, *args, tiled=False, splits=1) - want).abs().max().item() < tol


def dominant_case(g, T, H, G, d, rot, key, query, amp=40.0):
    """Key `key` and query `query` made large along the last dimension of a head - unrotated where rot < d, else the
    slowest pair, which a base of 1e6 hardly turns: that key takes all the weight wherever it is visible, and since
    values are keys the output is then that key."""
    qk, qb, kb = attn_case(g, T, H, G, d)
    qk.view(T, H + G, d)[key, H:, d - 2] = amp
    qk.view(T, H + G, d)[query, :H, d - 2] = amp
    return qk, qb, kb


@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("query,window,keep", [(70, 7, 0), (100, 37, 3), (128, 64, 2), (129, 65, 64), (140, 100, 20), (63, 64, 0),
                                               (64, 64, 1), (191, 128, 5), (192, 128, 63)])
def test_window_edge_with_a_dominant_key(ops, query, window, keep, f32):
    """The dominant key on the last visible position of the window and on the first invisible one, the query in a
    prompt and decoded alone."""
    H, G, d, rot, base, scale = (4, 2, 24, 24, 1e6, 0.5) if f32 else (4, 2, 64, 32, 1e6, 0.25)
    # bf16: a smaller peak (its score still stands 25 above the rest), so that what rounding q and k costs the OTHER
    # queries' sharp softmaxes stays small
    dt, tol, amp = (torch.float32, 3e-5, 40.0) if f32 else (torch.bfloat16, 0.25, 12.0)
    for inside in (True, False):
        key = query - window + 1 if inside else query - window
        if key < keep:
            continue
        g = torch.Generator().manual_seed(query + window)
        T = query + 1
        qk, qb, kb = dominant_case(g, T, H, G, d, rot, key, query, amp)
        args = (qk, qb, kb, H, G, d, rot, base, scale, window, keep, None, dt)
        want = attn_reference(*args[:-1])
        k_key = (qk[key, H * d:].double() + kb.double()).view(G, d)
        seen = (want[query] - k_key.repeat_interleave(H // G, 0)).abs().max().item() < 1e-3
        assert seen == inside                              # the case is what it claims to be
        cache = make_cache(kv={0: (G, d, d)}, dtype=dt)
        whole = attn_run(ops, cache, "w", 0, T, *args)
        assert (whole - want).abs().max().item() < tol
        assert ((whole[query] - k_key.repeat_interleave(H // G, 0)).abs().max().item() < max(0.1, tol)) == inside
        cache.free("w")
        first = attn_run(ops, cache, "p", 0, query, *args)
        last = attn_run(ops, cache, "p", query, T, *args)
        assert (torch.cat([first, last]) - want).abs().max().item() < tol
        cache.free("p")
        first = attn_run(ops, cache, "g", 0, query, *args, splits=1)
        last = attn_run(ops, cache, "g", query, T, *args, splits=2)
        assert (torch.cat([first, last]) - want).abs().max().item() < tol


@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("keep,window", [(1, 5), (5, 17), (20, 40), (64, 30), (65, 64), (70, 3), (128, 10)])
def test_kept_first_positions_with_a_dominant_key(ops, keep, window, f32):
    """Far behind the window: the dominant key on the last kept position (seen from anywhere, at its true position)
    and on the first position that is not kept (forgotten once the window has passed)."""
    H, G, d, rot, base, scale = (4, 1, 24, 8, 1e6, 0.5) if f32 else (2, 2, 128, 128, 1e6, 0.25)
    dt, tol, amp = (torch.float32, 3e-5, 40.0) if f32 else (torch.bfloat16, 0.25, 12.0)
    query = keep + window + 90
    T = query + 1
    for inside in (True, False):
        key = keep - 1 if inside else keep
        g = torch.Generator().manual_seed(keep + window)
        qk, qb, kb = dominant_case(g, T, H, G, d, rot, key, query, amp)
        args = (qk, qb, kb, H, G, d, rot, base, scale, window, keep, torch.zeros(H), dt)
        want = attn_reference(*args[:-1])
        k_key = (qk[key, H * d:].double() + kb.double()).view(G, d).repeat_interleave(H // G, 0)
        assert ((want[query] - k_key).abs().max().item() < 1e-3) == inside
        cache = make_cache(kv={0: (G, d, d)}, dtype=dt)
        whole = attn_run(ops, cache, "w", 0, T, *args)
        assert (whole - want).abs().max().item() < tol
        assert ((whole[query] - k_key).abs().max().item() < max(0.1, tol)) == inside
        cache.free("w")
        # the prompt cut right behind the kept positions and in the middle of nowhere, the query decoded alone
        cuts = [keep + 1, 2, window + 50]
        parts, at = [], 0
        for n in cuts + [T - 1 - sum(cuts)] + [1]:
            parts.append(attn_run(ops, cache, "p", at, at + n, *args))
            at += n
        assert at == T and (torch.cat(parts) - want).abs().max().item() < tol
        cache.free("p")
        parts, at = [], 0
        for n in cuts + [T - 1 - sum(cuts)] + [1]:
            parts.append(attn_run(ops, cache, "g", at, at + n, *args, splits=1 + at % 3))
            at += n
        assert (torch.cat(parts) - want).abs().max().item() < tol


def test_far_kept_key_among_hundreds_and_heavy_sink(ops):
    """The sequence's second token, 440 positions back and far outside the window, takes the weight of queries that are
    decoded one by one.  With a sink far above every score the output shrinks towards zero by exactly its share."""
    H, G, d, rot, base = 2, 1, 24, 24, 1e6
    g = torch.Generator().manual_seed(11)
    T = 450
    qk, qb, kb = attn_case(g, T, H, G, d)
    qk.view(T, H + G, d)[1, H:, d - 2] = 40.0
    qk.view(T, H + G, d)[440:, :H, d - 2] = 40.0
    args = [qk, qb, kb, H, G, d, rot, base, 0.5, 50, 3, None, torch.float32]
    want = attn_reference(*args[:-1])
    cache = make_cache(kv={0: (G, d, d)})
    first = attn_run(ops, cache, "p", 0, 441, *args)
    rest = [attn_run(ops, cache, "p", t, t + 1, *args, splits=t % 4) for t in range(441, T)]
    got = torch.cat([first] + rest)
    assert (got - want).abs().max().item() < 3e-5
    k1 = (qk[1, H * d:].double() + kb.double()).view(G, d)
    assert (got[445] - k1).abs().max().item() < 1e-3
    cache.free("p")
    args[8], args[11] = 0.1, torch.tensor([14.0, -30.0])
    want = attn_reference(*args[:-1])
    got = attn_run(ops, cache, "s", 0, 200, *args)
    assert (got - want[:200]).abs().max().item() < 3e-5
    assert got[150, 0].abs().max().item() < 1e-2 * got[150, 1].abs().max().item()
    for at, splits in ((200, 1), (210, 2)):      # the sink where the waves' and the splits' pieces meet
        late = attn_run(ops, cache, "s", at, at + 10, *args, splits=splits)
        assert (late - want[at:at + 10]).abs().max().item() < 3e-5
    # the same through the matrix-core kernel (bf16, a shape it takes)
    H, G, d, rot = 2, 2, 64, 64
    qk, qb, kb = attn_case(g, 200, H, G, d)
    args = [qk, qb, kb, H, G, d, rot, base, 0.1, 50, 3, torch.tensor([14.0, -30.0]), torch.bfloat16]
    want = attn_reference(*args[:-1])
    cache = make_cache(kv={0: (G, d, d)}, dtype=torch.bfloat16)
    got = attn_run(ops, cache, "t", 0, 200, *args)
    assert (got - want).abs().max().item() < 4e-2
    assert got[150, 0].abs().max().item() < 2e-2 * got[150, 1].abs().max().item()


def test_values_are_the_keys_before_rotation(ops):
    """What lands in the value page is the key with its bias and WITHOUT rotation; the key page holds the rotated one."""
    H, G, d, rot, base = 2, 2, 16, 8, 100.0
    g = torch.Generator().manual_seed(3)
    T = 70
    qk, qb, kb = attn_case(g, T, H, G, d)
    cache = make_cache(kv={0: (G, d, d)})
    attn_run(ops, cache, "v", 0, T, qk, qb, kb, H, G, d, rot, base, 0.3, 9, 2, None, torch.float32)
    k = (qk[:, H * d:].double() + kb.double()).view(T, G, d)
    pages = cache.get_blocks("v")
    vals = torch.cat([cache.v_caches[0][p] for p in pages])[:T].cpu().double()
    keys = torch.cat([cache.k_caches[0][p] for p in pages])[:T].cpu().double()
    assert (vals - k).abs().max().item() < 1e-6
    assert (keys - ref.rotate_adjacent(k, torch.arange(T), rot, base)).abs().max().item() < 1e-5
    assert (keys[5] - vals[5]).abs().max().item() > 0.1 and torch.equal(keys[:, :, rot:], vals[:, :, rot:])
    # the same launch with a feed-forward's gate | up columns behind q and k: both results as from separate launches
    ff = 150
    for dt in (torch.float32, torch.bfloat16):
        c2 = make_cache(kv={0: (G, d, d)}, dtype=dt)
        st = step_of(c2, [("x", [0] * T)])
        inv = (base ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot)).to(DEV)
        proj = torch.cat([qk, torch.randn(T, 2 * ff, generator=g) * 3], dim=1).to(DEV)
        both, alone = torch.empty(T, 8 + ff, dtype=dt, device=DEV)[:, 8:], torch.empty(T, ff, dtype=dt, device=DEV)
        ops.gated_act(proj[:, (H + G) * d:], alone, ops.GATE_GELU_TANH)
        x = proj.clone()
        ops.qk_rotary_store(x[:, :(H + G) * d], qb.to(DEV), kb.to(DEV), c2.k_caches[0], c2.v_caches[0], inv, st, H, G, d, rot,
                            act=(x[:, (H + G) * d:], both, ops.GATE_GELU_TANH, 0.0, 1.0))
        assert torch.equal(both, alone)
        pg = c2.get_blocks("x")
        k2 = torch.cat([c2.k_caches[0][p] for p in pg])[:T].float().cpu().double()
        assert (k2 - ref.rotate_adjacent(k, torch.arange(T), rot, base)).abs().max().item() < (1e-5 if dt == torch.float32 else 3e-2)
        q2 = x[:, :H * d].cpu().double().view(T, H, d)
        qw = ref.rotate_adjacent((qk[:, :H * d].double() + qb.double()).view(T, H, d), torch.arange(T), rot, base)
        assert (q2 - qw).abs().max().item() < 1e-5


@pytest.mark.parametrize("f32", [True, False])
def test_rotation_over_a_step_of_many_tokens(ops, f32):
    """Steps of many tokens form a position's sines and cosines once for several heads (a wave takes eight of them, a
    last group of fewer): queries in place, keys and values in their pages, all as head by head."""
    H, G, d, rot, base = 9, 3, 40, 24, 5000.0          # twelve heads: a group of eight and one of four
    dt = torch.float32 if f32 else torch.bfloat16
    g = torch.Generator().manual_seed(9)
    T = 700
    qk, qb, kb = attn_case(g, T, H, G, d)
    cache = make_cache(kv={0: (G, d, d)}, dtype=dt, max_tokens=1024)
    cache.k_caches[0].fill_(7.0)
    parts = []
    for lo, hi in ((0, 690), (690, 700)):              # the long step, then a short one (a wave per head) behind it
        st = step_of(cache, [("r", [0] * (hi - lo))])
        inv = (base ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / rot)).to(DEV)
        x = qk[lo:hi].to(DEV).clone()
        ops.qk_rotary_store(x, qb.to(DEV), kb.to(DEV), cache.k_caches[0], cache.v_caches[0], inv, st, H, G, d, rot)
        parts.append(x[:, :H * d].cpu().double())
    pos = torch.arange(T)
    k = (qk[:, H * d:].double() + kb.double()).view(T, G, d)
    q = (qk[:, :H * d].double() + qb.double()).view(T, H, d)
    pages = cache.get_blocks("r")
    vals = torch.cat([cache.v_caches[0][p] for p in pages])[:T].float().cpu().double()
    keys = torch.cat([cache.k_caches[0][p] for p in pages])[:T].float().cpu().double()
    tol = 1e-5 if f32 else 3e-2
    assert (torch.cat(parts).view(T, H, d) - ref.rotate_adjacent(q, pos, rot, base)).abs().max().item() < 1e-5
    assert (keys - ref.rotate_adjacent(k, pos, rot, base)).abs().max().item() < tol
    assert (vals - k).abs().max().item() < tol


# ---------------------------------------------------------------------------------------------------- experts
@pytest.mark.parametrize("f32", [False, True])
@pytest.mark.parametrize("E,n_id,top", [(5, 2, 3), (4, 0, 1), (1, 1, 2), (12, 3, 4), (40, 1, 6), (2, 4, 2)])
def test_routed_experts_with_pass_through(ops, f32, E, n_id, top):
    g = torch.Generator().manual_seed(E + top)
    dt = torch.float32 if f32 else torch.bfloat16
    T, W, ff, limit, scale = 37, 96, 40, 1.1, 1.7
    h = torch.randn(T, W, generator=g).to(dt)
    Wt = {"router": (torch.randn(E + n_id, W, generator=g) * 0.3).to(torch.bfloat16).float(),
          # a correction of the scores' own size: it overturns the order of the plain scores for many tokens
          "correction": (torch.randn(E + n_id, generator=g) * 0.2).to(torch.bfloat16).float()}
    for e in range(E):
        Wt[f"e{e}.gate"], Wt[f"e{e}.up"] = (torch.randn(ff, W, generator=g).to(dt).float() * 2 / math.sqrt(W) for _ in range(2))
        Wt[f"e{e}.down"] = torch.randn(W, ff, generator=g).to(dt).float() / math.sqrt(ff)
    mlp = {"router": {"experts": E, "identity": n_id, "top": top, "scale": scale}, "expert": {"ff": ff, "limit": limit}}
    want = ref.routed_with_identity(h.double(), {k: v.double() for k, v in Wt.items()}, "", mlp)
    hd = h.to(DEV)
    ids = torch.empty(T, top, dtype=torch.int32, device=DEV)
    wts = torch.empty(T, top, device=DEV)
    ops.moe_route_scored(hd, Wt["router"].to(DEV), Wt["correction"].to(DEV), ids, wts, scale, 1e-20)
    s = torch.softmax(h.double() @ Wt["router"].double().T, dim=-1)
    pick = (s + Wt["correction"].double()).topk(top, dim=1).indices
    assert torch.equal(ids.cpu().long().sort(dim=1).values, pick.sort(dim=1).values)
    if E + n_id > top:
        assert not torch.equal(pick.sort(dim=1).values, s.topk(top, dim=1).indices.sort(dim=1).values)   # the correction matters
    chosen = s.gather(1, ids.cpu().long())
    assert (wts.cpu().double() - chosen / chosen.sum(1, keepdim=True) * scale).abs().max().item() < 1e-5
    seg, order, place = (torch.empty(c, dtype=torch.int32, device=DEV) for c in (E + n_id + 1, T * top, T * top))
    ops.moe_plan(ids, seg, order, place, E + n_id)
    e_gu = torch.stack([torch.cat([Wt[f"e{e}.gate"], Wt[f"e{e}.up"]]) for e in range(E)]).to(dt).to(DEV)
    e_down = torch.stack([Wt[f"e{e}.down"] for e in range(E)]).to(dt).to(DEV)
    down = torch.full((T * top, W), float("nan"), device=DEV)          # rows of pass-through choices are never read
    gu = ops.linear_segments(hd, e_gu, torch.empty(T * top, 2 * ff, device=DEV), seg[:E + 1], order, top, T)
    act = torch.empty(T * top, ff, dtype=dt, device=DEV)
    ops.gated_act(gu, act, ops.GATE_CLAMPED, limit, 1.702)
    ops.linear_segments(act, e_down, down, seg[:E + 1], None, 1, T)
    y = torch.empty(T, W, device=DEV)
    ops.moe_combine(down, place, wts, None, None, y, ids=ids.view(-1), first_pass=E, passed=hd)
    assert (y.cpu().double() - want).abs().max().item() < (3e-5 if f32 else 4e-2)
