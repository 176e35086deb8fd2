"""Each mechanism the Fagunex stack adds to the ragged family alone: the HIP kernel against the plain
restatement in oracle/ref_fagunex.py (fp64 on the CPU), on random inputs and on inputs built so that a
fault shows (one key made dominant just inside / just outside a window, at a page border, far back; a
sink that outweighs every key; state slots dirtied before use)."""
import math

import pytest
import torch

from oracle import ref_fagunex as ref

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def ops():
    import micro_vllm_amd  # noqa: F401
    from micro_vllm_amd.kernel import ragged_ops
    return ragged_ops


def make_cache(kv=None, state=None, pages=16, slots=3, dtype=torch.float32, page=64, max_tokens=512):
    from micro_vllm_amd.core.state_cache import HybridCacheManager
    return HybridCacheManager(pages, page, slots, kv or {}, state or {}, dtype=dtype, device=DEV, max_tokens=max_tokens,
                              max_rows=4, max_step_tokens=1024)


def step_of(cache, rows):
    cache.reserve([(sid, len(t)) for sid, t in rows])
    st = cache.plan(rows)
    cache.advance([(sid, len(t)) for sid, t in rows])
    return st


def dyt(n, g):
    return (1.0 + 0.2 * torch.randn(n, generator=g), 0.1 * torch.randn(n, generator=g), torch.rand(1, generator=g) + 0.3)


def dev(norm):
    return tuple(t.to(DEV) for t in norm)


@pytest.mark.parametrize("f32", [False, True])
def test_dynamic_tanh_and_token_shift_over_steps(ops, f32):
    g = torch.Generator().manual_seed(3)
    dt = torch.float32 if f32 else torch.bfloat16
    n = 203
    norm, mix = dyt(n, g), torch.rand(n, generator=g)
    cache = make_cache(state={0: {"shift": (n,)}})
    cache.states[0]["shift"].fill_(7.0)                 # whatever a slot held before must not be seen
    seqs = {"a": torch.randn(40, n, generator=g) * 2, "b": torch.randn(9, n, generator=g) * 2,
            "c": torch.randn(3, n, generator=g)}
    want = {k: ref.token_shift(ref.dynamic_tanh(v.double(), *[t.double() for t in norm]), mix.double())
            for k, v in seqs.items()}
    got = {k: [] for k in seqs}
    # portions of unequal length side by side, single tokens among them
    plan = [[("a", 5), ("b", 1)], [("a", 1), ("b", 2), ("c", 3)], [("a", 30), ("b", 1)], [("b", 5), ("a", 4)]]
    at = {k: 0 for k in seqs}
    for rows in plan:
        xs = torch.cat([seqs[k][at[k]:at[k] + c] for k, c in rows])
        st = step_of(cache, [(k, [0] * c) for k, c in rows])
        h = torch.empty(xs.shape[0], n, dtype=dt, device=DEV)
        ops.dyt_shift(xs.to(DEV), dev(norm), mix.to(DEV), cache.states[0]["shift"], h, st)
        o = 0
        for k, c in rows:
            got[k].append(h[o:o + c].cpu().double())
            o, at[k] = o + c, at[k] + c
    for k in seqs:
        res = torch.cat(got[k])
        assert (res - want[k][:res.shape[0]]).abs().max().item() < (1e-5 if f32 else 2e-2), k
    # a slot given back and used again starts from zeros
    cache.free("c")
    st = step_of(cache, [("d", [0, 0])])
    h = torch.empty(2, n, dtype=dt, device=DEV)
    ops.dyt_shift(seqs["c"][:2].to(DEV), dev(norm), mix.to(DEV), cache.states[0]["shift"], h, st)
    assert (h.cpu().double() - want["c"][:2]).abs().max().item() < (1e-5 if f32 else 2e-2)


@pytest.mark.parametrize("f32", [False, True])
def test_rowwise_steps(ops, f32):
    g = torch.Generator().manual_seed(4)
    dt = torch.float32 if f32 else torch.bfloat16
    tol = 1e-5 if f32 else 3e-2
    rows, n, eps = 6, 150, 1e-5
    norm = dyt(n, g)
    nd = [t.double() for t in norm]
    x, y = torch.randn(rows, n, generator=g) * 3, torch.randn(rows, n, generator=g) * 2
    idx = torch.tensor([4, 0, 4], dtype=torch.int32)
    out = torch.empty(3, n, dtype=dt, device=DEV)
    ops.dyt_gather(x.to(DEV), idx.to(DEV), dev(norm), out)
    assert (out.cpu().double() - ref.dynamic_tanh(x.double()[idx.long()], *nd)).abs().max().item() < tol
    xd, h = x.to(DEV), torch.empty(rows, n, dtype=dt, device=DEV)
    ops.dyt_residual(y.to(DEV), dev(norm), xd, h)
    want = x.double() + ref.dynamic_tanh(y.double(), *nd)
    assert (xd.cpu().double() - want).abs().max().item() < 1e-5 and torch.equal(h.cpu(), xd.cpu().to(dt))
    ops.dyt_residual(y.to(DEV), dev(norm), xd)                      # without the copy
    want = want + ref.dynamic_tanh(y.double(), *nd)
    assert (xd.cpu().double() - want).abs().max().item() < 1e-5
    w = torch.randn(n, generator=g)
    ops.unitnorm_residual(y.to(DEV), w.to(DEV), eps, xd, h)
    want = want + ref.rms(y.double(), eps) * w.double()
    assert (xd.cpu().double() - want).abs().max().item() < 2e-5 and torch.equal(h.cpu(), xd.cpu().to(dt))
    # unit-RMS per group of a row, the rows a column slice of a wider buffer
    per, gn = 3, 24
    wide = torch.randn(rows, per * gn + 10, generator=g).to(DEV)
    wg = torch.randn(gn, generator=g)
    o = torch.empty(rows, per * gn, dtype=dt, device=DEV)
    ops.rmsnorm_rows(wide[:, 5:5 + per * gn], wg.to(DEV), eps, o, per=per)
    wantg = (ref.rms(wide[:, 5:5 + per * gn].cpu().double().view(rows, per, gn), eps) * wg.double()).reshape(rows, -1)
    assert (o.cpu().double() - wantg).abs().max().item() < tol
    # gelu gate times a slice of an embedding table
    table = torch.randn(31, 5 * 12, generator=g).to(dt)
    ids = torch.tensor([30, 0, 7, 7, 2, 19], dtype=torch.int32)
    a = torch.randn(rows, 12, generator=g) * 2
    o = torch.empty(rows, 12, dtype=dt, device=DEV)
    ops.gelu_gate_rows(a.to(DEV), table.to(DEV), 24, ids.to(DEV), o)
    assert (o.cpu().double() - ref.gelu_tanh(a.double()) * table.double()[ids.long(), 24:36]).abs().max().item() < tol
    gu = torch.randn(rows, 2 * 70, generator=g) * 2
    o = torch.empty(rows, 70, dtype=dt, device=DEV)
    ops.silu_mul(gu.to(DEV), o)
    assert (o.cpu().double() - torch.nn.functional.silu(gu.double()[:, :70]) * gu.double()[:, 70:]).abs().max().item() < tol
    gt = torch.randn(rows, n, generator=g) * 2
    o = torch.empty(rows, n, dtype=dt, device=DEV)
    ops.sigmoid_gate(y.to(DEV), gt.to(DEV), o)
    assert (o.cpu().double() - y.double() * torch.sigmoid(gt.double())).abs().max().item() < tol
    ops.sigmoid_gate(y.to(DEV), None, o)
    assert torch.equal(o.cpu(), y.to(dt))
    # the residual step that also hands out the next sublayer's norm of the new x
    norm2 = dyt(n, g)
    x1 = xd.cpu().double()
    ops.dyt_residual(y.to(DEV), dev(norm), xd, h, next_norm=dev(norm2))
    x2 = x1 + ref.dynamic_tanh(y.double(), *nd)
    assert (xd.cpu().double() - x2).abs().max().item() < 2e-5
    assert (h.cpu().double() - ref.dynamic_tanh(x2, *[t.double() for t in norm2])).abs().max().item() < tol


@pytest.mark.parametrize("f32", [False, True])
@pytest.mark.parametrize("m,heads,n,k", [(1, 3, 40, 24), (70, 2, 64, 64), (9, 5, 17, 100)])
def test_products_per_head(ops, f32, m, heads, n, k):
    g = torch.Generator().manual_seed(m + heads)
    dt = torch.float32 if f32 else torch.bfloat16
    x = torch.randn(m, heads * k, generator=g).to(dt)
    w = (torch.randn(heads, n, k, generator=g) / math.sqrt(k)).to(dt)
    wide = torch.full((m, heads, n + 6), 9.0, device=DEV)
    ops.linear_heads(x.to(DEV), w.to(DEV), wide[:, :, :n], heads)
    want = torch.einsum("mhk,hnk->mhn", x.double().view(m, heads, k), w.double())
    assert (wide[:, :, :n].cpu().double() - want).abs().max().item() < 1e-4 * math.sqrt(k)
    assert bool((wide[:, :, n:] == 9.0).all())


@pytest.mark.parametrize("m,n,k", [(300, 130, 96), (513, 256, 40), (260, 128, 64)])
def test_many_rows_take_the_wide_tile_with_the_same_bits(ops, m, n, k):
    g = torch.Generator().manual_seed(m)
    x = torch.randn(m, k, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(torch.bfloat16).to(DEV)
    lin = ops.AnyLinear(w, wave_tiles=False)
    got = lin(x)
    assert (got.cpu().double() - x.cpu().double() @ w.cpu().double().T).abs().max().item() < 1e-4 * math.sqrt(k)
    for lo in (0, 100, m - 70):           # the same rows in a launch of few rows: the 64 x 64 tile
        assert torch.equal(lin(x[lo:lo + 70]), got[lo:lo + 70])


@pytest.mark.parametrize("f32", [False, True])
@pytest.mark.parametrize("T,top,E,n,k", [(75, 2, 5, 40, 72), (300, 2, 5, 136, 64), (9, 3, 16, 48, 128)])
def test_products_by_segment(ops, f32, T, top, E, n, k):
    g = torch.Generator().manual_seed(5)
    dt = torch.float32 if f32 else torch.bfloat16
    x = torch.randn(T, k, generator=g).to(dt)
    w = (torch.randn(E, n, k, generator=g) / math.sqrt(k)).to(dt)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    seg, order, place = (torch.empty(c, dtype=torch.int32, device=DEV) for c in (E + 1, T * top, T * top))
    ops.moe_plan(ids.to(DEV), seg, order, place, E)
    flat = ids.view(-1).long()
    counts = torch.bincount(flat, minlength=E)
    assert seg.cpu().tolist() == [0] + torch.cumsum(counts, 0).tolist()
    assert sorted(order.cpu().tolist()) == list(range(T * top))
    assert bool((order.cpu()[place.cpu().long()] == torch.arange(T * top)).all())
    segl = seg.cpu().tolist()
    for e in range(E):
        assert bool((flat[order.cpu()[segl[e]:segl[e + 1]].long()] == e).all())
    out = torch.empty(T * top, n, device=DEV)
    ops.linear_segments(x.to(DEV), w.to(DEV), out, seg, order, top, T)
    tok = order.cpu().long() // top
    want = torch.einsum("rk,rnk->rn", x.double()[tok], w.double()[flat[order.cpu().long()]])
    assert (out.cpu().double() - want).abs().max().item() < 1e-4 * math.sqrt(k)


@pytest.mark.parametrize("heads,n,p", [(2, 32, 32), (3, 40, 24), (1, 128, 64), (4, 8, 100)])
def test_gated_recurrence_over_steps(ops, heads, n, p):
    g = torch.Generator().manual_seed(heads * 100 + n)
    cache = make_cache(state={0: {"gated": (heads, n, p)}})
    cache.states[0]["gated"].fill_(3.0)
    lens = {"a": 70, "b": 12}
    raw = {k: (torch.randn(L, heads * n, generator=g), torch.randn(L, heads * n, generator=g) * 2,
               torch.randn(L, heads * p, generator=g)) for k, L in lens.items()}
    bias, lower = torch.randn(heads * n, generator=g), torch.rand(heads * n, generator=g)
    lower[0], lower[1] = 0.0, 0.999           # a gate free to forget everything, one that keeps nearly all
    want = {}
    for k, (q, f, v) in raw.items():
        L = lens[k]
        fq = lower.double() + (1 - lower.double()) * torch.sigmoid(f.double() + bias.double())
        want[k], _ = ref.gated_write_recurrence(torch.nn.functional.silu(q.double()).view(L, heads, n),
                                                fq.view(L, heads, n), v.double().view(L, heads, p))
    got = {k: [] for k in raw}
    at = {k: 0 for k in raw}
    for rows in [[("a", 33), ("b", 1)], [("b", 2), ("a", 1)], [("a", 1), ("b", 9)], [("a", 35)]]:
        q, f, v = (torch.cat([raw[k][j][at[k]:at[k] + c] for k, c in rows]).to(DEV) for j in range(3))
        st = step_of(cache, [(k, [0] * c) for k, c in rows])
        ops.gate_lower_bound_(q, f, bias.to(DEV), lower.to(DEV))
        out = torch.empty(q.shape[0], heads * p, device=DEV)
        ops.scan_gated(q, f, v, cache.states[0]["gated"], out, st, heads, n, p)
        o = 0
        for k, c in rows:
            got[k].append(out[o:o + c].cpu().double())
            o, at[k] = o + c, at[k] + c
    for k in raw:
        assert (torch.cat(got[k]).view(lens[k], heads, p) - want[k]).abs().max().item() < 2e-5, k


@pytest.mark.parametrize("heads,n,p", [(2, 32, 32), (3, 40, 24), (1, 128, 128), (2, 8, 100)])
def test_gated_recurrence_in_chunks_against_token_by_token(ops, heads, n, p):
    """Long rows are cut into chunks of 64 that run side by side and are joined through the products of their
    gates: against the restatement and against the token-by-token kernel, with gates of exactly zero and one,
    chunks cut at odd places, a second portion that continues from the slot's state, a short row beside them."""
    g = torch.Generator().manual_seed(heads + n + p)
    cache = make_cache(state={0: {"gated": (heads, n, p)}, 1: {"gated": (heads, n, p)}}, max_tokens=1024)
    for st_ in cache.states.values():
        st_["gated"].fill_(-2.0)
    lens = {"a": 450, "b": 9, "c": 131}
    q = {k: torch.randn(L, heads * n, generator=g) for k, L in lens.items()}
    f = {k: torch.rand(L, heads * n, generator=g) ** 0.25 for k, L in lens.items()}
    v = {k: torch.randn(L, heads * p, generator=g) for k, L in lens.items()}
    f["a"][:, 0], f["a"][:, 1] = 1.0, 0.0
    f["a"][100:170, 2] = 0.05                       # a product over a chunk that underflows
    want = {k: ref.gated_write_recurrence(q[k].double().view(-1, heads, n), f[k].double().view(-1, heads, n),
                                          v[k].double().view(-1, heads, p))[0] for k in lens}
    got = {True: {k: [] for k in lens}, False: {k: [] for k in lens}}
    at = {k: 0 for k in lens}
    for rows in [[("a", 203), ("b", 9), ("c", 17)], [("c", 114), ("a", 247)]]:
        st = step_of(cache, [(k, [0] * c) for k, c in rows])
        qs, fs, vs = (torch.cat([x[k][at[k]:at[k] + c] for k, c in rows]).to(DEV) for x in (q, f, v))
        for li, chunked in ((0, True), (1, False)):
            out = torch.empty(qs.shape[0], heads * p, device=DEV)
            ops.scan_gated(qs, fs, vs, cache.states[li]["gated"], out, st, heads, n, p, chunked=chunked)
            o = 0
            for k, c in rows:
                got[chunked][k].append(out[o:o + c].cpu().double())
                o += c
        for k, c in rows:
            at[k] += c
    for k in lens:
        a, b = torch.cat(got[True][k]).view(-1, heads, p), torch.cat(got[False][k]).view(-1, heads, p)
        assert (b - want[k]).abs().max().item() < 2e-5 and (a - want[k]).abs().max().item() < 2e-5, k
    assert (cache.states[0]["gated"] - cache.states[1]["gated"]).abs().max().item() < 2e-5


def latent_case(g, T, H, d, r, dv, R, rot, base):
    q = torch.randn(T, H * (d + r), generator=g)
    dkv = torch.randn(T, R + r, generator=g)
    wn = 1.0 + 0.2 * torch.randn(R, generator=g)
    uk = torch.randn(H * d, R, generator=g) / math.sqrt(R)
    uv = torch.randn(H * dv, R, generator=g) / math.sqrt(R)
    return q, dkv, wn, uk, uv


def latent_reference(q, dkv, wn, uk, uv, H, d, r, dv, R, rot, base, interleaved, scale, window, sink, eps):
    T = q.shape[0]
    pos = torch.arange(T)
    rotate = ref.rotate_interleaved if interleaved else ref.rotate_halves
    qq = q.double().view(T, H, d + r)
    c = ref.rms(dkv.double()[:, :R], eps) * wn.double()
    k_rot = rotate(dkv.double()[:, R:], pos, rot, base)
    q_rot = rotate(qq[..., d:], pos, rot, base)
    kk = torch.cat([(c @ uk.double().T).view(T, H, d), k_rot[:, None, :].expand(T, H, r)], dim=-1)
    v = (c @ uv.double().T).view(T, H, dv)
    return ref.masked_softmax_attention(torch.cat([qq[..., :d], q_rot], dim=-1), kk, v, scale, window,
                                        None if sink is None else sink.double())


def latent_run(ops, cache, sid, lo, hi, q, dkv, wn, uk, uv, H, d, r, dv, R, rot, base, interleaved, scale, window, sink,
               eps, dt):
    """Tokens lo .. hi of sequence `sid` through prep, the per-head products and the attention kernel."""
    T = hi - lo
    st = step_of(cache, [(sid, [0] * T)])
    pages = cache.k_caches[0].view(cache.k_caches[0].shape[0], cache.page_size, R + r)
    inv = (base ** (-2.0 * torch.arange(max(rot // 2, 1), dtype=torch.float64) / max(rot, 1))).to(DEV)
    q_plain = torch.empty(T, H * d, dtype=dt, device=DEV)
    q_abs = torch.empty(T, H * (R + r), device=DEV)
    ops.latent_prep(dkv[lo:hi].to(DEV), wn.to(DEV), eps, pages, q[lo:hi].to(DEV), q_plain, q_abs, inv, st, H, d, r, R, rot,
                    interleaved)
    uk_t = uk.view(H, d, R).transpose(1, 2).contiguous().to(dt).to(DEV)
    ops.linear_heads(q_plain, uk_t, q_abs.view(T, H, R + r)[:, :, :R], H)
    lat = torch.empty(T, H * R, dtype=dt, device=DEV)
    ops.latent_attn(q_abs, pages, lat, st, None if sink is None else sink.to(DEV), H, R, r, scale, window or 0)
    val = torch.empty(T, H, dv, device=DEV)
    ops.linear_heads(lat, uv.view(H, dv, R).contiguous().to(dt).to(DEV), val, H)
    return val.cpu().double()


@pytest.mark.parametrize("f32", [False, True])
@pytest.mark.parametrize("H,d,r,dv,R,rot,interleaved,window,with_sink", [
    (4, 24, 32, 40, 64, 32, True, 75, True),         # window over more than a page, rotation over all of r
    (3, 24, 16, 40, 72, 8, False, None, False),      # causal, rotation over half of r, odd sizes
    (5, 16, 8, 16, 136, 8, True, 5, True),           # five heads (a group of four and one left over), small window
    (1, 64, 64, 64, 320, 64, False, 64, False),      # one head, window = page, five value columns a lane
    (2, 8, 0, 8, 24, 0, True, 3, True),              # no rotated part at all
    (2, 16, 64, 16, 128, 64, False, None, False),    # shapes the matrix-core kernel takes (bf16, rows above 16 tokens)
    (3, 16, 32, 24, 256, 32, True, 100, True),
    (2, 32, 64, 32, 512, 64, True, 70, True),
    (5, 8, 64, 8, 64, 16, False, 64, True),
])
def test_latent_attention_whole_portions_and_decoding(ops, f32, H, d, r, dv, R, rot, interleaved, window, with_sink):
    g = torch.Generator().manual_seed(H * 10 + R)
    dt = torch.float32 if f32 else torch.bfloat16
    T, eps, scale, base = 150, 1e-6, 0.17, 5000.0
    q, dkv, wn, uk, uv = latent_case(g, T, H, d, r, dv, R, rot, base)
    if not f32:     # the comparison is about the kernels, not about rounding the inputs
        q, dkv, wn, uk, uv = (t.to(dt).float() for t in (q, dkv, wn, uk, uv))
    sink = torch.randn(H, generator=g) * 2 if with_sink else None
    want = latent_reference(q, dkv, wn, uk, uv, H, d, r, dv, R, rot, base, interleaved, scale, window, sink, eps)
    tol = 3e-5 if f32 else 4e-2
    args = (q, dkv, wn, uk, uv, H, d, r, dv, R, rot, base, interleaved, scale, window, sink, eps, dt)
    cache = make_cache(kv={0: (1, R + r, 0)}, dtype=dt)
    cache.k_caches[0].fill_(50.0)                     # pages are not cleared: nothing unwritten may be read
    whole = latent_run(ops, cache, "w", 0, T, *args)
    assert (whole - want).abs().max().item() < tol
    cache.free("w")
    # portions cut inside a page and a window, down to two tokens, then token by token; pages used again
    parts, at = [], 0
    for n in [61, 2, 3, 40, 2, 17] + [1] * 25:
        parts.append(latent_run(ops, cache, "p", at, at + n, *args))
        at += n
    got = torch.cat(parts)
    assert at == T and (got - want).abs().max().item() < tol
    if f32:
        assert (got - whole).abs().max().item() < 1e-5


@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("interleaved", [True, False])
@pytest.mark.parametrize("query,window", [(70, 7), (100, 37), (128, 64), (129, 65), (140, 100), (63, 64), (64, 64)])
def test_latent_attention_window_edge_with_a_dominant_key(ops, interleaved, query, window, f32):
    """One key's rotated part is made large along the slowest pair, where rotation hardly turns it, and the
    query's likewise: that key takes all the weight while it is visible.  Placed on the last visible position and
    on the first invisible one, in a prompt and with the query decoded alone."""
    # fp32: a shape only the plain kernel takes; bf16: one that sends the prompt's rows to the matrix-core kernel
    H, d, r, dv, R, rot, base, eps, scale = (2, 16, 16, 16, 32, 16, 1e6, 1e-6, 1.0) if f32 else (2, 16, 32, 16, 64, 32, 1e6, 1e-6, 0.25)
    # bf16: what rounding the latents and the carried-over query costs at scores of this size; a key wrongly seen or
    # missed moves the output by the difference between two values, of order one
    dt, tol = (torch.float32, 3e-5) if f32 else (torch.bfloat16, 8e-2)
    for inside in (True, False):
        g = torch.Generator().manual_seed(query + window)
        T = query + 1
        q, dkv, wn, uk, uv = latent_case(g, T, H, d, r, dv, R, rot, base)
        if not f32:
            q, dkv, wn, uk, uv = (t.to(dt).float() for t in (q, dkv, wn, uk, uv))
        key = query - window + 1 if inside else query - window
        if key < 0:
            continue
        slow = (rot - 2, rot - 1) if interleaved else (rot // 2 - 1, rot - 1)
        dkv[key, R + slow[0]] = 30.0
        q.view(T, H, d + r)[query, :, d + slow[0]] = 30.0
        dkv[key, :R] = torch.arange(R) % 3 - 1.0          # a latent unlike the others
        args = (q, dkv, wn, uk, uv, H, d, r, dv, R, rot, base, interleaved, scale, window, None, eps, dt)
        want = latent_reference(*args[:-1])
        c_key = ref.rms(dkv.double()[key:key + 1, :R], eps) * wn.double()
        v_key = (c_key @ uv.double().T).view(H, dv)
        seen = (want[query] - v_key).abs().max().item() < 1e-3
        assert seen == inside                              # the case is what it claims to be
        cache = make_cache(kv={0: (1, R + r, 0)}, dtype=dt)
        whole = latent_run(ops, cache, "w", 0, T, *args)
        assert (whole - want).abs().max().item() < tol
        cache.free("w")
        first = latent_run(ops, cache, "p", 0, query, *args)
        last = latent_run(ops, cache, "p", query, T, *args)
        assert (torch.cat([first, last]) - want).abs().max().item() < tol


def test_latent_attention_far_key_and_heavy_sink(ops):
    """Causal: a key 400 tokens back among hundreds takes the weight.  With a sink far above every score the
    output shrinks towards zero by exactly the sink's share."""
    H, d, r, dv, R, rot, base, eps = 2, 16, 16, 16, 32, 16, 1e6, 1e-6
    g = torch.Generator().manual_seed(11)
    T = 450
    q, dkv, wn, uk, uv = latent_case(g, T, H, d, r, dv, R, rot, base)
    dkv[40, R + rot - 2] = 40.0
    q.view(T, H, d + r)[440:, :, d + rot - 2] = 40.0
    args = [q, dkv, wn, uk, uv, H, d, r, dv, R, rot, base, True, 1.0, None, None, eps, torch.float32]
    want = latent_reference(*args[:-1])
    cache = make_cache(kv={0: (1, R + r, 0)})
    first = latent_run(ops, cache, "p", 0, 441, *args)
    rest = [latent_run(ops, cache, "p", t, t + 1, *args) for t in range(441, T)]
    got = torch.cat([first] + rest)
    assert (got - want).abs().max().item() < 3e-5
    v40 = ((ref.rms(dkv.double()[40:41, :R], eps) * wn.double()) @ uv.double().T).view(H, dv)
    assert (got[445] - v40).abs().max().item() < 1e-3
    cache.free("p")
    args[13], args[14], args[15] = 0.2, 50, torch.tensor([12.0, -30.0])
    want = latent_reference(*args[:-1])
    got = latent_run(ops, cache, "s", 0, 200, *args)
    assert (got - want[:200]).abs().max().item() < 3e-5
    assert got[150, 0].abs().max().item() < 1e-2 * got[150, 1].abs().max().item()


@pytest.mark.parametrize("f32", [False, True])
@pytest.mark.parametrize("E,top,shared", [(12, 4, True), (5, 1, False), (3, 3, True), (40, 6, False)])
def test_routed_experts(ops, f32, E, top, shared):
    g = torch.Generator().manual_seed(E + top)
    dt = torch.float32 if f32 else torch.bfloat16
    T, W, ff, sf = 37, 96, 40, 56
    h = torch.randn(T, W, generator=g).to(dt)
    Wt = {"router": (torch.randn(E, W, generator=g) * 0.3).to(torch.bfloat16).float()}
    for e in range(E):
        Wt[f"e{e}.gate"], Wt[f"e{e}.up"] = (torch.randn(ff, W, generator=g).to(dt).float() / math.sqrt(W) for _ in range(2))
        Wt[f"e{e}.down"] = torch.randn(W, ff, generator=g).to(dt).float() / math.sqrt(ff)
    if shared:
        Wt["shared.gate"], Wt["shared.up"] = (torch.randn(sf, W, generator=g).to(dt).float() / math.sqrt(W) for _ in range(2))
        Wt["shared.down"] = torch.randn(W, sf, generator=g).to(dt).float() / math.sqrt(sf)
        Wt["shared.sg"] = torch.randn(1, W, generator=g) / math.sqrt(W)
    mlp = {"router": {"experts": E, "top": top}, "expert": {"ff": ff}, "shared": {"ff": sf} if shared else None}
    want = ref.routed_experts(h.double(), {k: v.double() for k, v in Wt.items()}, "", mlp)
    hd = h.to(DEV)
    ids = torch.empty(T, top, dtype=torch.int32, device=DEV)
    wts, sg = torch.empty(T, top, device=DEV), torch.empty(T, device=DEV)
    ops.moe_route(hd, Wt["router"].to(DEV), Wt["shared.sg"].view(-1).to(DEV) if shared else None, ids, wts, sg)
    z = h.double() @ Wt["router"].double().T
    assert torch.equal(ids.cpu().long().sort(dim=1).values, z.topk(top, dim=1).indices.sort(dim=1).values)
    assert (wts.cpu().double() - torch.softmax(z.gather(1, ids.cpu().long()), dim=1)).abs().max().item() < 1e-5
    seg, order, place = (torch.empty(c, dtype=torch.int32, device=DEV) for c in (E + 1, T * top, T * top))
    ops.moe_plan(ids, seg, order, place, E)
    e_gu = torch.stack([torch.cat([Wt[f"e{e}.gate"], Wt[f"e{e}.up"]]) for e in range(E)]).to(dt).to(DEV)
    e_down = torch.stack([Wt[f"e{e}.down"] for e in range(E)]).to(dt).to(DEV)
    gu = ops.linear_segments(hd, e_gu, torch.empty(T * top, 2 * ff, device=DEV), seg, order, top, T)
    act = torch.empty(T * top, ff, dtype=dt, device=DEV)
    ops.silu_mul(gu, act)
    down = ops.linear_segments(act, e_down, torch.empty(T * top, W, device=DEV), seg, None, 1, T)
    s_out = None
    if shared:
        s_gu = ops.AnyLinear(torch.cat([Wt["shared.gate"], Wt["shared.up"]]).to(dt).to(DEV))
        s_act = torch.empty(T, sf, dtype=dt, device=DEV)
        ops.silu_mul(s_gu(hd), s_act)
        s_out = ops.AnyLinear(Wt["shared.down"].to(dt).to(DEV))(s_act)
    y = torch.empty(T, W, device=DEV)
    ops.moe_combine(down, place, wts, s_out, sg if shared else None, y)
    assert (y.cpu().double() - want).abs().max().item() < (3e-5 if f32 else 4e-2)
    # the same sum sent through a norm into a residual stream, with the stream's copy in the activation type
    norm = dyt(W, g)
    x0 = torch.randn(T, W, generator=g)
    x, hx = x0.to(DEV), torch.empty(T, W, dtype=dt, device=DEV)
    ops.moe_combine(down, place, wts, s_out, sg if shared else None, x, norm=dev(norm), h=hx)
    fused = x0.double() + ref.dynamic_tanh(y.cpu().double(), *[t.double() for t in norm])
    assert (x.cpu().double() - fused).abs().max().item() < 1e-5 and torch.equal(hx.cpu(), x.cpu().to(dt))
