"""Each mechanism of the ragged family alone: the HIP kernel against the plain restatement in
oracle/ref_hybrid.py (fp64 on the CPU), on random inputs and on inputs built so that a fault shows
(one key made dominant just inside / just outside a window, far back, at a page border)."""
import math

import pytest
import torch

from oracle import ref_hybrid as ref

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


@pytest.mark.parametrize("f32", [False, True])
@pytest.mark.parametrize("m,n,k", [(1, 650, 200), (5, 37, 19), (70, 130, 288), (129, 64, 64), (3, 16, 2048)])
def test_linear_any(ops, f32, m, n, k):
    g = torch.Generator().manual_seed(m * 1000 + n)
    dt = torch.float32 if f32 else torch.bfloat16
    x = torch.randn(m, k, generator=g).to(dt)
    w = (torch.randn(n, k, generator=g) / math.sqrt(k)).to(dt)
    lin = ops.AnyLinear(w.to(DEV), wave_tiles=False)
    got = lin(x.to(DEV)).cpu().double()
    want = x.double() @ w.double().T
    assert (got - want).abs().max().item() <= (2e-5 if f32 else 2e-5) * max(1.0, want.abs().max().item()) * math.sqrt(k)
    # rows of a wider buffer, and a row's result does not depend on its neighbours
    wide = torch.zeros(m, k + 8, dtype=dt, device=DEV)
    wide[:, :k] = x.to(DEV)
    assert torch.equal(lin(wide[:, :k]).cpu().double(), got)
    assert torch.equal(lin(x[:1].to(DEV)).cpu().double(), got[:1])


def test_wave_tile_and_plain_projection_agree(ops):
    g = torch.Generator().manual_seed(1)
    w = (torch.randn(96, 128, generator=g) / 11).to(torch.bfloat16).to(DEV)
    a, b = ops.AnyLinear(w), ops.AnyLinear(w, wave_tiles=False)
    assert a.tiles is not None and b.tiles is None
    for m in (1, 7, 64, 65, 200):
        x = torch.randn(m, 128, generator=g).to(torch.bfloat16).to(DEV)
        assert (a(x) - b(x)).abs().max().item() < 1e-4


@pytest.mark.parametrize("f32", [False, True])
def test_stream_ops(ops, f32):
    g = torch.Generator().manual_seed(2)
    dt = torch.float32 if f32 else torch.bfloat16
    rows, n, eps = 5, 203, 1e-5
    table = torch.randn(50, n, generator=g).to(dt)
    ids = torch.tensor([3, 49, 0, 7, 7], dtype=torch.int32)
    x, h = torch.empty(rows, n, device=DEV), torch.empty(rows, n, dtype=dt, device=DEV)
    ops.embed_scaled(table.to(DEV), ids.to(DEV), 2.5, x, h)
    assert torch.equal(x.cpu(), table.float()[ids.long()] * 2.5) and torch.equal(h.cpu(), (table.float()[ids.long()] * 2.5).to(dt))
    y1, y2, w = torch.randn(rows, n, generator=g), torch.randn(rows, n, generator=g) * 3, torch.randn(n, generator=g) * 0.1
    x0 = x.cpu().double()
    ops.postnorm_residual(y1.to(DEV), w.to(DEV), eps, x, h, y2=y2.to(DEV), s1=1.2, s2=0.9)
    want = x0 + ref.offset_norm(1.2 * y1.double() + 0.9 * y2.double(), w.double(), eps)
    assert (x.cpu().double() - want).abs().max().item() < 1e-5
    assert torch.equal(h.cpu(), x.cpu().to(dt))
    ops.postnorm_residual(y1.to(DEV), w.to(DEV), eps, x, h)
    want = want + ref.offset_norm(y1.double(), w.double(), eps)
    assert (x.cpu().double() - want).abs().max().item() < 2e-5
    idx = torch.tensor([4, 0, 2], dtype=torch.int32)
    out = torch.empty(3, n, dtype=dt, device=DEV)
    ops.offset_rmsnorm_gather(x, idx.to(DEV), w.to(DEV), eps, out)
    wn = ref.offset_norm(x.cpu().double()[idx.long()], w.double(), eps)
    assert (out.cpu().double() - wn).abs().max().item() < (1e-5 if f32 else 0.04)
    r = torch.empty(rows, n, dtype=dt, device=DEV)
    ops.relu_squared(y1.to(DEV), r)
    assert (r.cpu().double() - torch.relu(y1.double()) ** 2).abs().max().item() < (1e-6 if f32 else 0.05)
    lg = (torch.randn(4, 77, generator=g) * 40).to(DEV)
    want = 30.0 * torch.tanh(lg.cpu().double() / 30.0)
    assert (ops.softcap_(lg, 30.0).cpu().double() - want).abs().max().item() < 1e-5


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_conv_whole_and_in_portions(ops, taps):
    g = torch.Generator().manual_seed(taps)
    C, T = 70, 23
    x, w, b = torch.randn(T, C + 6, generator=g), torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    want = ref.causal_conv_silu(x[:, 3:3 + C].double(), w.double(), b.double())
    for portions in ([T], [1] * T, [2, 1, 3, 2, 15], [5, 18]):
        cache = make_cache(state={0: {"conv": (taps - 1, C)}})
        cache.admit("other")                       # the request under test does not sit in slot 0
        cache.states[0]["conv"].fill_(7.0)         # what an earlier owner of the slot left behind
        out, pos = [], 0
        for n in portions:
            st = step_of(cache, [("s", [0] * n)])
            o = torch.empty(n, C, device=DEV)
            ops.conv_silu(x[pos:pos + n].to(DEV)[:, 3:3 + C], cache.states[0]["conv"], w.to(DEV), b.to(DEV), o, st)
            out.append(o.cpu())
            pos += n
        assert (torch.cat(out).double() - want).abs().max().item() < 1e-5, portions


def test_softplus_decay(ops):
    g = torch.Generator().manual_seed(5)
    raw = torch.randn(9, 11, generator=g) * 30         # far into both tails: no clamp anywhere
    bias, a_log = torch.randn(5, generator=g), torch.randn(5, generator=g)
    gain, decay, logd = torch.empty(9, 5, device=DEV), torch.empty(9, 5, device=DEV), torch.empty(9, 5, device=DEV)
    ops.softplus_decay(raw.to(DEV)[:, 4:9], bias.to(DEV), a_log.to(DEV), gain, decay, logd)
    v = raw[:, 4:9].double() + bias.double()
    dt = torch.where(v > 30, v, torch.log1p(torch.exp(v)))
    assert ((gain.cpu().double() - dt).abs() / dt.abs().clamp_min(1e-30)).max().item() < 1e-5
    assert (decay.cpu().double() - torch.exp(-torch.exp(a_log.double()) * dt)).abs().max().item() < 1e-6
    want = -torch.exp(a_log.double()) * dt
    assert ((logd.cpu().double() - want).abs() / want.abs().clamp_min(1e-30)).max().item() < 1e-5


@pytest.mark.parametrize("H,G,n,p", [(4, 2, 40, 24), (3, 3, 48, 20), (2, 1, 128, 64), (1, 1, 8, 128), (6, 1, 48, 48)])
def test_scan_whole_portions_and_rows(ops, H, G, n, p):
    g = torch.Generator().manual_seed(H * 100 + n)
    T = 19
    q, k = torch.randn(T, G * n, generator=g), torch.randn(T, G * n, generator=g)
    v = torch.randn(T, H * p, generator=g)
    decay, gain = torch.rand(T, H, generator=g), torch.rand(T, H, generator=g) + 0.1
    skip = torch.randn(H, generator=g)
    rep = H // G
    want, _ = ref.decayed_outer_product_scan(
        q.double().view(T, G, n).repeat_interleave(rep, 1), k.double().view(T, G, n).repeat_interleave(rep, 1),
        v.double().view(T, H, p), decay.double(), gain.double())
    want = (want + skip.double()[None, :, None] * v.double().view(T, H, p)).reshape(T, H * p)
    dv = lambda t: t.to(DEV)
    for portions in ([T], [1] * T, [2, 3, 2, 12]):
        cache = make_cache(state={0: {"s": (H, n, p)}})
        cache.admit("other")
        cache.states[0]["s"].fill_(3.0)
        out, pos = [], 0
        for m in portions:
            st = step_of(cache, [("a", [0] * m)])
            o = torch.empty(m, H * p, device=DEV)
            sl = slice(pos, pos + m)
            ops.scan_outer(dv(q[sl]), dv(k[sl]), dv(v[sl]), dv(decay[sl]), dv(gain[sl]), dv(skip), cache.states[0]["s"], o,
                           st, H, n, p, q_div=rep, k_div=rep)
            out.append(o.cpu())
            pos += m
        assert (torch.cat(out).double() - want).abs().max().item() < 2e-4, portions
    # two rows of unequal length in one launch, fixed decay per head, no gain, no skip
    cache = make_cache(state={0: {"s": (H, n, p)}})
    st = step_of(cache, [("a", [0] * 7), ("b", [0] * 12)])
    qq, kk = q.view(T, G, n).repeat_interleave(rep, 1).reshape(T, H * n), k.view(T, G, n).repeat_interleave(rep, 1).reshape(T, H * n)
    o = torch.empty(T, H * p, device=DEV)
    ops.scan_outer(dv(qq), dv(kk), dv(v), dv(decay[0].contiguous()), None, None, cache.states[0]["s"], o, st, H, n, p)
    for lo, hi in ((0, 7), (7, 19)):
        w2, _ = ref.decayed_outer_product_scan(qq[lo:hi].double().view(-1, H, n), kk[lo:hi].double().view(-1, H, n),
                                               v[lo:hi].double().view(-1, H, p), decay[0].double().repeat(hi - lo, 1),
                                               torch.ones(hi - lo, H, dtype=torch.float64))
        assert (o[lo:hi].cpu().double() - w2.reshape(hi - lo, H * p)).abs().max().item() < 2e-4


@pytest.mark.parametrize("H,G,n,p", [(4, 2, 40, 24), (2, 1, 128, 64), (1, 1, 8, 130), (3, 3, 64, 32)])
def test_scan_in_chunks_equals_token_by_token(ops, H, G, n, p):
    """Long rows: the chunked form against the restatement and against the token-by-token kernel, whole
    and cut at places that are no multiple of the chunk, beside a short row in the same launch; decays
    from nearly one down to values whose products underflow."""
    g = torch.Generator().manual_seed(H * 7 + p)
    T, rep = 333, H // G
    q, k = torch.randn(T, G * n, generator=g), torch.randn(T, G * n, generator=g)
    v = torch.randn(T, H * p, generator=g)
    logd = -torch.exp(torch.randn(T, H, generator=g) * 3.0 - 3.0)
    logd[100:110] = -120.0                       # a stretch that forgets everything
    decay, gain = torch.exp(logd), torch.rand(T, H, generator=g) + 0.1
    skip = torch.randn(H, generator=g)
    want, _ = ref.decayed_outer_product_scan(
        q.double().view(T, G, n).repeat_interleave(rep, 1), k.double().view(T, G, n).repeat_interleave(rep, 1),
        v.double().view(T, H, p), torch.exp(logd.double()), gain.double())
    want = (want + skip.double()[None, :, None] * v.double().view(T, H, p)).reshape(T, H * p)
    dv = lambda t: t.to(DEV)
    outs = {}
    for chunked in (True, False):
        for portions in ([T], [70, 3, 129, 17, 64, 50], [200] + [1] * 133):
            cache = make_cache(state={0: {"s": (H, n, p)}})
            cache.admit("other")
            cache.states[0]["s"].fill_(3.0)
            out, pos = [], 0
            for m in portions:
                rows = [("a", [0] * m)] + ([("b", [0] * 5)] if pos == 0 else [])     # a short row rides along once
                st = step_of(cache, rows)
                if chunked:
                    assert st.n_chunks == (m + 63) // 64 * (m > 16)
                tot = st.tokens
                o = torch.empty(tot, H * p, device=DEV)
                pad = lambda t: torch.cat([t[pos:pos + m], t[:tot - m]]).to(DEV)
                ops.scan_outer(pad(q), pad(k), pad(v), pad(decay), pad(gain), dv(skip), cache.states[0]["s"], o, st,
                               H, n, p, q_div=rep, k_div=rep, log_decay=pad(logd), chunked=chunked)
                out.append(o[:m].cpu())
                if pos == 0:
                    assert (o[m:].cpu().double() - want[:5]).abs().max().item() < 2e-4
                pos += m
            got = torch.cat(out).double()
            assert (got - want).abs().max().item() < 5e-4 * max(1.0, want.abs().max().item()), (chunked, portions)
            outs[(chunked, len(portions))] = got
    assert (outs[(True, 1)] - outs[(False, 1)]).abs().max().item() < 5e-4 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("dim,rot", [(48, 32), (64, 64), (40, 0), (6, 2)])
def test_rotary_pairs(ops, dim, rot):
    g = torch.Generator().manual_seed(dim)
    T, H, base = 6, 3, 1e6
    x = torch.randn(T, H * dim + 5, generator=g)
    pos = torch.tensor([0, 1, 63, 64, 1000, 70001], dtype=torch.int32)
    inv = base ** (-2.0 * torch.arange(rot // 2, dtype=torch.float64) / max(rot, 1))
    xd = x.to(DEV)
    ops.rotary_pairs_(xd[:, :H * dim], inv.to(DEV), pos.to(DEV), H, dim, rot, dim ** -0.5)
    want = ref.rotate_half_pairs(x[:, :H * dim].double().view(T, H, dim), pos, rot, base) * dim ** -0.5
    assert (xd[:, :H * dim].cpu().double() - want.reshape(T, H * dim)).abs().max().item() < 2e-6
    assert torch.equal(xd[:, H * dim:].cpu(), x[:, H * dim:])


@pytest.mark.parametrize("f32", [False, True])
def test_gated_group_norm_both_orders(ops, f32):
    g = torch.Generator().manual_seed(8)
    rows, n, eps = 7, 120, 1e-5
    y, z, w = torch.randn(rows, n, generator=g) * 4, torch.randn(rows, n, generator=g), torch.randn(n, generator=g)
    dt = torch.float32 if f32 else torch.bfloat16
    tol = 1e-5 if f32 else 0.05
    for groups in (1, 3, 120):
        out = torch.empty(rows, n, dtype=dt, device=DEV)
        ops.gated_group_norm(y.to(DEV), z.to(DEV), w.to(DEV), out, groups, True, eps)
        u = y.double() * z.double() * torch.sigmoid(z.double())
        want = ref.unit_rms(u.view(rows, groups, -1), eps).reshape(rows, n) * w.double()
        assert (out.cpu().double() - want).abs().max().item() < tol * max(1.0, want.abs().max().item())
        ops.gated_group_norm(y.to(DEV), z.to(DEV), None, out, groups, False, eps)
        want = ref.unit_rms(y.double().view(rows, groups, -1), eps).reshape(rows, n) * z.double() * torch.sigmoid(z.double())
        assert (out.cpu().double() - want).abs().max().item() < tol * max(1.0, want.abs().max().item())


def _attend(ops, q, k, v, H, G, d, dv, scale, window, slopes, portions, f32=True, pages=16, shuffle=True, tiled=True):
    """Feed q|k|v rows in portions through qk_unitnorm_store + window_attn; returns [T, H*dv]."""
    dt = torch.float32 if f32 else torch.bfloat16
    cache = make_cache(kv={0: (G, d, dv)}, pages=pages, dtype=dt, max_tokens=pages * 64)
    if shuffle:   # pages in no particular order, none of them page 0 for the first tokens
        order = list(cache._free_pages)
        order = order[1::2] + order[0::2]
        cache._free_pages.clear()
        cache._free_pages.extend(order)
    cache.k_caches[0].fill_(9.0)
    cache.v_caches[0].fill_(-9.0)
    T = q.shape[0]
    qkv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1).float()
    out, pos = [], 0
    for n in portions:
        st = step_of(cache, [("s", [0] * n)])
        rows = qkv[pos:pos + n].to(DEV).contiguous()
        ops.qk_unitnorm_store(rows, cache.k_caches[0], cache.v_caches[0], st, H, G, d, dv, 1e-6)
        o = torch.empty(n, H * dv, dtype=dt, device=DEV)
        ops.window_attn(rows, cache.k_caches[0], cache.v_caches[0], o, st, torch.tensor(slopes).float().to(DEV), H, G, d,
                        dv, scale, window, tiled=tiled)
        out.append(o.float().cpu())
        pos += n
    return torch.cat(out)


@pytest.mark.parametrize("H,G,d,dv,window", [(6, 2, 40, 56, 37), (2, 2, 64, 64, 5), (4, 1, 96, 130, 200), (3, 3, 8, 8, 1),
                                             (2, 1, 64, 64, 300)])
def test_window_attention_random(ops, H, G, d, dv, window):
    g = torch.Generator().manual_seed(d + window)
    T, scale = 150, 0.3
    q, k, v = torch.randn(T, H, d, generator=g), torch.randn(T, G, d, generator=g), torch.randn(T, G, dv, generator=g)
    slopes = [2.0 ** (-8.0 * (h + 1) / H) for h in range(H)]
    want = ref.windowed_softmax_attention(ref.unit_rms(q.double(), 1e-6), ref.unit_rms(k.double(), 1e-6), v.double(),
                                          scale, window, slopes).reshape(T, H * dv)
    for portions in ([T], [64, 64, 22], [3, 61, 2, 63, 1, 20], [100] + [1] * 50):
        got = _attend(ops, q, k, v, H, G, d, dv, scale, window, slopes, portions)
        assert (got.double() - want).abs().max().item() < 1e-4, portions
    got = _attend(ops, q, k, v, H, G, d, dv, scale, window, slopes, [T], f32=False, tiled=False)
    assert (got.double() - want).abs().max().item() < 0.05


@pytest.mark.parametrize("H,G,d,dv,window", [(2, 2, 64, 64, 5), (4, 2, 128, 64, 100), (3, 1, 96, 96, 72), (2, 1, 32, 32, 40),
                                             (8, 2, 128, 128, 64), (2, 2, 64, 128, 300)])
def test_window_attention_on_the_matrix_cores(ops, H, G, d, dv, window):
    """Long rows in bf16: the tiled kernel against the restatement and against the plain kernel, whole and
    in portions that start in the middle of a page, a short row riding along on the plain kernel."""
    g = torch.Generator().manual_seed(d * 3 + window)
    T, scale = 333, 0.3
    q, k, v = torch.randn(T, H, d, generator=g), torch.randn(T, G, d, generator=g), torch.randn(T, G, dv, generator=g)
    slopes = [2.0 ** (-8.0 * (h + 1) / H) for h in range(H)]
    want = ref.windowed_softmax_attention(ref.unit_rms(q.double(), 1e-6), ref.unit_rms(k.double(), 1e-6), v.double(),
                                          scale, window, slopes).reshape(T, H * dv)
    plain = _attend(ops, q, k, v, H, G, d, dv, scale, window, slopes, [T], f32=False, tiled=False)
    for portions in ([T], [70, 3, 129, 17, 64, 50], [200] + [1] * 133):
        got = _attend(ops, q, k, v, H, G, d, dv, scale, window, slopes, portions, f32=False)
        assert (got.double() - want).abs().max().item() < 0.06, portions
        assert (got - plain).abs().max().item() < 0.06, portions
    assert (got.double() - want).abs().mean().item() < 0.006


@pytest.mark.parametrize("window", [72, 64, 65, 130, 260])
@pytest.mark.parametrize("decode,f32", [(False, True), (True, True), (False, False)])
def test_window_edge_shows_in_the_output(ops, window, decode, f32):
    """One key carries a value of its own and is made to win the softmax whenever it is visible: the
    query that still sees it (distance window - 1) returns that value, the next one does not."""
    H = G = 1
    d = dv = 32              # a head shape the tiled bf16 kernel takes, so the bf16 prompt run goes through it
    T = 2 * window + 70
    g = torch.Generator().manual_seed(window)
    q, k, v = torch.randn(T, H, d, generator=g) * 0.01, torch.randn(T, G, d, generator=g) * 0.01, torch.zeros(T, G, dv)
    marks = (0, 5, 63, 64, window + 3)                    # first tokens, a page border, past one window
    for n, mark in enumerate(marks):
        k[mark, 0] = 0
        k[mark, 0, n] = 1.0                               # a direction of its own
        v[mark, 0, 0] = 100.0 + mark
    portions = [T] if not decode else [window // 2, 2] + [1] * (T - window // 2 - 2)
    seen = {}
    for n, mark in enumerate(marks):
        qq = q.clone()
        for i in (mark + window - 1, mark + window):     # just inside, just outside
            qq[i, 0] = 0
            qq[i, 0, n] = 1.0
        out = _attend(ops, qq, k, v, H, G, d, dv, 40.0, window, [0.0], portions, f32=f32)
        seen[mark] = (out[mark + window - 1, 0].item(), out[mark + window, 0].item())
        assert abs(seen[mark][0] - (100.0 + mark)) < (1.0 if f32 else 2.5), (mark, seen)
        assert abs(seen[mark][1]) < 60.0 and abs(seen[mark][1] - (100.0 + mark)) > 40.0, (mark, seen)


def test_distance_penalty_is_per_head_and_in_distance(ops):
    """Equal keys everywhere: the weights are softmax(-slope * distance), a different one per head."""
    H, G, d, dv, T, window = 4, 2, 8, 4, 40, 16
    q, k = torch.ones(T, H, d), torch.ones(T, G, d)
    v = torch.arange(T).float()[:, None, None].repeat(1, G, dv)      # value = position
    slopes = [2.0 ** (-8.0 * (h + 1) / H) for h in range(H)]
    out = _attend(ops, q, k, v, H, G, d, dv, 1.0, window, slopes, [7, 33]).view(T, H, dv)
    for h in range(H):
        for i in (0, 3, 15, 16, 39):
            js = torch.arange(max(0, i - window + 1), i + 1).double()
            p = torch.softmax(-slopes[h] * (i - js), 0)
            assert abs(out[i, h, 0].item() - (p * js).sum().item()) < 1e-3
