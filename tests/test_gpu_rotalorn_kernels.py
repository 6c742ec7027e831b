"""The kernels behind Rotalorn's mechanisms, each alone against the plain function of the same
mechanism (tests/plain/rotalorn_plain.py): the pair table with the previous token kept in a slot,
the norms over whole rows with rotation and the store of keys that are values, differential
attention over pages (and the kernel that joins two maps), the router with softmax scores, the
experts with scores on their outputs both ways, the gates, the closing kernel with a layer norm,
and the store of a latent whose queries lie elsewhere."""
import numpy as np
import pytest

from plain import rotalorn_plain as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    from zse_amd.runtime.device import Runtime
    rt = Runtime.get()
    return rt, rt.kernels("float32")


_alive = []          # uploaded operands stay allocated until the test that made them has ended


@pytest.fixture(autouse=True)
def _operands():
    yield
    _alive.clear()


def up(rt, a, dtype=None):
    _alive.append(rt.upload(np.ascontiguousarray(a), dtype))
    return _alive[-1]


def f32(rt, a):
    return up(rt, np.asarray(a, np.float32))


def i32(rt, a):
    return up(rt, np.asarray(a, np.int32))


def bf16(a):
    from zse_amd.weights.safetensors import bf16_bits_to_f32, f32_to_bf16_bits
    return bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(a, np.float32)))


def up16(rt, a):
    """Values that bfloat16 holds exactly, stored as bfloat16."""
    from zse_amd.weights.safetensors import f32_to_bf16_bits
    return up(rt, f32_to_bf16_bits(np.asarray(a, np.float32)), "bfloat16")


def close(got, want, tol=2e-5):
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max()), np.abs(got - want).max()


@pytest.mark.parametrize("buckets,mp,mc", [(61, 7, 3), (1, 1, 1), (523, 65521, 40503), (97, -5, 2)])
def test_pair_rows_and_the_previous_token(dev, buckets, mp, mc):
    """Two requests whose tokens come in portions of unequal sizes, single tokens among them: the
    token before a portion's first one comes from the request's slot, and the slot's other words
    stay as they are."""
    rt, k = dev
    rng = np.random.default_rng(buckets)
    V, H = 3000, 20
    table = rng.normal(size=(buckets + 1, H)).astype(np.float32)
    seqs = {0: rng.integers(0, V, 23).tolist(), 1: rng.integers(0, V, 17).tolist()}
    want = {r: table[P.bigram_rows(t, buckets, mp, mc)] for r, t in seqs.items()}
    cuts = {0: [1, 2, 9, 1, 1, 5, 4], 1: [6, 1, 2, 2, 1, 1, 4]}
    words, word = 9, 5
    state = up(rt, np.full((3, words), 7, np.int32))
    slot = {0: 2, 1: 0}
    at, got = {0: 0, 1: 0}, {0: [], 1: []}
    d_table = f32(rt, table)
    for step in range(7):
        toks, pos, req, q_start = [], [], [], [0]
        for i, r in enumerate((1, 0) if step % 2 else (0, 1)):
            n = cuts[r][step]
            toks += seqs[r][at[r]:at[r] + n]
            pos += list(range(at[r], at[r] + n))
            req += [i] * n
            q_start.append(q_start[-1] + n)
        order = (1, 0) if step % 2 else (0, 1)
        T = len(toks)
        out = up(rt, np.ones((T, H), np.float32))
        before = rt.empty((2,), "int32")
        d_tok, d_q = i32(rt, toks), i32(rt, q_start)
        k.zk_prev_token(d_tok.ptr, d_q.ptr, i32(rt, [slot[r] for r in order]).ptr, state.ptr, words, word, before.ptr, 2,
                        rt.stream)
        k.zk_add_pair_rows(out.ptr, d_table.ptr, d_tok.ptr, i32(rt, pos).ptr, i32(rt, req).ptr, d_q.ptr, before.ptr,
                           buckets, mp, mc, T, H, rt.stream)
        o = rt.download(out) - 1.0
        for i, r in enumerate(order):
            got[r].append(o[q_start[i]:q_start[i + 1]])
            at[r] += cuts[r][step]
    for r in (0, 1):
        close(np.concatenate(got[r]), want[r], 1e-6)
    st = rt.download(state)
    assert st[2, word] == seqs[0][-1] and st[0, word] == seqs[1][-1]
    st[[0, 2], word] = 7
    assert (st == 7).all()


@pytest.mark.parametrize("nh,nkv,D,R,transposed", [(4, 2, 24, 12, 0), (2, 2, 64, 64, 1), (1, 1, 10, 4, 0), (6, 2, 80, 80, 1),
                                                   (3, 1, 40, 0, 0)])
def test_norms_over_whole_rows_and_values_that_are_keys(dev, nh, nkv, D, R, transposed):
    rt, k = dev
    rng = np.random.default_rng(nh * 100 + D)
    T, bs, pages, eps = 9, 4, 7, 1e-5
    ld = (nh + nkv) * D + 5
    rows = rng.normal(size=(T, ld)).astype(np.float32)
    bias = rng.normal(0, 0.3, (nh + nkv) * D).astype(np.float32)
    gq, gk = rng.normal(1, 0.2, nh * D).astype(np.float32), rng.normal(1, 0.2, nkv * D).astype(np.float32)
    pos = np.array([0, 1, 2, 50, 51, 300, 7, -1, 9], np.int32)
    slots = rng.permutation(pages * bs)[:T].astype(np.int32)
    slots[6] = -1                                       # a token that is not stored
    freqs = P.rotary_frequencies(R, 300.0, {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 32}) if R else None
    q = rows[:, :nh * D].astype(np.float64) + bias[:nh * D]
    kk = rows[:, nh * D:(nh + nkv) * D].astype(np.float64) + bias[nh * D:]
    qn = P.rms_norm(q, gq, eps, np.float64).reshape(T, nh, D)
    kn = P.rms_norm(kk, gk, eps, np.float64).reshape(T, nkv, D)
    if R:
        qn, kn = P.rotate_half(qn, pos, freqs, np.float64), P.rotate_half(kn, pos, freqs, np.float64)
    d_rows = f32(rt, rows)
    kc, vc = rt.zeros((pages, nkv, bs, D), "float32"), rt.zeros((pages, nkv, D, bs) if transposed else (pages, nkv, bs, D), "float32")
    k.zk_row_prep(d_rows.ptr, ld, i32(rt, pos).ptr, i32(rt, slots).ptr, f32(rt, bias).ptr, f32(rt, gq).ptr, f32(rt, gk).ptr, eps,
                  f32(rt, freqs).ptr if R else None, R, kc.ptr, vc.ptr, T, nh, nkv, D, D, bs, transposed, 1, rt.stream)
    got, gk_, gv_ = rt.download(d_rows), rt.download(kc), rt.download(vc)
    if transposed:
        gv_ = gv_.transpose(0, 1, 3, 2)
    live = pos >= 0
    close(got[live, :nh * D], qn.reshape(T, -1)[live])
    assert np.array_equal(got[:, (nh + nkv) * D:], rows[:, (nh + nkv) * D:]) and np.array_equal(got[~live], rows[~live])
    seen = np.zeros((pages, bs), bool)
    for t in range(T):
        if live[t] and slots[t] >= 0:
            pg, off = divmod(int(slots[t]), bs)
            seen[pg, off] = True
            close(gk_[pg, :, off], kn[t])
            close(gv_[pg, :, off], kk[t].reshape(nkv, D))          # the key as projected: bias, no norm, no rotation
    assert not gk_.transpose(0, 2, 1, 3)[~seen].any() and not gv_.transpose(0, 2, 1, 3)[~seen].any()


def paged(rt, rng, lens, bs, spare=3):
    """Block tables over pages handed out in a shuffled order; returns (table, slot of (r, j))."""
    need = [-(-n // bs) for n in lens]
    ids = (rng.permutation(sum(need) + spare) + 1).tolist()
    table = np.full((len(lens), max(need) + 1), -1, np.int32)
    for r, n in enumerate(need):
        for b in range(n):
            table[r, b] = ids.pop()
    return table, (lambda r, j: int(table[r, j // bs]) * bs + j % bs), sum(need) + spare + 1


@pytest.mark.parametrize("H,G,D,E,window,cap,temp", [(4, 2, 12, 24, 0, 15.0, (0.5, 16)), (2, 2, 8, 8, 0, 0.0, (1.5, 5)),
                                                     (1, 1, 10, 6, 0, 2.0, (2.0, 1)), (2, 1, 32, 64, 37, 0.0, None),
                                                     (3, 3, 40, 80, 0, 25.0, (0.4, 32))])
def test_differential_attention_over_pages(dev, H, G, D, E, window, cap, temp):
    """Three requests: a whole prompt, a portion behind a context, one decoded token far behind;
    keys and values reach the cache through the storing kernel, in steps."""
    rt, k = dev
    rng = np.random.default_rng(H * 10 + D)
    bs, eps, diff, lam, scale = 8, 1e-5, 0.35, 0.62, D ** -0.5 * 1.7
    lens, new = [41, 150, 203], [41, 30, 1]
    q = {r: rng.normal(size=(n, H, 2, D)).astype(np.float32) for r, n in enumerate(lens)}
    kk = {r: rng.normal(size=(n, G, 2, D)).astype(np.float32) for r, n in enumerate(lens)}
    v = {r: rng.normal(size=(n, G, E)).astype(np.float32) for r, n in enumerate(lens)}
    table, slot_of, pages = paged(rt, rng, lens, bs)
    kc, vc = rt.zeros((pages, 2 * G, bs, D), "float32"), rt.zeros((pages, G, bs, E), "float32")
    ld = (H + G) * 2 * D + G * E + 3

    def rows_of(r, lo, hi):
        n = hi - lo
        return np.concatenate([q[r][lo:hi].reshape(n, -1), kk[r][lo:hi].reshape(n, -1), v[r][lo:hi].reshape(n, -1),
                               np.zeros((n, 3), np.float32)], axis=1)
    # the contexts first, then the step that is looked at
    for first in (True, False):
        rows, pos, req, slots = [], [], [], []
        for r, n in enumerate(lens):
            lo, hi = (0, n - new[r]) if first else (n - new[r], n)
            if hi > lo:
                rows.append(rows_of(r, lo, hi))
                pos += list(range(lo, hi))
                req += [r] * (hi - lo)
                slots += [slot_of(r, j) for j in range(lo, hi)]
        x = f32(rt, np.concatenate(rows))
        T = len(pos)
        k.zk_cache_store(x.ptr, ld, H * 2 * D, (H + G) * 2 * D, i32(rt, slots).ptr, kc.ptr, vc.ptr, T, 2 * G, D, G, E, bs, 0, rt.stream)
    out = rt.empty((T, H * E), "float32")
    k.zk_diff_attention_plain(x.ptr, ld, kc.ptr, vc.ptr, i32(rt, table).ptr, table.shape[1], i32(rt, req).ptr, i32(rt, pos).ptr,
                              out.ptr, T, H, G, D, E, bs, scale, cap, window, 0, lam, diff, eps,
                              temp[0] if temp else 0.0, temp[1] if temp else 0, rt.stream)
    got = rt.download(out)
    at = 0
    for r, n in enumerate(lens):
        qq = q[r].astype(np.float64)
        if temp:
            qq = qq * P.query_temperature(np.arange(n), temp[0], temp[1], np.float64)[:, None, None, None]
        a = [P.softmax_attention(qq[:, :, m], kk[r][:, :, m], v[r], scale, window or None, cap or None, np.float64) for m in (0, 1)]
        want = (P.unit_rms(a[0] - lam * a[1], eps, np.float64) * (1.0 - diff)).reshape(n, H * E)[n - new[r]:]
        close(got[at:at + new[r]], want, 3e-5)
        at += new[r]
    # the joining kernel alone: two maps' results as heads of their own
    a12 = rng.normal(size=(5, H, 2, E)).astype(np.float32)
    joined = rt.empty((5, H * E), "float32")
    k.zk_diff_join(f32(rt, a12).ptr, joined.ptr, 5, H, E, lam, diff, eps, rt.stream)
    close(rt.download(joined), (P.unit_rms(a12[:, :, 0] - lam * a12[:, :, 1].astype(np.float64), eps, np.float64)
                                * (1.0 - diff)).reshape(5, H * E))


def test_the_router_with_softmax_scores_and_ties(dev):
    rt, k = dev
    rng = np.random.default_rng(4)
    for E, top, ld in ((5, 2, 5), (16, 4, 17), (3, 3, 4), (70, 1, 70), (130, 16, 131)):
        T = 11
        z = rng.normal(0, 2.0, (T, ld)).astype(np.float32)
        z[3, :E] = 0.25                                    # all equal: the lowest indices win
        if E > 2:
            z[5, E - 1] = z[5, 0] = z[5, :E].max() + 1.0   # a tie for the first place
        ids, wts = rt.empty((T, top), "int32"), rt.empty((T, top), "float32")
        k.zk_moe_route_ext(f32(rt, z).ptr, ld, ids.ptr, wts.ptr, T, E, top, 1, rt.stream)
        s = np.exp(z[:, :E].astype(np.float64) - z[:, :E].max(axis=1, keepdims=True))
        s /= s.sum(axis=1, keepdims=True)
        order = np.argsort(-s.astype(np.float32), axis=1, kind="stable")[:, :top]
        got_ids, got_w = rt.download(ids), rt.download(wts)
        assert got_ids[3].tolist() == list(range(top))
        if E > 2:
            assert got_ids[5, 0] == 0 and (top == 1 or got_ids[5, 1] == E - 1)
        calm = np.ones(T, bool)
        srt = -np.sort(-s, axis=1)
        if E > top:
            calm = (srt[:, top - 1] - srt[:, top]) > 1e-6
        calm[[3, 5]] = False
        assert np.array_equal(got_ids[calm], order[calm])
        close(got_w, np.take_along_axis(s, got_ids.astype(np.int64), axis=1), 1e-6)
        assert np.allclose(got_w.sum(axis=1)[top == E:], 1.0, atol=1e-5) if top == E else (got_w.sum(axis=1) < 1.0).all()


def plain_mixture(x, ids, wts, wg, wu, wd):
    out = np.zeros((len(x), wd.shape[1]), np.float64)
    for t in range(len(x)):
        for e, s in zip(ids[t], wts[t]):
            out[t] += s * ((P.silu(x[t] @ wg[e].T) * (x[t] @ wu[e].T)) @ wd[e].T)
    return out


@pytest.mark.parametrize("T,E,top,W,F", [(3, 5, 2, 48, 24), (40, 4, 3, 36, 20), (1, 2, 2, 64, 96), (70, 16, 4, 64, 32)])
def test_experts_with_scores_on_their_outputs(dev, T, E, top, W, F):
    """Row by row in 32-bit, and through the grouped matrix-core product in bfloat16 where the sizes
    allow it; experts without tokens among them."""
    rt, k = dev
    rng = np.random.default_rng(T + E)
    x = bf16(rng.normal(size=(T, W)))
    wg, wu = bf16(rng.normal(0, W ** -0.5, (E, F, W))), bf16(rng.normal(0, W ** -0.5, (E, F, W)))
    wd = bf16(rng.normal(0, F ** -0.5, (E, W, F)))
    ids = np.stack([rng.permutation(E - 1 if E > top else E)[:top] for _ in range(T)]).astype(np.int32)     # the last expert idle
    wts = rng.uniform(0.05, 0.6, (T, top)).astype(np.float32)
    want = plain_mixture(x.astype(np.float64), ids, wts, wg, wu, wd)
    gu = np.concatenate([wg, wu], axis=1)
    y, out = rt.empty((T * top, F), "float32"), rt.empty((T, W), "float32")
    k.zk_moe_experts_ext(f32(rt, x).ptr, i32(rt, ids).ptr, f32(rt, wts).ptr, f32(rt, gu).ptr, f32(rt, wd).ptr, y.ptr, out.ptr,
                         T, top, W, F, 0.0, 1, 1, rt.stream)
    close(rt.download(out), want, 1e-5)
    if W % 8 or F % 8:
        return
    kb = rt.kernels("bfloat16")
    work = rt.empty((E + 1 + 2 * T * top,), "int32")
    xg, yb = rt.empty((T * top, W), "bfloat16"), rt.empty((T * top, F), "bfloat16")
    rows, outb = rt.empty((T * top, W), "float32"), rt.empty((T, W), "float32")
    kb.zk_moe_experts_grouped_ext(up16(rt, x).ptr, i32(rt, ids).ptr, f32(rt, wts).ptr, up16(rt, gu).ptr, up16(rt, wd).ptr, work.ptr,
                                  xg.ptr, yb.ptr, rows.ptr, outb.ptr, T, E, top, W, F, 0.0, 1, 1, rt.stream)
    close(rt.download(outb), want, 2e-2)
    outr = rt.empty((T, W), "float32")
    kb.zk_moe_experts_ext(up16(rt, x).ptr, i32(rt, ids).ptr, f32(rt, wts).ptr, up16(rt, gu).ptr, up16(rt, wd).ptr, yb.ptr, outr.ptr,
                          T, top, W, F, 0.0, 1, 1, rt.stream)
    close(rt.download(outr), want, 2e-2)


def test_the_gates(dev):
    rt, k = dev
    rng = np.random.default_rng(9)
    T, W, ld = 7, 30, 9
    rows, z = rng.normal(size=(T, W)).astype(np.float32), rng.normal(0, 2, (T, ld)).astype(np.float32)
    d = f32(rt, rows)
    k.zk_gate_rows(d.ptr, f32(rt, z).ptr + 4 * 6, ld, T, W, rt.stream)         # the seventh column of z
    close(rt.download(d), rows * P.sigmoid(z[:, 6:7].astype(np.float64)), 1e-6)
    H, E = 5, 6
    o, g = rng.normal(size=(T, H * E)).astype(np.float32), rng.normal(0, 2, (T, ld)).astype(np.float32)
    d = f32(rt, o)
    k.zk_gate_heads_per(d.ptr, f32(rt, g).ptr + 4 * 2, ld, T, H * E, E, rt.stream)     # columns 2..6 of g, one a head
    close(rt.download(d), (o.reshape(T, H, E) * P.sigmoid(g[:, 2:2 + H].astype(np.float64))[:, :, None]).reshape(T, H * E), 1e-6)


@pytest.mark.parametrize("W", [36, 48, 320, 1000])
def test_the_closing_kernel_with_a_layer_norm(dev, W):
    rt, k = dev
    rng = np.random.default_rng(W)
    T, eps = 6, 1e-5
    h = (rng.normal(size=(T, W)) * 3 + 5).astype(np.float32)
    a, planes = rng.normal(size=(T, W)).astype(np.float32), rng.normal(size=(2, T, W)).astype(np.float32)
    bias = rng.normal(size=W).astype(np.float32)
    w, c = rng.normal(1, 0.2, W).astype(np.float32), rng.normal(0, 0.3, W).astype(np.float32)
    d_h, out = f32(rt, h), rt.empty((T, W), "float32")
    k.zk_sum_layer_norm(d_h.ptr, f32(rt, a).ptr, 0, f32(rt, planes).ptr, 2, f32(rt, bias).ptr, f32(rt, w).ptr, f32(rt, c).ptr, eps,
                        out.ptr, T, W, rt.stream)
    new = h.astype(np.float64) + a + planes[0] + planes[1] + bias
    close(rt.download(d_h), new, 1e-6)
    close(rt.download(out), P.layer_norm(new, w, c, eps, np.float64), 1e-5)
    # the norm alone, of a stream that stays as it is
    k.zk_sum_layer_norm(d_h.ptr, None, 0, None, 0, None, f32(rt, w).ptr, None, eps, out.ptr, T, W, rt.stream)
    close(rt.download(out), P.layer_norm(new, w, np.zeros(W), eps, np.float64), 1e-5)
    close(rt.download(d_h), new, 1e-6)


@pytest.mark.parametrize("H,D,R,C", [(3, 8, 4, 20), (1, 12, 2, 9), (2, 16, 8, 56)])
def test_the_store_of_a_latent_whose_queries_lie_elsewhere(dev, H, D, R, C):
    rt, k = dev
    rng = np.random.default_rng(C)
    T, bs, pages, eps = 8, 4, 5, 1e-6
    ldq, ldd = H * (D + R) + 2, C + R + H
    q, down = rng.normal(size=(T, ldq)).astype(np.float32), rng.normal(size=(T, ldd)).astype(np.float32)
    gain = rng.normal(1, 0.2, C).astype(np.float32)
    pos = np.array([0, 1, 70, 71, 5, -1, 6, 300], np.int32)
    slots = rng.permutation(pages * bs)[:T].astype(np.int32)
    freqs = P.rotary_frequencies(R, 50.0)
    qa, kc = rt.zeros((T, H * (C + R)), "float32"), rt.zeros((pages, 1, bs, C + R), "float32")
    k.zk_latent_prep_ext(f32(rt, q).ptr, ldq, f32(rt, down).ptr, ldd, i32(rt, pos).ptr, i32(rt, slots).ptr, f32(rt, gain).ptr, eps,
                         f32(rt, freqs).ptr, 1.0, 0, qa.ptr, kc.ptr, T, H, D, R, C, bs, rt.stream)
    got_q, got_k = rt.download(qa).reshape(T, H, C + R), rt.download(kc).reshape(pages * bs, C + R)
    qr = P.rotate_half(q[:, :H * (D + R)].reshape(T, H, D + R)[:, :, D:], pos, freqs, np.float64)
    kr = P.rotate_half(down[:, None, C:C + R], pos, freqs, np.float64)[:, 0]
    c = P.rms_norm(down[:, :C], gain, eps, np.float64)
    for t in range(T):
        if pos[t] < 0:
            assert not got_q[t].any()
            continue
        close(got_q[t, :, C:], qr[t])
        close(got_k[slots[t]], np.concatenate([c[t], kr[t]]))
