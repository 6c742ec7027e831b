"""Kernels that Bumolix added or added to, each alone against the plain function of the same
mechanism or a few lines of NumPy: the square of relu as the epilogue of the matrix-core product
at every number of rows that picks another kernel of it; the matrix-core attention with a chunk
mask, the sink of score 0 and weights in two halves, against the plain softmax over the same
cached keys; the two recurrences over two steps of two requests whose states are carried in
slots, walked plainly and in segments."""
import numpy as np
import pytest

from plain import bumolix_plain as P

pytestmark = pytest.mark.gpu

_alive = []


@pytest.fixture(autouse=True)
def _operands():
    yield
    _alive.clear()


def bf16(a):
    from zse_amd.weights.safetensors import bf16_bits_to_f32, f32_to_bf16_bits
    return bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(a, np.float32)))


def up16(rt, a):
    from zse_amd.weights.safetensors import f32_to_bf16_bits
    _alive.append(rt.upload(f32_to_bf16_bits(np.ascontiguousarray(a, np.float32)), "bfloat16"))
    return _alive[-1]


def i32(rt, a):
    _alive.append(rt.upload(np.ascontiguousarray(a, np.int32)))
    return _alive[-1]


@pytest.mark.parametrize("M,K,N", [(3, 96, 80), (16, 96, 80), (40, 256, 144), (200, 96, 80), (700, 1024, 320), (2048, 512, 1024)])
def test_the_square_of_relu_in_the_products_epilogue(M, K, N):
    from zse_amd.runtime.device import Runtime
    rt = Runtime.get()
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(M)
    x = bf16(rng.normal(size=(M, K)))
    w = bf16(rng.normal(0, 1.5 / np.sqrt(K), (N, K)))
    want = np.maximum(x.astype(np.float64) @ w.T.astype(np.float64), 0.0) ** 2
    assert (want == 0).mean() > 0.3 and want.max() > 4.0
    out = rt.empty((M, N), "bfloat16")
    k.zk_gemm_bf16(up16(rt, x).ptr, K, up16(rt, w).ptr, out.ptr, N, 0, M, N, K, 7, 0.0, 0, None, 0, None, rt.stream)
    got = rt.download_f32(out)
    assert np.abs(got - want).max() < 0.01 * want.max()
    assert not got[want == 0].any()


def plain_attention(q, kk, v, pos0, scale, chunk, sink):
    """q [n, H, D] at positions pos0.., kk and v [ctx, G, D]: softmax over the keys of the query's own
    chunk up to itself, one more term exp(0) in the denominator where there is a sink."""
    n, H, D = q.shape
    G = kk.shape[1]
    out = np.zeros((n, H, D))
    for i in range(n):
        p = pos0 + i
        lo = p - p % chunk if chunk else 0
        for h in range(H):
            g = h // (H // G)
            s = (kk[lo:p + 1, g] @ q[i, h]) * scale
            m = max(s.max(), 0.0)
            e = np.exp(s - m)
            out[i, h] = (e @ v[lo:p + 1, g]) / (e.sum() + (np.exp(-m) if sink else 0.0))
    return out


@pytest.mark.parametrize("wide", [0, 1])
@pytest.mark.parametrize("D,H,G,bs,chunk,sink", [(16, 4, 2, 4, 24, 1), (64, 2, 1, 16, 100, 1), (128, 8, 2, 16, 700, 1),
                                                 (32, 3, 3, 8, 0, 1), (128, 4, 4, 16, 64, 0), (64, 4, 1, 16, 1, 1),
                                                 (32, 4, 2, 8, 33, 1), (256, 2, 2, 32, 1000, 1)])
def test_matrix_core_attention_with_chunks_and_the_sink(D, H, G, bs, chunk, sink, wide):
    """Three requests of one step: a long portion from position 0 (one request, few heads: its keys are
    cut into ranges), a portion that begins inside a chunk behind a cached context, and a single
    token far into its context (the split kernel, which begins at the chunk's first block)."""
    from zse_amd.runtime.device import Runtime
    rt = Runtime.get()
    k = rt.kernels("bfloat16")
    if not k.zk_attention_bf16_supports(H, G, D, bs):
        pytest.skip("head shape not taken by the matrix-core kernel")
    rng = np.random.default_rng(D + chunk)
    ctx = [900, 333, 1501]                 # context lengths after this step
    new = [900, 70, 1]                     # tokens the step brings
    R, T = 3, sum(new)
    max_ctx = 1536
    blocks = -(-max_ctx // bs)
    pages = R * blocks
    kc = np.zeros((pages, G, bs, D), np.float32)
    vc = np.zeros((pages, G, D, bs), np.float32)           # values lie transposed in a page
    table = np.arange(pages, dtype=np.int32).reshape(R, blocks)[:, ::-1].copy()     # pages in falling order
    keys, vals = [], []
    for r in range(R):
        kk = bf16(rng.normal(size=(ctx[r], G, D)))
        vv = bf16(rng.normal(size=(ctx[r], G, D)))
        kk *= np.sqrt(D) / np.linalg.norm(kk, axis=-1, keepdims=True)
        kk = bf16(kk)
        keys.append(kk)
        vals.append(vv)
        for p in range(ctx[r]):
            pg = table[r, p // bs]
            kc[pg, :, p % bs, :] = kk[p]
            vc[pg, :, :, p % bs] = vv[p]
    q = bf16(rng.normal(size=(T, H, D)))
    q = bf16(q * np.sqrt(D) / np.linalg.norm(q, axis=-1, keepdims=True))
    scale = 6.0 / D                                          # scores up to 6 either way: the sink weighs in
    q_start = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
    want = np.concatenate([plain_attention(q[q_start[r]:q_start[r + 1]].astype(np.float64), keys[r].astype(np.float64),
                                           vals[r].astype(np.float64), ctx[r] - new[r], scale, chunk, sink)
                           for r in range(R)])
    out = rt.empty((T, H * D), "bfloat16")
    need = (int(k.zk_attention_bf16_workspace(R, H, D, max_ctx)) + 255) // 256 * 256
    need += int(k.zk_attention_bf16_portion_workspace(2 * (928 + 128), H, G, D))
    ws = rt.zeros((need // 4 + 16,), "float32")
    _alive.append(ws)
    k.zk_attention_bf16_masked(up16(rt, q.reshape(T, H * D)).ptr, H * D, up16(rt, kc).ptr, up16(rt, vc).ptr,
                               i32(rt, table).ptr, blocks, i32(rt, q_start).ptr, i32(rt, ctx).ptr, out.ptr, R, 2, 928, max_ctx,
                               H, G, D, bs, scale, 0.0, 0, 64, ws.ptr, ws.nbytes, chunk, sink, wide, rt.stream)
    got = rt.download_f32(out).reshape(T, H, D)
    err = np.abs(got - want).max(axis=(1, 2))
    assert err.max() < (0.012 if wide else 0.03), (int(np.argmax(err)), float(err.max()))


def up32(rt, a):
    _alive.append(rt.upload(np.ascontiguousarray(a, np.float32)))
    return _alive[-1]


STEPS = ([150, 37], [70, 1], [1, 129])       # tokens of requests 0 and 1 in three steps


@pytest.mark.parametrize("seg", [0, 16, 64])
@pytest.mark.parametrize("H,D,E", [(3, 12, 40), (2, 64, 128), (1, 200, 24), (2, 32, 8)])
def test_gated_linear_attention_walk(H, D, E, seg):
    """decayed_outer_products, the unit RMS with its gain and the gate, against zk_gla in 32-bit."""
    from zse_amd.runtime.device import Runtime
    rt = Runtime.get()
    k = rt.kernels("float32")
    rng = np.random.default_rng(H * 1000 + D + seg)
    tau, eps, offset, slot_words = 3.0, 1e-5, 24, 24 + H * D * E + 8
    total = [sum(st[r] for st in STEPS) for r in range(2)]
    data = []
    for r in range(2):
        n = total[r]
        q, kk = rng.normal(size=(n, H, D)), rng.normal(size=(n, H, D))
        v, g, z = rng.normal(size=(n, H, E)), rng.normal(size=(n, H, E)), rng.normal(0.0, 2.0, (n, H, D))
        data.append((q, kk, v, g, z))
    bias, gain = rng.normal(1.5, 1.5, (H, D)), 1.0 + rng.normal(0, 0.3, E)
    want = []
    for q, kk, v, g, z in data:
        alpha = np.exp(P.log_sigmoid(z + bias) / tau)
        o = P.decayed_outer_products(q * D ** -0.5, kk, v, alpha, np.float64)
        want.append(P.unit_rms(o, eps, np.float64) * gain * P.silu(g))
    state = rt.zeros((2, slot_words), "float32")
    slots = i32(rt, [1, 0])
    done = [0, 0]
    for st in STEPS:
        T = sum(st)
        rows = np.concatenate([np.concatenate([d[i][done[r]:done[r] + st[r]].reshape(st[r], -1) for i in range(4)], axis=1)
                               for r, d in enumerate(data)])                      # q | k | v | g
        z = np.concatenate([d[4][done[r]:done[r] + st[r]].reshape(st[r], -1) for r, d in enumerate(data)])
        ld = 2 * H * D + 2 * H * E
        X, Z = up32(rt, rows), up32(rt, z)
        out, raw = rt.zeros((T, H * E), "float32"), rt.zeros((T, H * E), "float32")
        max_q = -(-max(st) // 32) * 32 if max(st) > 1 else 1
        nseg = 2 * -(-max_q // seg) if seg else 1
        ss, sd = rt.zeros((nseg, H * D * E), "float32"), rt.zeros((nseg, H * D), "float32")
        _alive.extend([out, raw, ss, sd])
        k.zk_gla(X.ptr, ld, H * D, 2 * H * D, X.ptr + (2 * H * D + H * E) * 4, ld, Z.ptr, H * D, up32(rt, bias).ptr, tau,
                 up32(rt, gain).ptr, state.ptr, slot_words, offset, i32(rt, [0, st[0], T]).ptr, slots.ptr,
                 i32(rt, np.zeros(T)).ptr, out.ptr, raw.ptr, T, 2, max_q, H, D, E, eps, seg, ss.ptr if seg else None,
                 sd.ptr if seg else None, rt.stream)
        got = rt.download(out).reshape(T, H, E)
        at = 0
        for r in range(2):
            ref = want[r][done[r]:done[r] + st[r]]
            assert np.abs(got[at:at + st[r]] - ref).max() < 2e-4 * max(1.0, np.abs(ref).max()), (st, r)
            at += st[r]
            done[r] += st[r]
    words = rt.download(state)
    assert not words[:, :offset].any() and not words[:, offset + H * D * E:].any()     # nothing beside the state is touched


@pytest.mark.parametrize("seg", [0, 16, 64])
@pytest.mark.parametrize("I,N", [(72, 5), (200, 16), (64, 40), (9, 1)])
def test_selective_scan_walk(I, N, seg):
    """selective_scan and the gate against zk_selective_scan in 32-bit."""
    from zse_amd.runtime.device import Runtime
    rt = Runtime.get()
    k = rt.kernels("float32")
    rng = np.random.default_rng(I + N + seg)
    offset, slot_words = 8, 8 + I * N + 4
    total = [sum(st[r] for st in STEPS) for r in range(2)]
    A_log, Dv, dt_bias = rng.normal(-1.0, 1.5, (I, N)), rng.normal(size=I), rng.normal(-1.0, 1.0, I)
    data, want = [], []
    for r in range(2):
        n = total[r]
        u, dt, z = rng.normal(size=(n, I)), rng.normal(0, 1.5, (n, I)), rng.normal(size=(n, I))
        B, C = rng.normal(size=(n, N)), rng.normal(size=(n, N))
        data.append((u, dt, z, B, C))
        y = P.selective_scan(u, P.softplus(dt + dt_bias), -np.exp(A_log), B, C, Dv, np.float64)
        want.append(y * P.silu(z))
    state = rt.zeros((2, slot_words), "float32")
    slots = i32(rt, [1, 0])
    done = [0, 0]
    for st in STEPS:
        T = sum(st)
        cut = lambda i: np.concatenate([d[i][done[r]:done[r] + st[r]] for r, d in enumerate(data)])
        bc = np.concatenate([np.zeros((T, 3)), cut(3), cut(4)], axis=1)            # three columns of something else first
        out = rt.zeros((T, I), "float32")
        max_q = -(-max(st) // 32) * 32 if max(st) > 1 else 1
        nseg = 2 * -(-max_q // seg) if seg else 1
        ss, sd = rt.zeros((nseg, I * N), "float32"), rt.zeros((nseg, I), "float32")
        _alive.extend([out, ss, sd])
        k.zk_selective_scan(up32(rt, cut(0)).ptr, I, up32(rt, cut(1)).ptr, I, up32(rt, dt_bias).ptr, up32(rt, bc).ptr, 3 + 2 * N,
                            3, 3 + N, up32(rt, A_log).ptr, up32(rt, Dv).ptr, up32(rt, cut(2)).ptr, I, state.ptr, slot_words,
                            offset, i32(rt, [0, st[0], T]).ptr, slots.ptr, out.ptr, T, 2, I, N, max_q, seg,
                            ss.ptr if seg else None, sd.ptr if seg else None, rt.stream)
        got = rt.download(out)
        at = 0
        for r in range(2):
            ref = want[r][done[r]:done[r] + st[r]]
            assert np.abs(got[at:at + st[r]] - ref).max() < 2e-4 * max(1.0, np.abs(ref).max()), (st, r)
            at += st[r]
            done[r] += st[r]
    words = rt.download(state)
    assert not words[:, :offset].any() and not words[:, offset + I * N:].any()
