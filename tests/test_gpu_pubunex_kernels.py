"""The kernels behind Pubunex's mechanisms, each alone against the plain function of the same
mechanism (tests/plain/pubunex_plain.py): the delta rule cut into steps, the convolution without
residual and with silu on strided rows, the router, the experts both ways, the per-head products
and the store of a latent attention, attention with sinks over keys that hold their values, the
biased and scaled rotation in front of an attention, and the kernel that joins two sublayers."""
import numpy as np
import pytest

from plain import pubunex_plain as P

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


def i32(rt, a):
    return up(rt, np.asarray(a, np.int32))


def bf16(a):
    from zse_amd.weights.safetensors import bf16_bits_to_f32, f32_to_bf16_bits
    return bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(a, np.float32)))


def up16(rt, a):
    """Values that bfloat16 holds exactly, stored as bfloat16."""
    from zse_amd.weights.safetensors import f32_to_bf16_bits
    return up(rt, f32_to_bf16_bits(np.asarray(a, np.float32)))


@pytest.mark.parametrize("H,G,D,E", [(4, 2, 16, 24), (1, 1, 100, 70), (2, 2, 32, 130), (3, 1, 8, 8), (2, 1, 200, 40)])
def test_delta_rule_cut_into_steps(dev, H, G, D, E):
    """Two requests whose rows come in portions of unequal sizes, single rows among them; the
    state in the slot carries S from step to step, and a slot's other words stay untouched."""
    rt, k = dev
    rng = np.random.default_rng(H * 100 + D)
    lens = {0: 37, 1: 21}
    cuts = {0: [1, 18, 1, 2, 15], 1: [5, 1, 1, 13, 1]}
    eps = 1e-5
    seq, want = {}, {}
    A_log, dtb, gain = rng.normal(0, 0.5, H), rng.normal(0, 0.5, H), rng.normal(1, 0.2, E)
    for r, n in lens.items():
        q, kk = rng.normal(size=(n, G, D)), rng.normal(size=(n, G, D))
        v, z = rng.normal(size=(n, H, E)), rng.normal(size=(n, H, E))
        b, a = rng.normal(size=(n, H)), rng.normal(size=(n, H))
        seq[r] = tuple(x.astype(np.float32) for x in (q, kk, v, z, b, a))
        q, kk, v, z, b, a = (x.astype(np.float64) for x in seq[r])
        qn = np.repeat(P.unit_vector(q, np.float64) * D ** -0.5, H // G, axis=1)
        kn = np.repeat(P.unit_vector(kk, np.float64), H // G, axis=1)
        decay = np.exp(-np.exp(A_log)[None] * P.softplus(a + dtb[None]))
        o, _ = P.delta_recurrence(qn, kn, v, P.sigmoid(b), decay, np.float64)
        want[r] = (P.unit_rms(o, eps, np.float64) * gain[None, None] * P.silu(z)).reshape(n, H * E)
    offset, words = 12, 12 + H * D * E + 7
    state = rt.zeros((3, words), "float32")
    slot = {0: 2, 1: 0}
    at, got = {0: 0, 1: 0}, {0: [], 1: []}
    ld = 2 * G * D + H * E
    for step in range(5):
        rows, q_start = [], [0]
        for r in (0, 1):
            n = cuts[r][step]
            q, kk, v, z, b, a = (x[at[r]:at[r] + n] for x in seq[r])
            rows.append((np.concatenate([q.reshape(n, -1), kk.reshape(n, -1), v.reshape(n, -1)], axis=1), z.reshape(n, -1),
                         np.concatenate([b, a], axis=1)))
            q_start.append(q_start[-1] + n)
            at[r] += n
        qkv, z, ba = (np.concatenate([x[i] for x in rows]) for i in range(3))
        T = len(qkv)
        d_o = rt.empty((T, H * E), "float32")
        k.zk_delta_rule(up(rt, qkv).ptr, ld, G * D, 2 * G * D, up(rt, z).ptr, H * E, up(rt, ba).ptr,
                        up(rt, A_log.astype(np.float32)).ptr, up(rt, dtb.astype(np.float32)).ptr,
                        up(rt, gain.astype(np.float32)).ptr, state.ptr, words, offset, i32(rt, q_start).ptr,
                        i32(rt, [slot[0], slot[1]]).ptr, i32(rt, list(range(T))).ptr, d_o.ptr,
                        rt.empty((T, H * E), "float32").ptr, T, 2, max(cuts[0][step], cuts[1][step]), H, G, D, E, eps,
                        rt.stream)
        o = rt.download(d_o)
        for i, r in enumerate((0, 1)):
            got[r].append(o[q_start[i]:q_start[i + 1]])
    for r in (0, 1):
        assert np.abs(np.concatenate(got[r]) - want[r]).max() < 2e-5 * max(1.0, np.abs(want[r]).max())
    st = rt.download(state)
    assert not st[1].any() and not st[:, :offset].any() and not st[:, offset + H * D * E:].any()


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_convolution_with_silu_on_strided_rows(dev, taps):
    rt, k = dev
    rng = np.random.default_rng(taps)
    C, ld = 50, 64
    w = rng.normal(size=(C, taps)).astype(np.float32)
    seqs = {0: rng.normal(size=(23, ld)).astype(np.float32), 1: rng.normal(size=(17, ld)).astype(np.float32)}
    want = {r: P.causal_conv_silu(h[:, :C], w, np.float64) for r, h in seqs.items()}
    words = 4 + (taps - 1) * C + 3
    state = rt.zeros((2, words), "float32")
    cuts = {0: [1, 2, 9, 1, 1, 5, 4], 1: [6, 1, 2, 2, 1, 1, 4]}
    at, got = {0: 0, 1: 0}, {0: [], 1: []}
    d_w = up(rt, w)
    for step in range(7):
        rows, pos, req, q_start = [], [], [], [0]
        for r in (0, 1):
            n = cuts[r][step]
            rows.append(seqs[r][at[r]:at[r] + n])
            pos += list(range(at[r], at[r] + n))
            req += [r] * n
            q_start.append(q_start[-1] + n)
            at[r] += n
        h = np.concatenate(rows)
        T = len(h)
        d_h, d_o = up(rt, h), rt.empty((T, C), "float32")
        args = (i32(rt, pos).ptr, i32(rt, req).ptr, i32(rt, q_start).ptr, i32(rt, [1, 0]).ptr)
        if all(cuts[r][step] == 1 for r in (0, 1)):
            k.zk_short_conv_token_ext(d_h.ptr, ld, d_w.ptr, state.ptr, words, 4, *args, d_o.ptr, C, T, C, taps, 0, 1, rt.stream)
        else:
            k.zk_short_conv_ext(d_h.ptr, ld, d_w.ptr, state.ptr, words, 4, *args, d_o.ptr, C, T, C, taps, 0, 1, rt.stream)
            k.zk_short_conv_state_ext(d_h.ptr, ld, state.ptr, words, 4, args[2], args[3], 2, C, taps, rt.stream)
        o = rt.download(d_o)
        for i, r in enumerate((0, 1)):
            got[r].append(o[q_start[i]:q_start[i + 1]])
    for r in (0, 1):
        assert np.abs(np.concatenate(got[r]) - want[r]).max() < 1e-5


def test_the_router_takes_the_largest_scores_and_the_lower_index_among_equals(dev):
    rt, k = dev
    rng = np.random.default_rng(3)
    T, E, top = 9, 70, 4
    z = rng.normal(0, 2, (T, E)).astype(np.float32)
    z[0, [5, 40, 41, 69]] = 9.0                      # four equal scores: all chosen, in the order of their numbers
    z[1, :] = 0.25                                   # all equal: the first four
    z[2, 66] = z[2, 3] = 7.0
    ids, wts = rt.empty((T, top), "int32"), rt.empty((T, top), "float32")
    k.zk_moe_route(up(rt, z).ptr, ids.ptr, wts.ptr, T, E, top, rt.stream)
    s = P.sigmoid(z.astype(np.float64))
    want_ids = np.argsort(-s.astype(np.float32), axis=1, kind="stable")[:, :top]
    got_ids, got_w = rt.download(ids), rt.download(wts)
    assert np.array_equal(got_ids, want_ids)
    assert list(got_ids[0]) == [5, 40, 41, 69] and list(got_ids[1]) == [0, 1, 2, 3] and list(got_ids[2][:2]) == [3, 66]
    assert np.abs(got_w - np.take_along_axis(s, want_ids, axis=1)).max() < 1e-6


def expert_weights(rng, E, W, F):
    w = {}
    for e in range(E):
        w[f"e{e}.gate"] = bf16(rng.normal(0, 2.0 / np.sqrt(W), (F, W)))
        w[f"e{e}.up"] = bf16(rng.normal(0, 2.0 / np.sqrt(W), (F, W)))
        w[f"e{e}.down"] = bf16(rng.normal(0, 1.0 / np.sqrt(F), (W, F)))
    return w


def plain_experts(x, ids, wts, w, limit):
    out = np.zeros(x.shape, np.float64)
    for t in range(len(x)):
        for e, s in zip(ids[t], wts[t]):
            out[t] += P.clamped_expert((s * x[t])[None].astype(np.float64), w, f"e{e}.", limit, np.float64)[0]
    return out


@pytest.mark.parametrize("T,E,top,W,F", [(5, 6, 2, 40, 24), (1, 3, 3, 36, 10), (33, 4, 1, 64, 48)])
def test_experts_row_by_row(dev, T, E, top, W, F):
    rt, k = dev
    rng = np.random.default_rng(T)
    w = expert_weights(rng, E, W, F)
    x = rng.normal(size=(T, W)).astype(np.float32)
    ids = np.stack([rng.permutation(E)[:top] for _ in range(T)]).astype(np.int32)
    wts = rng.uniform(0.1, 1.0, (T, top)).astype(np.float32)
    limit = 1.25
    want = plain_experts(x, ids, wts, w, limit)
    # the clamps bite: the test's own premise
    assert (np.abs(x @ w["e0.up"].T) > limit).mean() > 0.02
    gu = np.concatenate([w[f"e{e}.{r}"] for e in range(E) for r in ("gate", "up")])
    down = np.concatenate([w[f"e{e}.down"] for e in range(E)])
    y, out = rt.empty((T * top, F), "float32"), rt.empty((T, W), "float32")
    k.zk_moe_experts(up(rt, x).ptr, up(rt, ids).ptr, up(rt, wts).ptr, up(rt, gu).ptr, up(rt, down).ptr, y.ptr, out.ptr, T, top,
                     W, F, limit, rt.stream)
    assert np.abs(rt.download(out) - want).max() < 2e-5 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("T,E,top,W,F", [(70, 5, 2, 48, 24), (200, 16, 4, 64, 40), (64, 3, 1, 128, 72), (90, 7, 7, 32, 8)])
def test_experts_grouped_on_the_matrix_cores(T, E, top, W, F):
    """Sorted by expert and multiplied tile by tile: the same values as row by row (both round the
    scaled rows and the activations to bfloat16), whatever the groups' sizes; experts without a
    token, groups of one row and groups that end inside a tile among them."""
    from zse_amd.runtime.device import Runtime
    rt = Runtime.get()
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(E)
    w = expert_weights(rng, E, W, F)
    x = bf16(rng.normal(size=(T, W)))
    p = np.linspace(3.0, 0.2, E) ** 2
    ids = np.stack([rng.choice(E, top, replace=False, p=p / p.sum()) for _ in range(T)]).astype(np.int32)
    if top == 1:
        ids[ids == E - 1] = 0                    # the last expert gets no token
    wts = rng.uniform(0.1, 1.0, (T, top)).astype(np.float32)
    limit = 1.5
    gu = np.concatenate([w[f"e{e}.{r}"] for e in range(E) for r in ("gate", "up")])
    down = np.concatenate([w[f"e{e}.down"] for e in range(E)])
    d = [up16(rt, x), up(rt, ids), up(rt, wts), up16(rt, gu), up16(rt, down)]
    y, out = rt.empty((T * top, F), "bfloat16"), rt.empty((T, W), "float32")
    k.zk_moe_experts(d[0].ptr, d[1].ptr, d[2].ptr, d[3].ptr, d[4].ptr, y.ptr, out.ptr, T, top, W, F, limit, rt.stream)
    rows = rt.download(out)
    work = rt.empty((E + 1 + 2 * T * top,), "int32")
    xg, y2 = rt.empty((T * top, W), "bfloat16"), rt.empty((T * top, F), "bfloat16")
    tmp, out2 = rt.empty((T * top, W), "float32"), rt.empty((T, W), "float32")
    k.zk_moe_experts_grouped(d[0].ptr, d[1].ptr, d[2].ptr, d[3].ptr, d[4].ptr, work.ptr, xg.ptr, y2.ptr, tmp.ptr, out2.ptr,
                             T, E, top, W, F, limit, rt.stream)
    grouped = rt.download(out2)
    want = plain_experts(x, ids, wts, w, limit)
    big = max(1.0, np.abs(want).max())
    assert np.abs(rows - want).max() < 0.03 * big
    assert np.abs(grouped - want).max() < 0.03 * big
    assert np.abs(grouped - rows).max() < 0.01 * big          # a bfloat16 rounding of y apart at most


@pytest.mark.parametrize("M", [3, 16, 40, 200])
def test_the_clamped_gate_in_the_products_epilogue(M):
    """act(x Wg^T, x Wu^T) straight from the matrix-core product's float sums, for every kernel the
    number of rows picks; the clamps bite on both sides."""
    from zse_amd.runtime.device import Runtime
    rt = Runtime.get()
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(M)
    K, F, limit = 96, 80, 1.25
    x = bf16(rng.normal(size=(M, K)))
    w = bf16(rng.normal(0, 2.5 / np.sqrt(K), (2 * F, K)))
    g, u = x.astype(np.float64) @ w[:F].T, x.astype(np.float64) @ w[F:].T
    assert (g > limit).mean() > 0.05 and (np.abs(u) > limit).mean() > 0.1
    g, u = np.minimum(g, limit), np.clip(u, -limit, limit)
    want = g * P.sigmoid(1.702 * g) * (u + 1.0)
    out = rt.empty((M, F), "bfloat16")
    k.zk_gemm_bf16(up16(rt, x).ptr, K, up16(rt, w).ptr, out.ptr, F, 0, M, F, K, 6, limit, 0, None, 0, None, rt.stream)
    assert np.abs(rt.download_f32(out) - want).max() < 0.02 * np.abs(want).max()


@pytest.mark.parametrize("kn", [1, 0])
def test_products_per_head(dev, kn):
    rt, k = dev
    rng = np.random.default_rng(kn)
    T, H, K, N, ldx, ldo = 37, 3, 45, 70, 3 * 50 + 9, 3 * 80
    x = rng.normal(size=(T, ldx)).astype(np.float32)
    w = rng.normal(size=(H, K, N) if kn else (H, N, K)).astype(np.float32)
    out = rt.zeros((T, ldo), "float32")
    k.zk_heads_linear(up(rt, x).ptr, ldx, 50, up(rt, w).ptr, kn, out.ptr, ldo, 80, T, H, K, N, rt.stream)
    got = rt.download(out).reshape(T, H, 80)
    xs = np.stack([x[:, h * 50:h * 50 + K] for h in range(H)], axis=1).astype(np.float64)
    want = np.einsum("thk,hkn->thn", xs, w) if kn else np.einsum("thk,hnk->thn", xs, w)
    assert np.abs(got[:, :, :N] - want).max() < 1e-4 and not got[:, :, N:].any()


def test_latent_rows_queries_and_attention_with_sinks(dev):
    """The store of the normed latent and the rotated key part, the queries carried over to the
    latent's channels, and attention whose values are the first channels of its keys: together the
    plain attention over keys and values made from the latent."""
    rt, k = dev
    rng = np.random.default_rng(17)
    T, H, D, R, E, C, bs = 45, 3, 8, 6, 10, 20, 8
    eps, scale, base = 1e-5, 0.3, 40.0
    ld = H * (D + R) + C + R
    qd = rng.normal(size=(T, ld)).astype(np.float32)
    gain = rng.normal(1, 0.2, C).astype(np.float32)
    uk, uv = rng.normal(0, 0.3, (H * D, C)).astype(np.float32), rng.normal(0, 0.3, (H * E, C)).astype(np.float32)
    sinks = np.array([2.0, -1.0, 0.5], np.float32)
    f, _ = P.rotary_frequencies(R, base)
    pos = np.arange(T)
    q = qd[:, :H * (D + R)].reshape(T, H, D + R).astype(np.float64)
    c = P.rms_norm_plain(qd[:, H * (D + R):H * (D + R) + C], gain, eps, np.float64)
    k_rot = P.rotate(qd[:, None, H * (D + R) + C:], pos, f, 1.0, True, np.float64)
    q_rot = P.rotate(q[:, :, D:], pos, f, 1.0, True, np.float64)
    kk = np.concatenate([(c @ uk.T).reshape(T, H, D), np.broadcast_to(k_rot, (T, H, R))], axis=2)
    vv = (c @ uv.T).reshape(T, H, E)
    want = P.causal_attention(np.concatenate([q[:, :, :D], q_rot], axis=2), kk, vv, scale, sinks, np.float64)
    pages = -(-T // bs)
    table = np.arange(1, pages + 1)[::-1].copy()                   # pages in reverse: the table is really read
    slot_map = np.array([table[t // bs] * bs + t % bs for t in range(T)], np.int32)
    kcache = rt.zeros((pages + 1, 1, bs, C + R), "float32")
    qa = rt.zeros((T, H * (C + R)), "float32")
    k.zk_latent_prep(up(rt, qd).ptr, ld, i32(rt, pos).ptr, up(rt, slot_map).ptr, up(rt, gain).ptr, eps,
                     up(rt, f.astype(np.float32)).ptr, 1.0, 1, qa.ptr, kcache.ptr, T, H, D, R, C, bs, rt.stream)
    k.zk_heads_linear(up(rt, qd).ptr, ld, D + R, up(rt, uk).ptr, 1, qa.ptr, H * (C + R), C + R, T, H, D, C, rt.stream)
    o = rt.empty((T, H * C), "float32")
    k.zk_attention_plain_sink(qa.ptr, H * (C + R), kcache.ptr, kcache.ptr, i32(rt, table).ptr, pages, i32(rt, [0] * T).ptr,
                              i32(rt, pos).ptr, o.ptr, T, H, 1, C + R, C, bs, scale, 0.0, 0, 0, None, 0, up(rt, sinks).ptr, 1,
                              rt.stream)
    v = rt.empty((T, H * E), "float32")
    k.zk_heads_linear(o.ptr, H * C, C, up(rt, uv).ptr, 0, v.ptr, H * E, E, T, H, C, E, rt.stream)
    assert np.abs(rt.download(v).reshape(T, H, E) - want).max() < 2e-5
    cached = rt.download(kcache).reshape(-1, C + R)[slot_map]
    assert np.abs(cached[:, :C] - c).max() < 1e-5 and np.abs(cached[:, C:] - k_rot[:, 0]).max() < 1e-5


def test_wide_latent_rows(dev):
    """More channels than the attention kernel's narrow form holds (above 256)."""
    rt, k = dev
    rng = np.random.default_rng(5)
    T, H, C, R, bs = 20, 2, 300, 8, 4
    rows = rng.normal(0, 0.3, (T, C + R)).astype(np.float32)
    q = rng.normal(0, 0.3, (T, H, C + R)).astype(np.float32)
    sinks = np.array([0.3, -2.0], np.float32)
    want = P.causal_attention(q.astype(np.float64), rows[:, None].astype(np.float64), rows[:, None, :C].astype(np.float64), 0.5,
                              sinks, np.float64)
    pages = T // bs
    cache = np.zeros((pages + 1, 1, bs, C + R), np.float32)
    cache[1:] = rows.reshape(pages, 1, bs, C + R)
    o = rt.empty((T, H * C), "float32")
    d_c = up(rt, cache)
    k.zk_attention_plain_sink(up(rt, q).ptr, H * (C + R), d_c.ptr, d_c.ptr, i32(rt, np.arange(1, pages + 1)).ptr, pages,
                              i32(rt, [0] * T).ptr, i32(rt, np.arange(T)).ptr, o.ptr, T, H, 1, C + R, C, bs, 0.5, 0.0, 0, 0, None,
                              0, up(rt, sinks).ptr, 1, rt.stream)
    assert np.abs(rt.download(o).reshape(T, H, C) - want).max() < 2e-5


@pytest.mark.parametrize("H,C,R,bs", [(3, 20, 4, 8), (16, 256, 32, 16), (5, 96, 16, 4), (40, 64, 8, 16)])
def test_latent_attention_on_the_matrix_cores(H, C, R, bs):
    """Three requests in one step: a long portion from position 0, a portion behind a context, and
    one token behind a long context (its keys cut into ranges and joined); heads that do not fill
    a tile of rows, rows of one token that spread over two tiles, and sinks."""
    from zse_amd.runtime.device import Runtime
    rt = Runtime.get()
    k = rt.kernels("bfloat16")
    rng = np.random.default_rng(H)
    HD = C + R
    reqs = [(0, 150), (70, 37), (333, 1)]                          # (tokens already cached, tokens in the step)
    T = sum(n for _, n in reqs)
    sinks = rng.normal(0, 1, H).astype(np.float32)
    scale = 2.0 / np.sqrt(HD)
    max_ctx = max(a + n for a, n in reqs)
    max_blocks = -(-max_ctx // bs)
    pages = sum(-(-(a + n) // bs) for a, n in reqs)
    cache = np.zeros((pages + 1, 1, bs, HD), np.float32)
    table = np.full((len(reqs), max_blocks), -1, np.int32)
    order = rng.permutation(pages) + 1
    q_rows, want, q_start, ctx_len, positions, at = [], [], [0], [], [], 0
    for r, (a, n) in enumerate(reqs):
        L = a + n
        rows = bf16(rng.normal(0, 1, (L, HD)))
        mine = order[at:at + -(-L // bs)]
        at += len(mine)
        table[r, :len(mine)] = mine
        for j in range(L):
            cache[mine[j // bs], 0, j % bs] = rows[j]
        q = bf16(rng.normal(0, 1, (L, H, HD)))
        full = P.causal_attention(q.astype(np.float64), rows[:, None].astype(np.float64), rows[:, None, :C].astype(np.float64),
                                  scale, sinks, np.float64)
        q_rows.append(q[a:])
        want.append(full[a:])
        q_start.append(q_start[-1] + n)
        ctx_len.append(L)
        positions += list(range(a, L))
    q_all, want = np.concatenate(q_rows), np.concatenate(want)
    work = rt.empty((int(k.zk_latent_attention_bf16_workspace(32, H, C, 32)) // 4,), "float32")
    out = rt.empty((T, H * C), "bfloat16")
    d_cache = up16(rt, cache)
    for with_work in (True, False):
        k.zk_latent_attention_bf16(up16(rt, q_all).ptr, d_cache.ptr, up(rt, table).ptr, max_blocks, i32(rt, q_start).ptr,
                                   i32(rt, ctx_len).ptr, i32(rt, positions).ptr, up(rt, sinks).ptr, out.ptr,
                                   work.ptr if with_work else None, work.nbytes if with_work else 0, T, len(reqs), 160, 512, H,
                                   HD, C, bs, scale, rt.stream)
        got = rt.download_f32(out).reshape(T, H, C)
        assert np.abs(got - want).max() < 0.03 * np.abs(want).max(), with_work
    # the single token alone: few blocks, so its keys are cut into ranges
    a, n = reqs[2]
    k.zk_latent_attention_bf16(up16(rt, q_all[-1:]).ptr, d_cache.ptr, up(rt, table[2:]).ptr, max_blocks, i32(rt, [0, 1]).ptr,
                               i32(rt, [a + n]).ptr, i32(rt, [a]).ptr, up(rt, sinks).ptr, out.ptr, work.ptr, work.nbytes, 1, 1, 1,
                               512, H, HD, C, bs, scale, rt.stream)
    got = rt.download_f32(out).reshape(T, H, C)[0]
    assert np.abs(got - want[-1]).max() < 0.03 * np.abs(want).max()


def test_biases_and_scaled_rotation_in_front_of_an_attention(dev):
    rt, k = dev
    rng = np.random.default_rng(11)
    T, nh, nkv, D, E, bs, dims = 19, 4, 2, 12, 6, 4, 8
    width = (nh + nkv) * D + nkv * E
    qkv = rng.normal(size=(T, width)).astype(np.float32)
    bias = rng.normal(0, 0.5, width).astype(np.float32)
    pos = np.arange(3, 3 + T)
    f, mag = P.rotary_frequencies(dims, 100.0, {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0})
    x = (qkv + bias).astype(np.float64)
    q = P.rotate(x[:, :nh * D].reshape(T, nh, D), pos, f, mag, False, np.float64)
    kk = P.rotate(x[:, nh * D:(nh + nkv) * D].reshape(T, nkv, D), pos, f, mag, False, np.float64)
    vv = x[:, (nh + nkv) * D:].reshape(T, nkv, E)
    pages = -(-T // bs)
    slot_map = np.array([(1 + t // bs) * bs + t % bs for t in range(T)], np.int32)
    kc, vc = rt.zeros((pages + 1, nkv, bs, D), "float32"), rt.zeros((pages + 1, nkv, bs, E), "float32")
    d = up(rt, qkv)
    k.zk_head_prep_ext(d.ptr, i32(rt, pos).ptr, up(rt, slot_map).ptr, None, None, None, 1e-6, up(rt, f.astype(np.float32)).ptr,
                       dims, None, 0, kc.ptr, vc.ptr, T, nh, nkv, D, E, bs, 0, up(rt, bias).ptr, mag, 0, rt.stream)
    assert mag > 1.05
    assert np.abs(rt.download(d)[:, :nh * D].reshape(T, nh, D) - q).max() < 3e-5
    gk = rt.download(kc).transpose(0, 2, 1, 3).reshape(-1, nkv, D)[slot_map]
    gv = rt.download(vc).transpose(0, 2, 1, 3).reshape(-1, nkv, E)[slot_map]
    assert np.abs(gk - kk).max() < 3e-5 and np.abs(gv - vv).max() < 1e-6


@pytest.mark.parametrize("W", [36, 256, 1000])
def test_two_sublayers_join_the_stream(dev, W):
    """h <- h + (a + b + bias) and the next norm of it, a and b as activations or as float planes."""
    rt, k = dev
    rng = np.random.default_rng(W)
    T = 7
    h = rng.normal(size=(T, W)).astype(np.float32)
    a = rng.normal(size=(T, W)).astype(np.float32)
    planes = rng.normal(size=(3, T, W)).astype(np.float32)
    bias, g = rng.normal(size=W).astype(np.float32), rng.normal(0, 0.2, W).astype(np.float32)
    want_h = h.astype(np.float64) + (a.astype(np.float64) + planes.astype(np.float64).sum(axis=0) + bias)
    want = P.rms_norm_offset(want_h, g, 1e-5, np.float64)
    d_h, out = up(rt, h), rt.empty((T, W), "float32")
    k.zk_sum_norm(d_h.ptr, up(rt, a).ptr, 0, up(rt, planes).ptr, 3, up(rt, bias).ptr, up(rt, g).ptr, 1e-5, 1, out.ptr, T, W,
                  rt.stream)
    assert np.abs(rt.download(d_h) - want_h).max() < 1e-5 and np.abs(rt.download(out) - want).max() < 1e-5
    # one sublayer alone, no bias, no next norm
    d_h2 = up(rt, h)
    k.zk_sum_norm(d_h2.ptr, up(rt, planes).ptr, 1, None, 0, None, None, 0.0, 0, None, T, W, rt.stream)
    assert np.abs(rt.download(d_h2) - (h + planes[0])).max() < 1e-6
