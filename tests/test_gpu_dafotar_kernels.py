"""The kernels behind Dafotar's mechanisms, each alone against the plain function of the same
mechanism (tests/plain/dafotar_plain.py): residual streams with their layer norm, the short
convolution with its state over several steps, the matrix-memory recurrence cut into steps, and
the head norms / rotations in front of the attention."""
import numpy as np
import pytest

from plain import dafotar_plain as P

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


@pytest.mark.parametrize("S,W", [(1, 24), (2, 30), (3, 40), (8, 300)])
def test_streams_write_read_and_norm(dev, S, W):
    rt, k = dev
    rng = np.random.default_rng(S)
    T = 5
    xs = rng.normal(size=(T, S, W)).astype(np.float32)
    y = rng.normal(size=(T, W)).astype(np.float32)
    mix, out, win = (rng.normal(size=s).astype(np.float32) for s in ((S, S), (S,), (S,)))
    g, b = rng.normal(1, 0.2, W).astype(np.float32), rng.normal(0, 0.2, W).astype(np.float32)
    d_xs, d_o = up(rt, xs), rt.empty((T, W), "float32")
    k.zk_streams_step(d_xs.ptr, S, up(rt, y).ptr, 0, up(rt, mix).ptr, up(rt, out).ptr, up(rt, win).ptr, up(rt, g).ptr,
                      up(rt, b).ptr, 1e-5, None, d_o.ptr, T, T, W, rt.stream)
    want_xs = P.streams_write(xs, mix, out, y, np.float64)
    want = P.layer_norm(P.streams_read(want_xs, win, np.float64), g, b, 1e-5, np.float64)
    assert np.abs(rt.download(d_xs) - want_xs).max() < 1e-5
    assert np.abs(rt.download(d_o) - want).max() < 2e-5
    # the read of picked rows alone, streams summed with weight 1 (the model's last norm)
    rows = [4, 0, 2]
    d_p = rt.empty((3, W), "float32")
    k.zk_streams_step(d_xs.ptr, S, None, 0, None, None, None, up(rt, g).ptr, None, 1e-5, i32(rt, rows).ptr, d_p.ptr, 3, T, W,
                      rt.stream)
    want = P.layer_norm(want_xs.sum(axis=1)[rows], g, np.zeros(W), 1e-5, np.float64)
    assert np.abs(rt.download(d_p) - want).max() < 2e-5


def test_streams_write_from_partial_sums(dev):
    """A product that split K hands over float planes [P, T, W]; the kernel adds them up itself."""
    rt, k = dev
    rng = np.random.default_rng(9)
    T, S, W, Pn = 6, 4, 64, 3
    xs = rng.normal(size=(T, S, W)).astype(np.float32)
    planes = rng.normal(size=(Pn, T, W)).astype(np.float32)
    mix, out, win = (rng.normal(size=s).astype(np.float32) for s in ((S, S), (S,), (S,)))
    g, b = rng.normal(1, 0.2, W).astype(np.float32), rng.normal(0, 0.2, W).astype(np.float32)
    d_xs, d_o = up(rt, xs), rt.empty((T, W), "float32")
    k.zk_streams_step(d_xs.ptr, S, up(rt, planes).ptr, Pn, up(rt, mix).ptr, up(rt, out).ptr, up(rt, win).ptr, up(rt, g).ptr,
                      up(rt, b).ptr, 1e-5, None, d_o.ptr, T, T, W, rt.stream)
    y = planes[0] + planes[1] + planes[2]
    want_xs = P.streams_write(xs, mix, out, y, np.float64)
    want = P.layer_norm(P.streams_read(want_xs, win, np.float64), g, b, 1e-5, np.float64)
    assert np.abs(rt.download(d_xs) - want_xs).max() < 1e-5
    assert np.abs(rt.download(d_o) - want).max() < 2e-5


@pytest.mark.parametrize("taps", [2, 4, 7])
def test_short_convolution_over_steps(dev, taps):
    """Two requests whose rows come in portions of unequal sizes, also of one and two rows, side
    by side; the state carries the rows a portion cannot see."""
    rt, k = dev
    rng = np.random.default_rng(taps)
    W = 70
    w = rng.normal(size=(W, taps)).astype(np.float32)
    seqs = {0: rng.normal(size=(23, W)).astype(np.float32), 1: rng.normal(size=(17, W)).astype(np.float32)}
    want = {r: P.short_conv(h, w, np.float64) for r, h in seqs.items()}
    words = 8 + (taps - 1) * W + 5
    state = rt.zeros((3, words), "float32")
    slot = {0: 2, 1: 0}
    cuts = {0: [1, 2, 9, 1, 1, 5, 4], 1: [6, 1, 2, 2, 1, 1, 4]}
    at = {0: 0, 1: 0}
    got = {0: [], 1: []}
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
        d_h, d_o = up(rt, h), rt.empty((T, W), "float32")
        args = (i32(rt, q_start).ptr, i32(rt, [slot[0], slot[1]]).ptr)
        k.zk_short_conv(d_h.ptr, d_w.ptr, state.ptr, words, 8, i32(rt, pos).ptr, i32(rt, req).ptr, *args, d_o.ptr, T, W, taps,
                        rt.stream)
        k.zk_short_conv_state(d_h.ptr, state.ptr, words, 8, *args, 2, W, taps, rt.stream)
        o = rt.download(d_o)
        got[0].append(o[:q_start[1]])
        got[1].append(o[q_start[1]:])
    for r in (0, 1):
        assert np.abs(np.concatenate(got[r]) - want[r]).max() < 1e-5, r
    st = rt.download(state)
    assert not st[1].any() and not st[:, :8].any() and not st[:, 8 + (taps - 1) * W:].any()     # nothing outside its place


@pytest.mark.parametrize("H,D,E", [(1, 8, 8), (3, 12, 20), (2, 64, 128), (2, 20, 256), (1, 200, 256)])
def test_matrix_memory_cut_into_steps(dev, H, D, E):
    rt, k = dev
    rng = np.random.default_rng(D)
    T, W = 29, 16
    mx = {"heads": H, "dim": D, "vdim": E, "gate_cap": 5.0}
    # the recurrence alone: feed it projections directly (identity-free), compare with the plain
    # mixer given weights that reproduce them
    h = rng.normal(size=(T, W)).astype(np.float32)
    wts = {"q": rng.normal(size=(H * D, W)) * 0.5, "k": rng.normal(size=(H * D, W)) * 0.5,
           "v": rng.normal(size=(H * E, W)) * 0.5, "g": rng.normal(size=(H * E, W)) * 0.5,
           "i": rng.normal(size=(H, W)) * 2.0, "f": rng.normal(size=(H, W)) * 2.0,
           "i.b": rng.normal(size=H), "f.b": rng.normal(size=H) + 2.0, "norm": rng.normal(1, 0.2, H * E),
           "o": np.eye(H * E)}
    wts = {n: a.astype(np.float32) for n, a in wts.items()}
    want = P.mlstm(h, wts, "", mx, 1e-6, np.float64)
    qkvz = np.concatenate([h @ wts[n].T for n in ("q", "k", "v", "g")], axis=1).astype(np.float32)
    gates = np.concatenate([h @ wts["i"].T, h @ wts["f"].T], axis=1).astype(np.float32)
    words = 4 + k.zk_mlstm_state_bytes(H, D, E) // 4
    for cuts in ([T], [1] * T, [5, 2, 1, 13, 8]):
        state = rt.zeros((2, words), "float32")
        got, at = [], 0
        for n in cuts:
            d_o = rt.empty((n, H * E), "float32")
            k.zk_mlstm(up(rt, qkvz[at:at + n]).ptr, qkvz.shape[1], up(rt, gates[at:at + n]).ptr, up(rt, wts["i.b"]).ptr,
                       up(rt, wts["f.b"]).ptr, up(rt, wts["norm"]).ptr, state.ptr, words, 4, i32(rt, [0, n]).ptr,
                       i32(rt, [1]).ptr, d_o.ptr, 1, H, D, E, 5.0, 1e-6, rt.stream)
            got.append(rt.download(d_o))
            at += n
        got = np.concatenate(got)
        assert np.abs(got - want).max() < 3e-5 * max(1.0, np.abs(want).max()), cuts
        assert not rt.download(state)[0].any()


@pytest.mark.parametrize("side_by_side", [False, True])
@pytest.mark.parametrize("H,D,E", [(1, 8, 8), (3, 12, 20), (2, 64, 128), (1, 128, 48), (1, 256, 40)])
def test_matrix_memory_in_chunks(dev, H, D, E, side_by_side):
    """The chunked form of the recurrence with its finishing kernel: two requests side by side,
    portions of 1 to 150 tokens (chunks of 16, 32 and 64; full, partial and single-token ones),
    continuing from the state the portion before left.  ``side_by_side``: the three launches that
    run a step's chunks at once, instead of the kernel that walks them."""
    rt, k = dev
    rng = np.random.default_rng(D + E)
    W = 16
    mx = {"heads": H, "dim": D, "vdim": E, "gate_cap": 5.0}
    wts = {"q": rng.normal(size=(H * D, W)) * 0.5, "k": rng.normal(size=(H * D, W)) * 0.5,
           "v": rng.normal(size=(H * E, W)) * 0.5, "g": rng.normal(size=(H * E, W)) * 0.5,
           "i": rng.normal(size=(H, W)) * 2.0, "f": rng.normal(size=(H, W)) * 2.0,
           "i.b": rng.normal(size=H), "f.b": rng.normal(size=H) + 2.0, "norm": rng.normal(1, 0.2, H * E),
           "o": np.eye(H * E)}
    wts = {n: a.astype(np.float32) for n, a in wts.items()}
    lens = {0: 236, 1: 97}
    hs = {r: rng.normal(size=(n, W)).astype(np.float32) for r, n in lens.items()}
    want = {r: P.mlstm(h, wts, "", mx, 1e-6, np.float64) for r, h in hs.items()}
    proj = {r: np.concatenate([h @ wts[n].T for n in ("q", "k", "v", "g")], axis=1).astype(np.float32) for r, h in hs.items()}
    gate = {r: np.concatenate([h @ wts["i"].T, h @ wts["f"].T], axis=1).astype(np.float32) for r, h in hs.items()}
    cuts = {0: [150, 1, 17, 64, 4], 1: [30, 33, 1, 2, 31]}
    words = 4 + k.zk_mlstm_state_bytes(H, D, E) // 4
    state = rt.zeros((3, words), "float32")
    slots = [2, 0]
    at = {0: 0, 1: 0}
    got = {0: [], 1: []}
    bi, bf, g = up(rt, wts["i.b"]), up(rt, wts["f.b"]), up(rt, wts["norm"])
    for step in range(5):
        n0, n1 = cuts[0][step], cuts[1][step]
        T = n0 + n1
        rows = np.concatenate([proj[0][at[0]:at[0] + n0], proj[1][at[1]:at[1] + n1]])
        gts = np.concatenate([gate[0][at[0]:at[0] + n0], gate[1][at[1]:at[1] + n1]])
        d_rows, d_g = up(rt, rows), up(rt, gts)
        q_start, req = i32(rt, [0, n0, T]), i32(rt, [0] * n0 + [1] * n1)
        d_slots = i32(rt, slots)
        o_raw, nm, d_o = rt.zeros((T, H * E), "float32"), rt.zeros((2, H * (D + 1)), "float32"), rt.empty((T, H * E), "float32")
        if side_by_side:
            floats = k.zk_mlstm_scan_floats(T, 2, H, D, E, max(n0, n1))
            work = rt.zeros((floats,), "float32")
            k.zk_mlstm_scan(d_rows.ptr, rows.shape[1], d_g.ptr, bi.ptr, bf.ptr, state.ptr, words, 4, q_start.ptr, d_slots.ptr,
                            o_raw.ptr, work.ptr, floats, T, 2, H, D, E, 5.0, max(n0, n1), rt.stream)
        else:
            k.zk_mlstm_chunked(d_rows.ptr, rows.shape[1], d_g.ptr, bi.ptr, bf.ptr, state.ptr, words, 4, q_start.ptr, d_slots.ptr,
                               o_raw.ptr, nm.ptr, 2, H, D, E, 5.0, max(n0, n1), rt.stream)
        k.zk_mlstm_finish(o_raw.ptr, d_rows.ptr, rows.shape[1], g.ptr, None if side_by_side else nm.ptr, state.ptr, words, 4,
                          req.ptr, q_start.ptr, d_slots.ptr, d_o.ptr, T, H, D, E, 1e-6, rt.stream)
        o = rt.download(d_o)
        got[0].append(o[:n0])
        got[1].append(o[n0:])
        at[0] += n0
        at[1] += n1
    for r in (0, 1):
        err = np.abs(np.concatenate(got[r]) - want[r]).max()
        assert err < 5e-5 * max(1.0, np.abs(want[r]).max()), (r, err)
    # and the state it leaves is the one the token-by-token kernel leaves
    seq = rt.zeros((3, words), "float32")
    for r in (0, 1):
        d_o = rt.empty((lens[r], H * E), "float32")
        k.zk_mlstm(up(rt, proj[r]).ptr, proj[r].shape[1], up(rt, gate[r]).ptr, bi.ptr, bf.ptr, g.ptr, seq.ptr, words, 4,
                   i32(rt, [0, lens[r]]).ptr, i32(rt, [slots[r]]).ptr, d_o.ptr, 1, H, D, E, 5.0, 1e-6, rt.stream)
    a, b = rt.download(state), rt.download(seq)
    assert np.abs(a - b).max() < 1e-4 * max(1.0, np.abs(b).max())
    assert not a[1].any() and not a[:, :4].any()


def test_the_running_maximum_starts_at_zero(dev):
    """With strongly negative input gates the first outputs are governed by exp(-m) with m = 0
    in the denominator; a maximum that started at minus infinity would give other values."""
    rt, k = dev
    H, D, E, T, W = 1, 4, 4, 3, 4
    mx = {"heads": H, "dim": D, "vdim": E, "gate_cap": 20.0}
    rng = np.random.default_rng(0)
    h = rng.normal(size=(T, W)).astype(np.float32)
    wts = {n: (rng.normal(size=(s, W)) * 0.5).astype(np.float32) for n, s in (("q", D), ("k", D), ("v", E), ("g", E))}
    wts.update({"i": np.zeros((H, W), np.float32), "f": np.zeros((H, W), np.float32), "i.b": np.full(H, -8.0, np.float32),
                "f.b": np.full(H, 3.0, np.float32), "norm": np.ones(H * E, np.float32), "o": np.eye(H * E, dtype=np.float32)})
    want = P.mlstm(h, wts, "", mx, 1e-6, np.float64)
    qkvz = np.concatenate([h @ wts[n].T for n in ("q", "k", "v", "g")], axis=1).astype(np.float32)
    gates = np.zeros((T, 2), np.float32)
    words = k.zk_mlstm_state_bytes(H, D, E) // 4
    state = rt.zeros((1, words), "float32")
    d_o = rt.empty((T, E), "float32")
    k.zk_mlstm(up(rt, qkvz).ptr, qkvz.shape[1], up(rt, gates).ptr, up(rt, wts["i.b"]).ptr, up(rt, wts["f.b"]).ptr,
               up(rt, wts["norm"]).ptr, state.ptr, words, 0, i32(rt, [0, T]).ptr, i32(rt, [0]).ptr, d_o.ptr, 1, H, D, E, 20.0,
               1e-6, rt.stream)
    assert np.abs(rt.download(d_o) - want).max() < 1e-5
    # m went down from 0 by the forget gate alone, three times; from minus infinity it would have become i = -8
    f = float(P.log_sigmoid(np.float64(20.0 * np.tanh(3.0 / 20.0))))
    assert rt.download(state)[0, -1] == pytest.approx(3 * f, abs=1e-5)


@pytest.mark.parametrize("inter", [0, 1])
def test_head_norms_rotations_and_the_store(dev, inter):
    rt, k = dev
    rng = np.random.default_rng(4 + inter)
    T, nh, nkv, D, E, bs, dims = 6, 4, 2, 12, 20, 4, 8
    width = (nh + nkv) * D + nkv * E
    rows = rng.normal(size=(T, width)).astype(np.float32)
    gq, gk = rng.normal(1, 0.3, D).astype(np.float32), rng.normal(1, 0.3, D).astype(np.float32)
    temp = rng.normal(1, 0.3, nh).astype(np.float32)
    pos = np.array([3, 4, 5, 17, 0, 9])
    slots = np.array([5, 6, 7, 12, 20, 9])
    base = 100.0
    f = np.power(base, -2.0 * np.arange(dims // 2) / dims).astype(np.float32)
    vf = np.power(base, -2.0 * np.arange(E // 2) / E).astype(np.float32)
    pages = 8
    d_rows = up(rt, rows)
    kc, vc = rt.zeros((pages, nkv, bs, D), "float32"), rt.zeros((pages, nkv, bs, E), "float32")
    k.zk_head_prep(d_rows.ptr, i32(rt, pos).ptr, i32(rt, slots).ptr, up(rt, gq).ptr, up(rt, gk).ptr, up(rt, temp).ptr, 1e-5,
                   up(rt, f).ptr, dims, up(rt, vf).ptr, inter, kc.ptr, vc.ptr, T, nh, nkv, D, E, bs, 0, rt.stream)
    q = rows[:, :nh * D].reshape(T, nh, D)
    kk = rows[:, nh * D:(nh + nkv) * D].reshape(T, nkv, D)
    v = rows[:, (nh + nkv) * D:].reshape(T, nkv, E)
    want_q = P.rotate(P.unit_rms(q, 1e-5, np.float64) * gq, pos, base, dims, np.float64) * temp[None, :, None]
    want_k = P.rotate(P.unit_rms(kk, 1e-5, np.float64) * gk, pos, base, dims, np.float64)
    want_v = P.rotate(v, pos, base, E, np.float64, interleaved=bool(inter))
    got = rt.download(d_rows)
    assert np.abs(got[:, :nh * D].reshape(T, nh, D) - want_q).max() < 1e-5
    assert np.array_equal(got[:, nh * D:], rows[:, nh * D:])            # keys and values leave through the cache only
    gk_, gv_ = rt.download(kc), rt.download(vc)
    for t in range(T):
        pg, off = slots[t] // bs, slots[t] % bs
        assert np.abs(gk_[pg, :, off, :] - want_k[t]).max() < 1e-5
        assert np.abs(gv_[pg, :, off, :] - want_v[t]).max() < 1e-5
    # and back: an output turned by minus its position is the unrotated value again
    d_v = up(rt, want_v.reshape(T, nkv * E).astype(np.float32))
    k.zk_rotate_heads(d_v.ptr, i32(rt, pos).ptr, up(rt, vf).ptr, T, nkv, E, inter, -1.0, rt.stream)
    assert np.abs(rt.download(d_v).reshape(T, nkv, E) - v).max() < 1e-5
