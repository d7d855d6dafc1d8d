"""Gipozen on the GPU against the plain restatement (oracle/gipozen.py, float64): every kernel alone, then the model through the
engine -- whole prompts, token-by-token decoding, portions down to two tokens, unequal batches, reused pages and slots, decoding
far past every window, greedy generation through the scheduler, the trace replay command.  Small random configurations made
here; sizes are unlike one another and unlike any shipped model.  Unused cache memory is poisoned with NaN so that a read
outside a sequence's own keys or of a stale state shows."""
import numpy as np
import pytest
import torch

import gipozen_util as U
from oracle import gipozen as O

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def mops():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    torch.backends.cuda.matmul.allow_tf32 = False
    from aphrodite_engine_amd import mixer_ops
    return mixer_ops


def dev(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(DEV).to(dtype)


def i32(a):
    return torch.tensor(list(a), dtype=torch.int32, device=DEV)


def rounded(a, dtype):
    return U.bf16_round(a).astype(np.float64) if dtype == torch.bfloat16 else np.asarray(a, np.float32).astype(np.float64)


def tol_of(dtype):
    return 3e-5 if dtype == torch.float32 else 2e-2


# ---------------------------------------------------------------------------------------------------------------------
# norms and activations
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [72, 75, 200, 1032])      # 75: rows that cannot be read 16 bytes at a time
def test_depth_residual_rms_norm_every_step(mops, dtype, width):
    rng = np.random.default_rng(width)
    T, eps, entries = 5, 1e-5, 6
    for n_hist in (0, 1, 2, 5):
        hist = rng.standard_normal((entries, T, width)).astype(np.float32)
        x0 = rng.standard_normal((T, width)).astype(np.float32) * 3
        y = rounded(rng.standard_normal((T, width + 8)) * 2 + 0.5, dtype)
        w = rng.standard_normal(n_hist + 1).astype(np.float32)
        weight = rounded(1 + 0.3 * rng.standard_normal(width), dtype)
        h, x = dev(hist), dev(x0)
        out = mops.depth_residual_rms_norm(x, x_out=x, y=dev(y, dtype)[:, :width], history=h, n_hist=n_hist, depth_w=dev(w), gain=1.7,
                                           weight=dev(weight, dtype), eps=eps)
        r = x0.astype(np.float64) + y[:, :width]
        np.testing.assert_allclose(h[n_hist].cpu().numpy(), r, rtol=1e-6, atol=1e-6)
        avg = O.depth_average(list(hist[:n_hist].astype(np.float64)) + [r], w)
        np.testing.assert_allclose(x.cpu().numpy(), avg, rtol=2e-6, atol=2e-5)
        np.testing.assert_allclose(h[n_hist + 1:].cpu().numpy(), hist[n_hist + 1:])       # later entries untouched
        np.testing.assert_allclose(out.float().cpu().numpy(), O.scalar_rms_norm(avg, 1.7, eps) * weight, rtol=tol_of(dtype),
                                   atol=tol_of(dtype))
    # the plain steps alone: copy + norm, add + norm, add without a norm
    x0 = rng.standard_normal((T, width)).astype(np.float32)
    x = torch.empty(T, width, device=DEV)
    out = mops.depth_residual_rms_norm(dev(x0), x_out=x, gain=0.6, eps=eps, dtype=dtype)
    np.testing.assert_array_equal(x.cpu().numpy(), x0)
    np.testing.assert_allclose(out.float().cpu().numpy(), O.scalar_rms_norm(x0.astype(np.float64), 0.6, eps), rtol=tol_of(dtype),
                               atol=tol_of(dtype))
    y = rounded(rng.standard_normal((T, width)), dtype)
    assert mops.depth_residual_rms_norm(x, x_out=x, y=dev(y, dtype), want_out=False) is None
    np.testing.assert_allclose(x.cpu().numpy(), x0 + y, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n", [88, 75, 1032, 4104])
def test_poly_norm(mops, dtype, n):
    rng = np.random.default_rng(n)
    z = rounded(rng.standard_normal((4, n + 8)) * 1.5, dtype)
    z[1] *= 1e-3                                           # a row where eps matters
    coef = (0.8, -0.4, 0.3, 0.15)
    got = mops.poly_norm(dev(z, dtype)[:, :n], coef, 1e-5).float().cpu().numpy()
    np.testing.assert_allclose(got, O.poly_norm(z[:, :n], coef, 1e-5), rtol=tol_of(dtype), atol=tol_of(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,vdim,maps", [(3, 40, 2), (1, 200, 2), (5, 64, 1), (6, 24, 2)])
def test_differential_norm_gate(mops, dtype, heads, vdim, maps):
    rng = np.random.default_rng(heads * vdim)
    T, lam, sc, eps = 7, 0.37, 0.8, 1e-5
    a = rng.standard_normal((T, heads, maps, vdim)).astype(np.float32)
    g = rounded(rng.standard_normal((T, heads * vdim + 8)), dtype)
    out = torch.zeros(T, heads * vdim + 16, dtype=dtype, device=DEV)
    mops.differential_norm_gate(out[:, :heads * vdim], dev(a.reshape(T, -1)), dev(g, dtype)[:, :heads * vdim], heads, maps, vdim, lam, sc,
                                eps)
    o = a[:, :, 0].astype(np.float64) - (lam * a[:, :, 1] if maps == 2 else 0.0)
    want = (O.rms_unit(o, eps) * sc).reshape(T, -1) * O.sigmoid(g[:, :heads * vdim])
    np.testing.assert_allclose(out[:, :heads * vdim].float().cpu().numpy(), want, rtol=tol_of(dtype), atol=tol_of(dtype))
    assert float(out[:, heads * vdim:].abs().max()) == 0.0


# ---------------------------------------------------------------------------------------------------------------------
# short convolution with its state
# ---------------------------------------------------------------------------------------------------------------------
def conv_in_steps(mops, us, w, cuts, dtype, cq, ck, cv, slots=None, state=None, caches=None, block=4):
    """Sequences us[i] [T_i, C] cut as cuts[i] (sizes), one segment of each live sequence per step; returns per sequence the
    convolved q rows and the (k, v) rows read back from the caches."""
    n, C, taps = len(us), w.shape[0], w.shape[1]
    slots = slots if slots is not None else list(range(n))
    state = state if state is not None else torch.full((max(slots) + 1, taps - 1, C), float("nan"), dtype=dtype, device=DEV)
    total = sum(len(u) for u in us)
    kc = torch.full((total + n * block, max(ck, 1)), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((total + n * block, max(cv, 1)), float("nan"), dtype=dtype, device=DEV)
    base = np.cumsum([0] + [len(u) + block for u in us])
    at, outs = [0] * n, [[] for _ in us]
    wd = dev(w, dtype)
    for step in range(max(len(c) for c in cuts)):
        live = [i for i in range(n) if step < len(cuts[i])]
        rows = [us[i][at[i]:at[i] + cuts[i][step]] for i in live]
        lens = [len(r) for r in rows]
        starts = np.cumsum([0] + lens[:-1])
        u = dev(np.concatenate(rows), dtype)
        pad = torch.zeros(u.shape[0], C + 8, dtype=dtype, device=DEV)      # rows with a stride of their own
        pad[:, :C] = u
        seq_of = np.concatenate([[j] * n_ for j, n_ in enumerate(lens)])
        slot_map = torch.tensor(np.concatenate([base[i] + at[i] + np.arange(n_) for i, n_ in zip(live, lens)]), dtype=torch.int64,
                                device=DEV)
        q = mops.short_conv(pad[:, :C], wd, state, i32([slots[i] for i in live]), i32(starts), i32(lens), i32([at[i] for i in live]),
                            i32(seq_of), cq, ck, cv, kc.view(-1, 1, ck) if ck else None, vc.view(-1, 1, cv) if cv else None,
                            slot_map if ck else None)
        for j, i in enumerate(live):
            outs[i].append(q[starts[j]:starts[j] + lens[j]].float().cpu().numpy())
            at[i] += lens[j]
    res = []
    for i, u in enumerate(us):
        q = np.concatenate(outs[i])
        k = kc[base[i]:base[i] + len(u)].float().cpu().numpy()
        v = vc[base[i]:base[i] + len(u)].float().cpu().numpy()
        res.append(np.concatenate([q] + ([k, v] if ck else []), axis=1))
    return res, state


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 3, 4, 7])
@pytest.mark.parametrize("channels", [(52, 20, 37), (48, 16, 40)])      # the second: rows that are read 16 bytes at a time
def test_short_conv_in_steps_of_every_size(mops, dtype, taps, channels):
    rng = np.random.default_rng(taps)
    cq, ck, cv = channels
    C = cq + ck + cv
    w = rounded(rng.standard_normal((C, taps)), dtype)
    us = [rounded(rng.standard_normal((n, C)), dtype) for n in (29, 1, 12)]
    want = [O.short_causal_conv(u, w) for u in us]
    for cuts in ([[29], [1], [12]], [[1] * 29, [1], [1] * 12], [[2, 1, 1, 9, 3, 1, 12], [1], [5, 2, 2, 3]],
                 [[20, 2, 2, 2, 2, 1], [1], [1, 1, 10]]):
        got, _ = conv_in_steps(mops, us, w, cuts, dtype, cq, ck, cv)
        for g, x in zip(got, want):
            np.testing.assert_allclose(g, x, rtol=tol_of(dtype), atol=tol_of(dtype))


def test_short_conv_slot_taken_over_and_queries_alone(mops):
    rng = np.random.default_rng(5)
    C, taps = 24, 4
    w = rng.standard_normal((C, taps)).astype(np.float32)
    a, b = rng.standard_normal((9, C)).astype(np.float32), rng.standard_normal((6, C)).astype(np.float32)
    _, state = conv_in_steps(mops, [a], w, [[4, 5]], torch.float32, C, 0, 0, slots=[1])
    # the next request lands in the same slot and starts with single tokens: nothing of the old state may reach it
    got, _ = conv_in_steps(mops, [b], w, [[1, 1, 2, 2]], torch.float32, C, 0, 0, slots=[1], state=state)
    np.testing.assert_allclose(got[0], O.short_causal_conv(b.astype(np.float64), w.astype(np.float64)), rtol=3e-5, atol=3e-5)


# ---------------------------------------------------------------------------------------------------------------------
# attention under a window that keeps the first tokens
# ---------------------------------------------------------------------------------------------------------------------
def attend(mops, q, k, v, cuts, dtype, heads, kv_heads, maps, scale, window, keep_first, block=16):
    """One sequence: q [T, H * maps * d], k [T, G * maps * d], v [T, G * e]; its rows run in segments of sizes ``cuts`` over a
    paged cache whose pages are shuffled and whose unused memory is NaN.  -> fp32 [T, H * maps * e]"""
    T = q.shape[0]
    d, e = q.shape[1] // (heads * maps), v.shape[1] // kv_heads
    pages = (T + block - 1) // block
    perm = np.random.default_rng(1).permutation(pages + 3)[:pages]
    kc = torch.full((pages + 3, block, kv_heads * maps, d), float("nan"), dtype=dtype, device=DEV)
    vc = torch.full((pages + 3, block, kv_heads, e), float("nan"), dtype=dtype, device=DEV)
    outs, a = [], 0
    for n in cuts:
        pos = np.arange(a, a + n)
        slots = torch.tensor(perm[pos // block] * block + pos % block, dtype=torch.int64, device=DEV)
        kc.view(-1, k.shape[1])[slots] = dev(k[a:a + n], dtype)
        vc.view(-1, v.shape[1])[slots] = dev(v[a:a + n], dtype)
        outs.append(mops.windowed_attention(dev(q[a:a + n], dtype), kc, vc, i32(perm).view(1, -1), i32([0]), i32([n]), i32([a]),
                                            i32([0] * n), (n, n), heads, maps, scale, window, keep_first, max_kv_len=a + n))
        a += n
    assert a == T
    return torch.cat(outs).cpu().numpy()


def attention_oracle(q, k, v, heads, kv_heads, maps, scale, window, keep_first):
    T = q.shape[0]
    d, e = q.shape[1] // (heads * maps), v.shape[1] // kv_heads
    q, k, v = q.reshape(T, heads, maps, d), k.reshape(T, kv_heads, maps, d), v.reshape(T, kv_heads, e)
    out = np.zeros((T, heads, maps, e))
    for h in range(heads):
        g = h // (heads // kv_heads)
        for m in range(maps):
            out[:, h, m] = O.windowed_softmax_attention(q[:, h, m], k[:, g, m], v[:, g], scale, window if window > 0 else T, keep_first)
    return out.reshape(T, -1)


ATT_SHAPES = [  # heads, kv heads, maps, dim, vdim, window, keep_first
    (6, 2, 2, 24, 40, 23, 3), (4, 4, 2, 32, 64, 64, 0), (3, 1, 1, 16, 72, 17, 1), (8, 2, 2, 64, 32, 200, 5), (2, 1, 2, 20, 130, 0, 0),
    (4, 2, 2, 128, 128, 31, 40)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", ATT_SHAPES)
def test_attention_prompt_portions_and_decode(mops, dtype, shape):
    H, G, M, d, e, window, keep = shape
    rng = np.random.default_rng(H * d + e)
    T = 150
    q = rounded(rng.standard_normal((T, H * M * d)) * 1.5, dtype)
    k = rounded(rng.standard_normal((T, G * M * d)) * 1.5, dtype)
    v = rounded(rng.standard_normal((T, G * e)), dtype)
    want = attention_oracle(q, k, v, H, G, M, d ** -0.5, window, keep)
    for cuts in ([150], [70, 2, 33, 1, 1, 1, 42], [100] + [1] * 50, [9, 64, 77]):
        got = attend(mops, q, k, v, cuts, dtype, H, G, M, d ** -0.5, window, keep)
        np.testing.assert_allclose(got, want, rtol=tol_of(dtype), atol=tol_of(dtype), err_msg=str(cuts))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("decoded", [False, True])
def test_window_and_kept_tokens_end_exactly_where_they_should(mops, decoded, dtype):
    """One key made dominant (its value one-hot): the row's output shows whether it was seen.  Keys at the window's two sides,
    at the last kept token and the first one that is not, at page borders, and far back among hundreds."""
    H, G, M, d, e, window, keep = 2, 1, 2, 32, 64, 37, 5
    T = 300
    rng = np.random.default_rng(3)
    base_q = rng.standard_normal((T, H * M * d)) * 0.1
    base_k = rng.standard_normal((T, G * M * d)) * 0.1
    for row in (299, 150, 64, 48):
        for key, seen in ((row - window + 1, True), (row - window, False), (keep - 1, True), (keep, row - keep < window), (0, True),
                          (row, True), (16, row - 16 < window), (15, row - 15 < window)):
            q, k = base_q.copy(), base_k.copy()
            v = np.zeros((T, G * e))
            v[:, 1] = 1.0
            v[key] = 0.0
            v[key, 0] = 1.0
            q[row] = 0.0
            k[key] = 0.0
            q[row].reshape(H, M, d)[:, :, 7] = 6.0
            k[key].reshape(G, M, d)[:, :, 7] = 6.0          # score 36 * scale against ~0 for every other key
            cuts = [row, 1] if decoded else [row + 1]
            got = attend(mops, rounded(q, dtype)[:row + 1], rounded(k, dtype)[:row + 1], v[:row + 1], cuts, dtype, H, G, M, 1.0, window,
                         keep)
            col0 = got[row].reshape(H * M, e)[:, 0]
            assert (col0 > 0.99).all() if seen else (col0 < 1e-6).all(), (row, key, seen, col0)


FUSED_SHAPES = [  # heads, kv heads, dim, vdim, window, keep_first
    (4, 1, 32, 96, 17, 3), (6, 2, 64, 32, 64, 0), (2, 2, 128, 128, 100, 1), (8, 2, 96, 64, 0, 0), (3, 3, 32, 32, 5, 70), (4, 2, 64, 128, 1, 0)]


@pytest.mark.parametrize("shape", FUSED_SHAPES)
def test_fused_differential_attention_in_mixed_batches(mops, shape):
    """The one-launch form (both maps, join, unit RMS, gate) against the restatement: two sequences that advance together in
    unequal segments -- portions of 8 rows and more beside shorter ones and single tokens -- over shuffled pages.  Every seventh
    key is made loud, so a row that sees one key too many or too few at an edge of its window shows."""
    H, G, d, e, window, keep = shape
    assert mops.differential_window_attention_supported(H, G, d, e, torch.bfloat16)
    rng = np.random.default_rng(H * d + e)
    lens, block = (210, 77), 16
    lam, diff, eps = 0.45, 0.35, 1e-5
    seqs = []
    for T in lens:
        q = U.bf16_round(rng.standard_normal((T, H * 2 * d)))
        k = rng.standard_normal((T, G * 2 * d))
        k[3::7] *= 3.0
        seqs.append((q, U.bf16_round(k), U.bf16_round(rng.standard_normal((T, G * e))), U.bf16_round(rng.standard_normal((T, H * e + 4)))))
    want = [O.differential_attention(q.astype(np.float64), k.astype(np.float64), v.astype(np.float64), H, G, d, e, d ** -0.5,
                                     window if window > 0 else 10 ** 6, keep, lam, diff, eps) * O.sigmoid(g[:, :H * e])
            for q, k, v, g in seqs]
    pages = [(T + block - 1) // block for T in lens]
    perm = np.random.default_rng(2).permutation(sum(pages) + 2)
    tables = [perm[:pages[0]], perm[pages[0]:pages[0] + pages[1]]]
    bt = np.zeros((2, max(pages)), np.int32)
    for i in range(2):
        bt[i, :pages[i]] = tables[i]
    kc = torch.full((sum(pages) + 2, block, G * 2, d), float("nan"), dtype=torch.bfloat16, device=DEV)
    vc = torch.full((sum(pages) + 2, block, G, e), float("nan"), dtype=torch.bfloat16, device=DEV)
    plan = [(70, 1), (2, 9), (1, 1), (64, 3), (9, 7), (1, 40), (63, 16)]
    at, got = [0, 0], [[], []]
    for step in plan:
        live = [i for i in range(2) if step[i] and at[i] < lens[i]]
        ns = [min(step[i], lens[i] - at[i]) for i in live]
        order = sorted(range(len(live)), key=lambda j: ns[j] == 1 and at[live[j]] > 0)       # portions first, single tokens last
        live, ns = [live[j] for j in order], [ns[j] for j in order]
        starts = np.cumsum([0] + ns[:-1])
        for i, n in zip(live, ns):
            pos = np.arange(at[i], at[i] + n)
            slots = torch.tensor(tables[i][pos // block] * block + pos % block, dtype=torch.int64, device=DEV)
            kc.view(-1, G * 2 * d)[slots] = dev(seqs[i][1][at[i]:at[i] + n], torch.bfloat16)
            vc.view(-1, G * e)[slots] = dev(seqs[i][2][at[i]:at[i] + n], torch.bfloat16)
        q = dev(np.concatenate([seqs[i][0][at[i]:at[i] + n] for i, n in zip(live, ns)]), torch.bfloat16)
        gate = dev(np.concatenate([seqs[i][3][at[i]:at[i] + n] for i, n in zip(live, ns)]), torch.bfloat16)
        out = torch.zeros(q.shape[0], H * e + 8, dtype=torch.bfloat16, device=DEV)
        mops.differential_window_attention(out[:, :H * e], q, gate[:, :H * e], kc, vc, torch.from_numpy(bt[live]).to(DEV).contiguous(),
                                           i32(starts), i32(ns), i32([at[i] for i in live]),
                                           i32(np.concatenate([[j] * n for j, n in enumerate(ns)])), (min(ns), max(ns)), H, d ** -0.5,
                                           window, keep, lam, 1.0 - diff, eps)
        assert float(out[:, H * e:].abs().max()) == 0.0
        for j, (i, n) in enumerate(zip(live, ns)):
            got[i].append(out[starts[j]:starts[j] + n, :H * e].float().cpu().numpy())
            at[i] += n
    for i in range(2):
        assert at[i] == lens[i]
        np.testing.assert_allclose(np.concatenate(got[i]), want[i], rtol=3e-2, atol=3e-2)


def test_fused_decoded_rows_split_long_key_ranges(mops):
    """Decoded rows that see a thousand keys: their key range is cut over several workgroups and merged."""
    H, G, d, e, window, keep = 4, 2, 64, 128, 1000, 3
    lam, diff, eps = 0.3, 0.25, 1e-5
    rng = np.random.default_rng(11)
    T, block = 1300, 16
    q = U.bf16_round(rng.standard_normal((T, H * 2 * d)))
    k = U.bf16_round(rng.standard_normal((T, G * 2 * d)))
    v = U.bf16_round(rng.standard_normal((T, G * e)))
    pages = (T + block - 1) // block
    perm = np.random.default_rng(2).permutation(pages)
    pos = np.arange(T)
    slots = torch.tensor(perm[pos // block] * block + pos % block, dtype=torch.int64, device=DEV)
    kc = torch.zeros(pages, block, G * 2, d, dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros(pages, block, G, e, dtype=torch.bfloat16, device=DEV)
    kc.view(-1, G * 2 * d)[slots] = dev(k, torch.bfloat16)
    vc.view(-1, G * e)[slots] = dev(v, torch.bfloat16)
    rows = [1290, 1295, 1299]
    qq, kk, vv = q.reshape(T, H, 2, d), k.reshape(T, G, 2, d), v.reshape(T, G, e)
    for row in rows:
        out = torch.zeros(1, H * e, dtype=torch.bfloat16, device=DEV)
        mops.differential_window_attention(out, dev(q[row:row + 1], torch.bfloat16), None, kc, vc, i32(perm).view(1, -1), i32([0]), i32([1]),
                                           i32([row]), i32([0]), (1, 1), H, d ** -0.5, window, keep, lam, 1.0 - diff, eps, max_kv_len=row + 1)
        js = [j for j in range(row + 1) if O.visible(row, j, window, keep)]
        assert len(js) == window + keep
        want = np.zeros((H, e))
        for h in range(H):
            a = []
            for m in range(2):
                sc = kk[js, h // 2, m] @ qq[row, h, m] * d ** -0.5
                pr = np.exp(sc - sc.max())
                a.append((pr / pr.sum()) @ vv[js, h // 2])
            want[h] = O.rms_unit(a[0] - lam * a[1], eps) * (1.0 - diff)
        np.testing.assert_allclose(out.float().cpu().numpy().reshape(H, e), want, rtol=3e-2, atol=3e-2)


def test_decoded_rows_far_past_the_window(mops):
    H, G, M, d, e = 4, 2, 2, 32, 64
    rng = np.random.default_rng(9)
    T = 900
    q = U.bf16_round(rng.standard_normal((T, H * M * d)))
    k = U.bf16_round(rng.standard_normal((T, G * M * d)))
    v = U.bf16_round(rng.standard_normal((T, G * e)))
    got = attend(mops, q, k, v, [T - 3, 1, 1, 1], torch.bfloat16, H, G, M, d ** -0.5, 600, 2)
    qq, kk, vv = q.reshape(T, H, M, d), k.reshape(T, G, M, d), v.reshape(T, G, e)
    for row in (T - 3, T - 1):
        js = [j for j in range(row + 1) if O.visible(row, j, 600, 2)]
        for h in range(H):
            for m in range(M):
                s = kk[js, h // 2, m] @ qq[row, h, m] * d ** -0.5
                p = np.exp(s - s.max())
                np.testing.assert_allclose(got[row].reshape(H, M, e)[h, m], (p / p.sum()) @ vv[js, h // 2], rtol=2e-2, atol=2e-2)


# ---------------------------------------------------------------------------------------------------------------------
# experts
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("outputs,top", [(7, 2), (18, 4), (3, 3), (130, 1), (64, 8)])
def test_router_choice_uses_the_correction_and_the_weight_does_not(mops, outputs, top):
    rng = np.random.default_rng(outputs)
    T = 50
    z = rng.standard_normal((T, outputs)).astype(np.float32) * 2
    corr = (rng.standard_normal(outputs) * 0.3).astype(np.float32)
    ids, w = mops.experts_route(dev(z), dev(corr), top)
    # the restatement's router on an identity "hidden state": h = z, router = I
    want_ids, want_w = O.route(z.astype(np.float64), np.eye(outputs), corr.astype(np.float64), top)
    np.testing.assert_array_equal(ids.cpu().numpy(), want_ids)
    np.testing.assert_allclose(w.cpu().numpy(), want_w, rtol=1e-5, atol=1e-7)
    ids0, _ = mops.experts_route(dev(z), None, top)
    assert (ids0.cpu().numpy() != want_ids).any() or outputs == top


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(72, 88, 5, 1, 2, True, 45), (96, 64, 3, 0, 1, False, 45), (75, 40, 4, 2, 3, True, 45),
                                   (128, 32, 9, 1, 4, True, 45),
                                   # steps in which an expert has dozens / hundreds of rows: blocks of 64 and of 128 rows
                                   (128, 64, 3, 0, 2, False, 110), (128, 192, 3, 1, 2, True, 900), (192, 80, 2, 0, 2, False, 600)])
def test_experts_against_the_restatement_and_alone(mops, dtype, shape):
    width, ff, E, ident, top, shared, T = shape
    rng = np.random.default_rng(width + ff)
    cfg = U.make_config([U.attention_layer(mlp="moe", ff=ff, experts=E, identity=ident, top=top, shared_ff=56 if shared else 0)], width=width)
    W = {k[7:]: rounded(v, dtype) for k, v in U.make_weights(cfg, seed=1).items() if k.startswith("l0.mlp.")}
    h = rounded(rng.standard_normal((T, width)), dtype)
    want = O.moe_ff(h, W, "", cfg["layers"][0]["mlp"])
    from aphrodite_engine_amd.mixers import RoutedExperts
    m = RoutedExperts(width, ff, E, top, ident, 1.25, dtype, shared_ff=56 if shared else 0, shared_limit=2.0).to(DEV)
    m.router.copy_(dev(W["router"]))
    m.correction.copy_(dev(W["correction"]))
    for e in range(E):
        m.w_gate_up[e, :ff] = dev(W[f"e{e}.gate"], dtype)
        m.w_gate_up[e, ff:] = dev(W[f"e{e}.up"], dtype)
        m.w_down[e] = dev(W[f"e{e}.down"], dtype)
    if shared:
        m.shared_in.weight[:56] = dev(W["shared.gate"], dtype)
        m.shared_in.weight[56:112] = dev(W["shared.up"], dtype)
        m.shared_in.weight[112:113] = dev(W["shared.sg"], dtype)
        m.shared_down.weight.copy_(dev(W["shared.down"], dtype))
    with torch.no_grad():
        got = m(dev(h, dtype)).float().cpu().numpy()
        one = torch.cat([m(dev(h[t:t + 1], dtype)) for t in (0, 17, T - 1)]).float().cpu().numpy()
    tol = 1e-4 if dtype == torch.float32 else 6e-2
    np.testing.assert_allclose(got, want, rtol=tol, atol=tol)
    # a token's output does not depend on what else is in the batch
    np.testing.assert_allclose(one, got[[0, 17, T - 1]], rtol=1e-6 if dtype == torch.float32 else 1e-2, atol=1e-6 if dtype == torch.float32 else 1e-2)


# ---------------------------------------------------------------------------------------------------------------------
# the model through the engine
# ---------------------------------------------------------------------------------------------------------------------
A = U.attention_layer
CONFIGS = {
    # layers that differ in everything; a layer reads the keys and values of one two layers back; one layer has no feed-forward
    "mixed": lambda: U.make_config([A(), A(kv_from=0, window=11, keep_first=0, taps=2, diff=0.35, mlp="moe"),
                                    A(heads=3, kv_heads=3, dim=16, vdim=24, window=40, keep_first=1, taps=5, mlp=None),
                                    A(kv_from=0, window=64, keep_first=7, taps=1, diff=0.1, mlp="moe", identity=0, top=1, shared_ff=0)]),
    # sizes of the matrix-core kernels; one layer only
    "wide": lambda: U.make_config([A(heads=4, kv_heads=1, dim=32, vdim=96, window=48, keep_first=2, taps=4, mlp="moe", ff=64, experts=8,
                                     identity=2, top=3, shared_ff=64)], width=128, vocab=211, logit_scale=1.0),
    "pair": lambda: U.make_config([A(heads=8, kv_heads=2, dim=64, vdim=32, window=19, keep_first=4, mlp="dense", ff=96),
                                   A(heads=8, kv_heads=2, dim=64, vdim=32, window=100, keep_first=0, kv_from=0, mlp=None)], width=96),
}


def build(tmp_path, name, dtype, seed=0, **engine_args):
    from aphrodite_engine_amd.engine import LLMEngine
    cfg = CONFIGS[name]()
    W = U.make_weights(cfg, seed=seed)
    path = U.write_checkpoint(str(tmp_path / f"{name}-{seed}"), cfg, W)
    args = dict(max_tokens=512, max_num_seqs=4)
    args.update(engine_args)
    eng = LLMEngine.from_pretrained(path, dtype=dtype, device=DEV, **args)
    for c in eng.runner.caches:                   # poison: nothing may be read before it is written
        for t in (c if isinstance(c, (tuple, list)) else [c]):
            t.fill_(float("nan"))
    return cfg, W, eng


def prompts(cfg, lens, seed=0):
    rng = np.random.default_rng(seed)
    return [rng.integers(0, cfg["vocab"], n).tolist() for n in lens]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_prompt_and_layer_trace(mops, tmp_path, name, dtype):
    cfg, W, eng = build(tmp_path, name, dtype)
    toks = prompts(cfg, [83])[0]
    trace = []
    want = O.forward(cfg, W, toks, trace)
    model = eng.runner.model
    model.residual_trace = []
    got = eng.run_segments([("a", toks, list(range(len(toks))))]).cpu().numpy()
    U.assert_logits(got, want, dtype == torch.float32)
    assert len(model.residual_trace) == len(trace)
    for x, w in zip(model.residual_trace, trace):
        x = x.cpu().numpy()
        assert np.isfinite(x).all()
        if dtype == torch.float32:
            assert np.abs(x - w).max() < 2e-4 * max(1.0, np.abs(w).max() / 10)
    model.residual_trace = None
    eng.release("a")
    again = eng.run_segments([("b", toks, list(range(len(toks))))]).cpu().numpy()      # reused pages and slot
    U.assert_logits(again, want, dtype == torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["mixed", "wide"])
def test_portions_and_token_by_token_equal_the_whole_prompt(mops, tmp_path, name, dtype):
    cfg, W, eng = build(tmp_path, name, dtype)
    toks = prompts(cfg, [70], seed=1)[0]
    want = O.forward(cfg, W, toks)
    whole = eng.run_segments([("whole", toks, list(range(70)))]).cpu().numpy()
    eng.release("whole")
    for rid, sizes in (("tok", [1] * 70), ("two", [2] * 35), ("mix", [2, 15, 1, 16, 2, 17, 3, 1, 1, 12]), ("tail", [38] + [1] * 32)):
        got, a = [], 0
        for n in sizes:
            got.append(eng.run_segments([(rid, toks[a:a + n], list(range(n)))]).cpu().numpy())
            a += n
        eng.release(rid)
        assert a == 70
        U.assert_logits(np.concatenate(got), want, dtype == torch.float32, rid)
        # how a prompt is cut changes nothing beyond rounding -- in bfloat16 too
        assert np.quantile(U.logit_errors(np.concatenate(got), whole), 0.9) < (2e-4 if dtype == torch.float32 else 0.03), rid


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_unequal_requests_in_one_batch_equal_each_alone(mops, tmp_path, dtype):
    cfg, W, eng = build(tmp_path, "mixed", dtype, max_tokens=320)
    ps = prompts(cfg, [90, 1, 23, 47], seed=2)
    want = [O.forward(cfg, W, p) for p in ps]
    # a schedule with portions beside single tokens; request 1 ends early and request 3 takes its pages and slot
    plan = [[(0, 2), (1, 1)], [(0, 30), (2, 3)], [(0, 1), (2, 1), (3, 2)], [(0, 1), (2, 17), (3, 16)], [(2, 2), (3, 1), (0, 20)],
            [(3, 28), (0, 1)], [(0, 35)]]
    at, got = [0] * 4, [[] for _ in ps]
    for step in plan:
        entries = [(str(i), ps[i][at[i]:at[i] + n], list(range(n))) for i, n in step]
        out = eng.run_segments(entries).cpu().numpy()
        a = 0
        for i, n in step:
            got[i].append(out[a:a + n])
            a += n
            at[i] += n
            if at[i] == len(ps[i]):
                eng.release(str(i))
    for i in range(4):
        assert at[i] == len(ps[i])
        U.assert_logits(np.concatenate(got[i]), want[i], dtype == torch.float32, i)
    assert eng.pages.num_free == eng.pages.total and eng.slots.num_free == 4


def test_pages_and_slots_taken_over_from_a_finished_request(mops, tmp_path):
    cfg, W, eng = build(tmp_path, "pair", torch.float32, max_tokens=64, max_num_seqs=1)
    a, b = prompts(cfg, [60, 50], seed=3)
    eng.run_segments([("a", a, [])])
    with pytest.raises(Exception):
        eng.run_segments([("b", b, [])])             # neither pages nor a slot are left
    eng.requests.pop("b", None)
    eng.release("a")
    # the new request starts with single tokens in the slot the old one left: the convolution must not see its inputs
    got = [eng.run_segments([("b", b[:1], [0])]), eng.run_segments([("b", b[1:3], [0, 1])]), eng.run_segments([("b", b[3:31], list(range(28)))]),
           eng.run_segments([("b", b[31:], list(range(19)))])]
    U.assert_logits(torch.cat(got).cpu().numpy(), O.forward(cfg, W, b), True)


def test_long_decoding_passes_every_window(mops, tmp_path):
    cfg, W, eng = build(tmp_path, "mixed", torch.float32)
    toks = prompts(cfg, [180], seed=4)[0]
    want = O.forward(cfg, W, toks)
    got = [eng.run_segments([("a", toks[:5], [4])])]
    for t in toks[5:]:
        got.append(eng.run_segments([("a", [t], [0])]))
    U.assert_logits(torch.cat(got).cpu().numpy(), want[4:], True)


def test_greedy_generation_through_the_scheduler(mops, tmp_path):
    from aphrodite_engine_amd.engine import SamplingParams
    cfg, W, eng = build(tmp_path, "mixed", torch.float32, max_num_seqs=2, max_num_batched_tokens=24, max_tokens=192)
    ps = prompts(cfg, [40, 3, 1, 29], seed=5)
    outs = eng.generate(ps, SamplingParams(max_tokens=8))
    for p, out in zip(ps, outs):
        seq = list(p)
        for _ in range(8):
            seq.append(int(np.argmax(O.forward(cfg, W, seq)[-1])))
        assert out == seq[len(p):]
    assert eng.pages.num_free == eng.pages.total and eng.slots.num_free == 2 and not eng.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_command_on_an_unseen_shape(mops, tmp_path, dtype):
    """bin/trace_run end to end: a checkpoint of sizes no other test uses, a schedule with portions beside single tokens and a
    request that ends, the logits files against the restatement."""
    import json
    import os
    import subprocess
    cfg = U.make_config([A(heads=2, kv_heads=1, dim=48, vdim=80, window=9, keep_first=2, taps=6, mlp="moe", ff=48, experts=3, identity=3,
                           top=2, shared_ff=24),
                         A(heads=5, kv_heads=5, dim=8, vdim=16, window=30, keep_first=0, taps=2, mlp="dense", ff=100),
                         A(heads=2, kv_heads=1, dim=48, vdim=80, window=70, keep_first=1, taps=3, kv_from=0, mlp=None)],
                        vocab=300, width=104, logit_scale=1.3)
    W = U.make_weights(cfg, seed=21)
    model_dir = U.write_checkpoint(str(tmp_path / "m"), cfg, W)
    ps = prompts(cfg, [75, 20, 2], seed=9)
    want = [O.forward(cfg, W, p) for p in ps]
    plan = [[(0, 40), (1, 2)], [(0, 1), (1, 1), (2, 2)], [(0, 20), (1, 17)], [(0, 14)]]
    at, lines, rows = [0, 0, 0], [], []
    for n, step in enumerate(plan):
        entries, end = [], []
        for i, k in step:
            w = list(range(0, k, 2)) if k > 2 else list(range(k))
            entries.append({"id": "q%d" % i, "tokens": ps[i][at[i]:at[i] + k], "want": w})
            rows.append([(i, at[i] + x) for x in w])
            at[i] += k
            if at[i] == len(ps[i]):
                end.append("q%d" % i)
        lines.append(json.dumps({"step": n, "entries": entries, "end": end}))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", model_dir, "--dtype", dtype, "--out", str(out),
                        "--max-tokens", "128"], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == ["done %d" % n for n in range(len(plan))]
    got, exp, k = [], [], 0
    for n, step in enumerate(plan):
        g = np.fromfile(str(out / ("%d.f32" % n)), dtype="<f4").reshape(-1, cfg["vocab"])
        need = sum(len(rows[k + j]) for j in range(len(step)))
        assert g.shape[0] == need
        got.append(g)
        for j in range(len(step)):
            exp += [want[i][pos] for i, pos in rows[k + j]]
        k += len(step)
    U.assert_logits(np.concatenate(got), np.stack(exp), dtype == "float32")
