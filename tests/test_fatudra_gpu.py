"""Fatudra on the GPU against the plain restatement (oracle/fatudra.py, float64): every mixer kernel alone, then the model
through the engine -- whole prompts, token-by-token decoding, portions down to two tokens, unequal batches, reused pages
and slots, long decoding, greedy generation through the scheduler.  Small random configurations made here; sizes are
unlike one another and unlike any shipped model.  Unused cache memory is poisoned with NaN so that a read outside a
sequence's own keys or of a stale state shows."""
import math

import numpy as np
import pytest
import torch

import fatudra_util as U
from oracle import fatudra as O

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


# ---------------------------------------------------------------------------------------------------------------------
# kernels alone
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [72, 75, 200, 1032])      # 75: rows that cannot be read 16 bytes at a time
def test_residual_layer_norm_all_steps(mops, dtype, width):
    rng = np.random.default_rng(width)
    T, eps = 5, 1e-5
    r0 = rng.standard_normal((T, width)) * 3
    y = rounded(rng.standard_normal((T, width + 8)) * 2 + 0.5, dtype)
    yb = rng.standard_normal(width).astype(np.float32).astype(np.float64)
    vecs = [rounded(rng.standard_normal(width) * 0.3 + m, dtype) for m in (1, 0, 0, 1, 0)]
    pw, pb, add, qw, qb = vecs
    res = dev(r0)
    out = mops.residual_layer_norm(res, y=dev(y, dtype)[:, :width], post=(dev(pw, dtype), dev(pb, dtype)), y_bias=dev(yb),
                                   add_vec=dev(add, dtype), pre=(dev(qw, dtype), dev(qb, dtype)), eps=eps)
    want_r = r0.astype(np.float32).astype(np.float64) + O.layer_norm(y[:, :width] + yb, pw, pb, eps) + add
    np.testing.assert_allclose(res.cpu().numpy(), want_r, rtol=2e-6, atol=2e-5)
    want = O.layer_norm(want_r, qw, qb, eps)
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=tol, atol=tol)
    # the pre-norm alone leaves the residual untouched
    res2 = dev(r0)
    out2 = mops.residual_layer_norm(res2, pre=(dev(qw, dtype), dev(qb, dtype)), eps=eps)
    np.testing.assert_array_equal(res2.cpu().numpy(), r0.astype(np.float32))
    np.testing.assert_allclose(out2.float().cpu().numpy(), O.layer_norm(r0.astype(np.float32).astype(np.float64), qw, qb, eps),
                               rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_activations_and_group_norm(mops, dtype):
    rng = np.random.default_rng(1)
    T, d = 7, 45
    x = rounded(rng.standard_normal((T, 2 * d)) * 2, dtype)
    tol = 1e-5 if dtype == torch.float32 else 1.5e-2
    for act, fn in ((mops.ACT_GELU_TANH, O.gelu_tanh), (mops.ACT_SILU, O.silu)):
        got = mops.act_and_mul(dev(x, dtype), act).float().cpu().numpy()
        np.testing.assert_allclose(got, fn(x[:, :d]) * x[:, d:], rtol=tol, atol=tol)
    N = 3 * 28
    o = rng.standard_normal((T, N)).astype(np.float32).astype(np.float64) * 5
    w, g = rounded(rng.standard_normal(N) * 0.2 + 1, dtype), rounded(rng.standard_normal((T, N + 4)), dtype)
    for group in (N, 28):
        out = torch.zeros(T, N + 10, dtype=dtype, device=DEV)
        mops.gated_group_rms_norm(out[:, 6:6 + N], dev(o), dev(w, dtype), dev(g, dtype)[:, 4:], group, 1e-5, out_scale=0.7)
        want = 0.7 * O.rms_unit(o.reshape(T, N // group, group), 1e-5).reshape(T, N) * w * O.sigmoid(g[:, 4:])
        np.testing.assert_allclose(out[:, 6:6 + N].float().cpu().numpy(), want, rtol=tol, atol=tol)
        assert float(out[:, :6].abs().sum()) == 0 and float(out[:, 6 + N:].abs().sum()) == 0
    out = torch.zeros(T, N, dtype=dtype, device=DEV)
    mops.gated_group_rms_norm(out, dev(o), None, None, 28, 1e-5)
    np.testing.assert_allclose(out.float().cpu().numpy(), O.rms_unit(o.reshape(T, 3, 28), 1e-5).reshape(T, N), rtol=tol, atol=tol)


class Paged:
    """Keys and values of several sequences in a shuffled, NaN-poisoned page pool."""

    def __init__(self, mops, ks, vs, dtype, block=16, seed=0, spare=7):
        rng = np.random.default_rng(seed)
        G, d, e = ks[0].shape[1], ks[0].shape[2], vs[0].shape[2]
        need = [(k.shape[0] + block - 1) // block for k in ks]
        pool = sum(need) + spare
        perm = rng.permutation(pool)
        self.kc = torch.full((pool, block, G, d), float("nan"), dtype=dtype, device=DEV)
        self.vc = torch.full((pool, block, G, e), float("nan"), dtype=dtype, device=DEV)
        self.tables, a = [], 0
        for k, v, n in zip(ks, vs, need):
            pages = perm[a:a + n]
            a += n
            self.tables.append(pages)
            pos = np.arange(k.shape[0])
            slots = torch.from_numpy(pages[pos // block].astype(np.int64) * block + pos % block).to(DEV)
            mops.paged_kv_write(self.kc, self.vc, dev(k.reshape(k.shape[0], -1), dtype), dev(v.reshape(v.shape[0], -1), dtype), slots)
        width = max(need)
        bt = np.zeros((len(ks), width), np.int32)
        for s, p in enumerate(self.tables):
            bt[s, :len(p)] = p
        self.bt = torch.from_numpy(bt).to(DEV)


def run_attention(mops, pg, qs, ctx, H, scale, lut, coef, every, dtype, gate=None, out_scale=1.0, seqs=None):
    """qs: per segment its query rows (positions ctx[s] ..); seqs: which sequence of ``pg`` each segment continues."""
    bt = pg.bt if seqs is None else pg.bt[torch.tensor(seqs, device=DEV)].contiguous()
    lens = [q.shape[0] for q in qs]
    starts = np.concatenate([[0], np.cumsum(lens)[:-1]])
    seq_of = np.concatenate([np.full(n, s) for s, n in enumerate(lens)])
    q = dev(np.concatenate([x.reshape(x.shape[0], -1) for x in qs]), dtype)
    e = pg.vc.shape[3]
    out = torch.full((q.shape[0], H * e + 3), 7.0, dtype=dtype, device=DEV)
    mops.distance_bias_attention(out[:, :H * e], q, None if gate is None else dev(gate, dtype), pg.kc, pg.vc, bt,
                                 i32(starts), i32(lens), i32(ctx), i32(seq_of), (min(lens), max(lens)), H, scale, lut, coef, every,
                                 out_scale, max_kv_len=max(a + b for a, b in zip(ctx, lens)))
    assert float((out[:, H * e:] - 7.0).abs().sum()) == 0
    return out[:, :H * e].float().cpu().numpy().reshape(-1, H, e)


def make_lut(rel, far):
    from aphrodite_engine_amd.mixers import DistanceBiasAttention
    att = DistanceBiasAttention(rel.shape[1], 1, 8, 8, 1.0, bias_rows=rel.shape[0], bias_far=far)
    att.rel.copy_(torch.from_numpy(np.asarray(rel, np.float32)))
    att.to(DEV).finalize()
    return att.bias_lut


ATT_SHAPES = [  # H, G, d, e, rows, far, coef, every
    (4, 2, 24, 40, 12, 50, 0.5, 16),
    (3, 3, 20, 72, 9, 33.5, 2.0, 7),          # no grouping, odd table, sizes that force the scalar loads
    (8, 2, 64, 128, 16, 100, 0.0, 1),         # vector loads, two output columns per lane, no temperature
    (2, 1, 96, 200, 6, 20, 0.25, 5),
    (3, 3, 32, 64, 7, 45, 0.4, 11),           # one query head per kv head: the unpaired matrix-core form
    (6, 2, 64, 32, 8, 60, 0.3, 9),            # three query heads per kv head: no shared-key form, long segments only on the matrix cores
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", ATT_SHAPES)
def test_attention_prompt_portion_and_decode(mops, dtype, shape):
    H, G, d, e, rows, far, coef, every = shape
    rng = np.random.default_rng(H * 100 + d)
    lens = [150, 1, 37]
    scale = 0.9 * d ** -0.5
    q = [rounded(rng.standard_normal((n, H, d)), dtype) for n in lens]
    k = [rounded(rng.standard_normal((n, G, d)), dtype) for n in lens]
    v = [rounded(rng.standard_normal((n, G, e)), dtype) for n in lens]
    rel = rng.standard_normal((rows, H)).astype(np.float32) * 2
    gate = rounded(rng.standard_normal((sum(lens), H + 2)), dtype)
    want = [O.biased_softmax_attention(q[s], k[s], v[s], rel.astype(np.float64), scale, far, coef, every) for s in range(3)]
    pg, lut = Paged(mops, k, v, dtype), make_lut(rel, far)
    tol = 2e-5 if dtype == torch.float32 else 2.5e-2
    # whole prompts of unequal length in one batch, with the output gate and a scale
    got = run_attention(mops, pg, q, [0, 0, 0], H, scale, lut, coef, every, dtype, gate=gate[:, 1:H + 1], out_scale=1.7)
    w = np.concatenate(want) * O.sigmoid(gate[:, 1:H + 1])[:, :, None] * 1.7
    np.testing.assert_allclose(got, w, rtol=tol, atol=tol)
    # a portion in the middle (it starts inside a page), a decoded token, and a two-token portion
    got = run_attention(mops, pg, [q[2][36:37], q[0][37:99]], [36, 37], H, scale, lut, coef, every, dtype, seqs=[2, 0])
    np.testing.assert_allclose(got, np.concatenate([want[2][36:37], want[0][37:99]]), rtol=tol, atol=tol)
    got = run_attention(mops, pg, [q[0][148:150]], [148], H, scale, lut, coef, every, dtype, seqs=[0])
    np.testing.assert_allclose(got, want[0][148:150], rtol=tol, atol=tol)


def test_decoded_rows_over_long_contexts_split_their_keys(mops):
    """bfloat16 rows with a long context are split over several workgroups and merged; short and long contexts, a
    three-token portion and a prompt portion share the batch."""
    H, G, d, e = 8, 2, 64, 128
    rng = np.random.default_rng(11)
    lens = [1500, 700, 40, 900]
    dt = torch.bfloat16
    q = [rounded(rng.standard_normal((n, H, d)), dt) for n in lens]
    k = [rounded(rng.standard_normal((n, G, d)), dt) for n in lens]
    v = [rounded(rng.standard_normal((n, G, e)), dt) for n in lens]
    rel = rng.standard_normal((10, H)).astype(np.float32)
    want = [O.biased_softmax_attention(q[s], k[s], v[s], rel.astype(np.float64), d ** -0.5, 300, 0.3, 128) for s in range(4)]
    pg, lut = Paged(mops, k, v, dt), make_lut(rel, 300)
    got = run_attention(mops, pg, [q[3][880:900], q[0][1499:], q[1][697:], q[2][39:]], [880, 1499, 697, 39], H, d ** -0.5, lut, 0.3,
                        128, dt, seqs=[3, 0, 1, 2])
    w = np.concatenate([want[3][880:900], want[0][1499:], want[1][697:], want[2][39:]])
    np.testing.assert_allclose(got, w, rtol=2.5e-2, atol=2.5e-2)


@pytest.mark.parametrize("decoded", [False, True])
def test_attention_finds_one_far_key_among_hundreds(mops, decoded):
    """One early key is made to dominate a late query: the answer is that key's value, wherever its page lies."""
    H, G, d, e, T = 2, 1, 32, 48, 700
    rng = np.random.default_rng(7)
    q = rng.standard_normal((T, H, d)) * 0.1
    k = rng.standard_normal((T, G, d)) * 0.1
    v = rng.standard_normal((T, G, e))
    for far_key, query in ((3, T - 1), (15, T - 2), (16, T - 3), (T - 130, T - 4)):     # first page, a page's edges, mid
        # each query looks along its own key's direction only
        probe = rng.standard_normal(d)
        k[far_key, 0] = 9 * probe / np.linalg.norm(probe)
        q[query, :] = 9 * probe / np.linalg.norm(probe)
    pg = Paged(mops, [k], [v], torch.float32, seed=3)
    rel = np.zeros((4, H), np.float32)
    lut = make_lut(rel, 10)
    if decoded:
        got = np.concatenate([run_attention(mops, pg, [q[p:p + 1]], [p], H, 1.0, lut, 0.0, 1, torch.float32)
                              for p in (T - 4, T - 3, T - 2, T - 1)])
    else:
        got = run_attention(mops, pg, [q], [0], H, 1.0, lut, 0.0, 1, torch.float32)[T - 4:]
    want = O.biased_softmax_attention(q, k, v, rel.astype(np.float64), 1.0, 10, 0.0, 1)[T - 4:]
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=1e-4)
    for row, far_key in zip(got, (T - 130, 16, 15, 3)):
        np.testing.assert_allclose(row[0], v[far_key, 0], atol=1e-3)       # nearly all weight on that one key


@pytest.mark.parametrize("rows,far", [(12, 50), (16, 240), (5, 11)])
def test_attention_bias_rows_change_exactly_at_their_edges(mops, rows, far):
    """With q = 0 the weights are the bias alone; the table's rows are far apart, so a key in the wrong row shows.
    Values are one-hot in the distance row, so the output IS the share of each row.  Prompt rows and decoded rows."""
    H, G, d = 2, 1, 8
    T = int(far * 2.5)
    row_of = np.array([O.distance_bucket(n, rows, far) for n in range(T)])
    q, k = np.zeros((T, H, d)), np.ones((T, G, d))
    rel = (np.arange(rows)[:, None] * np.array([1.5, -1.0])[None, :]).astype(np.float32)
    lut = make_lut(rel, far)
    for pos in sorted({int(n) for n in np.flatnonzero(np.diff(row_of)) + 1} | {T - 1}):
        for delta in (-1, 0):                                  # the last distance of a row, the first of the next
            p = pos + delta
            v = np.zeros((p + 1, G, rows))
            v[np.arange(p + 1), 0, row_of[p - np.arange(p + 1)]] = 1.0
            pg = Paged(mops, [k[:p + 1]], [v], torch.float32, seed=p)
            want = O.biased_softmax_attention(q[:p + 1], k[:p + 1], v, rel.astype(np.float64), 1.0, far, 0.0, 1)
            got = run_attention(mops, pg, [q[p:p + 1]], [p], H, 1.0, lut, 0.0, 1, torch.float32)      # decoded
            np.testing.assert_allclose(got[0], want[p], rtol=1e-5, atol=1e-6)
            got = run_attention(mops, pg, [q[:p + 1]], [0], H, 1.0, lut, 0.0, 1, torch.float32)       # prompt
            np.testing.assert_allclose(got[p], want[p], rtol=1e-5, atol=1e-6)


def test_query_temperature_steps_at_multiples_of_its_period(mops):
    H, G, d, e, every, coef = 1, 1, 16, 8, 6, 3.0
    T = 40
    rng = np.random.default_rng(2)
    q, k, v = rng.standard_normal((T, H, d)), rng.standard_normal((T, G, d)), rng.standard_normal((T, G, e))
    pg = Paged(mops, [k], [v], torch.float32)
    want = O.biased_softmax_attention(q, k, v, np.zeros((2, 1)), 0.3, 4, coef, every)
    got = run_attention(mops, pg, [q], [0], H, 0.3, None, coef, every, torch.float32)
    np.testing.assert_allclose(got, want, rtol=2e-5, atol=2e-5)
    for p in (4, 5, 6, 11, 12, 35):          # position p uses floor((p + 1) / every): the step is at p = every - 1
        got = run_attention(mops, pg, [q[p:p + 1]], [p], H, 0.3, None, coef, every, torch.float32)
        np.testing.assert_allclose(got[0], want[p], rtol=2e-5, atol=2e-5)
    assert O.query_temperature(4, coef, every) == 1.0 and O.query_temperature(5, coef, every) > 1.0


MEM_SHAPES = [(3, 20, 72), (2, 32, 64), (1, 48, 36), (2, 96, 130), (1, 130, 40), (5, 8, 8)]


def scan_in_steps(mops, mode, q, k, v, cuts, dtype, decay=None, gi=None, gf=None, q_scale=1.0, cap=1.0, slots=5):
    """Every sequence cut into segments at ``cuts[s]``; step j runs the j-th segment of every sequence that still has one,
    in one launch.  Slots start poisoned."""
    H, d, e = q[0].shape[1], q[0].shape[2], v[0].shape[2]
    state = tuple(torch.full(s, float("nan"), device=DEV) for s in mops.memory_state_shapes(slots, H, d, e, mode))
    outs = [np.zeros((x.shape[0], H * e)) for x in q]
    bounds = [[0] + list(c) + [x.shape[0]] for c, x in zip(cuts, q)]
    slot_of = [4, 0, 2, 1, 3][:len(q)]
    for j in range(max(len(b) for b in bounds) - 1):
        live = [s for s in range(len(q)) if j + 1 < len(bounds[s])]
        seg = [(bounds[s][j], bounds[s][j + 1]) for s in live]
        lens = [b - a for a, b in seg]
        starts = np.concatenate([[0], np.cumsum(lens)[:-1]])

        def cat(xs, pad=0):
            a = np.concatenate([x[a:b].reshape(b - a, -1) for x, (a, b) in zip([xs[s] for s in live], seg)])
            t = torch.zeros(a.shape[0], a.shape[1] + pad, dtype=dtype, device=DEV)
            t[:, pad:] = dev(a, dtype)
            return t[:, pad:]
        kw = {}
        if mode == mops.MEMORY_MLSTM:
            gates = cat([np.concatenate([gi[s], gf[s]], 1) for s in range(len(q))], pad=3)
            kw = dict(gate_i=gates[:, :H], gate_f=gates[:, H:], q_scale=q_scale, gate_cap=cap)
        else:
            kw = dict(decay=torch.tensor(decay, dtype=torch.float32, device=DEV))
        o = mops.outer_memory_scan(cat(q, 5), cat(k), cat(v, 1), state, i32([slot_of[s] for s in live]), i32(starts), i32(lens),
                                   i32([a for a, _ in seg]), H, mode, max_q_len=max(lens), **kw).cpu().numpy()
        for s, (a, b), st in zip(live, seg, starts):
            outs[s][a:b] = o[st:st + b - a]
    return outs


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", MEM_SHAPES)
def test_decay_memory_in_steps(mops, dtype, shape):
    H, d, e = shape
    rng = np.random.default_rng(d * 7 + e)
    lens = [70, 1, 33]
    q = [rounded(rng.standard_normal((n, H, d)), dtype) for n in lens]
    k = [rounded(rng.standard_normal((n, H, d)), dtype) for n in lens]
    v = [rounded(rng.standard_normal((n, H, e)), dtype) for n in lens]
    decay = [0.999, 0.6, 0.9, 0.3, 0.97][:H]
    want = [O.decay_linear_attention(O.silu(q[s]), O.silu(k[s]), O.silu(v[s]), np.array(decay)).reshape(lens[s], -1)
            for s in range(3)]
    for cuts in ([[], [], []], [[16, 17, 19, 48, 64], [], [2, 4, 31]], [list(range(1, 70)), [], [32]], [[40], [], [32]], [[3, 69], [], []]):
        got = scan_in_steps(mops, mops.MEMORY_DECAY, q, k, v, cuts, dtype, decay=decay)
        for s in range(3):
            np.testing.assert_allclose(got[s], want[s], rtol=3e-5, atol=3e-5 * np.abs(want[s]).max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", MEM_SHAPES)
def test_mlstm_memory_in_steps(mops, dtype, shape):
    H, d, e = shape
    rng = np.random.default_rng(d * 11 + e)
    lens, cap = [70, 1, 33], 6.0
    q = [rounded(rng.standard_normal((n, H, d)), dtype) for n in lens]
    k = [rounded(rng.standard_normal((n, H, d)), dtype) for n in lens]
    v = [rounded(rng.standard_normal((n, H, e)), dtype) for n in lens]
    # raw gates wide enough to hit the cap on both sides; the first tokens get strongly negative input gates, where the
    # running maximum still holds its start value
    gi = [rounded(rng.standard_normal((n, H)) * 8 - (np.arange(n)[:, None] < 3) * 20, dtype) for n in lens]
    gf = [rounded(rng.standard_normal((n, H)) * 8 + 3, dtype) for n in lens]
    want = []
    for s in range(3):
        i_log = cap * np.tanh(gi[s] / cap)
        f_log = O.log_sigmoid(cap * np.tanh(gf[s] / cap))
        want.append(O.mlstm_memory(q[s] * d ** -0.5, k[s], v[s], i_log, f_log).reshape(lens[s], -1))
    for cuts in ([[], [], []], [[16, 17, 19, 48, 64], [], [2, 4, 31]], [list(range(1, 70)), [], [32]], [[40], [], [32]], [[3, 69], [], []]):
        got = scan_in_steps(mops, mops.MEMORY_MLSTM, q, k, v, cuts, dtype, gi=gi, gf=gf, q_scale=d ** -0.5, cap=cap)
        for s in range(3):
            np.testing.assert_allclose(got[s], want[s], rtol=1e-4, atol=1e-4 * np.abs(want[s]).max())


def test_decay_memory_remembers_a_token_from_long_ago(mops):
    """Decay 1 - 1e-3 over 900 tokens: the first token's value still comes back, scaled by decay^899."""
    H, d, e, T = 1, 16, 24, 900
    k = np.full((T, H, d), -20.0)                 # silu(-20) ~ 0: silent keys
    q = np.full((T, H, d), -20.0)
    v = np.zeros((T, H, e))
    k[0, 0, 3] = q[T - 1, 0, 3] = 5.0
    v[0, 0] = np.linspace(1, 2, e)
    got = scan_in_steps(mops, mops.MEMORY_DECAY, [q], [k], [v], [[500, 899]], torch.float32, decay=[0.999])[0]
    want = O.decay_linear_attention(O.silu(q), O.silu(k), O.silu(v), np.array([0.999])).reshape(T, -1)
    np.testing.assert_allclose(got[-1], want[-1], rtol=1e-4)
    assert want[-1].max() > 0.5


# ---------------------------------------------------------------------------------------------------------------------
# the model through the engine
# ---------------------------------------------------------------------------------------------------------------------
CONFIGS = {
    # looped from the first layer, a layer without feed-forward inside the loop, a plain layer after it
    "loop3": lambda: U.make_config([U.parallel_layer(), U.mlstm_layer(mlp=False), U.parallel_layer(heads=6, kv_heads=6, dim=16, vdim=8,
                                                                                                   rheads=1, rdim=40, rvdim=24)],
                                   loop=(0, 2, 3)),
    # no loop, mLSTM first, sizes that take the vector loads and two 64-column tiles of state
    "plain": lambda: U.make_config([U.mlstm_layer(heads=2, dim=32, vdim=96), U.parallel_layer(heads=8, kv_heads=2, dim=32, vdim=64,
                                                                                              rheads=2, rdim=64, rvdim=128, bias_max=40)],
                                   width=128, vocab=211),
    # one looped layer, run once; equal scales and a temperature period of 1
    "once": lambda: U.make_config([U.parallel_layer(every=1, left_scale=1.0, right_scale=1.0, mlp=False)], loop=(0, 1, 1), width=40),
}


def build(tmp_path, name, dtype, seed=0, bias_rows=12, **engine_args):
    from aphrodite_engine_amd.engine import LLMEngine
    cfg = CONFIGS[name]()
    W = U.make_weights(cfg, seed=seed, bias_rows=bias_rows)
    path = U.write_checkpoint(str(tmp_path / f"{name}-{seed}"), cfg, W)
    args = dict(max_tokens=512, max_num_seqs=4)
    args.update(engine_args)
    eng = LLMEngine.from_pretrained(path, dtype=dtype, device=DEV, **args)
    for c in eng.runner.caches:                   # poison: nothing may be read before it is written
        for t in c:
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
    again = eng.run_segments([("b", toks, list(range(len(toks))))]).cpu().numpy()      # fused norm path, reused pages
    U.assert_logits(again, want, dtype == torch.float32)
    if dtype == torch.bfloat16:                    # the same batch again: the same logits, whatever the pages
        assert U.logit_errors(again, got).max() < 0.02


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", ["loop3", "plain"])
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
    cfg, W, eng = build(tmp_path, "loop3", dtype, max_tokens=320)
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
    cfg, W, eng = build(tmp_path, "plain", torch.float32, max_tokens=64, max_num_seqs=1)
    a, b = prompts(cfg, [60, 50], seed=3)
    eng.run_segments([("a", a, [])])
    with pytest.raises(Exception):
        eng.run_segments([("b", b, [])])             # neither pages nor a slot are left
    eng.requests.pop("b", None)
    eng.release("a")
    got = [eng.run_segments([("b", b[:31], list(range(31)))]), eng.run_segments([("b", b[31:], list(range(19)))])]
    U.assert_logits(torch.cat(got).cpu().numpy(), O.forward(cfg, W, b), True)


def test_long_decoding_follows_the_restatement(mops, tmp_path):
    cfg, W, eng = build(tmp_path, "loop3", torch.float32)
    toks = prompts(cfg, [180], seed=4)[0]
    want = O.forward(cfg, W, toks)
    got = [eng.run_segments([("a", toks[:5], [4])])]
    for t in toks[5:]:
        got.append(eng.run_segments([("a", [t], [0])]))
    U.assert_logits(torch.cat(got).cpu().numpy(), want[4:], True)


def test_greedy_generation_through_the_scheduler(mops, tmp_path):
    from aphrodite_engine_amd.engine import SamplingParams
    cfg, W, eng = build(tmp_path, "loop3", torch.float32, max_num_seqs=2, max_num_batched_tokens=24, max_tokens=192)
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
    """bin/trace_run end to end: a checkpoint of sizes no other test uses (head sizes off the matrix-core list, one memory
    head, a loop in the middle run three times), a schedule with portions beside single tokens and a request that ends,
    the logits files against the restatement."""
    import json
    import os
    import subprocess
    import sys
    cfg = U.make_config([U.mlstm_layer(heads=1, dim=24, vdim=56), U.parallel_layer(heads=5, kv_heads=5, dim=48, vdim=80, rheads=1,
                                                                                   rdim=24, rvdim=40, bias_max=19, every=3),
                         U.parallel_layer(heads=4, kv_heads=1, dim=64, vdim=32, rheads=2, rdim=32, rvdim=16, mlp=False)],
                        vocab=300, width=96, loop=(1, 2, 3), embed_scale=3.0)
    W = U.make_weights(cfg, seed=21, bias_rows=9)
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
