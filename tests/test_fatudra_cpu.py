"""CPU-side parts of the Fatudra integration: config and layer schedule, registry dispatch, checkpoint loading into the
fused projections, the distance-bias table, the page / slot bookkeeping and the scheduler's batches, and the plain
restatement (oracle/fatudra.py) against itself where two formulations must agree."""
import json

import numpy as np
import pytest
import torch

import fatudra_util as U
from oracle import fatudra as O


def test_schedule_loops_a_range_and_counts_runs():
    from aphrodite_engine_amd.fatudra import FatudraConfig
    layers = [U.parallel_layer(), U.mlstm_layer(), U.parallel_layer(), U.mlstm_layer(mlp=False)]
    c = FatudraConfig.from_dict(U.make_config(layers, loop=(0, 2, 3)))
    assert c.schedule() == [(0, 0), (1, 0), (0, 1), (1, 1), (0, 2), (1, 2), (2, None), (3, None)]
    assert c.schedule() == O.layer_schedule(U.make_config(layers, loop=(0, 2, 3)))
    c = FatudraConfig.from_dict(U.make_config(layers))
    assert c.schedule() == [(i, None) for i in range(4)] and not c.looped
    c = FatudraConfig.from_dict(U.make_config(layers, loop=(2, 4, 1)))
    assert c.schedule() == [(0, None), (1, None), (2, 0), (3, 0)]
    with pytest.raises(ValueError):
        FatudraConfig.from_dict(U.make_config(layers, loop=(3, 5, 2)))
    bad = U.make_config(layers)
    bad["layers"][1]["type"] = "conv"
    with pytest.raises(ValueError):
        FatudraConfig.from_dict(bad)


def test_registry_chooses_the_class_by_config():
    from aphrodite_engine_amd import registry
    assert "Fatudra" in registry.supported_architectures() and "LlamaForCausalLM" in registry.supported_architectures()
    assert registry.architecture_of({"architectures": ["MistralForCausalLM"]}) == "MistralForCausalLM"
    assert registry.architecture_of({"architecture": "Fatudra"}) == "Fatudra"
    with pytest.raises(ValueError, match="not supported"):
        registry.resolve({"architecture": "Nonesuch"})


def test_checkpoint_fills_the_fused_projections(tmp_path):
    from aphrodite_engine_amd.loader import load_model
    cfg = U.make_config([U.parallel_layer(), U.mlstm_layer(mlp=False)], loop=(0, 1, 2))
    W = U.make_weights(cfg, seed=3)
    U.write_checkpoint(str(tmp_path), cfg, W)
    m = load_model(str(tmp_path), dtype=torch.float32, device="cpu")
    assert type(m).__name__ == "FatudraForCausalLM"
    mix = m.layers[0].mix
    a = 0
    for name, n in zip(mix.names, mix.splits):
        np.testing.assert_array_equal(mix.in_proj.weight[a:a + n].numpy(), W["l0.mix." + name])
        b = W.get("l0.mix." + name + ".b")
        np.testing.assert_array_equal(mix.in_proj.bias[a:a + n].numpy(), b if b is not None else np.zeros(n, np.float32))
        a += n
    np.testing.assert_array_equal(mix.out_proj.weight[:, :mix.left_out].numpy(), W["l0.mix.left.o"])
    np.testing.assert_array_equal(mix.out_proj.weight[:, mix.left_out:].numpy(), W["l0.mix.right.o"])
    np.testing.assert_allclose(mix.out_bias.numpy(), W["l0.mix.left.o.b"] * 1.3, rtol=1e-6)
    assert m.layers[1].mlp is None and len(m.specs) == 2 * 2 + 1 and m.run_caches == [[0, 1], [2, 3], [4]]
    # a tensor too many, one missing, one of the wrong shape
    W2 = dict(W)
    W2["l0.mix.left.extra"] = np.zeros(3, np.float32)
    U.write_checkpoint(str(tmp_path / "x"), cfg, W2)
    with pytest.raises(ValueError, match="unexpected"):
        load_model(str(tmp_path / "x"), dtype=torch.float32, device="cpu")
    W3 = {k: v for k, v in W.items() if k != "l1.mix.f.b"}
    U.write_checkpoint(str(tmp_path / "y"), cfg, W3)
    with pytest.raises(ValueError, match="lacks"):
        load_model(str(tmp_path / "y"), dtype=torch.float32, device="cpu")
    W4 = dict(W)
    W4["l0.mix.left.o"] = W["l0.mix.left.o"][:, :-1]
    U.write_checkpoint(str(tmp_path / "z"), cfg, W4)
    with pytest.raises(ValueError, match="does not fit"):
        load_model(str(tmp_path / "z"), dtype=torch.float32, device="cpu")


@pytest.mark.parametrize("rows,far", [(12, 50), (16, 240), (7, 9.5), (32, 256), (2, 5), (1, 3)])
def test_distance_table_matches_the_bucket_rule(rows, far):
    from aphrodite_engine_amd.mixers import DistanceBiasAttention, log_distance_bucket
    att = DistanceBiasAttention(2, 1, 8, 8, 1.0, bias_rows=rows, bias_far=far)
    att.rel.copy_(torch.arange(rows * 2, dtype=torch.float32).reshape(rows, 2))
    att.finalize()
    lut = att.bias_lut.numpy()
    for n in range(0, int(far) * 3 + 5):
        want = O.distance_bucket(n, rows, far) if rows > 1 else 0
        assert log_distance_bucket(n, rows, far) == want
        assert lut[1, min(n, lut.shape[1] - 1)] == want * 2 + 1
    half = rows // 2
    if rows > 2:      # exact rows below the half, the last row from `far` on, never decreasing
        assert [O.distance_bucket(n, rows, far) for n in range(half)] == list(range(half))
        assert O.distance_bucket(int(np.ceil(far)), rows, far) == rows - 1
        b = [O.distance_bucket(n, rows, far) for n in range(int(far) + 3)]
        assert all(y >= x for x, y in zip(b, b[1:]))


def test_pages_and_slots_are_reused_last_in_first_out():
    from aphrodite_engine_amd.engine import FreeList, NoFreePages
    f = FreeList(4, "pages")
    a = f.take(3)
    assert a == [0, 1, 2] and f.num_free == 1
    f.give([1])
    assert f.take(1) == [1]
    with pytest.raises(NoFreePages):
        f.take(2)
    with pytest.raises(ValueError):
        f.give([3])
    f.give(a)
    with pytest.raises(ValueError):
        f.give([0])


def test_step_batch_indices():
    from aphrodite_engine_amd.step_batch import StepBatch
    b = StepBatch.build([[5, 6, 7], [9], [1, 2]], [14, 0, 31], [[3, 0], [2], [7, 5, 1]], [1, 0, 3], 16, "cpu")
    assert b.positions.tolist() == [14, 15, 16, 0, 31, 32]
    assert b.slot_mapping.tolist() == [3 * 16 + 14, 3 * 16 + 15, 0, 2 * 16, 5 * 16 + 15, 1 * 16]
    assert b.seq_of_token.tolist() == [0, 0, 0, 1, 2, 2] and b.q_start.tolist() == [0, 3, 4]
    assert b.last_rows() == [2, 3, 5]
    with pytest.raises(ValueError, match="pages"):
        StepBatch.build([[1] * 5], [30], [[0, 1]], [0], 16, "cpu")
    with pytest.raises(ValueError, match="slot"):
        StepBatch.build([[1], [2]], [0, 0], [[0], [1]], [2, 2], 16, "cpu")
    # portions first, decoded tokens last is what the attention metadata assumes
    assert StepBatch.build([[1, 2], [3]], [0, 4], [[0], [1]], [0, 1], 16, "cpu").decode_split() == 1
    with pytest.raises(ValueError):
        StepBatch.build([[3], [1, 2]], [4, 0], [[1], [0]], [1, 0], 16, "cpu").decode_split()


def test_scheduler_batches_portions_and_decodes():
    from aphrodite_engine_amd.engine import Request, Scheduler
    s = Scheduler(max_num_seqs=2, max_num_batched_tokens=8)
    rs = [Request(str(i), list(range(n)), n) for i, n in enumerate((11, 3, 4))]
    for r in rs:
        s.add(r)
    free = {"slots": 2}

    def admit():
        return free["slots"] > 0

    def pages(r, n):
        if r.slot < 0:
            r.slot = 2 - free["slots"]
            free["slots"] -= 1
        return True
    p = s.plan(admit, pages)
    assert [(r.request_id, n) for r, n in p] == [("0", 8)]
    rs[0].num_computed = 8
    p = s.plan(admit, pages)                       # the rest of the first prompt, then the second one
    assert [(r.request_id, n) for r, n in p] == [("0", 3), ("1", 3)]
    rs[0].num_computed, rs[1].num_computed = 11, 3
    rs[0].tokens.append(1)
    rs[1].tokens.append(1)
    p = s.plan(admit, pages)                       # both decode; the third waits for a slot
    assert [(r.request_id, n) for r, n in p] == [("0", 1), ("1", 1)]
    s.retire(rs[1])
    free["slots"] += 1
    rs[0].num_computed = 12
    rs[0].tokens.append(2)
    p = s.plan(admit, pages)
    assert [(r.request_id, n) for r, n in p] == [("2", 4), ("0", 1)]     # portions first, decoded tokens last


def test_restatement_recurrences_agree_with_their_closed_forms():
    rng = np.random.default_rng(0)
    T, H, d, e = 9, 2, 5, 3
    q, k, v = rng.standard_normal((T, H, d)), rng.standard_normal((T, H, d)), rng.standard_normal((T, H, e))
    dec = np.array([0.7, 0.95])
    o = O.decay_linear_attention(q, k, v, dec)
    for t in range(T):
        for h in range(H):
            want = sum(dec[h] ** (t - j) * (q[t, h] @ k[j, h]) * v[j, h] for j in range(t + 1))
            np.testing.assert_allclose(o[t, h], want, rtol=1e-10, atol=1e-12)
    # the stabilised mLSTM equals the unstabilised one where nothing overflows (the guard then is exp(-m) > 0 only)
    ig, fg = rng.standard_normal((T, H)), O.log_sigmoid(rng.standard_normal((T, H)) + 2)
    o = O.mlstm_memory(q, k, v, ig, fg)
    for h in range(H):
        S, n, m = np.zeros((d, e)), np.zeros(d), 0.0
        for t in range(T):
            S = np.exp(fg[t, h]) * S + np.exp(ig[t, h]) * np.outer(k[t, h], v[t, h])
            n = np.exp(fg[t, h]) * n + np.exp(ig[t, h]) * k[t, h]
            m = max(fg[t, h] + m, ig[t, h])
            want = S.T @ q[t, h] / (max(abs(n @ q[t, h]), 1.0) + 1e-6 * np.exp(m))
            np.testing.assert_allclose(o[t, h], want, rtol=1e-9, atol=1e-12)
