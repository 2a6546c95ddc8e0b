"""CPU checks of the Sanazen design: configuration and tensor table of zig_gpt2_amd/lm.py, the registry, and the float64 oracle's
own consistency (portions against whole prompts, the mask, the recurrence, the router and the experts on hand-made inputs)."""
import json

import numpy as np

import sanazen_oracle as so
import sanazen_testlib as sl
from zig_gpt2_amd import lm, models


def small_cfg():
    return sl.config([sl.pair_layer(mlp=sl.moe_mlp()), sl.pair_layer(heads=2, kv_heads=1, dim=6, vdim=10, window=5, keep_first=7, conv=2, mlp=None),
                      sl.pair_layer(window=0, conv=0, mlp=sl.moe_mlp(top=1, shared=None))])


def test_configuration_round_trip_and_tensor_table():
    cfg = small_cfg()
    c = lm.LMConfig.from_json(cfg)
    assert c.architecture == "Sanazen" and [l.mixer for l in c.layers] == ["window_linear"] * 3
    assert lm.LMConfig.from_json(json.loads(json.dumps(c.to_json()))) == c
    assert c.layers[1].keep_first == 7 and c.layers[1].window == 5 and c.layers[2].window == 0 and c.layers[2].conv == 0
    assert c.layers[0].shared_width == 20 and c.layers[2].shared_width == 0 and c.layers[1].ff == "none"
    t = c.tensor_shapes()
    assert t["l0.mix.left.q"] == (48, 48) and t["l0.mix.left.k.conv"] == (24, 3) and t["l1.mix.left.k.norm"] == (6,)
    assert t["l0.mlp.shared.sg"] == (1, 48) and "l2.mlp.shared.sg" not in t and "l1.norm2" not in t and "l2.mix.left.q.conv" not in t
    assert "l0.norm1b" not in t and "l0.mlp.correction" not in t and "head" in t
    assert set(c.derived_tensors()) == {f"l{i}.mix.right.decay" for i in range(3)}
    assert c.flags() & lm._lib.LM_SIDE_BY_SIDE and c.flags() & lm._lib.LM_SINUSOID_POSITIONS
    assert "Sanazen" in models.ARCHITECTURES


def test_taps_come_from_the_checkpoint_when_the_configuration_is_silent():
    cfg = small_cfg()
    del cfg["layers"][0]["mixer"]["left"]["conv"]
    c = lm.LMConfig.from_json(cfg, {"l0.mix.left.q.conv": (48, 4)})
    assert c.layers[0].conv == 4
    assert lm.LMConfig.from_json(cfg).layers[0].conv == 0


def test_oracle_portions_equal_whole_prompts():
    cfg = small_cfg()
    w = sl.weights(cfg, seed=1)
    toks = sl.tokens(1, 40, cfg["vocab"])
    ref, _, tr = so.forward(w, cfg, toks, trace=True)
    assert tr.shape == (3, 40, 48)
    for cuts in ([1, 2, 3, 17, 19], [10, 30], list(range(1, 40))):
        st, rows, lo = None, [], 0
        for hi in cuts + [40]:
            out, st = so.forward(w, cfg, toks[lo:hi], st)
            rows.append(out)
            lo = hi
        assert np.abs(np.concatenate(rows) - ref).max() < 1e-9
    assert so.greedy(w, cfg, toks[:5], 4) == so.greedy(w, cfg, toks[:5], 6)[:4]


def test_mask_and_weights_on_hand_made_scores():
    ok = so.visible([0, 5, 9], np.arange(10), 3, 2)
    assert ok[0].tolist() == [True] + [False] * 9
    assert ok[1].tolist() == [True, True, False, True, True, True, False, False, False, False]
    assert ok[2].tolist() == [True, True, False, False, False, False, False, True, True, True]
    assert so.visible([4], np.arange(6), 0, 0)[0].tolist() == [True] * 5 + [False]
    q = np.zeros((1, 2, 3))
    k = np.zeros((4, 1, 3))
    a = so.softmax_weights(q, k, 1.0, np.array([[True, False, True, True]]), 2, 1)
    assert np.allclose(a[:, 0], [[1 / 3, 0, 1 / 3, 1 / 3]] * 2)


def test_position_vectors_conv_recurrence_router_and_experts():
    pe = so.position_vectors([0, 3], 6)
    assert np.allclose(pe[0], [0, 1, 0, 1, 0, 1])
    assert np.allclose(pe[1, :2], [np.sin(3.0), np.cos(3.0)]) and np.allclose(pe[1, 2], np.sin(3.0 * 10000.0 ** (-2 / 6)), atol=1e-6)
    y, tail = so.causal_conv(np.arange(8.0).reshape(4, 2), np.array([[1.0, 10.0, 100.0]] * 2), None)
    assert y[:, 0].tolist() == [0.0, 200.0, 420.0, 642.0] and tail[:, 0].tolist() == [4.0, 6.0]
    q = np.ones((3, 1, 2))
    k = np.ones((3, 1, 2))
    v = np.array([1.0, 2.0, 4.0]).reshape(3, 1, 1)
    o, S = so.decayed_linear_attention(q, k, v, np.array([0.5]), None)
    assert np.allclose(o[:, 0, 0], [2.0, 5.0, 10.5]) and np.allclose(S[0, :, 0], [5.25, 5.25])
    w = {"r.router": np.array([[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]])}
    pick, score = so.sigmoid_router(np.array([[2.0, -1.0]]), w, "r.", 2)
    assert pick.tolist() == [[0, 2]] and np.allclose(score, [[so.sigmoid(2.0), so.sigmoid(1.0)]])
    e = {"e.gate": np.array([[1.0]]), "e.up": np.array([[1.0]]), "e.down": np.array([[2.0]])}
    # gate capped at 1.5, linear part clipped to [-1.5, 1.5] and lifted by one
    assert np.allclose(so.clipped_expert(np.array([[5.0]]), e, "e.", 1.5), 2.0 * 1.5 * so.sigmoid(1.702 * 1.5) * 2.5)
    assert np.allclose(so.clipped_expert(np.array([[-5.0]]), e, "e.", 1.5), 2.0 * -5.0 * so.sigmoid(1.702 * -5.0) * -0.5)
