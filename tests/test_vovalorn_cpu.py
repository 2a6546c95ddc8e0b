"""CPU checks of the Vovalorn design: configuration and tensor table of zig_gpt2_amd/lm.py, the registry, layers that run another
layer's tensors, and the float64 oracle's own consistency (portions against whole prompts, the router's groups, the attention's
score shaping and the decays on hand-made inputs)."""
import json

import numpy as np
import pytest

import vovalorn_oracle as vo
import vovalorn_testlib as vl
from zig_gpt2_amd import lm, models


def small_cfg():
    return vl.config([vl.gla_layer(mlp=vl.moe_mlp()), vl.attn_layer(mlp=None), vl.gla_layer(weights_of=0, mlp=vl.moe_mlp()),
                      vl.attn_layer(heads=2, kv_heads=2, dim=6, softcap=0.0, q_temp=None, mlp=vl.moe_mlp(experts=4, top=1, groups=None, shared=None)),
                      vl.attn_layer(weights_of=1)])


def test_configuration_round_trip_and_tensor_table():
    cfg = small_cfg()
    c = lm.LMConfig.from_json(cfg)
    assert c.architecture == "Vovalorn" and [l.mixer for l in c.layers] == ["gla", "attention", "gla", "attention", "attention"]
    assert lm.LMConfig.from_json(json.loads(json.dumps(c.to_json()))) == c
    assert c.residual_mult == 0.45 and c.layers[0].tau == 4.0 and c.layers[1].qtemp_every == 5 and c.layers[3].qtemp_every == 0
    assert c.layers[0].route_groups == 3 and c.layers[0].route_keep == 2 and c.layers[0].route_scale == 1.7 and c.layers[0].shared_width == 14
    assert c.layers[3].route_groups == 1 and c.layers[3].shared_width == 0 and c.layers[1].ff == "none"
    assert [l.weights_of for l in c.layers] == [None, None, 0, None, 1]
    t = c.tensor_shapes()
    assert t["l0.mix.q"] == (36, 40) and t["l0.mix.v"] == (30, 40) and t["l0.mix.a1"] == (6, 40) and t["l0.mix.a2"] == (36, 6) and t["l0.mix.norm"] == (10,)
    assert t["l1.mix.q"] == (48, 40) and t["l1.mix.k"] == (24, 40) and t["l1.mix.o"] == (40, 48) and "l1.mix.v" not in t
    assert t["l0.norm1b.alpha"] == () and t["l0.norm2.b"] == (40,) and t["embed.norm"] == (40,) and t["final.norm.alpha"] == ()
    assert "l1.norm2" not in t and "l0.shift" not in t and "l0.mlp.shared.sg" not in t and t["l0.mlp.shared.gate"] == (14, 40)
    assert t["l0.mlp.correction"] == (6,) and "l3.mlp.shared.up" not in t
    assert not [k for k in t if k.startswith("l2.") or k.startswith("l4.")]  # layers without tensors of their own
    assert c.flags() & lm._lib.LM_TANH_NORMS and c.flags() & lm._lib.LM_EMBED_NORM
    assert c.layers[2].to_c().weights_of == 1 and c.layers[4].to_c().weights_of == 2 and c.layers[0].to_c().weights_of == 0
    assert "Vovalorn" in models.ARCHITECTURES


def test_inner_size_comes_from_the_checkpoint_when_the_configuration_is_silent():
    cfg = small_cfg()
    for i in (0, 2):
        del cfg["layers"][i]["mixer"]["decay_rank"]
    c = lm.LMConfig.from_json(cfg, {"l0.mix.a1": (9, 40)})
    assert c.layers[0].decay_rank == 9 and c.layers[2].decay_rank == 9  # the layer without tensors reads its owner's
    with pytest.raises(KeyError):
        lm.LMConfig.from_json(cfg)


def test_bad_configurations_are_refused():
    cfg = small_cfg()
    cfg["layers"][1]["mixer"]["vdim"] = 7  # values reuse the key projection
    with pytest.raises(ValueError):
        lm.LMConfig.from_json(cfg)
    cfg = small_cfg()
    cfg["layers"][2]["weights_of"] = 2
    with pytest.raises(ValueError):
        lm.LMConfig.from_json(cfg)
    cfg = small_cfg()
    cfg["layers"][0]["type"] = "hgrn2"
    with pytest.raises(ValueError):
        lm.LMConfig.from_json(cfg)


def test_oracle_portions_equal_whole_prompts():
    cfg = small_cfg()
    w = vl.weights(cfg, seed=1)
    toks = vl.tokens(1, 40, cfg["vocab"])
    tr = []
    ref = vo.forward(w, cfg, toks, trace=tr)
    assert len(tr) == 5 and tr[0].shape == (40, 40)
    for cuts in ([1, 2, 3, 17, 19], [10, 30], list(range(1, 40))):
        seq, rows, lo = vo.Sequence(cfg), [], 0
        for hi in cuts + [40]:
            rows.append(vo.forward(w, cfg, toks[lo:hi], seq))
            lo = hi
        assert np.abs(np.concatenate(rows) - ref).max() < 1e-9
    assert vo.generate(w, cfg, toks[:5], 4) == vo.generate(w, cfg, toks[:5], 6)[:4]


def test_layers_that_share_tensors_keep_states_of_their_own():
    cfg = small_cfg()
    w = vl.weights(cfg, seed=2)
    toks = vl.tokens(2, 12, cfg["vocab"])
    seq = vo.Sequence(cfg)
    vo.forward(w, cfg, toks, seq)
    assert np.abs(seq.state[0] - seq.state[2]).max() > 1e-3  # same tensors, other inputs
    assert seq.state[1][0].shape == seq.state[4][0].shape and np.abs(seq.state[1][0] - seq.state[4][0]).max() > 1e-3


def test_router_on_hand_made_scores():
    r = {"experts": 6, "top": 2, "scale": 2.0, "groups": {"count": 3, "keep": 1}}
    z = np.array([[3.0, -9.0, 2.0, 2.5, -9.0, -9.0]])  # the largest score sits alone in its group; the pair next door outweighs it
    picks, wts = vo.route(z, np.zeros(6), r)
    assert picks[0].tolist() == [3, 2]
    s = vo.sigmoid(np.array([2.5, 2.0]))
    assert np.allclose(wts[0], s / s.sum() * 2.0)
    # the correction moves the choice, not the weights
    corr = np.array([0.0, 0.0, 0.0, 0.0, 2.0, 2.0])
    picks, wts = vo.route(z, corr, r)
    assert sorted(picks[0].tolist()) == [4, 5]
    s = vo.sigmoid(np.array([-9.0, -9.0]))
    assert np.allclose(wts[0], s / (s.sum() + 1e-20) * 2.0)
    # negative ranking scores: a group that is out of the race is set to -inf, not as zero
    corr = np.full(6, -5.0)
    picks, _ = vo.route(np.array([[0.1, 0.0, -9.0, -9.0, 0.3, -8.0]]), corr, {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 1}})
    assert sorted(picks[0].tolist()) == [0, 1]  # the pair 0.1, 0.0 outweighs 0.3 with its weak neighbour; all scores are below zero
    # groups of one expert: the group's score is that expert's; no groups at all: the plain top
    picks, _ = vo.route(z, np.zeros(6), {"experts": 6, "top": 2, "groups": {"count": 6, "keep": 2}})
    assert picks[0].tolist() == [0, 3]
    picks, _ = vo.route(z, np.zeros(6), {"experts": 6, "top": 3})
    assert picks[0].tolist() == [0, 3, 2]


def test_attention_weights_on_hand_made_scores():
    m = {"heads": 2, "kv_heads": 1, "dim": 2, "scale": 1.0, "softcap": 1.0}
    q = np.zeros((1, 2, 2))
    k = np.zeros((4, 1, 2))
    a = vo.attention_weights(q, k, [3], [0, 1, 2, 3], m)
    sl = vo.head_slopes(2)
    assert np.allclose(sl, [2.0 ** -4, 2.0 ** -8])
    for h in range(2):  # equal scores: the distance alone orders the weights
        want = np.exp(-sl[h] * np.array([3.0, 2.0, 1.0, 0.0]))
        assert np.allclose(a[h, 0], want / want.sum())
    # the cap flattens large scores: 100 and 50 both end close to the cap of one
    q[0, :, 0] = 10.0
    k[1, 0, 0], k[2, 0, 0] = 10.0, 5.0
    a = vo.attention_weights(q, k, [3], [0, 1, 2, 3], m)
    assert abs(a[1, 0, 1] / a[1, 0, 2] - np.exp(-sl[1])) < 1e-6
    # a key behind the query has no weight
    a = vo.attention_weights(q, k, [1], [0, 1, 2, 3], m)
    assert a[:, 0, 2:].max() == 0.0
    assert np.allclose(vo.query_factor([0, 3, 4, 9], {"coef": 0.5, "every": 5}), [1.0, 1.0, 1.0 + 0.5 * np.log(2.0), 1.0 + 0.5 * np.log(3.0)])


def test_decay_and_recurrence_on_hand_made_inputs():
    m = {"heads": 1, "dim": 2, "vdim": 1, "tau": 2.0}
    w = {"a1": np.eye(2), "a2": np.eye(2), "a2.b": np.array([0.0, 100.0])}
    f = vo.gla_decay(w, "", m, np.zeros((1, 2)))
    assert np.allclose(f[0, 0], [np.sqrt(0.5), 1.0])
    q = np.ones((3, 1, 2))
    k = np.array([[[1.0, 1.0]], [[0.0, 0.0]], [[0.0, 0.0]]])
    v = np.ones((3, 1, 1))
    o, S = vo.gla_recurrence(q, k, v, np.repeat(f, 3, axis=0), None)
    assert np.allclose(o[:, 0, 0], [2.0, np.sqrt(0.5) + 1.0, 0.5 + 1.0])  # the first token's own decay meets an empty state
    o2, _ = vo.gla_recurrence(q[2:], k[2:], v[2:], np.repeat(f, 1, axis=0), vo.gla_recurrence(q[:2], k[:2], v[:2], np.repeat(f, 2, axis=0), None)[1])
    assert np.allclose(o2[0], o[2])
