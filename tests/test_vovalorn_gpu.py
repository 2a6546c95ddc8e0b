"""The Vovalorn design on the layered-model tier (zig_gpt2_amd/lm.py) against the float64 oracle of tests/vovalorn_oracle.py: every
mechanism alone, whole prompts against portions and token-by-token decoding, ragged batches, slots and pages that go round,
layers that run another layer's tensors, heavy keys hundreds of tokens back, a cap, a query factor and a distance slope that
show, a state that forgets slowly across the chunks of the recurrence, other sizes, and generation through the library's entry
points, the scheduler, the host program and the trace replay."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import lm_testlib as tl
import vovalorn_oracle as vo
import vovalorn_testlib as vl
from zig_gpt2_amd import lm, models, weights_io

pytestmark = pytest.mark.gpu


def make(cfg, w, dtype="float32", **kw):
    kw.setdefault("max_tokens", 512)
    kw.setdefault("max_seqs", 4)
    m = lm.LayeredLM(lm.LMConfig.from_json(cfg), dtype=dtype, **kw)
    m.load_weights(w)
    return m


def run_whole(m, toks, want=None, trace=False):
    s = m.open()
    out = m.step([(s, toks, list(range(len(toks))) if want is None else want)], trace=trace)
    m.close_seq(s)
    return out


def run_cut(m, toks, cuts):
    """Feed toks in portions that end at `cuts`; all logits."""
    s = m.open()
    rows, lo = [], 0
    for hi in list(cuts) + [len(toks)]:
        if hi > lo:
            rows.append(m.step([(s, toks[lo:hi], list(range(hi - lo)))]))
        lo = hi
    m.close_seq(s)
    return np.concatenate(rows)


SINGLE = {
    "gla": [vl.gla_layer()],
    "gla_one_head": [vl.gla_layer(heads=1, dim=21, vdim=3, tau=1.0, decay_rank=1)],  # key channels on two lanes of a column, tau one
    "gla_wide_values": [vl.gla_layer(heads=2, dim=5, vdim=70, tau=30.0, decay_rank=11)],  # more columns than a workgroup takes at once
    "attention": [vl.attn_layer()],  # grouped keys, cap, query factor
    "attention_plain": [vl.attn_layer(heads=3, kv_heads=3, dim=8, softcap=0.0, q_temp=None)],  # every head its own keys, no cap, no factor
    "attention_one_key_head": [vl.attn_layer(heads=5, kv_heads=1, dim=7, scale=0.9, softcap=2.0, q_temp=(1.5, 1))],  # a factor that grows every token
    "attention_one_head": [vl.attn_layer(heads=1, kv_heads=1, dim=70, scale=0.05, softcap=50.0, q_temp=(0.2, 64))],  # beyond one lane row of channels
    "moe": [vl.gla_layer(mlp=vl.moe_mlp())],
    "moe_top1_no_shared": [vl.attn_layer(mlp=vl.moe_mlp(ff=9, experts=3, top=1, groups=None, shared=None))],
    "moe_all": [vl.gla_layer(mlp=vl.moe_mlp(ff=8, experts=4, top=4, groups=(2, 2), scale=0.5, shared=5))],  # every group stays, every expert is chosen
    "moe_groups_of_one": [vl.attn_layer(mlp=vl.moe_mlp(ff=8, experts=5, top=2, groups=(5, 3)))],
    "moe_one_group_kept": [vl.gla_layer(mlp=vl.moe_mlp(ff=12, experts=12, top=3, groups=(4, 1), scale=1.0))],
    "moe_many": [vl.attn_layer(mlp=vl.moe_mlp(ff=8, experts=70, top=3, groups=(7, 2)))],  # more experts than a wave has lanes
    "shared_tensors": [vl.gla_layer(mlp=vl.moe_mlp()), vl.attn_layer(), vl.attn_layer(weights_of=1), vl.gla_layer(weights_of=0, mlp=vl.moe_mlp())],
    "shared_tensors_backwards": [vl.attn_layer(weights_of=1, mlp=vl.moe_mlp(groups=(2, 1))), vl.attn_layer(mlp=vl.moe_mlp(groups=(2, 1)))],
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mechanism_alone(name, dtype):
    cfg = vl.config(SINGLE[name], width=50 if "one_head" in name else 40, residual_mult=1.0 if "plain" in name else 0.45)
    w = vl.weights(cfg, seed=sum(map(ord, name)), correction_std=0.4 if "moe" in name else 0.1)
    toks = vl.tokens(1, 83 if "one_head" in name else 37, cfg["vocab"])
    ref_tr = []
    ref = vo.forward(w, cfg, toks, trace=ref_tr)
    m = make(cfg, w, dtype)
    got, tr = run_whole(m, toks, trace=True)
    tl.assert_close(tr, np.stack(ref_tr), dtype, "residual stream")
    tl.assert_close(got, ref, dtype, "logits")
    # the same prompt token by token: the decode kernels, state carried by the slot
    step = run_cut(m, toks, range(1, len(toks)))
    tl.assert_close(step, ref, dtype, "decoded")
    m.close()


def _router_case(groups, experts, top):
    cfg = vl.config([vl.gla_layer(mlp=vl.moe_mlp(ff=10, experts=experts, top=top, groups=groups, shared=None))])
    w = vl.weights(cfg, seed=experts, correction_std=0.3)
    w["l0.mlp.router"] = w["l0.mlp.router"] * np.float32(8.0)  # scores that differ from token to token as much as the corrections do
    if experts == 9:
        w["l0.mlp.correction"] = w["l0.mlp.correction"] - np.float32(2.0)  # every ranking score below zero
    toks = vl.tokens(experts, 60, cfg["vocab"])
    vo.PROBE = []
    try:
        ref = vo.forward(w, cfg, toks)
        picks = [p for p in vo.PROBE if p[0] == "route"][0][1]
    finally:
        vo.PROBE = None
    return cfg, w, toks, ref, picks


ROUTER_CASES = [((4, 1), 12, 2), ((3, 2), 9, 3), ((6, 2), 6, 2), (None, 7, 2)]


def test_router_choices_equal_the_oracle():
    """Correction terms as large as the differences between the scores (in one case every ranking score is below zero), groups
    that lose the race with the best single expert inside: the residual stream behind the layer moves by a whole expert's
    output if one choice differs."""
    for groups, experts, top in ROUTER_CASES:
        cfg, w, toks, ref, picks = _router_case(groups, experts, top)
        if groups and experts // groups[0] > 1:  # the construction: without the groups other experts are chosen
            cfg2 = json.loads(json.dumps(cfg))
            del cfg2["layers"][0]["mlp"]["router"]["groups"]
            assert tl.rel_err(vo.forward(w, cfg2, toks), ref) > 1e-2, groups
        assert len({tuple(sorted(p)) for p in picks.tolist()}) >= 3, "the construction always chooses the same experts"
        m = make(cfg, w)
        tl.assert_close(run_whole(m, toks), ref, "float32", groups)
        tl.assert_close(run_cut(m, toks, range(50, 60)), ref, "float32", groups)
        m.close()


def full_cfg(**kw):
    return vl.config([vl.gla_layer(mlp=vl.moe_mlp()), vl.attn_layer(mlp=vl.moe_mlp(experts=8, top=3, groups=(4, 2), shared=None)),
                      vl.gla_layer(heads=2, dim=20, vdim=6, tau=9.0, decay_rank=3, mlp=None), vl.attn_layer(weights_of=1, mlp=vl.moe_mlp(experts=8, top=3, groups=(4, 2), shared=None)),
                      vl.gla_layer(weights_of=0, mlp=vl.moe_mlp()), vl.attn_layer(heads=6, kv_heads=3, dim=4, scale=0.5, softcap=3.0, q_temp=(0.7, 3), mlp=vl.moe_mlp(top=1, groups=None, shared=9))],
                     **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_several_sizes(dtype):
    cfg = full_cfg()
    w = vl.weights(cfg, seed=5)
    toks = vl.tokens(2, 90, cfg["vocab"])
    ref = vo.forward(w, cfg, toks)
    m = make(cfg, w, dtype, page_tokens=8)
    tl.assert_close(run_whole(m, toks), ref, dtype)
    for cuts in ([2, 4, 7, 15, 16, 24, 25, 57, 88], [1, 2, 3, 40, 41, 43], list(range(9, 90, 9)), [64]):
        tl.assert_close(run_cut(m, toks, cuts), ref, dtype, cuts)
    # portions longer than one pass of the library are cut inside the step
    m2 = make(cfg, w, dtype, max_step_tokens=16, page_tokens=8)
    tl.assert_close(run_whole(m2, toks), ref, dtype)
    tl.assert_close(run_cut(m2, toks, [33, 35]), ref, dtype)
    m.close()
    m2.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_in_one_batch(dtype):
    cfg = full_cfg()
    w = vl.weights(cfg, seed=7)
    lens = [41, 3, 17, 1]
    prompts = [vl.tokens(10 + i, n, cfg["vocab"]) for i, n in enumerate(lens)]
    refs = [vo.forward(w, cfg, p) for p in prompts]
    m = make(cfg, w, dtype, page_tokens=4)
    seqs = [m.open() for _ in prompts]
    first = [30, 2, 9, 1]
    got = m.step([(s, p[:k], list(range(k))) for s, p, k in zip(seqs, prompts, first)])
    off = 0
    for r, k in zip(refs, first):
        tl.assert_close(got[off:off + k], r[:k], dtype)
        off += k
    entries = [(s, p[k:], list(range(len(p) - k))) for s, p, k in zip(seqs, prompts, first) if len(p) > k]
    got = m.step(entries)
    off = 0
    for r, p, k in zip(refs, prompts, first):
        if len(p) > k:
            tl.assert_close(got[off:off + len(p) - k], r[k:], dtype)
            off += len(p) - k
    # lock-step decoding of three sequences at different positions against each alone
    more = [vl.tokens(20 + i, 6, cfg["vocab"]) for i in range(3)]
    alone = [vo.forward(w, cfg, np.concatenate([prompts[i], more[i]]))[len(prompts[i]):] for i in range(3)]
    rows = [m.step([(seqs[i], [more[i][t]], [0]) for i in range(3)]) for t in range(6)]
    for i in range(3):
        tl.assert_close(np.stack([r[i] for r in rows]), alone[i], dtype, i)
    m.close()


def test_slots_and_pages_are_reused():
    """Two slots and a cache of 96 tokens in pages of 4.  A closed sequence gives its pages and its slot back; the next one
    starts from an empty state and from positions that count from zero, on pages that held other keys."""
    cfg = full_cfg()
    w = vl.weights(cfg, seed=8)
    m = make(cfg, w, max_tokens=96, max_seqs=2, page_tokens=4)
    total = m.free_tokens()
    a, b, c = (vl.tokens(30 + i, n, cfg["vocab"]) for i, n in enumerate((50, 38, 44)))
    ra, rb, rc = (vo.forward(w, cfg, t) for t in (a, b, c))
    for rnd in range(2):
        sa, sb = m.open(), m.open()
        with pytest.raises(Exception):
            m.open()  # both slots taken
        for lo in range(0, 30, 10):
            got = m.step([(sa, a[lo:lo + 10], list(range(10))), (sb, b[lo:lo + 10], [9])])
            tl.assert_close(got[:10], ra[lo:lo + 10], "float32", (rnd, lo))
            tl.assert_close(got[10], rb[lo + 9], "float32", (rnd, lo))
        assert total - m.free_tokens() == 2 * 32  # whole pages per sequence
        with pytest.raises(Exception):
            m.step([(sa, np.concatenate([a, a]), [])])  # more than the cache holds
        m.close_seq(sb)  # its slot and pages go to a new sequence that starts from nothing
        sc = m.open()
        got = m.step([(sc, c, list(range(44))), (sa, a[30:], list(range(20)))])
        tl.assert_close(got[:44], rc, "float32", rnd)
        tl.assert_close(got[44:], ra[30:], "float32", rnd)
        assert m.seq_len(sa) == 50 and m.seq_len(sc) == 44
        m.close_seq(sa)
        m.close_seq(sc)
        assert m.free_tokens() == total
    m.close()


def test_general_attention_kernel(monkeypatch):
    """The one-workgroup-per-row form of the attention (what a step takes when the split form's workspace would not fit), on
    prompts, portions and decoded tokens over several key tiles."""
    monkeypatch.setenv("ZGPT2_LM_WINDOW_GENERAL", "1")
    cfg = vl.config([vl.attn_layer(), vl.attn_layer(heads=2, kv_heads=1, dim=70, scale=0.08, softcap=4.0, q_temp=(0.3, 50))])
    w = vl.weights(cfg, seed=21)
    toks = vl.tokens(22, 200, cfg["vocab"])
    ref = vo.forward(w, cfg, toks)
    for dtype in ("float32", "bfloat16"):
        m = make(cfg, w, dtype)
        tl.assert_close(run_whole(m, toks), ref, dtype)
        tl.assert_close(run_cut(m, toks, [3, 64, 65, 130] + list(range(180, 200))), ref, dtype)
        m.close()


@pytest.mark.parametrize("hook", ["ZGPT2_LM_WINDOW_NO_TILES", "ZGPT2_LM_WINDOW_TILES"])
def test_both_score_kernels_on_all_steps(monkeypatch, hook):
    """Prompt portions take their scores from matrix-core tiles of 32 rows x 32 keys, steps of few rows from the wave-per-key
    kernel; the hooks send every step through one of them (ragged row blocks, two entries): the cap and the slopes sit in both."""
    monkeypatch.setenv(hook, "1")
    cfg = vl.config([vl.attn_layer(heads=6, kv_heads=2, dim=18, softcap=1.5, q_temp=(0.9, 4)), vl.attn_layer(heads=1, kv_heads=1, dim=5, softcap=0.0),
                     vl.attn_layer(heads=18, kv_heads=6, dim=4, scale=0.7)])  # more heads than the tiled value product takes
    w = vl.weights(cfg, seed=23)
    a, b = vl.tokens(24, 150, cfg["vocab"]), vl.tokens(25, 47, cfg["vocab"])
    ra, rb = vo.forward(w, cfg, a), vo.forward(w, cfg, b)
    m = make(cfg, w)
    tl.assert_close(run_whole(m, a), ra, "float32")
    tl.assert_close(run_cut(m, a, [3, 35, 36, 100] + list(range(140, 150))), ra, "float32")
    sa, sb = m.open(), m.open()
    got = m.step([(sa, a[:70], list(range(70))), (sb, b, list(range(47)))])
    tl.assert_close(got[:70], ra[:70], "float32")
    tl.assert_close(got[70:], rb, "float32")
    m.close()


def _sharp(n, seed, **kw):
    """One attention layer whose softmax is sharp (normed q and k of 16 channels times a large factor): most queries put nearly all
    their weight on one key.  Returns (cfg, weights, tokens, logits, the softmax weights [heads, queries, keys])."""
    kw.setdefault("softcap", 60.0)
    kw.setdefault("q_temp", None)
    cfg = vl.config([vl.attn_layer(heads=4, kv_heads=2, dim=16, scale=2.5, **kw)], width=32, residual_mult=1.0)
    w = vl.weights(cfg, seed=seed)
    toks = vl.tokens(seed, n, cfg["vocab"])
    return (cfg, w, toks) + _probe_attention(cfg, w, toks)


def _probe_attention(cfg, w, toks):
    vo.PROBE = []
    try:
        ref = vo.forward(w, cfg, toks)
        att = [p for p in vo.PROBE if p[0] == "attention"][0][1]
    finally:
        vo.PROBE = None
    return ref, att


def test_far_keys_among_hundreds():
    """Every key stays visible.  One key is made to stand out: in the first layer a token's query and key depend on the token
    alone, so the key of one token id and the query of another are given a large common direction (through a vector of the input
    space that every other token of the prompt is orthogonal to).  That key sits at position 5, its queries hundreds of tokens
    later — across pages, key tiles and the shares of a split row; the values are the un-normalised key heads, the scores use the normed
    ones; the head with the flattest slope carries the pair."""
    n, D, W = 420, 16, 32
    cfg, w, _, _, _ = _sharp(n, 19)
    rng = np.random.default_rng(19)
    ids = rng.permutation(cfg["vocab"])[:22]  # the prompt's tokens: fewer than the width, so the orthogonal vectors exist
    key_tok, query_tok, rest = ids[0], ids[1], ids[2:]
    toks = rng.choice(rest, n).astype(np.int32)
    toks[5] = key_tok
    toks[[230, 300, 301, 388, 419]] = query_tok
    u = vo.tanh_norm(w, "l0.norm1", vo.embed(w, ids))  # the mixer's input of every token of the prompt
    dual = np.linalg.pinv(u)  # column t: a vector whose product with u[t] is one and with every other row zero
    d = rng.normal(0.0, 1.0, D)
    w = dict(w)
    wq, wk = w["l0.mix.q"].astype(np.float64).copy(), w["l0.mix.k"].astype(np.float64).copy()
    wq[3 * D:4 * D] += 30.0 * np.outer(d, dual[:, 1])  # head 3 (on key head 1): the flattest slope
    wk[1 * D:2 * D] += 30.0 * np.outer(d, dual[:, 0])
    w["l0.mix.q"], w["l0.mix.k"] = vl.round_bf16(wq.astype(np.float32)), vl.round_bf16(wk.astype(np.float32))
    ref, att = _probe_attention(cfg, w, toks)
    assert all(att[3, i, 5] > 0.8 for i in (230, 300, 301, 388, 419)), "the construction puts no heavy key far back"
    moved = toks.copy()
    moved[5], moved[6] = toks[6], toks[5]  # the heavy key one position later: its value is another token's neighbour
    assert tl.rel_err(vo.forward(w, cfg, moved)[300], ref[300]) < 1e-2 < tl.rel_err(vo.forward(w, cfg, np.delete(toks, 5))[299], ref[300])
    m = make(cfg, w, page_tokens=16)
    assert tl.rel_err(run_whole(m, toks), ref) < 2e-4
    assert tl.rel_err(run_cut(m, toks, [4, 5, 6, 100, 229, 230, 231, 333] + list(range(380, n))), ref) < 2e-4
    m.close()
    # the same weights with the slopes given to other heads differ clearly
    flipped = dict(w)
    flipped["l0.mix.q"] = w["l0.mix.q"].reshape(4, 16, -1)[[1, 0, 3, 2]].reshape(64, -1)
    assert tl.rel_err(vo.forward(flipped, cfg, toks), ref) > 1e-2


def test_cap_query_factor_and_slopes_show():
    """Each constant of the score's way to the softmax moves the logits clearly when it is left out or a little off, and the
    library follows the oracle with all of them: a cap well inside the scores' range, a query factor that steps up every seven
    tokens (inside portions and between decoded tokens), slopes that outweigh the scores at a distance."""
    n = 130
    cfg, w, toks, ref, att = _sharp(n, 27, softcap=6.0, q_temp=(0.8, 7))
    for key, other in (("softcap", None), ("softcap", 9.0), ("q_temp", None), ("q_temp", {"coef": 0.8, "every": 8}), ("q_temp", {"coef": 0.5, "every": 7}),
                       ("scale", 2.0)):
        cfg2 = json.loads(json.dumps(cfg))
        if other is None:
            del cfg2["layers"][0]["mixer"][key]
        else:
            cfg2["layers"][0]["mixer"][key] = other
        assert tl.rel_err(vo.forward(w, cfg2, toks), ref) > 1e-2, (key, other)
    near = np.arange(n)[None, :] - att[0].argmax(axis=-1)  # the head with the steepest slope looks at its neighbours
    assert np.median(near[0, 20:]) < np.median((np.arange(n)[None, :] - att[3].argmax(axis=-1))[0, 20:])
    m = make(cfg, w, page_tokens=8)
    assert tl.rel_err(run_whole(m, toks), ref) < 2e-4
    assert tl.rel_err(run_cut(m, toks, [5, 6, 7, 8, 13, 14, 15, 48, 49, 50, 100]), ref) < 2e-4
    assert tl.rel_err(run_cut(m, toks, range(20, n)), ref) < 2e-4  # decoded one by one, the factor stepping up on the way
    m.close()


def test_state_remembers_far_tokens_across_chunks():
    """Decays close to one (a large root, logits well above zero): the state forgets slowly, so the first tokens still weigh in
    hundreds of tokens later — a state that is lost, reset or carried wrongly between portions, chunks of the long-step form or
    decode steps shows.  Long steps run chunks of 64 tokens side by side; cuts sit at, before and behind their edges."""
    cfg = vl.config([vl.gla_layer(heads=2, dim=16, vdim=12, tau=64.0, decay_rank=4)], width=32, residual_mult=1.0)
    w = vl.weights(cfg, seed=11, decay_bias=(3.0, 0.5))
    n = 600
    toks = vl.tokens(41, n, cfg["vocab"])
    other = toks.copy()
    other[:40] = (other[:40] + 1) % cfg["vocab"]
    ref, ref_other = vo.forward(w, cfg, toks), vo.forward(w, cfg, other)
    assert tl.rel_err(ref_other[-1], ref[-1]) > 1e-3, "the construction does not carry the first tokens to the end"
    m = make(cfg, w, max_tokens=1024)
    tl.assert_close(run_whole(m, toks), ref, "float32")  # long enough for the chunks that run side by side
    tl.assert_close(run_cut(m, toks, [2, 4, 63, 64, 65, 127, 129, 385, 386]), ref, "float32")
    tl.assert_close(run_cut(m, toks, [300] + list(range(540, n))), ref, "float32")
    m.close()
    # a fast-forgetting layer beside it: tau one and logits below zero halve the state every token or faster
    cfg = vl.config([vl.gla_layer(heads=2, dim=16, vdim=12, tau=1.0, decay_rank=4)], width=32)
    w = vl.weights(cfg, seed=12, decay_bias=(-2.0, 2.0))
    ref = vo.forward(w, cfg, toks[:300])
    m = make(cfg, w)
    tl.assert_close(run_whole(m, toks[:300]), ref, "float32")
    tl.assert_close(run_cut(m, toks[:300], [64, 128, 290, 295]), ref, "float32")
    m.close()


def test_first_tokens_and_single_token_sequences():
    cfg = full_cfg()
    w = vl.weights(cfg, seed=12)
    m = make(cfg, w)
    for n in (1, 2, 3, 6):
        toks = vl.tokens(50 + n, n, cfg["vocab"])
        ref = vo.forward(w, cfg, toks)
        tl.assert_close(run_whole(m, toks), ref, "float32")
        tl.assert_close(run_cut(m, toks, range(1, n)), ref, "float32")
    m.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    cfg = full_cfg()
    w = vl.weights(cfg, seed=13)
    toks = vl.tokens(60, 200, cfg["vocab"])
    ref = vo.forward(w, cfg, toks)
    m = make(cfg, w, dtype, page_tokens=8)
    got = run_cut(m, toks, range(8, 200))
    tl.assert_close(got, ref, dtype)
    m.close()


def test_decoding_across_length_buckets():
    """Decode steps replay a graph per bucket of the longest sequence's length (512, 1024, ... tokens: a row's keys are split into
    shares by the bucket's capacity).  Two sequences decode in lock step while the longer one crosses 512 and 1024."""
    cfg = vl.config([vl.attn_layer(heads=4, kv_heads=2, dim=8, q_temp=(0.5, 100)), vl.gla_layer(heads=1, dim=8, vdim=8)], width=24, vocab=61)
    w = vl.weights(cfg, seed=31)
    a, b = vl.tokens(65, 1040, cfg["vocab"]), vl.tokens(66, 560, cfg["vocab"])
    ra, rb = vo.forward(w, cfg, a), vo.forward(w, cfg, b)
    m = make(cfg, w, max_tokens=2048)
    sa, sb = m.open(), m.open()
    m.step([(sa, a[:505], []), (sb, b[:25], [])])
    for lo, n in ((505, 15), (1015, 25)):  # 505 .. 519 and 1015 .. 1039 of the longer sequence
        if lo == 1015:
            m.step([(sa, a[520:1015], []), (sb, b[40:535], [])])
        rows = [m.step([(sa, a[lo + t:lo + t + 1], [0]), (sb, b[lo - 480 + t:lo - 479 + t], [0])]) for t in range(n)]
        tl.assert_close(np.stack([r[0] for r in rows]), ra[lo:lo + n], "float32", lo)
        tl.assert_close(np.stack([r[1] for r in rows]), rb[lo - 480:lo - 480 + n], "float32", lo)
    m.close()


def test_decode_steps_with_and_without_the_captured_graph():
    """A decode step replays the graph captured for its batch size; every replay, with eager prompt steps of other sequences
    between them, equals the same step launched kernel by kernel."""
    cfg = full_cfg()
    w = vl.weights(cfg, seed=17)
    a, b = vl.tokens(63, 40, cfg["vocab"]), vl.tokens(64, 25, cfg["vocab"])
    outs = []
    for use_graph in (True, False):
        m = make(cfg, w, use_graph=use_graph)
        sa, sb = m.open(), m.open()
        rows = [m.step([(sa, a[:10], [9])])]
        for t in range(10, 40):
            rows.append(m.step([(sa, a[t:t + 1], [0])]))
            if t % 7 == 0:  # eager work of another sequence between two replays
                lo = (t // 7 - 1) * 5
                rows.append(m.step([(sb, b[lo:lo + 5], [4])]))
        outs.append(np.concatenate(rows))
        m.close()
    assert np.array_equal(outs[0], outs[1])


def test_larger_odd_sizes_take_the_tiled_products():
    """Sizes that are not multiples of the kernels' tiles and vectors, enough rows for grouped products and for the chunks of the
    recurrence, heads of 128 and more channels, a width no vector load divides."""
    cfg = vl.config([vl.gla_layer(heads=3, dim=40, vdim=24, tau=11.0, decay_rank=7, mlp=vl.moe_mlp(ff=36, experts=6, top=2, groups=(2, 1), shared=50)),
                     vl.attn_layer(heads=6, kv_heads=3, dim=20, scale=0.2, mlp=vl.moe_mlp(ff=100, experts=3, top=2, groups=None, shared=3)),
                     vl.gla_layer(heads=1, dim=130, vdim=7, tau=20.0, decay_rank=2),
                     vl.attn_layer(heads=2, kv_heads=1, dim=128, scale=0.09, softcap=30.0, q_temp=(0.3, 100))],
                    vocab=203, width=77)
    w = vl.weights(cfg, seed=14)
    toks = vl.tokens(61, 330, cfg["vocab"])
    ref = vo.forward(w, cfg, toks)
    for dtype in ("float32", "bfloat16"):
        m = make(cfg, w, dtype)
        tl.assert_close(run_whole(m, toks), ref, dtype, dtype)
        tl.assert_close(run_cut(m, toks, [7, 140, 141, 215, 325]), ref, dtype, dtype)
        m.close()
    wide = vl.config([vl.gla_layer(mlp=vl.moe_mlp()), vl.attn_layer()], width=4100, vocab=50)
    w = vl.weights(wide, seed=15)
    toks = vl.tokens(62, 12, 50)
    m = make(wide, w)
    tl.assert_close(run_cut(m, toks, [9, 10]), vo.forward(w, wide, toks), "float32")
    m.close()


def test_greedy_and_sampled_generation():
    cfg = full_cfg()
    w = vl.weights(cfg, seed=15)
    prompts = [vl.tokens(70, 9, cfg["vocab"]), vl.tokens(71, 2, cfg["vocab"]), vl.tokens(72, 30, cfg["vocab"])]
    m = make(cfg, w, max_step_tokens=16)
    total = m.free_tokens()
    got = m.generate(prompts, 12)
    for p, g in zip(prompts, got):
        seq = vo.Sequence(cfg)
        lg = vo.forward(w, cfg, p, seq)
        for t in range(12):
            order = np.argsort(-lg[-1])
            if lg[-1][order[0]] - lg[-1][order[1]] < 1e-3 * np.abs(lg[-1]).max():
                break  # a near tie: fp32 and fp64 may differ from here on
            assert g[t] == order[0], (t, g, order[:3])
            lg = vo.forward(w, cfg, [int(g[t])], seq)
    assert m.free_tokens() == total  # generate gave every slot and page back
    a = m.generate(prompts, 10, temp=2.0, seed=3)
    assert np.array_equal(a, m.generate(prompts, 10, temp=2.0, seed=3)) and not np.array_equal(a, m.generate(prompts, 10, temp=2.0, seed=4))
    assert np.array_equal(m.generate(prompts, 4, temp=1e-3, seed=1), got[:, :4])
    m.close()


def test_checkpoint_folder_through_registry_host_program_and_trace_replay(tmp_path):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = full_cfg()
    for i in (0, 2, 4):
        del cfg["layers"][i]["mixer"]["decay_rank"]  # the inner size of the decay's projection only in the checkpoint's tensor shapes
    w = vl.weights(full_cfg(), seed=16)
    path = str(tmp_path / "ckpt")
    os.makedirs(path)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    weights_io.write_safetensors(os.path.join(path, "model.safetensors"), w)
    cfg = full_cfg()
    prompts = [vl.tokens(80, 11, cfg["vocab"]), vl.tokens(81, 4, cfg["vocab"])]
    m = models.load_model(path, dtype="float32", max_tokens=256, max_seqs=4)
    assert isinstance(m, lm.LayeredLM) and m.config.architecture == "Vovalorn" and m.config.layers[2].decay_rank == 3 and m.config.layers[4].decay_rank == 6
    want = m.generate(prompts, 9)
    ref = vo.forward(w, cfg, prompts[0])
    s = m.open()
    tl.assert_close(m.step([(s, prompts[0], list(range(11)))]), ref, "float32")
    m.close()
    exe = os.path.join(root, "zig_gpt2_amd", "bin", "zgpt2_main")
    arg = ";".join(",".join(str(int(t)) for t in p) for p in prompts)
    out = subprocess.run([exe, "lm", path, arg, "9", "--dtype", "float32"], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    got = np.array([[int(t) for t in line.split()] for line in out.stdout.strip().splitlines()])
    assert np.array_equal(got, want)
    a, b = [int(t) for t in prompts[0]], [int(t) for t in prompts[1]]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [5]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[6:9], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b, "want": [0, 3]}], "end": ["b"]},
             {"step": 3, "entries": [{"id": "a", "tokens": a[9:10], "want": [0]}], "end": []},
             {"step": 4, "entries": [{"id": "a", "tokens": a[10:11], "want": [0]}], "end": ["a"]},
             {"step": 5, "entries": [{"id": "c", "tokens": a, "want": [10]}], "end": ["c"]}]
    outdir = tmp_path / "out"
    for dtype in ("float32", "bfloat16"):
        run = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", dtype, "--out", str(outdir),
                              "--max-tokens", "64"], input="\n".join(json.dumps(x) for x in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert run.returncode == 0, run.stderr
        assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(6)]
        refb = vo.forward(w, cfg, prompts[1])
        rd = lambda i: np.fromfile(str(outdir / f"{i}.f32"), dtype="<f4").reshape(-1, cfg["vocab"])  # noqa: E731
        assert not (outdir / "1.f32").exists()
        tol = 3e-5 if dtype == "float32" else 4e-2
        for i, want_rows in ((0, ref[5:6]), (2, refb[[0, 3]]), (3, ref[9:10]), (4, ref[10:11]), (5, ref[10:11])):
            assert tl.rel_err(rd(i), want_rows) < tol, (dtype, i)


def test_scheduler_serves_more_requests_than_slots():
    """Continuous batching: seven requests of unequal lengths on two slots — every request's tokens equal its generation alone,
    slots and pages go round."""
    cfg = full_cfg()
    w = vl.weights(cfg, seed=18)
    m = make(cfg, w, max_tokens=128, max_seqs=2, page_tokens=8)
    reqs = [(vl.tokens(90 + i, n, cfg["vocab"]), k) for i, (n, k) in enumerate([(30, 6), (3, 9), (17, 2), (1, 12), (41, 5), (8, 8), (2, 1)])]
    alone = [m.generate([p], k)[0] for p, k in reqs]
    total = m.free_tokens()
    sch = lm.Scheduler(m, portion=16)
    ids = [sch.submit(p, k) for p, k in reqs]
    out = sch.run()
    for rid, want in zip(ids, alone):
        assert np.array_equal(out[rid], want), (rid, out[rid], want)
    assert m.free_tokens() == total and sch._reserved == 0
    assert sch.steps < sum(-(-len(p) // 16) + k for p, k in reqs)  # requests shared steps
    m.close()


def test_errors_are_reported():
    cfg = vl.config([vl.gla_layer(), vl.attn_layer(weights_of=0)])  # a layer cannot run the tensors of another kind of layer
    with pytest.raises(Exception):
        lm.LayeredLM(lm.LMConfig.from_json(cfg), dtype="float32", max_tokens=64, max_seqs=1)
    cfg = vl.config([vl.gla_layer(mlp=vl.moe_mlp(experts=6, top=5, groups=(3, 2)))])  # more experts chosen than the kept groups hold
    with pytest.raises(Exception):
        lm.LayeredLM(lm.LMConfig.from_json(cfg), dtype="float32", max_tokens=64, max_seqs=1)
    cfg = vl.config([vl.gla_layer()])
    w = vl.weights(cfg, seed=3)
    m = lm.LayeredLM(lm.LMConfig.from_json(cfg), dtype="float32", max_tokens=64, max_seqs=1)
    s = m.open()
    with pytest.raises(Exception):
        m.step([(s, [1, 2], [0])])  # no weights yet
    del w["l0.norm1b.alpha"]
    with pytest.raises(KeyError):
        m.load_weights(w)
    m.close()


def _random_cfg(rng):
    """A stack with sizes drawn at random: odd and even widths, heads on fewer key heads, groups of every shape, layers with and
    without experts or a shared one, layers that run the tensors of an earlier or later layer of their kind."""
    layers = []
    for _ in range(int(rng.integers(1, 5))):
        mlp = None
        if rng.random() < 0.75:
            count = int(rng.choice([1, 2, 3, 5]))
            size = int(rng.integers(1, 5))
            keep = int(rng.integers(1, count + 1))
            mlp = vl.moe_mlp(ff=int(rng.integers(1, 40)), experts=count * size, top=int(rng.integers(1, keep * size + 1)), groups=(count, keep) if rng.random() < 0.8 else None,
                             scale=float(rng.choice([0.5, 1.0, 2.5])), shared=int(rng.integers(1, 40)) if rng.random() < 0.6 else None)
            if mlp["router"].get("groups") is None:
                mlp["router"]["top"] = int(rng.integers(1, count * size + 1))
        if rng.random() < 0.5:
            layers.append(vl.gla_layer(heads=int(rng.integers(1, 5)), dim=int(rng.integers(1, 50)), vdim=int(rng.integers(1, 50)), tau=float(rng.choice([1.0, 4.0, 16.0, 50.0])),
                                       decay_rank=int(rng.integers(1, 20)), mlp=mlp))
        else:
            kv = int(rng.choice([1, 2, 3]))
            layers.append(vl.attn_layer(heads=kv * int(rng.choice([1, 2, 4])), kv_heads=kv, dim=int(rng.integers(1, 40)), scale=float(rng.choice([0.1, 0.5, 2.0])),
                                        softcap=float(rng.choice([0.0, 1.0, 5.0, 40.0])), q_temp=(float(rng.uniform(0.05, 1.0)), int(rng.choice([1, 2, 9, 64, 1000]))) if rng.random() < 0.7 else None,
                                        mlp=mlp))
    for _ in range(int(rng.integers(0, 3))):  # a copy of a layer, run again somewhere in the stack with separate state
        j = int(rng.integers(0, len(layers)))
        if "weights_of" in layers[j]:
            continue
        at = int(rng.integers(0, len(layers) + 1))
        twin = json.loads(json.dumps(layers[j]))
        layers.insert(at, twin)
        for e in layers:  # the indices behind the new entry move up
            if e is not twin and e.get("weights_of") is not None and e["weights_of"] >= at:
                e["weights_of"] += 1
        twin["weights_of"] = j + 1 if at <= j else j
    return vl.config(layers, vocab=int(rng.integers(2, 300)), width=int(rng.integers(3, 90)), eps=float(rng.choice([1e-6, 1e-5, 1e-3])),
                     residual_mult=float(rng.uniform(0.2, 1.2)))


@pytest.mark.parametrize("seed", range(12))
def test_sizes_drawn_at_random(seed):
    rng = np.random.default_rng(8000 + seed)
    cfg = _random_cfg(rng)
    w = vl.weights(cfg, seed=seed, correction_std=0.5)
    n = int(rng.integers(20, 300))
    toks = vl.tokens(seed, n, cfg["vocab"])
    ref = vo.forward(w, cfg, toks)
    m = make(cfg, w, page_tokens=int(rng.choice([4, 16, 64])))
    tl.assert_close(run_whole(m, toks), ref, "float32", cfg)
    cuts = sorted(set(int(c) for c in rng.integers(1, n, 6))) + list(range(max(1, n - 12), n))
    tl.assert_close(run_cut(m, toks, sorted(set(cuts))), ref, "float32", (cfg, cuts))
    m.close()
