"""The Sanazen design on the layered-model tier (zig_gpt2_amd/lm.py) against the float64 oracle of tests/sanazen_oracle.py: every
mechanism alone, whole prompts against portions and token-by-token decoding, ragged batches, slots and pages that go round (also
the pages between the kept first tokens and the window), keys at the window's edge and at the edge of the kept tokens made to
stand out, a linear-attention state that forgets slowly, other sizes, and generation through the library's entry points, the
scheduler, the host program and the trace replay."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import lm_testlib as tl
import sanazen_oracle as so
import sanazen_testlib as sl
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
    "pair": [sl.pair_layer()],  # grouped keys, a window with kept first tokens
    "pair_no_window": [sl.pair_layer(heads=3, kv_heads=3, dim=8, vdim=12, window=0, conv=1, lin_heads=1, lin_dim=5, lin_vdim=7)],
    "pair_one_head": [sl.pair_layer(heads=1, kv_heads=1, dim=6, vdim=4, window=70, keep_first=5, conv=5, lin_heads=1, lin_dim=20, lin_vdim=3)],  # a window beyond one key tile
    "pair_keeps_more_than_it_sees": [sl.pair_layer(heads=2, kv_heads=1, dim=10, vdim=6, window=4, keep_first=11, conv=2)],
    "pair_window_of_one": [sl.pair_layer(window=1, keep_first=1, lin_heads=2, lin_dim=18, lin_vdim=34)],
    "pair_no_conv": [sl.pair_layer(conv=0, keep_first=0, decay=[1.0, 0.5, 0.0])],
    "moe": [sl.pair_layer(mlp=sl.moe_mlp())],
    "moe_top1_no_shared": [sl.pair_layer(mlp=sl.moe_mlp(ff=20, experts=3, top=1, shared=None))],
    "moe_all": [sl.pair_layer(mlp=sl.moe_mlp(ff=8, experts=4, top=4, limit=0.3, shared=(5, 2.5)))],
    "moe_many": [sl.pair_layer(mlp=sl.moe_mlp(ff=8, experts=70, top=3))],  # more experts than a wave has lanes
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(SINGLE))
def test_each_mechanism_alone(name, dtype):
    cfg = sl.config(SINGLE[name], softcap=0.0 if "no_window" in name else 12.0, logit_scale=None if "no_conv" in name else 0.6,
                    width=50 if "one_head" in name else 48)
    w = sl.weights(cfg, seed=sum(map(ord, name)))
    toks = sl.tokens(1, 83 if "one_head" in name else 37, cfg["vocab"])
    ref, _, ref_tr = so.forward(w, cfg, toks, trace=True)
    m = make(cfg, w, dtype)
    got, tr = run_whole(m, toks, trace=True)
    tl.assert_close(tr, ref_tr, dtype, "residual stream")
    tl.assert_close(got, ref, dtype, "logits")
    # the same prompt token by token: the decode kernels, state carried by the slot
    step = run_cut(m, toks, range(1, len(toks)))
    tl.assert_close(step, ref, dtype, "decoded")
    m.close()


def full_cfg(**kw):
    return sl.config([sl.pair_layer(mlp=sl.moe_mlp()), sl.pair_layer(heads=2, kv_heads=1, dim=10, vdim=14, window=19, keep_first=2, conv=2, mlp=None),
                      sl.pair_layer(heads=6, kv_heads=3, dim=4, vdim=6, window=6, keep_first=9, conv=4, lin_heads=2, lin_dim=12, lin_vdim=6,
                                    mlp=sl.moe_mlp(experts=7, top=3, shared=None)),
                      sl.pair_layer(window=13, keep_first=0, mlp=sl.moe_mlp(top=1, shared=(9, 1.0)))], **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_portions_of_several_sizes(dtype):
    cfg = full_cfg()
    w = sl.weights(cfg, seed=5)
    toks = sl.tokens(2, 90, cfg["vocab"])
    ref = so.forward(w, cfg, toks)[0]
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
    w = sl.weights(cfg, seed=7)
    lens = [41, 3, 17, 1]
    prompts = [sl.tokens(10 + i, n, cfg["vocab"]) for i, n in enumerate(lens)]
    refs = [so.forward(w, cfg, p)[0] for p in prompts]
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
    more = [sl.tokens(20 + i, 6, cfg["vocab"]) for i in range(3)]
    alone = [so.forward(w, cfg, np.concatenate([prompts[i], more[i]]))[0][len(prompts[i]):] for i in range(3)]
    rows = [m.step([(seqs[i], [more[i][t]], [0]) for i in range(3)]) for t in range(6)]
    for i in range(3):
        tl.assert_close(np.stack([r[i] for r in rows]), alone[i], dtype, i)
    m.close()


def test_slots_and_pages_are_reused():
    """Two slots and a cache of 96 tokens.  The pages between the kept first tokens and the longest window go back to the pool
    while a sequence grows, so two sequences of 80 tokens fit together."""
    cfg = full_cfg()
    w = sl.weights(cfg, seed=8)
    m = make(cfg, w, max_tokens=96, max_seqs=2, page_tokens=4)
    total = m.free_tokens()
    a, b = sl.tokens(30, 80, cfg["vocab"]), sl.tokens(31, 80, cfg["vocab"])
    ra, rb = so.forward(w, cfg, a)[0], so.forward(w, cfg, b)[0]
    for rnd in range(2):
        sa, sb = m.open(), m.open()
        with pytest.raises(Exception):
            m.open()  # both slots taken
        for lo in range(0, 80, 10):
            got = m.step([(sa, a[lo:lo + 10], list(range(10))), (sb, b[lo:lo + 10], [9])])
            tl.assert_close(got[:10], ra[lo:lo + 10], "float32", (rnd, lo))
            tl.assert_close(got[10], rb[lo + 9], "float32", (rnd, lo))
            assert total - m.free_tokens() <= 2 * (12 + 19 + 2 * 4)  # per sequence: three pages of first tokens, the window, the edges
        m.close_seq(sb)  # its slot goes to a new sequence that starts from nothing
        sb = m.open()
        got = m.step([(sb, b[:21], list(range(21)))])
        tl.assert_close(got, rb[:21], "float32", rnd)
        with pytest.raises(Exception):
            m.step([(sa, a, [])])  # a sequence cannot outgrow the page table while first tokens are kept
        assert m.seq_len(sa) == 80 and m.seq_len(sb) == 21
        m.close_seq(sa)
        m.close_seq(sb)
        assert m.free_tokens() == total
    m.close()
    # no first tokens kept anywhere: the window's pages go round and a sequence grows far beyond the cache
    cfg = sl.config([sl.pair_layer(keep_first=0, mlp=sl.moe_mlp()), sl.pair_layer(window=17, keep_first=0)])
    w = sl.weights(cfg, seed=9)
    m = make(cfg, w, max_tokens=64, max_seqs=2, page_tokens=4)
    total = m.free_tokens()
    long = sl.tokens(32, 300, cfg["vocab"])
    rl = so.forward(w, cfg, long)[0]
    s = m.open()
    rows = [m.step([(s, long[i:i + 10], list(range(10)))]) for i in range(0, 300, 10)]
    tl.assert_close(np.concatenate(rows), rl, "float32")
    m.close_seq(s)
    assert m.free_tokens() == total
    m.close()


def test_general_window_kernel(monkeypatch):
    """The one-workgroup-per-row form of the windowed attention (what a step takes when the split form's workspace would not
    fit), on prompts, portions and decoded tokens, windows of several key tiles and kept first tokens included."""
    monkeypatch.setenv("ZGPT2_LM_WINDOW_GENERAL", "1")
    cfg = sl.config([sl.pair_layer(window=0), sl.pair_layer(heads=2, kv_heads=1, dim=70, vdim=6, window=90, keep_first=33)])
    w = sl.weights(cfg, seed=21)
    toks = sl.tokens(22, 200, cfg["vocab"])
    ref = so.forward(w, cfg, toks)[0]
    for dtype in ("float32", "bfloat16"):
        m = make(cfg, w, dtype)
        tl.assert_close(run_whole(m, toks), ref, dtype)
        tl.assert_close(run_cut(m, toks, [3, 64, 65, 130] + list(range(180, 200))), ref, dtype)
        m.close()


@pytest.mark.parametrize("hook", ["ZGPT2_LM_WINDOW_NO_TILES", "ZGPT2_LM_WINDOW_TILES"])
def test_both_score_kernels_on_all_steps(monkeypatch, hook):
    """Prompt portions take their scores from matrix-core tiles of 32 rows x 32 keys, steps of few rows from the wave-per-key
    kernel; the hooks send every step through one of them (ragged row blocks, windows that start inside a tile, kept tokens
    that end inside one, two entries)."""
    monkeypatch.setenv(hook, "1")
    cfg = sl.config([sl.pair_layer(heads=6, kv_heads=2, dim=18, vdim=4, window=41, keep_first=37), sl.pair_layer(heads=1, kv_heads=1, dim=5, vdim=3, window=0),
                     sl.pair_layer(heads=18, kv_heads=6, dim=4, vdim=34, window=9, keep_first=2)])  # more heads than the tiled value product takes
    w = sl.weights(cfg, seed=23)
    a, b = sl.tokens(24, 150, cfg["vocab"]), sl.tokens(25, 47, cfg["vocab"])
    ra, rb = so.forward(w, cfg, a)[0], so.forward(w, cfg, b)[0]
    m = make(cfg, w)
    tl.assert_close(run_whole(m, a), ra, "float32")
    tl.assert_close(run_cut(m, a, [3, 35, 36, 100] + list(range(140, 150))), ra, "float32")
    sa, sb = m.open(), m.open()
    got = m.step([(sa, a[:70], list(range(70))), (sb, b, list(range(47)))])
    tl.assert_close(got[:70], ra[:70], "float32")
    tl.assert_close(got[70:], rb, "float32")
    m.close()


def _edge_model(window, keep, n, seed):
    """One layer whose attention is sharp (a large score factor): most queries put nearly all their weight on one key.
    Returns (cfg, weights, tokens, the softmax weights [heads, queries, keys])."""
    lay = sl.pair_layer(heads=2, kv_heads=1, dim=16, vdim=8, window=window, keep_first=keep, scale=2.5, left_scale=1.5, right_scale=0.2)
    cfg = sl.config([lay], width=32)
    w = sl.weights(cfg, seed=seed)
    toks = sl.tokens(seed, n, cfg["vocab"])
    so.PROBE = []
    try:
        so.forward(w, cfg, toks)
        att = so.PROBE[0]
    finally:
        so.PROBE = None
    return cfg, w, toks, att


def test_keys_at_the_edges_stand_out():
    """A sharp softmax: a key that is one token too many or too few at the window's far edge or at the end of the kept first
    tokens, or read from a wrong page, changes a row by its whole value.  The same prompt with a window or a number of kept
    tokens that is one off must differ clearly."""
    window, n = 23, 150
    for keep in range(3, 20):  # a number of kept tokens whose last one is the heavy key of several rows far behind it
        cfg, w, toks, att = _edge_model(window, keep, n, 9)
        top, arg = att.max(axis=-1), att.argmax(axis=-1)
        far = np.arange(n)[None, :] - arg
        if ((top > 0.8) & (arg == keep - 1) & (far >= window)).sum() >= 3:
            break
    else:
        raise AssertionError("the construction puts no heavy key on the last kept token")
    assert ((top > 0.8) & (far == window - 1)).sum() >= 3, "the construction puts no heavy key on the window's edge"
    ref = so.forward(w, cfg, toks)[0]
    for key, other in (("size", window - 1), ("size", window + 1), ("keep_first", keep - 1), ("keep_first", keep + 1)):
        cfg2 = json.loads(json.dumps(cfg))
        cfg2["layers"][0]["mixer"]["left"]["mask"][key] = other
        assert tl.rel_err(so.forward(w, cfg2, toks)[0], ref) > 1e-2, (key, other)
    m = make(cfg, w, page_tokens=8)
    assert tl.rel_err(run_whole(m, toks), ref) < 2e-4
    assert tl.rel_err(run_cut(m, toks, [5, 6, 7, 22, 23, 24, 28, 29, 30, 46, 100]), ref) < 2e-4
    assert tl.rel_err(run_cut(m, toks, range(20, n)), ref) < 2e-4  # decoded one by one, the window sliding over pages
    m.close()


def test_far_keys_among_hundreds():
    """No window: every key stays visible.  With a sharp softmax the heavy keys lie hundreds of tokens back, across pages, key
    tiles and the shares of a split row."""
    n = 420
    lay = sl.pair_layer(heads=2, kv_heads=2, dim=16, vdim=8, window=0, scale=2.5, left_scale=1.5, right_scale=0.2)
    cfg = sl.config([lay], width=32)
    w = sl.weights(cfg, seed=19)
    toks = sl.tokens(19, n, cfg["vocab"])
    so.PROBE = []
    try:
        ref = so.forward(w, cfg, toks)[0]
        att = so.PROBE[0]
    finally:
        so.PROBE = None
    far = np.arange(n)[None, :] - att.argmax(axis=-1)
    assert ((att.max(axis=-1) > 0.8) & (far > 200)).sum() >= 10, "the construction puts no heavy key far back"
    m = make(cfg, w, page_tokens=16)
    assert tl.rel_err(run_whole(m, toks), ref) < 2e-4
    assert tl.rel_err(run_cut(m, toks, [100, 101, 333] + list(range(380, n))), ref) < 2e-4
    m.close()


@pytest.mark.parametrize("scan", [False, True])
def test_linear_attention_remembers_far_tokens(monkeypatch, scan):
    """Decays close to one: the state forgets slowly, so the first tokens still weigh in hundreds of tokens later (far beyond
    the window) — a state that is lost, reset or carried wrongly between portions, chunks or steps shows.  Prompt portions take
    chunks of 32 tokens as matrix products; the hook sends them through the token-serial scan (what wider heads take)."""
    if scan:
        monkeypatch.setenv("ZGPT2_LM_LINEAR_NO_CHUNKS", "1")
    cfg = sl.config([sl.pair_layer(window=5, keep_first=0, lin_heads=2, lin_dim=16, lin_vdim=12, decay=[0.9995, 0.998], left_scale=0.3, right_scale=1.0)], width=32)
    w = sl.weights(cfg, seed=11)
    n = 600
    toks = sl.tokens(41, n, cfg["vocab"])
    other = toks.copy()
    other[:40] = (other[:40] + 1) % cfg["vocab"]
    ref, ref_other = so.forward(w, cfg, toks)[0], so.forward(w, cfg, other)[0]
    assert tl.rel_err(ref_other[-1], ref[-1]) > 1e-3, "the construction does not carry the first tokens to the end"
    m = make(cfg, w, max_tokens=1024)
    tl.assert_close(run_whole(m, toks), ref, "float32")  # long enough for the chunks that run side by side
    tl.assert_close(run_cut(m, toks, [2, 4, 100, 101, 103, 200, 231, 232, 233, 264, 500]), ref, "float32")
    tl.assert_close(run_cut(m, toks, [300] + list(range(540, n))), ref, "float32")
    m.close()


def test_first_tokens_and_single_token_sequences():
    cfg = full_cfg()
    w = sl.weights(cfg, seed=12)
    m = make(cfg, w)
    for n in (1, 2, 3, 6):
        toks = sl.tokens(50 + n, n, cfg["vocab"])
        ref = so.forward(w, cfg, toks)[0]
        tl.assert_close(run_whole(m, toks), ref, "float32")
        tl.assert_close(run_cut(m, toks, range(1, n)), ref, "float32")
    m.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    cfg = full_cfg()
    w = sl.weights(cfg, seed=13)
    toks = sl.tokens(60, 200, cfg["vocab"])
    ref = so.forward(w, cfg, toks)[0]
    m = make(cfg, w, dtype, page_tokens=8)
    got = run_cut(m, toks, range(8, 200))
    tl.assert_close(got, ref, dtype)
    m.close()


def test_larger_odd_sizes_take_the_tiled_products():
    """Sizes that are not multiples of the kernels' tiles and vectors, enough rows for grouped products and for the chunks of the
    recurrence, a window of several key tiles, a width beyond the register-held norm kernel."""
    cfg = sl.config([sl.pair_layer(heads=6, kv_heads=3, dim=20, vdim=10, window=150, keep_first=40, conv=4, lin_heads=3, lin_dim=40, lin_vdim=24,
                                   mlp=sl.moe_mlp(ff=36, experts=6, top=2, shared=(50, 1.0))),
                     sl.pair_layer(heads=2, kv_heads=1, dim=128, vdim=64, window=64, keep_first=64, lin_heads=1, lin_dim=130, lin_vdim=7,
                                   mlp=sl.moe_mlp(ff=100, experts=3, top=2, shared=(3, 0.5)))],
                    vocab=203, width=76)
    w = sl.weights(cfg, seed=14)
    toks = sl.tokens(61, 330, cfg["vocab"])
    ref = so.forward(w, cfg, toks)[0]
    for dtype in ("float32", "bfloat16"):
        m = make(cfg, w, dtype)
        tl.assert_close(run_whole(m, toks), ref, dtype, dtype)
        tl.assert_close(run_cut(m, toks, [7, 140, 141, 215, 325]), ref, dtype, dtype)
        m.close()
    wide = sl.config([sl.pair_layer(mlp=sl.moe_mlp())], width=4100, vocab=50)
    w = sl.weights(wide, seed=15)
    toks = sl.tokens(62, 12, 50)
    m = make(wide, w)
    tl.assert_close(run_cut(m, toks, [9, 10]), so.forward(w, wide, toks)[0], "float32")
    m.close()


def test_greedy_and_sampled_generation():
    cfg = full_cfg(softcap=30.0)
    w = sl.weights(cfg, seed=15, embed_std=0.5)
    prompts = [sl.tokens(70, 9, cfg["vocab"]), sl.tokens(71, 2, cfg["vocab"]), sl.tokens(72, 30, cfg["vocab"])]
    m = make(cfg, w, max_step_tokens=16)
    total = m.free_tokens()
    got = m.generate(prompts, 12)
    for p, g in zip(prompts, got):
        lg, st = so.forward(w, cfg, p)
        for t in range(12):
            order = np.argsort(-lg[-1])
            if lg[-1][order[0]] - lg[-1][order[1]] < 1e-3 * np.abs(lg[-1]).max():
                break  # a near tie: fp32 and fp64 may differ from here on
            assert g[t] == order[0], (t, g, order[:3])
            lg, st = so.forward(w, cfg, [int(g[t])], st)
    assert m.free_tokens() == total  # generate gave every slot and page back
    a = m.generate(prompts, 10, temp=2.0, seed=3)
    assert np.array_equal(a, m.generate(prompts, 10, temp=2.0, seed=3)) and not np.array_equal(a, m.generate(prompts, 10, temp=2.0, seed=4))
    assert np.array_equal(m.generate(prompts, 4, temp=1e-3, seed=1), got[:, :4])
    m.close()


def test_checkpoint_folder_through_registry_host_program_and_trace_replay(tmp_path):
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = full_cfg()
    del cfg["layers"][2]["mixer"]["left"]["conv"]  # the taps of this layer only in the checkpoint's tensor shapes
    w = sl.weights(full_cfg(), seed=16, embed_std=0.5)
    path = str(tmp_path / "ckpt")
    os.makedirs(path)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    weights_io.write_safetensors(os.path.join(path, "model.safetensors"), w)
    cfg = full_cfg()
    prompts = [sl.tokens(80, 11, cfg["vocab"]), sl.tokens(81, 4, cfg["vocab"])]
    m = models.load_model(path, dtype="float32", max_tokens=256, max_seqs=4)
    assert isinstance(m, lm.LayeredLM) and m.config.architecture == "Sanazen" and m.config.layers[2].conv == 4
    want = m.generate(prompts, 9)
    ref = so.forward(w, cfg, prompts[0])[0]
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
    run = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32", "--out", str(outdir),
                          "--max-tokens", "64"], input="\n".join(json.dumps(x) for x in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(6)]
    refb = so.forward(w, cfg, prompts[1])[0]
    rd = lambda i: np.fromfile(str(outdir / f"{i}.f32"), dtype="<f4").reshape(-1, cfg["vocab"])  # noqa: E731
    assert not (outdir / "1.f32").exists()
    tl.assert_close(rd(0), ref[5:6], "float32")
    tl.assert_close(rd(2), refb[[0, 3]], "float32")
    tl.assert_close(rd(3), ref[9:10], "float32")
    tl.assert_close(rd(4), ref[10:11], "float32")
    tl.assert_close(rd(5), ref[10:11], "float32")


def test_scheduler_serves_more_requests_than_slots():
    """Continuous batching: seven requests of unequal lengths on two slots — every request's tokens equal its generation alone,
    slots and pages go round, also the pages that the windows leave behind while a request is still running."""
    cfg = full_cfg(softcap=30.0)
    w = sl.weights(cfg, seed=18, embed_std=0.5)
    m = make(cfg, w, max_tokens=128, max_seqs=2, page_tokens=8)
    reqs = [(sl.tokens(90 + i, n, cfg["vocab"]), k) for i, (n, k) in enumerate([(30, 6), (3, 9), (17, 2), (1, 12), (41, 5), (8, 8), (2, 1)])]
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
    cfg = sl.config([sl.pair_layer()])
    w = sl.weights(cfg, seed=3)
    m = lm.LayeredLM(lm.LMConfig.from_json(cfg), dtype="float32", max_tokens=64, max_seqs=1)
    s = m.open()
    with pytest.raises(Exception):
        m.step([(s, [1, 2], [0])])  # no weights yet
    del w["l0.mix.left.o.b"]
    with pytest.raises(KeyError):
        m.load_weights(w)
    bad = json.loads(json.dumps(cfg))
    bad["layers"][0]["mixer"]["right"]["decay"] = [0.5]
    with pytest.raises(ValueError):
        lm.LMConfig.from_json(bad)
    m.close()


def _random_cfg(rng):
    """A stack with sizes drawn at random: odd and even widths, heads on fewer key heads, unequal key and value sizes, windows
    from one token to none, kept tokens below and above the window, 0 to 6 taps, experts with and without a shared one."""
    layers = []
    for _ in range(int(rng.integers(1, 4))):
        kv = int(rng.choice([1, 2, 3]))
        heads = kv * int(rng.choice([1, 2, 4]))
        window = int(rng.choice([0, 1, 2, 5, 16, 33, 64, 100]))
        lh = int(rng.integers(1, 4))
        mlp = None
        if rng.random() < 0.75:
            experts = int(rng.integers(1, 10))
            mlp = sl.moe_mlp(ff=int(rng.integers(1, 40)), experts=experts, top=int(rng.integers(1, experts + 1)), limit=float(rng.choice([0.25, 1.0, 7.0])),
                             shared=(int(rng.integers(1, 40)), float(rng.choice([0.5, 3.0]))) if rng.random() < 0.6 else None)
        layers.append(sl.pair_layer(heads=heads, kv_heads=kv, dim=int(rng.integers(1, 40)), vdim=int(rng.integers(1, 40)), window=window,
                                    keep_first=int(rng.choice([0, 1, 3, 8, 40])), scale=float(rng.choice([0.1, 0.5])), conv=int(rng.integers(0, 7)),
                                    lin_heads=lh, lin_dim=int(rng.integers(1, 50)), lin_vdim=int(rng.integers(1, 50)),
                                    decay=[float(v) for v in rng.uniform(0.3, 1.0, lh)], left_scale=float(rng.uniform(0.3, 1.5)),
                                    right_scale=float(rng.uniform(0.3, 1.5)), mlp=mlp))
    return sl.config(layers, vocab=int(rng.integers(2, 300)), width=int(rng.integers(3, 90)), eps=float(rng.choice([1e-6, 1e-5, 1e-3])),
                     embed_scale=float(rng.uniform(0.5, 9.0)), logit_scale=float(rng.uniform(0.2, 2.0)), softcap=float(rng.choice([0.0, 5.0, 40.0])))


@pytest.mark.parametrize("seed", range(12))
def test_sizes_drawn_at_random(seed):
    rng = np.random.default_rng(7000 + seed)
    cfg = _random_cfg(rng)
    w = sl.weights(cfg, seed=seed)
    n = int(rng.integers(20, 300))
    toks = sl.tokens(seed, n, cfg["vocab"])
    ref = so.forward(w, cfg, toks)[0]
    m = make(cfg, w, page_tokens=int(rng.choice([4, 16, 64])))
    tl.assert_close(run_whole(m, toks), ref, "float32", cfg)
    cuts = sorted(set(int(c) for c in rng.integers(1, n, 6))) + list(range(max(1, n - 12), n))
    tl.assert_close(run_cut(m, toks, sorted(set(cuts))), ref, "float32", (cfg, cuts))
    m.close()
