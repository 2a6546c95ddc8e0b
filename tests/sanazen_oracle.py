"""Plain, slow float64 restatement of the Sanazen design that zig_gpt2_amd/lm.py serves.

One function per mechanism, numpy only, written from the design's equations; it shares no code with the product path
(zig_gpt2_amd/ is not imported).  Weights are a dict name -> numpy array with the checkpoint's tensor names, the
configuration is the dict of config.json.

Notation: x residual stream [T, W]; h a sublayer's input; positions p count from 0 per sequence;
rms(v) = sqrt(mean(v^2) + eps).  Every function that carries something from token to token takes the state the tokens
before left (None: the start of a sequence) and returns the new one.

  x_t   = embed[token_t] * s_e + pe(p_t),    pe(p)[2i] = sin(p b^(-2i/W)), pe(p)[2i+1] = cos(p b^(-2i/W)), b = 10000
  layer : x <- x + mixer(n1(x)) + ff(n2(x)),   n(v) = v / rms(v) * w          (both sublayers read the same x)
  mixer : c_l * A(h) + c_r * L(h)
    A   : u = conv(W_u h + b_u) for u in q, k, v;  q <- q / rms(q) * w_q, k likewise (over the whole projection);
          a_ij = softmax_j(scale q_i . k_j) over j <= i with i - j < window or j < keep;  W_o (concat_h(a v) * sigmoid(W_g h)) + b_o
    L   : q, k, v = silu(W. h);  S_t = lambda_h S_(t-1) + k_t v_t^T;  o_t = S_t^T q_t;  W_o (o / rms(o) * w * sigmoid(W_g h))
  ff    : s = sigmoid(W_r h), the `top` largest;  sum_e E_e(s_e h) + sigmoid(w_sg . h) E_shared(h)
          E(z) = W_down (g sigmoid(1.702 g) (u + 1)),  g = min(W_gate z, lim),  u = clip(W_up z, -lim, lim)
  logits = cap tanh(s_l (W_head n_f(x)) / cap)
"""
import numpy as np

F = np.float64
PROBE = None  # a list: every call of the left branch appends its softmax weights [heads, queries, keys] (for tests that build on them)


def rms_unit(v, eps):
    return v / np.sqrt(np.mean(v * v, axis=-1, keepdims=True) + eps)


def norm_plain(v, w, eps):
    return rms_unit(v, eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


# ----------------------------------------------------------------------------------------------- embedding
def position_vectors(positions, width):
    """Interleaved sines and cosines; the angle is formed as a 32-bit product of the position and a 32-bit frequency."""
    half = (width + 1) // 2
    freq = np.array([10000.0 ** (-2.0 * i / width) for i in range(half)], F).astype(np.float32)
    ang = (np.asarray(positions, np.float32)[:, None] * freq[None, :]).astype(F)
    out = np.zeros((len(positions), 2 * half), F)
    out[:, 0::2] = np.sin(ang)
    out[:, 1::2] = np.cos(ang)
    return out[:, :width]


def embed(w, cfg, tokens, positions):
    scale = float((cfg.get("embedding") or {}).get("scale", 1.0))
    return w["embed"].astype(F)[np.asarray(tokens)] * scale + position_vectors(positions, int(cfg["width"]))


# ----------------------------------------------------------------------------------------------- causal convolution over time
def causal_conv(v, w, tail):
    """v [T, C], w [C, taps] (the last column multiplies the current token), tail: the taps - 1 inputs before v (None: zeros).
    Returns (conv [T, C], new tail)."""
    taps = w.shape[1]
    T, C = v.shape
    before = np.zeros((taps - 1, C), F) if tail is None else tail
    full = np.concatenate([before, v], axis=0)
    out = np.zeros((T, C), F)
    for j in range(taps):
        out += full[j:j + T] * w[:, j][None, :]
    return out, full[full.shape[0] - (taps - 1):].copy()


# ----------------------------------------------------------------------------------------------- windowed attention, first tokens kept
def visible(q_pos, k_pos, window, keep_first):
    """[queries, keys]: a key at or before the query that is inside the window or among the first tokens.  window 0: no window."""
    dist = np.asarray(q_pos)[:, None] - np.asarray(k_pos)[None, :]
    ok = dist >= 0
    if window:
        ok &= (dist < window) | (np.asarray(k_pos)[None, :] < keep_first)
    return ok


def softmax_weights(q, k, scale, ok, H, G):
    """q [T, H, D], k [N, G, D] -> weights [H, T, N]; query head h reads key head h // (H / G)."""
    s = np.einsum("thd,nhd->htn", q, np.repeat(k, H // G, axis=1)) * scale
    s = np.where(ok[None], s, -np.inf)
    e = np.exp(s - s.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


def gated_window_attention(h, w, p, m, eps, positions, state):
    """The left branch.  state: dict(q=, k=, v= convolution tails, keys=[n, G, D], values=[n, G, V]) of the tokens before."""
    H, G, D, V = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"])
    mask = m.get("mask") or {}
    st = dict(state) if state else {}
    proj = {}
    for u in ("q", "k", "v"):
        z = h @ w[p + u].astype(F).T + w[p + u + ".b"].astype(F)
        if p + u + ".conv" in w:
            z, st[u] = causal_conv(z, w[p + u + ".conv"].astype(F), st.get(u))
        proj[u] = z
    q = norm_plain(proj["q"], w[p + "q.norm"].astype(F), eps).reshape(-1, H, D)
    k = norm_plain(proj["k"], w[p + "k.norm"].astype(F), eps).reshape(-1, G, D)
    v = proj["v"].reshape(-1, G, V)
    n_before = 0 if "keys" not in st else st["keys"].shape[0]
    keys = k if n_before == 0 else np.concatenate([st["keys"], k], axis=0)
    values = v if n_before == 0 else np.concatenate([st["values"], v], axis=0)
    st["keys"], st["values"] = keys, values
    k_pos = np.arange(keys.shape[0])
    ok = visible(positions, k_pos, int(mask.get("size", 0)), int(mask.get("keep_first", 0)))
    a = softmax_weights(q, keys, float(m["scale"]), ok, H, G)
    if PROBE is not None:
        PROBE.append(a)
    o = np.einsum("htn,nhv->thv", a, np.repeat(values, H // G, axis=1)).reshape(-1, H * V)
    o = o * sigmoid(h @ w[p + "g"].astype(F).T)
    return o @ w[p + "o"].astype(F).T + w[p + "o.b"].astype(F), st


# ----------------------------------------------------------------------------------------------- linear attention with a fixed decay per head
def decayed_linear_attention(q, k, v, decay, S):
    """q, k [T, H, D], v [T, H, V], decay [H], S [H, D, V] (None: zeros): S <- decay S + k v^T, o = S^T q, token by token."""
    T, H, D = q.shape
    S = np.zeros((H, D, v.shape[2]), F) if S is None else S.copy()
    out = np.zeros((T, H, v.shape[2]), F)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = np.einsum("hdv,hd->hv", S, q[t])
    return out, S


def lightning_branch(h, w, p, m, eps, state):
    """The right branch.  state: S [H, D, V] or None."""
    H, D, V = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(h @ w[p + "q"].astype(F).T).reshape(-1, H, D)
    k = silu(h @ w[p + "k"].astype(F).T).reshape(-1, H, D)
    v = silu(h @ w[p + "v"].astype(F).T).reshape(-1, H, V)
    o, S = decayed_linear_attention(q, k, v, np.asarray(m["decay"], F), state)
    o = norm_plain(o.reshape(-1, H * V), w[p + "norm"].astype(F), eps) * sigmoid(h @ w[p + "g"].astype(F).T)
    return o @ w[p + "o"].astype(F).T, S


def pair_mixer(h, w, p, m, eps, positions, state):
    st = state or {}
    left, ls = gated_window_attention(h, w, p + "left.", m["left"], eps, positions, st.get("left"))
    right, rs = lightning_branch(h, w, p + "right.", m["right"], eps, st.get("right"))
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right, {"left": ls, "right": rs}


# ----------------------------------------------------------------------------------------------- experts
def clipped_expert(z, w, p, limit):
    """W_down(g sigmoid(1.702 g) (u + 1)) with the gate capped from above and the linear part clipped on both sides."""
    g = np.minimum(z @ w[p + "gate"].astype(F).T, limit)
    u = np.clip(z @ w[p + "up"].astype(F).T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].astype(F).T


def sigmoid_router(h, w, p, top, logits_dtype=np.float32):
    """(chosen experts [T, top], their scores): the largest sigmoid scores, lowest index first among equals."""
    z = (h.astype(logits_dtype) @ w[p + "router"].astype(logits_dtype).T).astype(F)
    s = sigmoid(z)
    pick = np.argsort(-s, axis=-1, kind="stable")[:, :top]
    return pick, np.take_along_axis(s, pick, axis=-1)


def expert_mixture(h, w, p, mlp):
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    pick, score = sigmoid_router(h, w, p, top, F)
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]), F)
    for t in range(h.shape[0]):
        for e, s in zip(pick[t], score[t]):
            out[t] += clipped_expert((s * h[t])[None], w, f"{p}e{e}.", float(mlp["expert"]["limit"]))[0]
    if mlp.get("shared"):
        gate = sigmoid(h @ w[p + "shared.sg"].astype(F).T)  # [T, 1]
        out += gate * clipped_expert(h, w, p + "shared.", float(mlp["shared"]["limit"]))
    assert E >= top
    return out


# ----------------------------------------------------------------------------------------------- the model
def layer(x, w, i, entry, eps, positions, state):
    p = f"l{i}."
    y, st = pair_mixer(norm_plain(x, w[p + "norm1"].astype(F), eps), w, p + "mix.", entry["mixer"], eps, positions, state)
    if entry.get("mlp"):
        y = y + expert_mixture(norm_plain(x, w[p + "norm2"].astype(F), eps), w, p + "mlp.", entry["mlp"])
    return x + y, st


def logits_of(x, w, cfg):
    z = norm_plain(x, w["final.norm"].astype(F), float(cfg["norm"]["eps"])) @ w["head"].astype(F).T * float(cfg.get("logit_scale", 1.0))
    cap = cfg.get("logit_softcap")
    return cap * np.tanh(z / cap) if cap else z


def forward(w, cfg, tokens, state=None, trace=False):
    """The next tokens of one sequence.  state: what the tokens before left (None: a new sequence).  Returns (logits [T, vocab],
    new state) and, with trace, the residual stream behind every layer [layers, T, W]."""
    eps = float(cfg["norm"]["eps"])
    st = {"n": 0, "layers": [None] * len(cfg["layers"])} if state is None else {"n": state["n"], "layers": list(state["layers"])}
    positions = np.arange(st["n"], st["n"] + len(tokens))
    x = embed(w, cfg, tokens, positions)
    tr = []
    for i, entry in enumerate(cfg["layers"]):
        if entry["type"] != "parallel":
            raise ValueError(f"unknown layer type {entry['type']!r}")
        x, st["layers"][i] = layer(x, w, i, entry, eps, positions, st["layers"][i])
        tr.append(x.copy())
    st["n"] += len(tokens)
    out = logits_of(x, w, cfg)
    return (out, st, np.stack(tr)) if trace else (out, st)


def greedy(w, cfg, prompt, n_new):
    out, st = forward(w, cfg, prompt)
    toks = [int(np.argmax(out[-1]))]
    while len(toks) < n_new:
        out, st = forward(w, cfg, [toks[-1]], st)
        toks.append(int(np.argmax(out[-1])))
    return toks
