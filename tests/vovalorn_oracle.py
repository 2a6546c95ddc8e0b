"""Plain, slow float64 restatement of the Vovalorn design that zig_gpt2_amd/lm.py serves.

One function per mechanism, numpy only, written from the design's equations; it shares no code with the product path
(zig_gpt2_amd/ is not imported).  Weights are a dict name -> numpy array with the checkpoint's tensor names, the
configuration is the dict of config.json.

Notation: x residual stream [T, W]; u a sublayer's input; positions p count from 0 per sequence; rms(v) = sqrt(mean(v^2) + eps);
c the residual factor.  Every function that carries something from token to token takes what the tokens before left (None: the
start of a sequence) and returns the new one.

  n(v)   = tanh(a v) * w + b                       a scalar a and vectors w, b per norm; no reduction over the row
  x_t    = n_e(embed[token_t])
  layer  : x <- x + c n_1b(mixer(n_1(x)));  x <- x + c n_2b(ff(n_2(x)))        (a layer may have no ff)
           a layer that names another layer runs that layer's tensors with separate state
  gla    : q = W_q u / sqrt(D), k = W_k u, v = W_v u per head;  f = sigmoid(W_a2 W_a1 u + b_a)^(1/tau) per head and key channel
           S_t = diag(f_t) S_(t-1) + k_t v_t^T;  o_t = S_t^T q_t;  W_o (concat_h(o / rms(o) * w) * silu(W_g u))
  attention : q = W_q u, k = W_k u; the VALUE of a key head is that head's un-normalised k;  q, k <- q / rms(q), k / rms(k) per head
           q_i <- q_i (1 + t_c ln(floor((i + 1) / t_e) + 1))
           s_ij = cap tanh(scale (q_i . k_j) / cap) - 2^(-8 (h + 1) / H) (i - j),  j <= i;  softmax over j;  W_o concat_h(sum_j a_ij v_j)
  ff     : z = W_r u, s = sigmoid(z), experts ranked by r = s + correction; the expert list in `count` contiguous blocks, a block ranked by
           its best r plus its second-best r, experts outside the `keep` top blocks get r = -inf; the `top` highest r win;
           weights s_e / (sum of the chosen s + 1e-20) * route_scale;  sum_e w_e E_e(u) + E_shared(u),
           E(u) = W_down (silu(W_gate u) * W_up u)
  logits = W_head n_f(x)
"""
import math

import numpy as np

F = np.float64
PROBE = None  # a list: every attention call appends its softmax weights [heads, queries, keys]; every router call its choices


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def rms_unit(v, eps):
    return v / np.sqrt(np.mean(v * v, axis=-1, keepdims=True) + eps)


# ----------------------------------------------------------------------------------------------- the norm
def tanh_norm(w, name, v):
    """tanh(alpha v) * weight + bias with the three tensors of `name`."""
    return np.tanh(float(w[name + ".alpha"]) * v) * w[name].astype(F) + w[name + ".b"].astype(F)


# ----------------------------------------------------------------------------------------------- embedding
def embed(w, tokens):
    return tanh_norm(w, "embed.norm", w["embed"].astype(F)[np.asarray(tokens)])


# ----------------------------------------------------------------------------------------------- gated linear attention
def gla_decay(w, p, m, u):
    """[T, heads, dim]: the factor of every key channel's row of the state."""
    H, D = int(m["heads"]), int(m["dim"])
    z = (u @ w[p + "a1"].astype(F).T) @ w[p + "a2"].astype(F).T + w[p + "a2.b"].astype(F)
    return (sigmoid(z) ** (1.0 / float(m["tau"]))).reshape(-1, H, D)


def gla_recurrence(q, k, v, f, state):
    """q, k, f [T, H, D], v [T, H, V]; state [H, D, V] or None.  Returns (o [T, H, V], state)."""
    T, H, D = q.shape
    S = np.zeros((H, D, v.shape[2]), F) if state is None else state.copy()
    o = np.zeros((T, H, v.shape[2]), F)
    for t in range(T):
        S = f[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = np.einsum("hdv,hd->hv", S, q[t])
    return o, S


def gla(w, p, m, u, state, eps):
    H, D, V = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    T = u.shape[0]
    q = (u @ w[p + "q"].astype(F).T).reshape(T, H, D) / math.sqrt(D)
    k = (u @ w[p + "k"].astype(F).T).reshape(T, H, D)
    v = (u @ w[p + "v"].astype(F).T).reshape(T, H, V)
    o, state = gla_recurrence(q, k, v, gla_decay(w, p, m, u), state)
    o = rms_unit(o, eps) * w[p + "norm"].astype(F)
    gate = silu(u @ w[p + "g"].astype(F).T)
    return (o.reshape(T, H * V) * gate) @ w[p + "o"].astype(F).T, state


# ----------------------------------------------------------------------------------------------- attention
def query_factor(positions, q_temp):
    if not q_temp:
        return np.ones(len(positions), F)
    p = np.asarray(positions, np.int64)
    return 1.0 + float(q_temp["coef"]) * np.log((p + 1) // int(q_temp["every"]) + 1.0)


def head_slopes(H):
    return np.array([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)], F)


def attention_weights(q, k, q_pos, k_pos, m):
    """q [Tq, H, D] (normed, with its factor), k [Tk, G, D] (normed) -> softmax weights [H, Tq, Tk]."""
    H, G = int(m["heads"]), int(m.get("kv_heads", m["heads"]))
    rep = H // G
    s = np.einsum("ihd,jhd->hij", q, np.repeat(k, rep, axis=1)) * float(m["scale"])
    cap = float(m.get("softcap") or 0.0)
    if cap > 0.0:
        s = cap * np.tanh(s / cap)
    dist = np.asarray(q_pos, F)[:, None] - np.asarray(k_pos, F)[None, :]
    s = s - head_slopes(H)[:, None, None] * dist[None]
    s = np.where(dist[None] >= 0, s, -np.inf)
    s = s - s.max(axis=2, keepdims=True)
    e = np.exp(s)
    return e / e.sum(axis=2, keepdims=True)


def attention(w, p, m, u, positions, cache, eps):
    """cache: (normed keys [T0, G, D], values [T0, G, D]) of the tokens before, or None."""
    H, G, D = int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"])
    T = u.shape[0]
    q = rms_unit((u @ w[p + "q"].astype(F).T).reshape(T, H, D), eps) * query_factor(positions, m.get("q_temp"))[:, None, None]
    k_raw = (u @ w[p + "k"].astype(F).T).reshape(T, G, D)
    k = rms_unit(k_raw, eps)
    if cache is not None:
        k = np.concatenate([cache[0], k], axis=0)
        k_raw = np.concatenate([cache[1], k_raw], axis=0)
    n0 = k.shape[0] - T
    k_pos = np.concatenate([np.arange(n0), np.asarray(positions)]) if n0 else np.asarray(positions)
    a = attention_weights(q, k, positions, k_pos, m)
    if PROBE is not None:
        PROBE.append(("attention", a))
    o = np.einsum("hij,jhd->ihd", a, np.repeat(k_raw, H // G, axis=1)).reshape(T, H * D)
    return o @ w[p + "o"].astype(F).T, (k, k_raw)


# ----------------------------------------------------------------------------------------------- experts
def route(z, correction, r):
    """z [T, E] router logits -> (chosen experts [T, top], weights [T, top])."""
    E, top = int(r["experts"]), int(r["top"])
    groups = r.get("groups") or {"count": 1, "keep": 1}
    count, keep = int(groups["count"]), int(groups["keep"])
    size = E // count
    s = sigmoid(z)
    choice = s + correction
    picks, weights = [], []
    for t in range(z.shape[0]):
        c = choice[t].copy()
        if count > 1:
            gs = [np.sort(c[g * size:(g + 1) * size])[::-1][:2].sum() for g in range(count)]
            best = sorted(range(count), key=lambda g: (-gs[g], g))[:keep]
            for g in range(count):
                if g not in best:
                    c[g * size:(g + 1) * size] = -np.inf
        chosen = sorted(range(E), key=lambda e: (-c[e], e))[:top]
        sc = s[t][chosen]
        picks.append(chosen)
        weights.append(sc / (sc.sum() + 1e-20) * float(r.get("scale", 1.0)))
    return np.array(picks), np.array(weights, F)


def expert(w, p, u):
    return (silu(u @ w[p + "gate"].astype(F).T) * (u @ w[p + "up"].astype(F).T)) @ w[p + "down"].astype(F).T


def experts_ff(w, p, mlp, u):
    picks, weights = route(u @ w[p + "router"].astype(F).T, w[p + "correction"].astype(F), mlp["router"])
    if PROBE is not None:
        PROBE.append(("route", picks, weights))
    y = np.zeros_like(u)
    for t in range(u.shape[0]):
        for e, a in zip(picks[t], weights[t]):
            y[t] += a * expert(w, f"{p}e{e}.", u[t:t + 1])[0]
    if mlp.get("shared"):
        y += expert(w, p + "shared.", u)
    return y


# ----------------------------------------------------------------------------------------------- the stack
def weights_layer(cfg, i):
    """Index of the layer whose tensors layer i runs."""
    seen = set()
    while cfg["layers"][i].get("weights_of") is not None and i not in seen:
        seen.add(i)
        i = int(cfg["layers"][i]["weights_of"])
    return i


class Sequence:
    """What a sequence carries between calls: per layer the recurrent state or the keys and values, and the token count."""

    def __init__(self, cfg):
        self.state = [None] * len(cfg["layers"])
        self.n = 0


def forward(w, cfg, tokens, seq=None, trace=None):
    """Logits [T, vocab] of the next `tokens` of a sequence (seq: a Sequence that is moved on; None: a new one).
    trace: a list that receives the residual stream behind every layer."""
    seq = seq or Sequence(cfg)
    eps, c = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    positions = np.arange(seq.n, seq.n + len(tokens))
    x = embed(w, tokens)
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{weights_layer(cfg, i)}."
        u = tanh_norm(w, p + "norm1", x)
        if layer["type"] == "gla":
            y, seq.state[i] = gla(w, p + "mix.", layer["mixer"], u, seq.state[i], eps)
        elif layer["type"] == "attention":
            y, seq.state[i] = attention(w, p + "mix.", layer["mixer"], u, positions, seq.state[i], eps)
        else:
            raise ValueError(layer["type"])
        x = x + c * tanh_norm(w, p + "norm1b", y)
        if layer.get("mlp"):
            y = experts_ff(w, p + "mlp.", layer["mlp"], tanh_norm(w, p + "norm2", x))
            x = x + c * tanh_norm(w, p + "norm2b", y)
        if trace is not None:
            trace.append(x.copy())
    seq.n += len(tokens)
    return tanh_norm(w, "final.norm", x) @ w["head"].astype(F).T


def generate(w, cfg, prompt, n_new):
    seq = Sequence(cfg)
    out, logits = [], forward(w, cfg, prompt, seq)
    for _ in range(n_new):
        out.append(int(np.argmax(logits[-1])))
        logits = forward(w, cfg, [out[-1]], seq)
    return out
