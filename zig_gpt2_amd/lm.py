"""Layered language models over the C ABI's layered-model tier (zg_lm_* of include/zgpt2.h).

A model of this family is DATA: config.json lists the layers — which token mixer, which feed-forward, their sizes — and the
library runs whatever list it is given.  This module turns a checkpoint's config.json into the library's layer descriptors
(`LMConfig`), loads tensors by their checkpoint names, and wraps the handle (`LayeredLM`): sequences are opened, stepped with
any number of tokens at a time (several sequences per step), and closed; `generate` runs prompts through the same step with
the library's greedy / sampling head.

config.json (zig_gpt2_amd/models.py maps architecture names to loaders; `DESIGNS` below holds what a name fixes):
  vocab, width, norm.eps, layers[i] = {type, mixer: {...sizes...}, mlp: null | {kind: "dense", ff}
  | {kind: "moe", expert: {ff}, router: {experts, top}}}, loop: null | {start, stop, times}.
  Tokosun: type "hgrn2" | "latent_attention"; token shift in front of the mixer; gated experts, softmax router with correction.
  Gupizen: type "parallel" (mixer.left: windowed attention with sink, mixed heads and rotated values; mixer.right: gated linear
  recurrent unit) | "channel_delta" (gated delta rule); canon.taps: input convolution of both sublayers; embedding.scale; tied
  head; the embedding output added again in front of every repetition of the loop but the first; plain gelu experts, the
  router's largest logits.  Sizes the configuration does not list (the inner sizes of two-step projections) come from the
  checkpoint's tensor shapes.
  Sanazen: type "parallel" (mixer.left: grouped-query attention without rotation — q, k, v with biases through a short causal
  convolution, q and k normed over the whole projection, a sliding window that keeps the first mask.keep_first tokens in sight,
  heads gated by sigmoid(W_g h); mixer.right: linear attention with the fixed per-head `decay`; the branches summed with
  left_scale / right_scale); a layer is x += mixer(norm1(x)) + mlp(norm2(x)) with plain norm weights; sinusoidal position
  vectors added to the scaled embedding; experts with a clipped gated activation (`expert.limit`), chosen by their sigmoid
  scores, the score multiplying the expert's input; mlp.shared: an expert every token uses, times sigmoid(shared.sg . h);
  logit_scale, logit_softcap.
  Vovalorn: type "gla" (gated linear attention: a decay per key channel, sigmoid(W_a2 W_a1 h + b)^(1 / tau); heads normed over
  vdim, gated by silu(W_g h)) | "attention" (grouped-query attention over the whole sequence with no value projection —
  a key head's un-normalised projection serves as its value —, q and k divided by their root mean square per head, a query factor that grows with the logarithm of the position
  (q_temp: coef, every), scores capped (softcap) and lowered by a slope per head times the distance); a layer with "weights_of": j
  runs layer j's tensors with separate cache and state; every norm is tanh(alpha v) * w + b (tensors `<name>`, `<name>.b`,
  `<name>.alpha`), also behind the embedding (`embed.norm`); residual_mult: factor of every sublayer's normed output in the
  residual sum; experts chosen by sigmoid scores + correction among the best contiguous blocks of experts (router.groups:
  count, keep), weights normalised over the chosen, times router.scale; mlp.shared: an expert every token uses.
"""
import ctypes as C
import json
import os
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

from . import _lib
from ._lib import check_lm as check

MIXERS = {"hgrn2": _lib.LM_MIX_HGRN2, "latent_attention": _lib.LM_MIX_LATENT_ATTENTION, "parallel": _lib.LM_MIX_PARALLEL,
          "channel_delta": _lib.LM_MIX_CHANNEL_DELTA, "window_linear": _lib.LM_MIX_WINDOW_LINEAR, "gla": _lib.LM_MIX_GLA,
          "attention": _lib.LM_MIX_ATTENTION}
ROT_STYLES = {"yarn": _lib.LM_ROT_YARN, "bands": _lib.LM_ROT_BANDS}
EXPERT_ACTS = {"glu_silu": _lib.LM_ACT_GLU_SILU, "gelu": _lib.LM_ACT_GELU, "glu_clipped": _lib.LM_ACT_GLU_CLIPPED}
ROUTERS = {"softmax_all": _lib.LM_ROUTE_SOFTMAX_ALL, "top_logits": _lib.LM_ROUTE_TOP_LOGITS, "sigmoid_input": _lib.LM_ROUTE_SIGMOID_INPUT,
           "sigmoid_groups": _lib.LM_ROUTE_SIGMOID_GROUPS}

# what an architecture name fixes beyond config.json.  mixers: layer type of config.json -> mixer of the library (two designs
# call different pairs of branches "parallel")
DESIGNS = {
    "Tokosun": dict(mixers={"hgrn2": "hgrn2", "latent_attention": "latent_attention"}, tied_head=False, loop_readd=False, expert_act="glu_silu",
                    router="softmax_all"),
    "Gupizen": dict(mixers={"parallel": "parallel", "channel_delta": "channel_delta"}, tied_head=True, loop_readd=True, expert_act="gelu",
                    router="top_logits"),
    "Sanazen": dict(mixers={"parallel": "window_linear"}, tied_head=False, loop_readd=False, expert_act="glu_clipped", router="sigmoid_input",
                    side_by_side=True, sinusoid_positions=True),
    "Vovalorn": dict(mixers={"gla": "gla", "attention": "attention"}, tied_head=False, loop_readd=False, expert_act="glu_silu", router="sigmoid_groups",
                     tanh_norms=True, embed_norm=True),
}


@dataclass
class LayerSpec:
    """One entry of config['layers'], flattened into the fields of zg_lm_layer."""

    mixer: str
    heads: int
    dim: int
    vdim: int
    rot_dim: int = 0
    kv_rank: int = 0
    q_rank: int = 0
    scale: float = 1.0
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: Optional[dict] = None  # {factor, original, fast, slow}
    rot_style: str = "yarn"  # yarn: {factor, original, fast, slow} | bands: {factor, original, low, high}
    ff: str = "none"  # none | dense | moe
    ff_width: int = 0
    experts: int = 0
    top: int = 0
    expert_act: str = "glu_silu"
    router: str = "softmax_all"
    kv_heads: int = 0
    window: int = 0
    lru_width: int = 0
    lru_blocks: int = 0
    lru_conv: int = 0
    conv: int = 0
    decay_rank: int = 0
    gate_rank: int = 0
    keep_first: int = 0
    left_scale: float = 1.0
    right_scale: float = 1.0
    lin_heads: int = 0
    lin_dim: int = 0
    lin_vdim: int = 0
    decay: Optional[list] = None  # one factor per head of the linear-attention branch
    ff_limit: float = 0.0
    shared_width: int = 0
    shared_limit: float = 0.0
    tau: float = 0.0  # gla: the decay is sigmoid(.)^(1 / tau)
    softcap: float = 0.0  # attention: cap of the scores (0: none)
    qtemp_coef: float = 0.0  # attention: the query factor 1 + coef ln(floor((p + 1) / every) + 1) ...
    qtemp_every: int = 0  # ... 0: none
    dist_bias: bool = False  # attention: head h loses 2^(-8 (h + 1) / heads) per position of distance
    route_groups: int = 1  # sigmoid_groups: contiguous blocks of experts, how many of them stay in the race, factor of the weights
    route_keep: int = 1
    route_scale: float = 1.0
    weights_of: Optional[int] = None  # this layer runs the tensors of that layer

    @classmethod
    def from_json(cls, entry, design="Tokosun", shapes=None, prefix=""):
        """entry: one element of config['layers'].  shapes: {tensor name: shape} of the checkpoint, for the sizes that only
        tensor shapes give (prefix: 'l<i>.')."""
        kind, m = entry["type"], entry["mixer"]
        fixed = DESIGNS[design]
        if kind not in fixed["mixers"]:
            raise ValueError(f"unknown mixer type {kind!r} (known to {design}: {sorted(fixed['mixers'])})")
        kind = fixed["mixers"][kind]

        def inner(key, tensor):
            """A size the configuration may leave to the checkpoint: rows of `tensor`."""
            if key in m:
                return int(m[key])
            if shapes is None or prefix + tensor not in shapes:
                raise KeyError(f"{prefix}mix: the inner size {key!r} needs the shape of tensor {prefix + tensor!r}")
            return int(shapes[prefix + tensor][0])

        if kind == "gla":
            kw = dict(mixer=kind, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]), tau=float(m["tau"]),
                      decay_rank=inner("decay_rank", "mix.a1"))
        elif kind == "attention":
            qt = m.get("q_temp") or {}
            kw = dict(mixer=kind, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                      vdim=int(m.get("vdim", m["dim"])), scale=float(m["scale"]), softcap=float(m.get("softcap") or 0.0),
                      qtemp_coef=float(qt.get("coef", 0.0)), qtemp_every=int(qt.get("every", 0)), dist_bias=bool(m.get("dist_bias", True)))
            if kw["vdim"] != kw["dim"]:
                raise ValueError(f"{prefix}mix: values reuse the key projection, so vdim {kw['vdim']} cannot differ from dim {kw['dim']}")
        elif kind == "window_linear":
            l, r = m["left"], m["right"]
            mask = l.get("mask") or {}
            conv = l.get("conv")
            if conv is None:  # the taps of the convolutions from the checkpoint; no such tensor: no convolution
                conv = int(shapes[prefix + "mix.left.q.conv"][1]) if shapes and prefix + "mix.left.q.conv" in shapes else 0
            kw = dict(mixer=kind, heads=int(l["heads"]), kv_heads=int(l.get("kv_heads", l["heads"])), dim=int(l["dim"]), vdim=int(l["vdim"]),
                      scale=float(l["scale"]), window=int(mask.get("size", 0)), keep_first=int(mask.get("keep_first", 0)), conv=int(conv),
                      left_scale=float(m.get("left_scale", 1.0)), right_scale=float(m.get("right_scale", 1.0)), lin_heads=int(r["heads"]),
                      lin_dim=int(r["dim"]), lin_vdim=int(r["vdim"]), decay=[float(v) for v in r["decay"]])
            if len(kw["decay"]) != kw["lin_heads"]:
                raise ValueError(f"{prefix}mix.right: {len(kw['decay'])} decays for {kw['lin_heads']} heads")
        elif kind == "parallel":
            l, r = m["left"], m["right"]
            rot = l.get("rot") or {}
            kw = dict(mixer=kind, heads=int(l["heads"]), kv_heads=int(l.get("kv_heads", l["heads"])), dim=int(l["dim"]), vdim=int(l["vdim"]),
                      scale=float(l["scale"]), window=int((l.get("mask") or {}).get("size", 0)), rot_dims=int(rot.get("dims", 0)),
                      rot_base=float(rot.get("base", 10000.0)), rot_scaling=dict(rot["scaling"]) if rot.get("scaling") else None,
                      rot_style="bands", lru_width=int(r["width"]), lru_blocks=int(r["blocks"]), lru_conv=int(r["conv"]))
        elif kind == "channel_delta":
            kw = dict(mixer=kind, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m["vdim"]),
                      conv=int(m["conv"]), decay_rank=inner("decay_rank", "mix.a1"), gate_rank=inner("gate_rank", "mix.g1"))
        else:
            kw = dict(mixer=kind, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]))
        kw.update(expert_act=fixed["expert_act"], router=fixed["router"])
        if kind == "latent_attention":
            rot = m.get("rot") or {}
            kw.update(rot_dim=int(m["rot_dim"]), kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]), scale=float(m["scale"]),
                      rot_dims=int(rot.get("dims", m["rot_dim"])), rot_base=float(rot.get("base", 10000.0)),
                      rot_scaling=dict(rot["scaling"]) if rot.get("scaling") else None)
        mlp = entry.get("mlp")
        if mlp:
            if mlp["kind"] == "dense":
                kw.update(ff="dense", ff_width=int(mlp["ff"]))
            elif mlp["kind"] == "moe":
                kw.update(ff="moe", ff_width=int(mlp["expert"]["ff"]), experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]))
                if fixed["expert_act"] == "glu_clipped":
                    kw.update(ff_limit=float(mlp["expert"]["limit"]))
                    if mlp.get("shared"):
                        kw.update(shared_width=int(mlp["shared"]["ff"]), shared_limit=float(mlp["shared"]["limit"]))
                elif mlp.get("shared"):
                    kw.update(shared_width=int(mlp["shared"]["ff"]))
                if fixed["router"] == "sigmoid_groups":
                    groups = mlp["router"].get("groups") or {}
                    count = int(groups.get("count", 1))
                    kw.update(route_groups=count, route_keep=int(groups.get("keep", count)), route_scale=float(mlp["router"].get("scale", 1.0)))
            else:
                raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
        if entry.get("weights_of") is not None:
            kw.update(weights_of=int(entry["weights_of"]))
        return cls(**kw)

    def to_json(self):
        mixer = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim}
        if self.mixer == "parallel":
            rot = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling:
                rot["scaling"] = dict(self.rot_scaling)
            left = dict(mixer, kv_heads=self.kv_heads, scale=self.scale, rot=rot)
            if self.window:
                left["mask"] = {"size": self.window}
            mixer = {"left": left, "right": {"width": self.lru_width, "blocks": self.lru_blocks, "conv": self.lru_conv}}
        elif self.mixer == "channel_delta":
            mixer.update(kv_heads=self.kv_heads, conv=self.conv, decay_rank=self.decay_rank, gate_rank=self.gate_rank)
        elif self.mixer == "window_linear":
            left = dict(mixer, kv_heads=self.kv_heads, scale=self.scale, conv=self.conv)
            if self.window:
                left["mask"] = {"size": self.window, "keep_first": self.keep_first}
            mixer = {"left": left, "left_scale": self.left_scale, "right_scale": self.right_scale,
                     "right": {"heads": self.lin_heads, "dim": self.lin_dim, "vdim": self.lin_vdim, "decay": list(self.decay)}}
        if self.mixer == "latent_attention":
            rot = {"base": self.rot_base, "dims": self.rot_dims}
            if self.rot_scaling:
                rot["scaling"] = dict(self.rot_scaling)
            mixer.update(rot_dim=self.rot_dim, kv_rank=self.kv_rank, q_rank=self.q_rank, scale=self.scale, rot=rot)
        if self.mixer == "gla":
            mixer.update(tau=self.tau, decay_rank=self.decay_rank)
        elif self.mixer == "attention":
            mixer.update(kv_heads=self.kv_heads, scale=self.scale)
            if self.softcap:
                mixer["softcap"] = self.softcap
            if self.qtemp_every:
                mixer["q_temp"] = {"coef": self.qtemp_coef, "every": self.qtemp_every}
            if not self.dist_bias:
                mixer["dist_bias"] = False
        mlp = None
        if self.ff == "dense":
            mlp = {"kind": "dense", "ff": self.ff_width}
        elif self.ff == "moe":
            mlp = {"kind": "moe", "expert": {"ff": self.ff_width}, "router": {"experts": self.experts, "top": self.top}}
            if self.expert_act == "glu_clipped":
                mlp["expert"]["limit"] = self.ff_limit
                mlp["shared"] = {"ff": self.shared_width, "limit": self.shared_limit} if self.shared_width else None
            elif self.shared_width:
                mlp["shared"] = {"ff": self.shared_width}
            if self.router == "sigmoid_groups":
                mlp["router"].update(groups={"count": self.route_groups, "keep": self.route_keep}, scale=self.route_scale)
        out = {"type": "parallel" if self.mixer == "window_linear" else self.mixer, "mixer": mixer, "mlp": mlp}
        if self.weights_of is not None:
            out["weights_of"] = self.weights_of
        return out

    def to_c(self):
        sc = self.rot_scaling or {}
        bands = self.rot_style == "bands"  # the bands' `high` / `low` travel in the fields of the blend's `fast` / `slow`
        return _lib.LmLayer(MIXERS[self.mixer], self.heads, self.dim, self.vdim, self.rot_dim, self.kv_rank, self.q_rank, self.scale, self.rot_dims,
                            self.rot_base, ROT_STYLES[self.rot_style] if self.rot_scaling else 0, float(sc.get("factor", 1.0)),
                            float(sc.get("original", 1.0)), float(sc.get("high" if bands else "fast", 1.0)),
                            float(sc.get("low" if bands else "slow", 1.0)),
                            {"none": _lib.LM_FF_NONE, "dense": _lib.LM_FF_DENSE, "moe": _lib.LM_FF_MOE}[self.ff], self.ff_width, self.experts,
                            self.top, self.kv_heads, self.window, self.lru_width, self.lru_blocks, self.lru_conv, self.conv, self.decay_rank,
                            self.gate_rank, EXPERT_ACTS[self.expert_act], ROUTERS[self.router], self.keep_first, self.left_scale, self.right_scale,
                            self.lin_heads, self.lin_dim, self.lin_vdim, self.ff_limit, self.shared_width, self.shared_limit, self.tau, self.softcap,
                            self.qtemp_coef, self.qtemp_every, int(self.dist_bias), self.route_groups, self.route_keep, self.route_scale,
                            0 if self.weights_of is None else self.weights_of + 1)

    def tensor_shapes(self, prefix, width, canon_taps=0, tanh_norms=False):
        """{checkpoint tensor name: shape} of this layer (none for a layer that runs another layer's tensors)."""
        if self.weights_of is not None:
            return {}
        H, D, V, W = self.heads, self.dim, self.vdim, width
        t = {prefix + "norm1": (W,), prefix + "norm1b": (W,)}
        if self.mixer == "window_linear":  # plain norms in front of the sublayers only, nothing between norm and mixer
            t = {prefix + "norm1": (W,)}
        elif tanh_norms:  # the mixer reads the norm as it is
            pass
        elif canon_taps:
            t[prefix + "canon1"] = (W, canon_taps)
            if self.ff != "none":
                t[prefix + "canon2"] = (W, canon_taps)
        else:
            t[prefix + "shift"] = (W,)
        m = prefix + "mix."
        if self.mixer == "parallel":
            G, C, NB = self.kv_heads, self.lru_width, self.lru_blocks
            l, r = m + "left.", m + "right."
            t.update({l + "q": (H * D, W), l + "k": (G * D, W), l + "v": (G * V, W), l + "talk": (H, H), l + "sink": (H,), l + "o": (W, H * V),
                      l + "out": (W,), r + "out": (W,), r + "y": (C, W), r + "y.b": (C,), r + "x": (C, W), r + "x.b": (C,),
                      r + "conv": (C, self.lru_conv), r + "conv.b": (C,), r + "ra": (NB, C // NB, C // NB), r + "ra.b": (NB, C // NB),
                      r + "ri": (NB, C // NB, C // NB), r + "ri.b": (NB, C // NB), r + "lam": (C,), r + "o": (W, C)})
        elif self.mixer == "window_linear":
            G, HR, DR, VR = self.kv_heads, self.lin_heads, self.lin_dim, self.lin_vdim
            l, r = m + "left.", m + "right."
            for u, n in (("q", H * D), ("k", G * D), ("v", G * V)):
                t.update({l + u: (n, W), l + u + ".b": (n,)})
                if self.conv:
                    t[l + u + ".conv"] = (n, self.conv)
            t.update({l + "q.norm": (H * D,), l + "k.norm": (G * D,), l + "g": (H * V, W), l + "o": (W, H * V), l + "o.b": (W,),
                      r + "q": (HR * DR, W), r + "k": (HR * DR, W), r + "v": (HR * VR, W), r + "g": (HR * VR, W), r + "o": (W, HR * VR),
                      r + "norm": (HR * VR,)})
        elif self.mixer == "channel_delta":
            G = self.kv_heads
            t.update({m + "q": (G * D, W), m + "q.conv": (G * D, self.conv), m + "k": (G * D, W), m + "k.conv": (G * D, self.conv),
                      m + "v": (H * V, W), m + "v.conv": (H * V, self.conv), m + "b": (H, W), m + "A_log": (H,), m + "norm": (V,),
                      m + "a1": (self.decay_rank, W), m + "a2": (H * D, self.decay_rank), m + "dt_bias": (H * D,),
                      m + "g1": (self.gate_rank, W), m + "g2": (H * V, self.gate_rank), m + "o": (W, H * V)})
        elif self.mixer == "gla":
            R = self.decay_rank
            t.update({m + "q": (H * D, W), m + "k": (H * D, W), m + "v": (H * V, W), m + "g": (H * V, W), m + "o": (W, H * V), m + "norm": (V,),
                      m + "a1": (R, W), m + "a2": (H * D, R), m + "a2.b": (H * D,)})
        elif self.mixer == "attention":
            t.update({m + "q": (H * D, W), m + "k": (self.kv_heads * D, W), m + "o": (W, H * D)})
        elif self.mixer == "hgrn2":
            t.update({m + "q": (H * D, W), m + "f": (H * D, W), m + "f.b": (H * D,), m + "lower": (H * D,), m + "v": (H * V, W), m + "norm": (V,),
                      m + "o": (W, H * V)})
        elif self.mixer == "latent_attention":
            R, KR, QR = self.rot_dim, self.kv_rank, self.q_rank
            t.update({m + "dq": (QR, W), m + "dq.norm": (QR,), m + "uq": (H * (D + R), QR), m + "dkv": (KR + R, W), m + "dkv.norm": (KR,),
                      m + "uk": (H * D, KR), m + "uv": (H * V, KR), m + "o": (W, H * V)})
        f = prefix + "mlp."
        if self.ff != "none":
            t.update({prefix + "norm2": (W,), prefix + "norm2b": (W,)})
            if self.mixer == "window_linear":
                del t[prefix + "norm2b"]
        if self.ff == "dense":
            t.update({f + "up": (self.ff_width, W), f + "down": (W, self.ff_width)})
        elif self.ff == "moe":
            for e in range(self.experts):
                t.update({f"{f}e{e}.up": (self.ff_width, W), f"{f}e{e}.down": (W, self.ff_width)})
                if self.expert_act in ("glu_silu", "glu_clipped"):
                    t[f"{f}e{e}.gate"] = (self.ff_width, W)
            t[f + "router"] = (self.experts, W)
            if self.router != "sigmoid_input":
                t[f + ("router.b" if self.router == "top_logits" else "correction")] = (self.experts,)
            if self.shared_width:
                S = self.shared_width
                t.update({f + "shared.gate": (S, W), f + "shared.up": (S, W), f + "shared.down": (W, S)})
                if self.expert_act == "glu_clipped":
                    t[f + "shared.sg"] = (1, W)
        if tanh_norms:  # every norm's bias and scalar beside its weight
            for name in [k for k in t if k[len(prefix):] in ("norm1", "norm1b", "norm2", "norm2b")]:
                t.update({name + ".b": (W,), name + ".alpha": ()})
        return t

    def derived_tensors(self, prefix):
        """{tensor name of the library: values} that the configuration holds instead of the checkpoint."""
        if self.mixer == "window_linear":
            return {prefix + "mix.right.decay": np.asarray(self.decay, np.float32)}
        return {}


@dataclass
class LMConfig:
    vocab: int
    width: int
    layers: List[LayerSpec]
    norm_eps: float = 1e-6
    loop: Optional[dict] = None  # {start, stop, times}
    architecture: str = "Tokosun"
    embed_scale: float = 1.0
    canon_taps: int = 0  # > 0: both sublayers read h + conv(h) over this many tokens; 0: token shift in front of the mixer
    logit_scale: float = 1.0
    logit_softcap: float = 0.0  # > 0: logits <- cap tanh(logits / cap)
    residual_mult: float = 1.0  # designs with tanh norms: factor of a sublayer's normed output in the residual sum
    extra: dict = field(default_factory=dict)

    @classmethod
    def from_json(cls, cfg, shapes=None):
        """cfg: the dict of config.json; shapes: {tensor name: shape} of the checkpoint (for sizes only shapes give)."""
        arch = cfg.get("architecture", "Tokosun")
        if arch not in DESIGNS:
            raise ValueError(f"architecture {arch!r} is not a layered design (known: {sorted(DESIGNS)})")
        entries = cfg["layers"]

        def owner(i):  # the layer whose tensors layer i runs
            seen = set()
            while entries[i].get("weights_of") is not None:
                if i in seen or not 0 <= int(entries[i]["weights_of"]) < len(entries):
                    raise ValueError(f"layer {i}: weights_of {entries[i]['weights_of']!r} names no layer with tensors")
                seen.add(i)
                i = int(entries[i]["weights_of"])
            return i

        layers = [LayerSpec.from_json(e, arch, shapes, f"l{owner(i)}.") for i, e in enumerate(entries)]
        return cls(vocab=int(cfg["vocab"]), width=int(cfg["width"]), layers=layers,
                   norm_eps=float(cfg["norm"]["eps"]), loop=dict(cfg["loop"]) if cfg.get("loop") else None, architecture=arch,
                   embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)), canon_taps=int((cfg.get("canon") or {}).get("taps", 0)),
                   logit_scale=float(cfg.get("logit_scale") or 1.0), logit_softcap=float(cfg.get("logit_softcap") or 0.0),
                   residual_mult=float(cfg.get("residual_mult", 1.0)))

    @classmethod
    def from_dir(cls, path):
        from . import weights_io

        with open(os.path.join(path, "config.json")) as f:
            cfg = json.load(f)
        st = os.path.join(path, "model.safetensors")
        shapes = {k: tuple(a.shape) for k, (_, a) in weights_io.read_safetensors(st).items()} if os.path.exists(st) else None
        return cls.from_json(cfg, shapes)

    def to_json(self):
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "layers": [l.to_json() for l in self.layers], "loop": dict(self.loop) if self.loop else None}
        if self.embed_scale != 1.0:
            out["embedding"] = {"scale": self.embed_scale}
        if self.canon_taps:
            out["canon"] = {"taps": self.canon_taps}
        if self.logit_scale != 1.0:
            out["logit_scale"] = self.logit_scale
        if self.logit_softcap:
            out["logit_softcap"] = self.logit_softcap
        if self.residual_mult != 1.0:
            out["residual_mult"] = self.residual_mult
        if out["loop"] is None and DESIGNS[self.architecture].get("tanh_norms"):
            del out["loop"]
        return out

    @property
    def tied_head(self):
        return DESIGNS[self.architecture]["tied_head"]

    def flags(self):
        d = DESIGNS[self.architecture]
        return ((_lib.LM_TIED_HEAD if d["tied_head"] else 0) | (_lib.LM_LOOP_READD if d["loop_readd"] else 0) |
                (_lib.LM_SIDE_BY_SIDE if d.get("side_by_side") else 0) | (_lib.LM_SINUSOID_POSITIONS if d.get("sinusoid_positions") else 0) |
                (_lib.LM_TANH_NORMS if d.get("tanh_norms") else 0) | (_lib.LM_EMBED_NORM if d.get("embed_norm") else 0))

    def passes(self):
        """Layer index of every pass, in execution order."""
        n = len(self.layers)
        if not self.loop or int(self.loop["times"]) <= 1:
            return list(range(n))
        a, b, k = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        return list(range(a)) + list(range(a, b)) * k + list(range(b, n))

    def tensor_shapes(self):
        t = {"embed": (self.vocab, self.width), "final.norm": (self.width,)}
        d = DESIGNS[self.architecture]
        tanh_norms = bool(d.get("tanh_norms"))
        if tanh_norms:
            t.update({"final.norm.b": (self.width,), "final.norm.alpha": ()})
            if d.get("embed_norm"):
                t.update({"embed.norm": (self.width,), "embed.norm.b": (self.width,), "embed.norm.alpha": ()})
        if not self.tied_head:
            t["head"] = (self.vocab, self.width)
        for i, l in enumerate(self.layers):
            t.update(l.tensor_shapes(f"l{i}.", self.width, self.canon_taps, tanh_norms))
        return t

    def derived_tensors(self):
        """Tensors of the library that the configuration fills (constants listed per head), by name."""
        t = {}
        for i, l in enumerate(self.layers):
            t.update(l.derived_tensors(f"l{i}."))
        return t


class LayeredLM:
    """A handle of the layered-model tier: weights, state slots, the step function and generation."""

    def __init__(self, config: LMConfig, dtype="bfloat16", max_tokens=4096, max_seqs=8, max_step_tokens=0, page_tokens=0, device=0,
                 build_if_missing=False, use_graph=True):
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"dtype {dtype!r}: bfloat16 or float32")
        self.config, self.dtype = config, dtype
        L = self._L = _lib.load_lm(build_if_missing=build_if_missing)
        self._layers = (_lib.LmLayer * len(config.layers))(*[l.to_c() for l in config.layers])
        loop = config.loop or {"start": 0, "stop": 0, "times": 1}
        cfg = _lib.LmConfig(config.vocab, config.width, len(config.layers), self._layers, int(loop["start"]), int(loop["stop"]), int(loop["times"]),
                            config.norm_eps, max_tokens, max_seqs, max_step_tokens, page_tokens,
                            (_lib.LM_F32 if dtype == "float32" else 0) | (0 if use_graph else _lib.LM_NO_GRAPH) | config.flags(),
                            config.embed_scale, config.canon_taps, config.logit_scale, config.logit_softcap, config.residual_mult)
        h = C.c_void_p()
        check(L.zg_lm_create(C.byref(h), C.byref(cfg), device))
        self.h = h
        self._load_derived()
        self.n_passes = len(config.passes())
        self.page_tokens = int(page_tokens) or 64  # (the library's default)

    @classmethod
    def from_dir(cls, path, dtype="bfloat16", **kw):
        """config.json + model.safetensors of a checkpoint folder."""
        from . import weights_io

        m = cls(LMConfig.from_dir(path), dtype=dtype, **kw)
        # tensors the configuration does not name are left alone (a checkpoint may carry tables of other tools); every tensor it
        # does name must be there
        m.load_weights(weights_io.load_safetensors_f32(os.path.join(path, "model.safetensors")), strict=False)
        missing = m.missing_tensors()
        if missing:
            raise KeyError(f"{path}: {len(missing)} tensors missing from the checkpoint: {' '.join(missing[:8])}")
        return m

    def close(self):
        if getattr(self, "h", None):
            self._L.zg_lm_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # ------------------------------------------------------------------ weights
    def load_weights(self, weights, strict=True):
        """weights: dict checkpoint name -> array (fp32 values; matrices [out, in]).  strict: every tensor of the configuration
        must be there, with its shape, and nothing else."""
        shapes = self.config.tensor_shapes()
        for name, a in weights.items():
            if name not in shapes:
                if strict:
                    raise KeyError(f"tensor {name!r} is not part of this configuration")
                continue
            scalar = np.size(a) == 1 and int(np.prod(shapes[name], dtype=np.int64)) == 1  # a scalar may be stored as [] or [1]
            if tuple(np.shape(a)) != tuple(shapes[name]) and not scalar:
                raise ValueError(f"tensor {name!r} has shape {tuple(np.shape(a))}, the configuration needs {tuple(shapes[name])}")
            a = np.ascontiguousarray(a, dtype=np.float32)
            check(self._L.zg_lm_load_tensor(self.h, name.encode(), a.ctypes.data, a.size))
        if strict:
            missing = self.missing_tensors()
            if missing:
                raise KeyError(f"{len(missing)} tensors missing from the checkpoint: {' '.join(missing[:8])}")

    def _load_derived(self):
        for name, a in self.config.derived_tensors().items():
            a = np.ascontiguousarray(a, dtype=np.float32)
            check(self._L.zg_lm_load_tensor(self.h, name.encode(), a.ctypes.data, a.size))

    def missing_tensors(self):
        n, buf = C.c_size_t(), C.create_string_buffer(1 << 16)
        check(self._L.zg_lm_missing_tensors(self.h, C.byref(n), buf, len(buf)))
        return buf.value.decode().split() if n.value else []

    def init_random(self, seed=0, std=0.02):
        check(self._L.zg_lm_init_random(self.h, seed, std))
        self._load_derived()

    # ------------------------------------------------------------------ sequences and steps
    def open(self):
        s = C.c_int()
        check(self._L.zg_lm_seq_open(self.h, C.byref(s)))
        return s.value

    def close_seq(self, seq):
        check(self._L.zg_lm_seq_close(self.h, seq))

    def seq_len(self, seq):
        n = C.c_size_t()
        check(self._L.zg_lm_seq_len(self.h, seq, C.byref(n)))
        return n.value

    def free_tokens(self):
        n = C.c_size_t()
        check(self._L.zg_lm_free_tokens(self.h, C.byref(n)))
        return n.value

    def step(self, entries, trace=False):
        """entries: [(seq, tokens, want)] — the next tokens of every sequence and the places among them whose logits are asked
        for.  Returns the logits [sum of wants, vocab] in entry order then want order (with trace=True also the residual stream
        behind every layer pass, [passes, rows, width])."""
        arr = (_lib.LmEntry * max(1, len(entries)))()
        keep, n_want, rows = [], 0, 0
        for i, (seq, tokens, want) in enumerate(entries):
            t = np.ascontiguousarray(tokens, dtype=np.int32).reshape(-1)
            w = np.ascontiguousarray(want, dtype=np.int32).reshape(-1)
            keep += [t, w]
            arr[i] = _lib.LmEntry(int(seq), t.ctypes.data if t.size else None, t.size, w.ctypes.data if w.size else None, w.size)
            n_want += w.size
            rows += t.size
        logits = np.empty((n_want, self.config.vocab), np.float32)
        tr = None
        if trace:
            tr = np.zeros((self.n_passes, rows, self.config.width), np.float32)
            check(self._L.zg_lm_set_trace(self.h, tr.ctypes.data, tr.size))
        try:
            check(self._L.zg_lm_step(self.h, arr, len(entries), logits.ctypes.data if n_want else None, logits.size))
        finally:
            if trace:
                self._L.zg_lm_set_trace(self.h, None, 0)
        return (logits, tr) if trace else logits

    def generate(self, prompts, n_new, temp=0.0, seed=0):
        """Greedy (temp == 0) or sampled continuation of every prompt; returns tokens [len(prompts), n_new]."""
        prompts = [np.ascontiguousarray(p, dtype=np.int32).reshape(-1) for p in prompts]
        stride = max(len(p) for p in prompts)
        mat = np.zeros((len(prompts), stride), np.int32)
        lens = np.zeros(len(prompts), np.uint64)
        for b, p in enumerate(prompts):
            mat[b, : len(p)] = p
            lens[b] = len(p)
        out = np.zeros((len(prompts), n_new), np.int32)
        check(self._L.zg_lm_generate(self.h, mat.ctypes.data, stride, lens.ctypes.data, len(prompts), n_new, float(temp), int(seed), out.ctypes.data,
                                     out.size))
        return out

    def last_ms(self):
        """(device ms of the last step, mean device ms per decode step of the last generate)."""
        a, b = C.c_float(), C.c_float()
        check(self._L.zg_lm_last_ms(self.h, C.byref(a), C.byref(b)))
        return a.value, b.value

    def last_kernel(self):
        buf = C.create_string_buffer(160)
        self._L.zg_debug_last_kernel(buf, len(buf))
        return buf.value.decode()


class Scheduler:
    """Continuous batching over one LayeredLM.  Requests wait in a queue and are admitted while a state slot and enough cache
    pages for their whole life (prompt + new tokens) are free; every iteration is ONE ragged step of the library: the next
    portion (at most `portion` tokens) of every prompt that is still being fed, beside the single last token of every sequence
    that is decoding.  A finished request gives its slot and pages back at once, and the next one in the queue takes them.
    Token choice: greedy (temp == 0, first maximum) or softmax(logits / temp) sampling from a generator seeded per request."""

    def __init__(self, model: LayeredLM, portion=256, temp=0.0, seed=0):
        self.model, self.portion, self.temp, self.seed, self.page = model, int(portion), float(temp), int(seed), model.page_tokens
        self.queue, self.active, self.done, self._next_id, self._reserved = [], [], {}, 0, 0
        self.steps = 0

    def submit(self, prompt, n_new):
        rid = self._next_id
        self._next_id += 1
        prompt = np.ascontiguousarray(prompt, dtype=np.int32).reshape(-1)
        if prompt.size < 1 or n_new < 1:
            raise ValueError("a request needs a prompt and at least one new token")
        self.queue.append({"id": rid, "prompt": prompt, "n_new": int(n_new), "fed": 0, "out": [], "seq": None,
                           "rng": np.random.default_rng([self.seed, rid])})
        return rid

    def _pages(self, r):
        return -(-(r["prompt"].size + r["n_new"]) // self.page) * self.page

    def _admit(self):
        while self.queue:
            r = self.queue[0]
            if self.model.free_tokens() - self._reserved < self._pages(r):
                break
            try:
                r["seq"] = self.model.open()
            except _lib.ZgError:
                break  # no slot
            self._reserved += self._pages(r)
            self.active.append(self.queue.pop(0))

    def _choose(self, r, logits):
        if self.temp <= 0.0:
            return int(np.argmax(logits))
        z = logits.astype(np.float64) / self.temp
        p = np.exp(z - z.max())
        return int(r["rng"].choice(p.size, p=p / p.sum()))

    def run(self):
        """Serve every submitted request; returns {request id: new tokens}."""
        while self.queue or self.active:
            self._admit()
            if not self.active:
                raise RuntimeError("a request does not fit the cache even when it is alone")
            entries, asked = [], []
            for r in self.active:
                n = r["prompt"].size
                if r["fed"] < n:  # still feeding the prompt
                    hi = min(n, r["fed"] + self.portion)
                    last = hi == n
                    entries.append((r["seq"], r["prompt"][r["fed"]:hi], [hi - r["fed"] - 1] if last else []))
                    r["fed"] = hi
                    if last:
                        asked.append(r)
                else:
                    entries.append((r["seq"], [r["out"][-1]], [0]))
                    asked.append(r)
            before = {r["seq"]: self.model.seq_len(r["seq"]) for r in self.active}
            logits = self.model.step(entries)
            for r in self.active:  # pages the step took are no longer merely promised (a windowed model may have given others back)
                self._reserved -= (-(-self.model.seq_len(r["seq"]) // self.page) - -(-before[r["seq"]] // self.page)) * self.page
            self.steps += 1
            for r, row in zip(asked, logits):
                r["out"].append(self._choose(r, row))
            for r in [r for r in self.active if len(r["out"]) >= r["n_new"]]:
                held = -(-self.model.seq_len(r["seq"]) // self.page) * self.page
                self._reserved -= self._pages(r) - held  # what was promised and never taken
                self.model.close_seq(r["seq"])
                self.active.remove(r)
                self.done[r["id"]] = np.array(r["out"][: r["n_new"]], np.int32)
        return self.done
