"""Small random Sanazen configurations and weights for the tests (bf16-representable values, so that the float64 oracle and the
bf16-storage device path see the same numbers)."""
import numpy as np

from zig_gpt2_amd.synth import round_bf16


def pair_layer(heads=4, kv_heads=2, dim=12, vdim=8, window=9, keep_first=3, scale=0.3, conv=3, lin_heads=3, lin_dim=8, lin_vdim=10, decay=None,
               left_scale=0.7, right_scale=1.2, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if conv:
        left["conv"] = conv
    if window:
        left["mask"] = {"size": window, "keep_first": keep_first}
    if decay is None:
        decay = [float(np.exp(-1.0 / (1.5 + 4.0 * i))) for i in range(lin_heads)]
    right = {"heads": lin_heads, "dim": lin_dim, "vdim": lin_vdim, "decay": list(decay)}
    return {"type": "parallel", "mixer": {"left": left, "left_scale": left_scale, "right": right, "right_scale": right_scale}, "mlp": mlp}


def moe_mlp(ff=24, experts=5, top=2, limit=1.5, shared=(20, 0.8)):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top},
            "shared": {"ff": shared[0], "limit": shared[1]} if shared else None}


def config(layers, vocab=97, width=48, eps=1e-5, embed_scale=3.0, logit_scale=0.6, softcap=12.0):
    cfg = {"architecture": "Sanazen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers, "embedding": {"scale": embed_scale}}
    if logit_scale is not None:
        cfg["logit_scale"] = logit_scale
    if softcap:
        cfg["logit_softcap"] = softcap
    return cfg


def weights(cfg, seed=0, embed_std=1.0, head_std=None):
    """Random tensors for every name of the configuration.  Matrices ~ N(0, 1 / fan_in); norm weights around one."""
    from zig_gpt2_amd import lm

    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in lm.LMConfig.from_json(cfg).tensor_shapes().items():
        leaf = name.split(".")[-1]
        if name == "embed":
            a = rng.normal(0.0, embed_std, shape)
        elif name == "head" and head_std is not None:
            a = rng.normal(0.0, head_std, shape)
        elif leaf == "conv":
            a = rng.normal(0.0, 0.5, shape)
        elif leaf == "b":
            a = rng.normal(0.0, 0.4, shape)
        elif len(shape) == 2:
            a = rng.normal(0.0, 1.0 / np.sqrt(shape[1]), shape)
        else:  # plain norm weights
            a = 1.0 + rng.normal(0.0, 0.1, shape)
        out[name] = round_bf16(a.astype(np.float32)).reshape(shape)
    return out


def tokens(seed, n, vocab):
    return np.random.default_rng(3000 + seed).integers(0, vocab, n).astype(np.int32)
