"""Small random Vovalorn configurations and weights for the tests (bf16-representable values, so that the float64 oracle and the
bf16-storage device path see the same numbers)."""
import numpy as np

from zig_gpt2_amd.synth import round_bf16  # noqa: F401  (also for the tests that build weights by hand)


def gla_layer(heads=3, dim=12, vdim=10, tau=4.0, decay_rank=6, mlp=None, weights_of=None):
    e = {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "decay_rank": decay_rank}, "mlp": mlp}
    if weights_of is not None:
        e["weights_of"] = weights_of
    return e


def attn_layer(heads=4, kv_heads=2, dim=12, scale=0.3, softcap=8.0, q_temp=(0.4, 5), mlp=None, weights_of=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if softcap:
        m["softcap"] = softcap
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    e = {"type": "attention", "mixer": m, "mlp": mlp}
    if weights_of is not None:
        e["weights_of"] = weights_of
    return e


def moe_mlp(ff=20, experts=6, top=2, groups=(3, 2), scale=1.7, shared=14):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": r, "shared": {"ff": shared} if shared else None}


def config(layers, vocab=89, width=40, eps=1e-5, residual_mult=0.45):
    return {"architecture": "Vovalorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": residual_mult, "layers": layers}


def weights(cfg, seed=0, embed_std=1.0, decay_bias=(1.0, 1.5), correction_std=0.1):
    """Random tensors for every name of the configuration.  Matrices ~ N(0, 1 / fan_in); norm weights around one, their biases
    around zero, their scalars in (0.4, 1.2); the bias of the decay's logit ~ N(decay_bias)."""
    from zig_gpt2_amd import lm

    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in lm.LMConfig.from_json(cfg).tensor_shapes().items():
        leaf = name.split(".")[-1]
        if name == "embed":
            a = rng.normal(0.0, embed_std, shape)
        elif leaf == "alpha":
            a = rng.uniform(0.4, 1.2, shape)
        elif name.endswith("a2.b"):
            a = rng.normal(decay_bias[0], decay_bias[1], shape)
        elif leaf == "b":
            a = rng.normal(0.0, 0.1, shape)
        elif leaf == "correction":
            a = rng.normal(0.0, correction_std, shape)
        elif len(shape) == 2:
            a = rng.normal(0.0, 1.0 / np.sqrt(shape[1]), shape)
        else:  # norm weights
            a = 1.0 + rng.normal(0.0, 0.1, shape)
        out[name] = round_bf16(np.asarray(a, np.float32)).reshape(shape)
    return out


def tokens(seed, n, vocab):
    return np.random.default_rng(4000 + seed).integers(0, vocab, n).astype(np.int32)
