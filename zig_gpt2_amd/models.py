"""Model registry: which class serves which checkpoint architecture.

A checkpoint folder is recognised by its files: `config.json` with an "architecture" names a family of lm.py (layer lists
served by the layered-model tier); a reference-format raw weight directory (`model-wte`, ... — weights_io.py) is GPT-2 and needs
its GPTConfig named, since that format carries no configuration.
"""
import json
import os

from . import synth

# architecture name of config.json -> loader(path, dtype, **serving options)
ARCHITECTURES = {}


def register(name):
    def deco(fn):
        ARCHITECTURES[name] = fn
        return fn

    return deco


@register("Tokosun")
def _load_tokosun(path, dtype="bfloat16", **kw):
    from . import lm

    return lm.LayeredLM.from_dir(path, dtype=dtype, **kw)


@register("Gupizen")
def _load_gupizen(path, dtype="bfloat16", **kw):
    from . import lm

    return lm.LayeredLM.from_dir(path, dtype=dtype, **kw)


@register("Sanazen")
def _load_sanazen(path, dtype="bfloat16", **kw):
    from . import lm

    return lm.LayeredLM.from_dir(path, dtype=dtype, **kw)


@register("Vovalorn")
def _load_vovalorn(path, dtype="bfloat16", **kw):
    from . import lm

    return lm.LayeredLM.from_dir(path, dtype=dtype, **kw)


@register("gpt2")
def _load_gpt2(path, dtype="float32", config="124M", **kw):
    from . import gpt

    cfg = synth.CONFIGS[config] if isinstance(config, str) else config
    return gpt.GPT.from_raw_dir(path, cfg, **kw)


def architecture_of(path):
    """Name of the architecture a checkpoint folder holds."""
    cj = os.path.join(path, "config.json")
    if os.path.exists(cj):
        with open(cj) as f:
            cfg = json.load(f)
        name = cfg.get("architecture")
        if name not in ARCHITECTURES:
            raise ValueError(f"{cj}: architecture {name!r} is not served (known: {sorted(ARCHITECTURES)})")
        return name
    if os.path.exists(os.path.join(path, "model-wte")):
        return "gpt2"
    raise ValueError(f"{path}: neither config.json nor a raw GPT-2 weight directory")


def load_model(path, dtype="bfloat16", **kw):
    """The model of a checkpoint folder, weights loaded, on the class its architecture is registered with."""
    return ARCHITECTURES[architecture_of(path)](path, dtype=dtype, **kw)
