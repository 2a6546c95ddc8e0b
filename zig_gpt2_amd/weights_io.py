"""Raw weight directory format of the reference: one little-endian fp32 file per
tensor under `<dir>/`, named `model-<tf variable with '/' -> '-'>` (download_weights.py:57-64),
`*/w` matrices already transposed to [out, in] (download_weights.py:60-61) — exactly what
load_linear / load_layer_norm / load_embedding of src/main.zig:210-269 read with hard-coded
`models/124M/raw/` paths.  Here the directory and the config are arguments.

  model-wte, model-wpe, model-ln_f-{g,b},
  model-h{i}-ln_1-{g,b}, model-h{i}-attn-c_attn-{w,b}, model-h{i}-attn-c_proj-{w,b},
  model-h{i}-ln_2-{g,b}, model-h{i}-mlp-c_fc-{w,b}, model-h{i}-mlp-c_proj-{w,b}
"""
import os

import numpy as np

from .synth import GPTConfig, tensor_specs

# our tensor name -> reference file stem
_BLOCK_FILES = {
    "ln_1_g": "ln_1-g", "ln_1_b": "ln_1-b", "c_attn_w": "attn-c_attn-w", "c_attn_b": "attn-c_attn-b",
    "c_proj_w": "attn-c_proj-w", "c_proj_b": "attn-c_proj-b", "ln_2_g": "ln_2-g", "ln_2_b": "ln_2-b",
    "c_fc_w": "mlp-c_fc-w", "c_fc_b": "mlp-c_fc-b", "mlp_proj_w": "mlp-c_proj-w", "mlp_proj_b": "mlp-c_proj-b",
}
_TOP_FILES = {"wte": "wte", "wpe": "wpe", "ln_f_g": "ln_f-g", "ln_f_b": "ln_f-b"}


def file_name(tensor_name):
    if "." in tensor_name:
        layer, slot = tensor_name.split(".")
        return f"model-{layer}-{_BLOCK_FILES[slot]}"
    return f"model-{_TOP_FILES[tensor_name]}"


def load_raw_dir(path, cfg: GPTConfig):
    """Read every tensor of `cfg` from a reference-format directory.  Unlike the reference's
    load_tensor (src/ops.zig:318, short reads silently ignored) a size mismatch is an error."""
    out = {}
    for name, shape, _, _ in tensor_specs(cfg):
        f = os.path.join(path, file_name(name))
        a = np.fromfile(f, dtype="<f4")
        want = int(np.prod(shape))
        if a.size != want:
            raise ValueError(f"{f}: {a.size} floats on disk, config needs {want} for {name}{tuple(shape)}")
        out[name] = np.ascontiguousarray(a.reshape(shape))
    return out


def save_raw_dir(path, cfg: GPTConfig, weights):
    os.makedirs(path, exist_ok=True)
    for name, shape, _, _ in tensor_specs(cfg):
        np.ascontiguousarray(weights[name], dtype="<f4").reshape(-1).tofile(os.path.join(path, file_name(name)))


def bf16_representable(a):
    """True when rounding `a` to bf16 changes nothing (its low 16 mantissa bits are zero)."""
    b = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    return not bool(np.any(b & np.uint32(0xFFFF)))


def flags_for_checkpoint(weights):
    """How a handle should store the matrices of THIS checkpoint: bf16 storage is lossless only for bf16-representable
    weights (the synthetic ones); on an ordinary fp32 checkpoint it moves the logits by about 1e-2 of their scale
    (tests/test_weight_storage_gpu.py), outside north_star's 1e-3 — such a checkpoint gets ZG_GPT_WEIGHTS_F32, the reference's
    own precision (src/main.zig:210-269 keeps fp32).  Returns keyword arguments for gpt.GPT."""
    mats = [v for k, v in weights.items() if np.ndim(v) == 2]
    return {"weights_f32": not all(bf16_representable(m) for m in mats)}


# ------------------------------------------------------------------------------------------------
# safetensors checkpoints (the layered models of lm.py): an 8-byte little-endian header length, that many bytes of JSON
# (tensor name -> dtype, shape, data_offsets relative to the end of the header), then the raw little-endian data.
# Read with numpy alone; nothing in the file is executed.
# ------------------------------------------------------------------------------------------------
_ST_DTYPES = {"F32": ("<f4", 4), "F16": ("<f2", 2), "BF16": ("<u2", 2), "I32": ("<i4", 4), "I64": ("<i8", 8), "F64": ("<f8", 8),
              "U8": ("u1", 1), "I8": ("i1", 1), "U16": ("<u2", 2), "I16": ("<i2", 2), "U32": ("<u4", 4), "BOOL": ("u1", 1)}


def read_safetensors(path):
    """dict name -> (dtype string of the file, numpy array).  BF16 tensors come back as their uint16 bit patterns (numpy has
    no bfloat16); everything else in its own type.  The arrays are views of one memory map of the file."""
    import json
    import struct

    with open(path, "rb") as f:
        head = f.read(8)
        if len(head) != 8:
            raise ValueError(f"{path}: too short for a safetensors header")
        (n,) = struct.unpack("<Q", head)
        size = os.path.getsize(path)
        if n > size - 8:
            raise ValueError(f"{path}: header length {n} exceeds the file")
        meta = json.loads(f.read(n).decode("utf-8"))
    data = np.memmap(path, dtype=np.uint8, mode="r", offset=8 + n) if size > 8 + n else np.zeros(0, np.uint8)
    out = {}
    for name, info in meta.items():
        if name == "__metadata__":
            continue
        if info["dtype"] not in _ST_DTYPES:
            raise ValueError(f"{path}: tensor {name} has unsupported dtype {info['dtype']}")
        dt, width = _ST_DTYPES[info["dtype"]]
        lo, hi = info["data_offsets"]
        count = int(np.prod(info["shape"], dtype=np.int64)) if info["shape"] else 1
        if hi - lo != count * width or hi > data.size:
            raise ValueError(f"{path}: tensor {name}: {hi - lo} bytes on disk, shape {info['shape']} needs {count * width}")
        out[name] = (info["dtype"], np.frombuffer(data, dtype=dt, count=count, offset=lo).reshape(info["shape"]))
    return out


def bf16_bits_to_f32(bits):
    """uint16 bf16 bit patterns -> fp32 values (exact)."""
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32).reshape(np.shape(bits))


def load_safetensors_f32(path):
    """dict name -> fp32 array (integer tables stay integer): the form the model classes' load_weights take."""
    out = {}
    for name, (dt, a) in read_safetensors(path).items():
        if dt == "BF16":
            out[name] = bf16_bits_to_f32(a)
        elif dt in ("F16", "F64", "F32"):
            out[name] = np.ascontiguousarray(a, dtype=np.float32)
        else:
            out[name] = np.ascontiguousarray(a)
    return out


def write_safetensors(path, tensors, bf16=True):
    """Write fp32 arrays as BF16 (rounded to nearest even; bf16=False: F32) and integer arrays as I32 — the inverse of
    load_safetensors_f32 for the layered models' checkpoints."""
    import json
    import struct

    from .synth import to_bf16_bits

    meta, blobs, off = {}, [], 0
    for name, a in tensors.items():
        a = np.asarray(a)
        if np.issubdtype(a.dtype, np.integer):
            dt, raw = "I32", np.ascontiguousarray(a, dtype="<i4").tobytes()
        elif bf16:
            dt, raw = "BF16", to_bf16_bits(np.ascontiguousarray(a, dtype=np.float32)).astype("<u2").tobytes()
        else:
            dt, raw = "F32", np.ascontiguousarray(a, dtype="<f4").tobytes()
        meta[name] = {"dtype": dt, "shape": list(a.shape), "data_offsets": [off, off + len(raw)]}
        blobs.append(raw)
        off += len(raw)
    head = json.dumps(meta, separators=(",", ":")).encode("utf-8")
    head += b" " * (-len(head) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(head)))
        f.write(head)
        for b in blobs:
            f.write(b)
