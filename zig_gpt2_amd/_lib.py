"""ctypes binding of libzgpt2_hip.so (the C ABI of include/zgpt2.h).

There is no fallback: if the HIP library is missing, load() raises.  build() compiles it in-tree
with hipcc for gfx950 (zig_gpt2_amd/csrc/Makefile), so the .so travels with the repo snapshot.
"""
import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
SO_PATH = os.environ.get("ZGPT2_LIB") or os.path.join(_HERE, "lib", "libzgpt2_hip.so")  # ZGPT2_LIB: diagnostic builds
HEADER = os.path.join(os.path.dirname(_HERE), "include", "zgpt2.h")

LM_SO_PATH = os.path.join(_HERE, "lib", "libzgpt2_lm.so")  # the layered-model tier alone (make lm)

_lib = None
_lm_lib = None

f32p = C.POINTER(C.c_float)
szp = C.POINTER(C.c_size_t)
vp = C.c_void_p
sz = C.c_size_t


class ZgError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__(f"libzgpt2_hip error {code}: {msg}")
        self.code = code


class GptConfig(C.Structure):
    """zg_gpt_config == GPTConfig of src/main.zig:5-23."""

    _fields_ = [("vocab_size", sz), ("context_size", sz), ("n_layer", sz), ("n_heads", sz), ("n_embed", sz)]


class GptOptions(C.Structure):
    """zg_gpt_options of include/zgpt2.h."""

    _fields_ = [("share_weights_with", vp), ("own_stream", C.c_int), ("stream_priority", C.c_int)]


class LmLayer(C.Structure):
    """zg_lm_layer of include/zgpt2.h."""

    _fields_ = [("mixer", C.c_int), ("heads", C.c_int), ("dim", C.c_int), ("vdim", C.c_int), ("rot_dim", C.c_int), ("kv_rank", C.c_int),
                ("q_rank", C.c_int), ("scale", C.c_float), ("rot_dims", C.c_int), ("rot_base", C.c_float), ("rot_scaled", C.c_int),
                ("rot_factor", C.c_float), ("rot_original", C.c_float), ("rot_fast", C.c_float), ("rot_slow", C.c_float), ("ff", C.c_int),
                ("ff_width", C.c_int), ("experts", C.c_int), ("top", C.c_int), ("kv_heads", C.c_int), ("window", C.c_int), ("lru_width", C.c_int),
                ("lru_blocks", C.c_int), ("lru_conv", C.c_int), ("conv", C.c_int), ("decay_rank", C.c_int), ("gate_rank", C.c_int),
                ("ff_act", C.c_int), ("router", C.c_int), ("keep_first", C.c_int), ("left_scale", C.c_float), ("right_scale", C.c_float),
                ("lin_heads", C.c_int), ("lin_dim", C.c_int), ("lin_vdim", C.c_int), ("ff_limit", C.c_float), ("shared_width", C.c_int),
                ("shared_limit", C.c_float), ("tau", C.c_float), ("softcap", C.c_float), ("qtemp_coef", C.c_float), ("qtemp_every", C.c_int),
                ("dist_bias", C.c_int), ("route_groups", C.c_int), ("route_keep", C.c_int), ("route_scale", C.c_float), ("weights_of", C.c_int)]


class LmConfig(C.Structure):
    """zg_lm_config of include/zgpt2.h."""

    _fields_ = [("vocab", sz), ("width", sz), ("n_layers", sz), ("layers", C.POINTER(LmLayer)), ("loop_start", C.c_int), ("loop_stop", C.c_int),
                ("loop_times", C.c_int), ("norm_eps", C.c_float), ("max_tokens", sz), ("max_seqs", sz), ("max_step_tokens", sz),
                ("page_tokens", sz), ("flags", C.c_uint), ("embed_scale", C.c_float), ("canon_taps", C.c_int), ("logit_scale", C.c_float),
                ("logit_softcap", C.c_float), ("residual_mult", C.c_float)]


class LmEntry(C.Structure):
    """zg_lm_entry of include/zgpt2.h."""

    _fields_ = [("seq", C.c_int), ("tokens", vp), ("n_tokens", sz), ("want", vp), ("n_want", sz)]


LM_MIX_HGRN2, LM_MIX_LATENT_ATTENTION, LM_MIX_PARALLEL, LM_MIX_CHANNEL_DELTA, LM_MIX_WINDOW_LINEAR = 1, 2, 3, 4, 5
LM_MIX_GLA, LM_MIX_ATTENTION = 6, 7
LM_FF_NONE, LM_FF_DENSE, LM_FF_MOE = 0, 1, 2
LM_ACT_GLU_SILU, LM_ACT_GELU, LM_ACT_GLU_CLIPPED = 0, 1, 2
LM_ROUTE_SOFTMAX_ALL, LM_ROUTE_TOP_LOGITS, LM_ROUTE_SIGMOID_INPUT = 0, 1, 2
LM_ROUTE_SIGMOID_GROUPS = 3
LM_ROT_PLAIN, LM_ROT_YARN, LM_ROT_BANDS = 0, 1, 2
LM_F32, LM_NO_GRAPH, LM_TIED_HEAD, LM_LOOP_READD, LM_SIDE_BY_SIDE, LM_SINUSOID_POSITIONS = 1, 2, 4, 8, 16, 32
LM_TANH_NORMS, LM_EMBED_NORM = 64, 128

# the layered-model tier (present in both libraries)
LM_SIGNATURES = {
    "zg_last_error": (C.c_char_p, []),
    "zg_debug_last_kernel": (C.c_int, [C.c_char_p, sz]),
    "zg_lm_create": (C.c_int, [C.POINTER(vp), C.POINTER(LmConfig), C.c_int]),
    "zg_lm_destroy": (C.c_int, [vp]),
    "zg_lm_load_tensor": (C.c_int, [vp, C.c_char_p, vp, sz]),
    "zg_lm_missing_tensors": (C.c_int, [vp, szp, C.c_char_p, sz]),
    "zg_lm_init_random": (C.c_int, [vp, C.c_uint64, C.c_float]),
    "zg_lm_seq_open": (C.c_int, [vp, C.POINTER(C.c_int)]),
    "zg_lm_seq_close": (C.c_int, [vp, C.c_int]),
    "zg_lm_seq_len": (C.c_int, [vp, C.c_int, szp]),
    "zg_lm_free_tokens": (C.c_int, [vp, szp]),
    "zg_lm_step": (C.c_int, [vp, C.POINTER(LmEntry), sz, vp, sz]),
    "zg_lm_generate": (C.c_int, [vp, vp, sz, vp, sz, sz, C.c_float, C.c_uint64, vp, sz]),
    "zg_lm_set_trace": (C.c_int, [vp, vp, sz]),
    "zg_lm_last_ms": (C.c_int, [vp, f32p, f32p]),
}

# name -> (restype, argtypes); every symbol include/zgpt2.h declares
SIGNATURES = {
    "zg_init": (C.c_int, [C.c_int]),
    "zg_init_ex": (C.c_int, [C.c_int, sz]),
    "zg_shutdown": (C.c_int, []),
    "zg_last_error": (C.c_char_p, []),
    "zg_set_stream": (C.c_int, [vp]),
    "zg_synchronize": (C.c_int, []),
    "zg_register_tensor": (C.c_int, [vp, sz]),
    "zg_unregister_tensor": (C.c_int, [vp]),
    "zg_unregister_all": (C.c_int, []),
    "zg_debug_gemm_launches": (C.c_ulonglong, []),
    "zg_debug_gemm_stamps": (C.c_int, [vp, sz]),
    "zg_debug_last_kernel": (C.c_int, [C.c_char_p, sz]),
    "zg_debug_attn_prefill": (C.c_int, [vp, vp, sz, sz, sz, sz, vp, vp, sz, vp, sz, C.c_int]),
    "zg_debug_prefill_route": (C.c_int, [C.c_int, C.c_int]),
    "zg_debug_prefill_linear": (C.c_int, [vp, vp, vp, vp, sz, sz, sz, C.c_int, C.c_int, C.c_int, vp, sz]),
    "zg_linear_forward": (C.c_int, [sz, sz, vp, vp, vp, sz, vp, sz]),
    "zg_embedding_forward": (C.c_int, [sz, vp, sz, vp, sz, vp, sz]),
    "zg_layernorm_forward": (C.c_int, [sz, vp, vp, C.c_float, vp, sz]),
    "zg_attn_forward": (C.c_int, [sz, sz, vp, vp, vp, vp, sz, vp, sz] + [vp, sz] * 8),
    "zg_split_qkv": (C.c_int, [sz, sz, vp, sz, sz, vp, sz]),
    "zg_transpose": (C.c_int, [sz, sz, sz, vp, sz, vp, sz]),
    "zg_scaled_dot_product_attention": (C.c_int, [vp, sz, vp, sz, vp, sz, sz, sz, sz, vp, sz, vp, sz]),
    "zg_gemm_bf16_nt": (C.c_int, [vp, vp, vp, vp, sz, sz, sz, C.c_int, C.c_int]),
    "zg_f32_to_bf16": (C.c_int, [vp, vp, sz]),
    "zg_gelu": (C.c_int, [vp, sz]),
    "zg_softmax": (C.c_int, [vp, sz]),
    "zg_gpt_create": (C.c_int, [C.POINTER(vp), C.POINTER(GptConfig), sz, C.c_uint]),
    "zg_gpt_destroy": (C.c_int, [vp]),
    "zg_gpt_create_ex": (C.c_int, [C.POINTER(vp), C.POINTER(GptConfig), sz, C.c_uint, vp]),
    "zg_gpt_stream": (C.c_int, [vp, C.POINTER(vp)]),
    "zg_gpt_generate_enqueue_many": (C.c_int, [vp, sz, vp, sz, vp, sz]),
    "zg_gpt_generate_fetch_many": (C.c_int, [vp, sz, sz, vp, sz]),
    "zg_gpt_load_block_tensor": (C.c_int, [vp, sz, C.c_int, vp, sz]),
    "zg_gpt_load_tensor": (C.c_int, [vp, C.c_int, vp, sz]),
    "zg_gpt_weight_arena": (C.c_int, [vp, C.POINTER(vp), szp]),
    "zg_dist_available": (C.c_int, []),
    "zg_dist_unique_id": (C.c_int, [vp, sz]),
    "zg_dist_init": (C.c_int, [vp, sz, C.c_int, C.c_int]),
    "zg_dist_world": (C.c_int, [C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "zg_gpt_broadcast_weights": (C.c_int, [vp, C.c_int, f32p]),
    "zg_dist_allgather": (C.c_int, [vp, vp, sz]),
    "zg_dist_finalize": (C.c_int, []),
    "zg_gpt_step_bytes": (C.c_int, [vp, sz, szp, szp]),
    "zg_gpt_forward": (C.c_int, [vp, sz, vp, sz, C.c_int, vp, sz]),
    "zg_gpt_prefill": (C.c_int, [vp, vp, sz, sz, C.c_int, vp, sz]),
    "zg_gpt_argmax": (C.c_int, [vp, vp, sz]),
    "zg_gpt_sample": (C.c_int, [vp, sz, vp, sz, C.c_float, vp, C.c_uint64, vp, vp, sz]),
    "zg_gpt_hidden": (C.c_int, [vp, vp, sz]),
    "zg_gpt_generate_greedy": (C.c_int, [vp, vp, sz, vp, sz, vp, sz]),
    "zg_gpt_generate_enqueue": (C.c_int, [vp, vp, sz, vp, sz]),
    "zg_gpt_generate_fetch": (C.c_int, [vp, sz, vp, sz]),
    "zg_gpt_generate_sample_enqueue": (C.c_int, [vp, vp, sz, vp, sz, C.c_float, C.c_uint64]),
    "zg_gpt_generate_sample": (C.c_int, [vp, vp, sz, vp, sz, C.c_float, C.c_uint64, vp, sz]),
    "zg_gpt_time_kernel": (C.c_int, [vp, C.c_int, C.c_int, f32p, szp]),
    "zg_gpt_profile_step": (C.c_int, [vp, sz, C.c_int, f32p, sz]),
    "zg_debug_prefetch_stats": (C.c_int, [vp, vp, sz]),
    "zg_bpe_create": (C.c_int, [C.POINTER(vp), vp, vp, sz, vp, vp, sz]),
    "zg_bpe_destroy": (C.c_int, [vp]),
    "zg_bpe_encode": (C.c_int, [vp, C.c_char_p, sz, vp, sz, szp]),
    "zg_bpe_decode": (C.c_int, [vp, vp, sz, vp, sz, szp]),
}
SIGNATURES.update(LM_SIGNATURES)

# flags / slots of include/zgpt2.h
GPT_WEIGHTS_BF16, GPT_WEIGHTS_F32, GPT_NO_GRAPH, GPT_KV_F16, GPT_NO_PREFILL, GPT_PREFILL_2PLANE, GPT_NO_PREFETCH = 0, 1, 2, 4, 8, 16, 32
GPT_KV_B24 = 64
GPT_SAMPLED_GENERATE = 128
BLOCK_SLOTS = ["ln_1_g", "ln_1_b", "c_attn_w", "c_attn_b", "c_proj_w", "c_proj_b",
               "ln_2_g", "ln_2_b", "c_fc_w", "c_fc_b", "mlp_proj_w", "mlp_proj_b"]
TOP_SLOTS = ["wte", "wpe", "ln_f_g", "ln_f_b"]
TIME_LM_HEAD = 6


def build(force=False):
    """hipcc --offload-arch=gfx950 build of every HIP source into lib/libzgpt2_hip.so."""
    args = ["make", "-C", CSRC, "-j8"]
    if force:
        args.append("-B")
    subprocess.check_call(args, stdout=subprocess.DEVNULL)
    if not os.path.exists(SO_PATH):
        raise RuntimeError(f"build did not produce {SO_PATH}")
    return SO_PATH


def load():
    """Load the HIP library; raises if it is not built (no CPU fallback exists)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(SO_PATH):
        raise RuntimeError(
            f"{SO_PATH} is missing: the HIP extension is required (run `python -c 'import __graft_entry__ as g; g.build()'`)"
        )
    # One HIP runtime per process: PyTorch-ROCm bundles its own libamdhip64 (SONAME libamdhip64.so.7,
    # requested by torch as "libamdhip64.so").  If this library pulled in /opt/rocm's copy first, a
    # later `import torch` would load a second runtime that finds no GPU.  Importing torch first makes
    # the dynamic linker resolve our DT_NEEDED libamdhip64.so.7 to the copy torch already loaded.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(SO_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def build_lm():
    """hipcc build of the layered-model tier alone into lib/libzgpt2_lm.so (`make lm`: a handful of files)."""
    subprocess.check_call(["make", "-C", CSRC, "-j16", "lm"], stdout=subprocess.DEVNULL)
    if not os.path.exists(LM_SO_PATH):
        raise RuntimeError(f"build did not produce {LM_SO_PATH}")
    return LM_SO_PATH


def load_lm(build_if_missing=False):
    """The library that holds the layered-model tier (zg_lm_*): the full library when it is built, else the tier's own small
    library; with build_if_missing a fresh checkout compiles the latter (and only that) first.  No CPU fallback."""
    global _lm_lib
    if _lm_lib is not None:
        return _lm_lib
    if _lib is not None or os.path.exists(SO_PATH):
        _lm_lib = load()
        return _lm_lib
    if not os.path.exists(LM_SO_PATH):
        if not build_if_missing:
            raise RuntimeError(f"{LM_SO_PATH} is missing: build it with `make -C {CSRC} lm` (or the whole library)")
        build_lm()
    try:
        import torch  # noqa: F401  (one HIP runtime per process: see load())
    except ImportError:
        pass
    lib = C.CDLL(LM_SO_PATH)
    for name, (res, args) in LM_SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lm_lib = lib
    return lib


def check(code):
    if code != 0:
        raise ZgError(code, load().zg_last_error().decode(errors="replace"))


def check_lm(code):
    if code != 0:
        raise ZgError(code, load_lm().zg_last_error().decode(errors="replace"))


def ptr(a):
    """Raw address of a numpy array (host) or torch tensor (host or device); None -> NULL."""
    if a is None:
        return None
    if hasattr(a, "data_ptr"):
        return a.data_ptr()
    return a.ctypes.data
