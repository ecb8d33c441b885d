"""ctypes binding of include/dashinfer_hip_seq.h: the operators of the ragged-batch sequence engine.

The library is small (two translation units); when it is missing it is built on the spot with `make seq`, so that a fresh
checkout serves a model of the sequence engine without building the quantised-decode library first.  There is no fallback
path: a build that fails raises.
"""
import ctypes as C
import os
import subprocess

from . import PKG_DIR

SEQ_LIB_PATH = os.path.join(os.environ.get("DIHIP_LIB_DIR") or os.path.join(PKG_DIR, "lib"), "libdashinfer_hip_seq.so")
F32, BF16 = 0, 2
MATH_F32, MATH_BF16, MATH_F32_STREAM = 0, 1, 2
ACT = {None: 0, "none": 0, "tanh": 1, "gelu_erf": 2, "gelu_tanh": 3, "relu": 4, "silu": 5, "sigmoid": 6}

vp, sz, i32, f32, lng = C.c_void_p, C.c_size_t, C.c_int, C.c_float, C.c_long

_SIGS = {
    "dihip_seq_version": (C.c_char_p, []),
    "dihip_seq_last_error": (C.c_char_p, []),
    "dihip_linear": (i32, [vp, vp, i32, lng, lng, i32, vp, i32, vp, vp, i32, lng, lng, vp, lng, i32, i32, i32, i32, i32, i32, i32, i32]),
    "dihip_embed_sum": (i32, [vp, vp, vp, vp, vp, vp, i32, i32, i32]),
    "dihip_embed_rows": (i32, [vp, vp, i32, lng, vp, vp, i32, lng, lng, f32, i32, i32]),
    "dihip_rmsnorm_strided": (i32, [vp, vp, i32, lng, vp, lng, vp, vp, i32, f32, f32, f32, i32, i32]),
    "dihip_residual_norm_step": (i32, [vp, vp, vp, vp, lng, vp, f32, vp, f32, i32, f32, vp, i32, lng, vp, i32, lng, i32, i32]),
    "dihip_norm_span_append": (i32, [vp, vp, i32, i32, i32, vp, lng, vp, i32, f32, vp, vp, i32, i32]),
    "dihip_norm_residual_mix": (i32, [vp, vp, vp, vp, lng, vp, i32, f32, vp, sz, vp, i32, vp, vp, i32, i32]),
    "dihip_latent_window_attn": (i32, [vp, vp, lng, vp, lng, vp, i32, i32, i32, vp, i32, vp, vp, i32, i32, i32, i32, f32, i32]),
    "dihip_latent_window_attn_mc_supported": (i32, [i32, i32, i32]),
    "dihip_latent_window_attn_mc_workspace_bytes": (sz, [i32, i32, i32, i32]),
    "dihip_latent_window_attn_mc": (i32, [vp, vp, lng, vp, lng, vp, i32, i32, vp, i32, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, i32,
                                          vp, sz]),
    "dihip_causal_conv_state": (i32, [vp, vp, lng, vp, lng, vp, vp, i32, vp, vp, vp, i32, i32, i32, i32]),
    "dihip_conv_tail_update": (i32, [vp, vp, vp, lng, vp, vp, vp, i32, i32, i32]),
    "dihip_gated_recurrence_chunked_workspace_bytes": (sz, [i32, i32, i32]),
    "dihip_gated_recurrence_chunked": (i32, [vp, vp, lng, vp, vp, lng, vp, lng, vp, lng, vp, i32, f32, vp, vp, vp, vp, i32, i32, i32, vp, sz]),
    "dihip_linear_segmented": (i32, [vp, vp, i32, lng, vp, i32, vp, vp, i32, lng, i32, i32, i32, i32, vp, vp, i32, i32, i32]),
    "dihip_add_dyt": (i32, [vp, vp, vp, vp, lng, vp, lng, vp, f32, vp, vp, i32, vp, vp, i32, i32]),
    "dihip_qkv_prep_append": (i32, [vp, vp, lng, i32, i32, i32, i32, i32, i32, i32, i32, vp, vp, i32, f32, vp, i32, i32, f32, f32, vp, vp, lng, vp, vp,
                                    i32, i32, i32, vp, vp, i32]),
    "dihip_gqa_attn": (i32, [vp, vp, lng, vp, lng, vp, vp, i32, i32, i32, vp, i32, i32, f32, vp, lng, vp, vp, i32, i32, i32, i32, i32, f32, i32, i32,
                             i32]),
    "dihip_maps_diff_norm": (i32, [vp, vp, i32, lng, vp, lng, f32, f32, f32, i32, i32, i32]),
    "dihip_gqa_attn_mc_supported": (i32, [i32, i32, i32, i32]),
    "dihip_gqa_attn_mc_workspace_bytes": (sz, [i32, i32, i32, i32]),
    "dihip_gqa_attn_mc": (i32, [vp, vp, lng, vp, lng, vp, vp, i32, i32, vp, i32, i32, f32, vp, lng, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32,
                                i32, f32, i32, i32, i32, i32, vp, sz, vp, i32, lng, f32, f32, f32]),
    "dihip_gla_workspace_bytes": (sz, [i32, i32, i32, i32, i32, i32, i32]),
    "dihip_gla": (i32, [vp, vp, lng, vp, lng, vp, lng, vp, lng, vp, lng, f32, f32, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, vp, sz]),
    "dihip_head_rmsnorm_mul": (i32, [vp, vp, i32, lng, vp, lng, vp, i32, f32, vp, lng, i32, i32, i32]),
    "dihip_seq_moe_route": (i32, [vp, vp, lng, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp, i32, i32, i32]),
    "dihip_seq_moe_glu": (i32, [vp, vp, i32, lng, vp, lng, i32, i32, f32, f32, i32]),
    "dihip_seq_moe_combine": (i32, [vp, vp, lng, vp, lng, vp, vp, i32, i32, i32, vp, i32, vp, i32, lng, vp, lng]),
    "dihip_residual_layernorm": (i32, [vp, vp, vp, vp, lng, vp, lng, f32, vp, vp, vp, i32, f32, vp, i32, lng, i32, i32]),
    "dihip_polynorm": (i32, [vp, vp, i32, lng, vp, lng, vp, i32, f32, i32, i32]),
    "dihip_rmsnorm_pair": (i32, [vp, vp, lng, vp, lng, vp, vp, lng, vp, i32, f32, f32, i32, i32]),
    "dihip_gate_group_rmsnorm": (i32, [vp, vp, i32, lng, vp, lng, vp, lng, vp, vp, lng, vp, i32, f32, i32, i32, i32, i32]),
    "dihip_latent_rope_append": (i32, [vp, vp, i32, i32, i32, vp, lng, vp, i32, f32, i32, i32, i32, vp, vp, lng, vp, lng, i32, vp, vp, i32]),
    "dihip_ssd": (i32, [vp, vp, lng, vp, lng, vp, lng, vp, lng, vp, lng, vp, vp, i32, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, i32, vp, sz]),
    "dihip_talk_attn_workspace_bytes": (sz, [i32, i32, i32, i32]),
    "dihip_talk_attn": (i32, [vp, vp, i32, lng, vp, lng, vp, vp, i32, i32, i32, vp, vp, i32, vp, lng, vp, vp, i32, i32, i32, i32, i32, f32, i32, i32,
                              vp, sz]),
    "dihip_talk_attn_few_workspace_bytes": (sz, [i32, i32, i32, i32]),
    "dihip_talk_attn_few": (i32, [vp, vp, i32, lng, vp, lng, vp, vp, i32, i32, i32, vp, vp, i32, vp, lng, vp, vp, i32, i32, i32, i32, i32, f32, i32, i32,
                                  vp, sz]),
    "dihip_talk_attn_mc_supported": (i32, [i32, i32, i32, i32, i32, i32]),
    "dihip_talk_attn_mc_workspace_bytes": (sz, [i32, i32]),
    "dihip_talk_attn_mc": (i32, [vp, vp, i32, lng, vp, lng, vp, vp, i32, i32, vp, i32, vp, vp, lng, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32,
                                 f32, i32, vp, sz]),
    "dihip_gated_recurrence": (i32, [vp, vp, lng, vp, vp, lng, vp, lng, vp, lng, vp, i32, f32, vp, vp, vp, vp, i32, i32]),
}

_lib = None


def build():
    """hipcc of csrc/seq/*.hip -> lib/libdashinfer_hip_seq.so"""
    jobs = str(min(os.cpu_count() or 4, 16))
    r = subprocess.run(["make", "-C", os.path.join(PKG_DIR, "csrc"), "-j", jobs, "seq"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
    if r.returncode != 0:
        raise RuntimeError("building libdashinfer_hip_seq.so failed:\n" + r.stdout.decode(errors="replace")[-4000:])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(SEQ_LIB_PATH):
            build()
        try:  # torch's libamdhip64 must be the HIP runtime of the process
            import torch  # noqa: F401
        except ImportError:
            pass
        l = C.CDLL(SEQ_LIB_PATH)
        for name, (res, args) in _SIGS.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


class SeqError(RuntimeError):
    def __init__(self, code, what):
        super().__init__(f"{what}: status {code}: {lib().dihip_seq_last_error().decode()}")
        self.code = code


def check(code, what):
    if code != 0:
        raise SeqError(code, what)
