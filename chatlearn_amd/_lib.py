"""ctypes binding of libclgrpo.so (the C ABI declared in include/clgrpo.h).

The library is the only compute path of this package: there is no torch or CPU
fallback.  If the shared object is missing, importing succeeds (so that
host-only helpers stay usable) but the first call that needs it raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# CLGRPO_LIB_PATH selects another build of the same library (e.g. a tuning variant).
LIB_PATH = os.environ.get("CLGRPO_LIB_PATH") or os.path.join(_HERE, "csrc", "libclgrpo.so")

BF16, F32, F64, U8 = 0, 1, 2, 3
LOSS_GRPO, LOSS_GSPO = 0, 1

STATUS_NAMES = {0: "CLGRPO_OK", -1: "CLGRPO_EINVAL", -2: "CLGRPO_EDTYPE", -3: "CLGRPO_ESHAPE",
                -4: "CLGRPO_ENULL", -5: "CLGRPO_ELAUNCH", -6: "CLGRPO_EWORKSPACE"}

vp, i64, i32, f32, f64, sz = C.c_void_p, C.c_int64, C.c_int32, C.c_float, C.c_double, C.c_size_t


class ClgrpoError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"{STATUS_NAMES.get(code, code)}: {message}")
        self.code = code


class LmheadFwdArgs(C.Structure):
    _fields_ = [("hidden", vp), ("weight", vp), ("labels", vp), ("T", i64), ("H", i64), ("V", i64),
                ("dtype", i32), ("inv_temperature", f32), ("logprob", vp), ("entropy", vp),
                ("rowmax", vp), ("lse", vp), ("workspace", vp), ("workspace_bytes", sz),
                ("saved_logits", vp), ("ld_saved", i64), ("saved_row_map", vp), ("saved_rows", i64)]


class LmheadBwdArgs(C.Structure):
    _fields_ = [("hidden", vp), ("weight", vp), ("labels", vp), ("lse", vp), ("entropy", vp),
                ("g_logprob", vp), ("g_entropy", vp), ("T", i64), ("H", i64), ("V", i64),
                ("dtype", i32), ("inv_temperature", f32), ("dhidden", vp), ("dweight", vp),
                ("accumulate_dweight", i32), ("workspace", vp), ("workspace_bytes", sz),
                ("saved_logits", vp), ("ld_saved", i64), ("weight_t", vp), ("weight_t_ready", i32),
                ("saved_rows", i64)]


class SoftmaxStatsArgs(C.Structure):
    _fields_ = [("logits", vp), ("labels", vp), ("R", i64), ("V", i64), ("ld", i64), ("dtype", i32),
                ("logprob", vp), ("entropy", vp), ("lse", vp)]


class SoftmaxStatsBwdArgs(C.Structure):
    _fields_ = [("logits", vp), ("labels", vp), ("g_logprob", vp), ("g_entropy", vp), ("R", i64),
                ("V", i64), ("ld", i64), ("dtype", i32), ("dlogits", vp), ("lse", vp), ("entropy", vp)]


class PolicyLossArgs(C.Structure):
    _fields_ = [("mode", i32), ("compute_dtype", i32), ("n", i64), ("B", i64), ("S", i64),
                ("cu_seqlens", vp), ("logprob", vp), ("old_logprob", vp), ("ref_logprob", vp),
                ("entropy", vp), ("loss_mask", vp), ("advantages", vp),
                ("diff_clip_ratio", f64), ("pos_clip_ratio", f64), ("neg_clip_ratio", f64),
                ("final_clip_ratio", f64), ("kl_coef", f64), ("entropy_coef", f64), ("grad_scale", f64),
                ("loss", vp), ("dloss_dlogprob", vp), ("kl", vp), ("is_positive_clipped", vp),
                ("is_negative_clipped", vp), ("is_clipped", vp), ("g_logprob", vp), ("g_entropy", vp),
                ("sums", vp), ("flags", vp), ("workspace", vp), ("workspace_bytes", sz),
                ("token_offset", i64)]


class MaskedSumsArgs(C.Structure):
    _fields_ = [("n", i64), ("k", i32), ("src", vp * 16), ("dtype", i32 * 16), ("average", i32 * 16),
                ("mask", vp), ("out", vp), ("count", vp)]


class GroupAdvantageArgs(C.Structure):
    _fields_ = [("n_samples", i64), ("n_groups", i64), ("rewards", vp), ("group_of", vp), ("pool", vp),
                ("pool_offsets", vp), ("eps", f64), ("advantages", vp), ("all_zeros", vp), ("all_ones", vp)]


class BuildMasksArgs(C.Structure):
    _fields_ = [("B", i64), ("S", i64), ("prompt_len", vp), ("response_len", vp), ("attn_mask", vp),
                ("loss_mask", vp), ("position_ids", vp)]


class ShiftLabelsArgs(C.Structure):
    _fields_ = [("B", i64), ("S", i64), ("tokens", vp), ("loss_mask", vp), ("labels", vp),
                ("shifted_mask", vp), ("zero_last", i32)]


class UnpadIndicesArgs(C.Structure):
    _fields_ = [("B", i64), ("S", i64), ("attn_mask", vp), ("indices", vp), ("cu_seqlens", vp),
                ("seqlens", vp), ("total", vp), ("row_offsets", vp)]


class ThdPackArgs(C.Structure):
    _fields_ = [("B", i64), ("S", i64), ("tokens", vp), ("prompt_len", vp), ("response_len", vp),
                ("align", i32), ("cp_size", i32), ("cp_rank", i32), ("pad_token", i64), ("total_padded", i64),
                ("cu_seqlens_padded", vp), ("seqlens", vp), ("seqlens_padded", vp), ("stats", vp), ("status", vp),
                ("indices", vp), ("seq_indices", vp), ("out_tokens", vp), ("out_labels", vp), ("out_loss_mask", vp),
                ("out_position_ids", vp)]


class RowsArgs(C.Structure):
    _fields_ = [("src", vp), ("dst", vp), ("indices", vp), ("n_idx", i64), ("row_bytes", i64), ("n_rows", i64)]


# name -> (restype, argtypes); every symbol include/clgrpo.h declares.
SIGNATURES = {
    "clgrpo_version": (C.c_int, []),
    "clgrpo_last_error_string": (C.c_char_p, []),
    "clgrpo_lmhead_fwd_workspace_bytes": (sz, [i64, i64, i64, i32]),
    "clgrpo_lmhead_fwd": (C.c_int, [C.POINTER(LmheadFwdArgs), vp]),
    "clgrpo_lmhead_fwd_launch_plan": (C.c_int, [i64, i64, i32, vp]),
    "clgrpo_lmhead_bwd_dhidden_plan": (C.c_int, [i64, i64, i64, i32, i32, vp]),
    "clgrpo_lmhead_bwd_dweight_plan": (C.c_int, [i64, i64, i64, i32, i32, vp]),
    "clgrpo_saved_logits_ld": (i64, [i64]),
    "clgrpo_lmhead_bwd_workspace_bytes": (sz, [i64, i64, i64, i32, i64, i32]),
    "clgrpo_lmhead_bwd": (C.c_int, [C.POINTER(LmheadBwdArgs), vp]),
    "clgrpo_lmhead_fwd_shard": (C.c_int, [C.POINTER(LmheadFwdArgs), i64, vp, vp]),
    "clgrpo_lmhead_merge_shards": (C.c_int, [vp, i64, i64, vp, i64, f32, vp, vp, vp, vp, vp]),
    "clgrpo_lmhead_bwd_shard": (C.c_int, [C.POINTER(LmheadBwdArgs), i64, vp]),
    "clgrpo_softmax_stats": (C.c_int, [C.POINTER(SoftmaxStatsArgs), vp]),
    "clgrpo_softmax_stats_bwd": (C.c_int, [C.POINTER(SoftmaxStatsBwdArgs), vp]),
    "clgrpo_policy_loss_workspace_bytes": (sz, [i64, i64]),
    "clgrpo_policy_loss": (C.c_int, [C.POINTER(PolicyLossArgs), vp]),
    "clgrpo_policy_loss_launches": (C.c_int, [i64, i32]),
    "clgrpo_policy_loss_static": (C.c_int, [C.POINTER(PolicyLossArgs), vp]),
    "clgrpo_policy_loss_static_max_sequences": (i64, []),
    "clgrpo_masked_sums": (C.c_int, [C.POINTER(MaskedSumsArgs), vp]),
    "clgrpo_masked_sums_bwd": (C.c_int, [i64, vp, vp, vp, i32, vp]),
    "clgrpo_group_advantage": (C.c_int, [C.POINTER(GroupAdvantageArgs), vp]),
    "clgrpo_build_masks": (C.c_int, [C.POINTER(BuildMasksArgs), vp]),
    "clgrpo_shift_labels": (C.c_int, [C.POINTER(ShiftLabelsArgs), vp]),
    "clgrpo_unpad_indices": (C.c_int, [C.POINTER(UnpadIndicesArgs), vp]),
    "clgrpo_thd_pack": (C.c_int, [C.POINTER(ThdPackArgs), vp]),
    "clgrpo_gather_rows": (C.c_int, [C.POINTER(RowsArgs), vp]),
    "clgrpo_scatter_rows": (C.c_int, [C.POINTER(RowsArgs), vp]),
    "clgrpo_bin_packing": (C.c_int, [vp, i64, i64, vp, vp, vp]),
    "clgrpo_bin_packing_fix_bin": (C.c_int, [vp, i64, i64, vp, vp]),
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m chatlearn_amd.build` "
                "(this package has no fallback path)")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(code):
    if code != 0:
        raise ClgrpoError(code, lib().clgrpo_last_error_string().decode())


def call(name, args_struct, stream=None):
    """Invoke a launching entry point with an args struct and a stream handle."""
    check(getattr(lib(), name)(C.byref(args_struct), vp(stream or 0)))
