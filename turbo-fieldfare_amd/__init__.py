"""ctypes binding of ``libtf_kernels.so`` — the C ABI declared in ``include/tf_kernels.h``.

The product is the HIP library; this module only loads it and passes device pointers through.  PyTorch is used
by callers for device memory and streams, never for arithmetic.  There is no CPU fallback: if the shared object is
missing or cannot be loaded, importing :func:`load` raises.

Load with ``importlib.import_module("turbo-fieldfare_amd")`` (the directory name is not a Python identifier).
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtf_kernels.so")

TF_OK = 0
TF_ERR_INVALID_ARGUMENT = -1
TF_ERR_UNAVAILABLE = -2
TF_ERR_DIMENSION_MISMATCH = -3
TF_ERR_SCRATCH_TOO_SMALL = -4
TF_ERR_UNSUPPORTED_BITS = -5
TF_ERR_NO_DEVICE = -6
TF_ERR_DEVICE = -7
TF_ERR_OUT_OF_MEMORY = -8

TF_BF16, TF_FP16, TF_FP32 = 0, 1, 2

vp = C.c_void_p
u64 = C.c_uint64
u32 = C.c_uint32
i32 = C.c_int32


class ExpertOffsets(C.Structure):
    """tf_expert_offsets (36 bytes)."""
    _fields_ = [(n, C.c_uint32) for n in (
        "gate_W_off", "gate_s_off", "gate_b_off", "up_W_off", "up_s_off", "up_b_off",
        "down_W_off", "down_s_off", "down_b_off")]


class Projection(C.Structure):
    """tf_projection."""
    _fields_ = [("weights", vp), ("weights_offset", u64), ("scales", vp), ("scales_offset", u64),
                ("biases", vp), ("biases_offset", u64), ("rows", u32), ("cols", u32)]


class PrefillAttentionParams(C.Structure):
    """PrefillAttentionParams (Kernels/Attention/PrefillAttention.swift:4-40)."""
    _fields_ = [("start_position", C.c_uint32), ("query_count", C.c_uint32), ("head_dim", C.c_uint32), ("num_q_heads", C.c_uint32),
                ("num_kv_heads", C.c_uint32), ("kv_valid_count", C.c_uint32), ("sliding_window", C.c_uint32),
                ("kv_token_stride_elements", C.c_uint32), ("q_token_stride_elements", C.c_uint32), ("o_token_stride_elements", C.c_uint32),
                ("scale", C.c_float)]


class AttentionSplitGeometry(C.Structure):
    """AttentionSplitGeometry (Kernels/Attention/Attention.swift:5-11)."""
    _fields_ = [("effective_length", C.c_int32), ("num_chunks", C.c_int32), ("chunk_length", C.c_int32),
                ("partial_threadgroups", C.c_int32), ("use_swa_grouped_partial", C.c_int32)]


class ScratchLimits(C.Structure):
    """tf_scratch_limits: what the context's wrapper scratch is sized for (tf_ctx_reserve raises it)."""
    _fields_ = [(n, C.c_uint32) for n in ("max_vocab", "max_block_tokens", "max_experts", "max_shared_intermediate", "max_q_heads",
                                          "max_head_dim", "max_attention_block_tokens")]


class RoutedBlobs(C.Structure):
    """tf_routed_blobs."""
    _fields_ = [("blobs", vp * 8), ("pool", vp), ("pool_stride", u64), ("indices", vp), ("num_experts", u32)]


class PrefillPair(C.Structure):
    """tf_prefill_pair (16 bytes)."""
    _fields_ = [("token", u32), ("expert", u32), ("rank", u32), ("weight_bits_and_reserved", u32)]


class PrefillGroup(C.Structure):
    """tf_prefill_group."""
    _fields_ = [("expert", u32), ("pair_start", u32), ("pair_count", u32)]


class PrefillTile(C.Structure):
    """tf_prefill_tile."""
    _fields_ = [("group_start", u32), ("group_count", u32), ("pair_start", u32), ("pair_count", u32)]


class StreamedParams(C.Structure):
    """tf_prefill_streamed_params (128 bytes)."""
    _fields_ = ([(n, u32) for n in ("pair_start", "pair_count", "d", "routed_intermediate", "top_k", "hidden_stride_elements",
                                    "live_expert_count")]
                + [("local_expert", u32 * 16)]
                + [(n, u32) for n in ("gate_W_off", "gate_s_off", "gate_b_off", "up_W_off", "up_s_off", "up_b_off",
                                      "down_W_off", "down_s_off", "down_b_off")])


GROUP_ERRORS = {-101: "invalidQueryCount", -102: "invalidTopK", -103: "invalidNumExperts", -104: "invalidTileExpertCount",
                -105: "pairCountMismatch", -106: "tokenOutOfRange", -107: "rankOutOfRange", -108: "expertOutOfRange",
                -109: "duplicateTokenRank", -110: "expertSortKeyCountMismatch"}


class TFError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"tf_kernels status {status}: {message}")
        self.status = status


# every symbol include/tf_kernels.h declares; tests check that the library exports each one
EXPORTS = {
    "tf_ctx_create": (i32, [i32, C.POINTER(vp)]),
    "tf_ctx_destroy": (None, [vp]),
    "tf_ctx_reserve": (i32, [vp, C.POINTER(ScratchLimits)]),
    "tf_ctx_scratch_limits": (i32, [vp, C.POINTER(ScratchLimits)]),
    "tf_stream_synchronize": (i32, [vp, vp]),
    "tf_status_string": (C.c_char_p, [i32]),
    "tf_last_error": (C.c_char_p, [vp]),
    "tf_abi_version": (u32, []),
    "tf_ctx_set_step_timing": (i32, [vp, i32]),
    "tf_ctx_last_step_timing": (i32, [vp, C.POINTER(C.c_float)]),
    "tf_router_logits": (vp, [vp]),
    "tf_prefill_router_logits": (vp, [vp]),
    "tf_dequantize_int4_affine": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, i32]),
    "tf_dequantize_int8_affine": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, i32]),
    "tf_dequant_int4_gemv": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, i32, i32]),
    "tf_dequant_int8_gemv": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, i32, i32]),
    "tf_fused_qkv_gemv": (i32, [vp, vp] + [vp, u64] * 9 + [vp] + [vp, u64] * 3 + [u32, u32, u32, i32]),
    "tf_fused_norm_qkv_gemv": (i32, [vp, vp, vp, u64, C.c_float] + [vp, u64] * 9 + [vp] + [vp, u64] * 3 + [u32, u32, u32, i32]),
    "tf_fused_layer_tail_norm_qkv_gemv": (i32, [vp, vp, vp, vp, vp, vp] + [vp, u64] * 3 + [C.c_float, C.c_float, vp, u64, C.c_float] + [vp, u64] * 9 +
                                          [vp, u64] * 3 + [u32, u32, u32, i32]),
    "tf_gelu_mul_fp16": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, u32]),
    "tf_rmsnorm_bf16w": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, u32, C.c_float]),
    "tf_fused_post_attn_setup": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, u64, vp, u64, vp, u64, u32, C.c_float]),
    "tf_prefill_post_attn_setup_block": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64,
                                               u32, u32, u32, u32, u32, u32, u32, C.c_float]),
    "tf_fused_layer_tail": (i32, [vp, vp, vp, vp, vp, vp, u64, vp, u64, u32, C.c_float, C.c_float]),
    "tf_fused_layer_tail_shared_norm": (i32, [vp, vp, vp, vp, vp, vp, u64, vp, u64, vp, u64, u32, C.c_float, C.c_float]),
    "tf_prefill_layer_tail_block": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, u32, u32, u32,
                                          C.c_float, C.c_float]),
    "tf_shared_expert_int4": (i32, [vp, vp, vp, u64, u64, C.POINTER(Projection), C.POINTER(Projection), C.POINTER(Projection),
                                    vp, u64, u64, vp, u64, u64, vp, u64, u64, vp, u64, u64, u32, i32]),
    "tf_shared_expert_int8": (i32, [vp, vp, vp, u64, u64, C.POINTER(Projection), C.POINTER(Projection), C.POINTER(Projection), vp, u64, u64,
                                    vp, u64, u64, i32]),
    "tf_shared_expert_int8_phase1": (i32, [vp, vp, vp, u64, u64, C.POINTER(Projection), C.POINTER(Projection), vp, u64, u64, i32]),
    "tf_shared_expert_int8_down": (i32, [vp, vp, C.POINTER(Projection), vp, u64, u64, vp, u64, u64, i32]),
    "tf_prefill_shared_expert_int4_block": (i32, [vp, vp, vp, u64, vp, u64, C.POINTER(Projection), C.POINTER(Projection),
                                                  C.POINTER(Projection), vp, u64, u64, vp, u64, u64, vp, u64, u64, u32, u32, u32,
                                                  u32, u32, u32, i32]),
    "tf_rope_default_neox": (i32, [vp, vp, vp, u64, u32, u32, u32, u32, C.c_float]),
    "tf_rope_proportional_neox": (i32, [vp, vp, vp, u64, u32, u32, u32, u32, u32, C.c_float]),
    "tf_fused_qkv_epilogue": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, u32, u32, C.c_float, u32, C.c_float]),
    "tf_rmsnorm_no_scale": (i32, [vp, vp, vp, u64, vp, u64, u32, C.c_float]),
    "tf_rmsnorm_bf16w_perhead": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, u32, u32, C.c_float]),
    "tf_rmsnorm_no_scale_perhead": (i32, [vp, vp, vp, u64, vp, u64, u32, u32, C.c_float]),
    "tf_prefill_rmsnorm_bf16w_block": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, u32, u32, C.c_float]),
    "tf_prefill_rmsnorm_bf16w_perhead_block": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, u32, u32, u32, u32, C.c_float]),
    "tf_prefill_rmsnorm_no_scale_perhead_block": (i32, [vp, vp, vp, u64, vp, u64, u32, u32, u32, u32, C.c_float]),
    "tf_prefill_rope_default_neox_block": (i32, [vp, vp, vp, u64, u32, u32, u32, u32, u32, C.c_float]),
    "tf_prefill_rope_proportional_neox_block": (i32, [vp, vp, vp, u64, u32, u32, u32, u32, u32, u32, C.c_float]),
    "tf_prefill_qkv_epilogue_block": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, u32, u32, u32, u32, u32, C.c_float, u32,
                                            C.c_float]),
    "tf_attention_swa": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, u32, u32, u32, C.c_float, u32]),
    "tf_attention_full": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, u32, u32, C.c_float]),
    "tf_prefill_attention_causal": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, C.POINTER(PrefillAttentionParams), u32]),
    "tf_attention_split_geometry": (None, [u32, u32, u32, u32, i32, C.POINTER(AttentionSplitGeometry)]),
    "tf_router_gemma4": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, vp, u64, vp, u64, vp, vp, u32, u32, u32]),
    "tf_moe_phase1_gate_up_act": (i32, [vp, vp, C.POINTER(RoutedBlobs), C.POINTER(ExpertOffsets), vp, vp, u32, u32, u32, i32]),
    "tf_moe_phase1_gate_up_act_subset": (i32, [vp, vp, C.POINTER(RoutedBlobs), C.POINTER(ExpertOffsets), vp, vp, vp, u32,
                                               u32, u32, u32, i32]),
    "tf_moe_phase2_down_reduce": (i32, [vp, vp, C.POINTER(RoutedBlobs), C.POINTER(ExpertOffsets), vp, vp, vp, vp, u32, u32,
                                        u32, i32]),
    "tf_moe_decode_step": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, vp, u64, vp, u64, vp, u64, u32, C.POINTER(ExpertOffsets),
                                 vp, vp, vp, vp, vp, vp, u32, u32, u32, i32]),
    "tf_moe_decode_step_static": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, vp, u64, vp, u64, vp, u64, u32, C.POINTER(ExpertOffsets),
                                        vp, vp, vp, vp, vp, vp, u32, u32, u32, i32]),
    "tf_moe_decode_step_shared": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, vp, u64, vp, u64, vp, u64, u32, C.POINTER(ExpertOffsets),
                                        vp, vp, vp, vp, vp, vp, u32, u32, u32, i32, vp, C.POINTER(Projection), C.POINTER(Projection),
                                        C.POINTER(Projection), vp, vp, vp, vp]),
    "tf_moe_decode_step_shared_post_attn": (i32, [vp, vp, vp, vp, vp, vp, u64, vp, u64, vp, u64, C.c_float,
                                                  vp, u64, vp, u64, vp, u64, vp, vp, u64, vp, u64, vp, u64, u32, C.POINTER(ExpertOffsets),
                                                  vp, vp, vp, vp, vp, vp, u32, u32, u32, i32, vp, C.POINTER(Projection),
                                                  C.POINTER(Projection), C.POINTER(Projection), vp, vp, vp, vp]),
    "tf_prefill_router_gemma4_block": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64,
                                             u32, u32, u32, u32, u32]),
    "tf_prefill_router_group_block": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64,
                                            u32, u32, u32, u32, u32, vp, vp, vp, vp, vp]),
    "tf_prefill_routed_moe_few_tokens": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64,
                                               u32, u32, u32, u32, u32, vp, u64, u32, vp, u64, C.POINTER(ExpertOffsets), vp, vp, vp, u64,
                                               u32, i32]),
    "tf_prefill_make_token_expert_pairs": (i32, [vp, vp, i32, i32, vp]),
    "tf_prefill_group_token_expert_pairs": (i32, [vp, u64, i32, i32, i32, i32, vp, u64, vp, vp, vp, vp, vp, vp, vp]),
    "tf_prefill_group_pairs_device": (i32, [vp, vp, vp, vp, u32, u32, u32, vp, vp, vp, vp, vp]),
    "tf_prefill_grouped_routed_moe_streamed": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp,
                                                     C.POINTER(StreamedParams), vp, u32, i32, C.POINTER(i32), i32]),
    "tf_prefill_grouped_routed_moe_resident": (i32, [vp, vp, vp, u64, u32, vp, vp, vp, u32, u32, vp, u64, u32,
                                                     C.POINTER(ExpertOffsets), vp, vp, u32, u32, u32, i32]),
    "tf_prefill_grouped_routed_moe_resident_shared": (i32, [vp, vp, vp, u64, u32, vp, vp, vp, u32, u32, vp, u64, u32,
                                                            C.POINTER(ExpertOffsets), vp, vp, u32, u32, u32, i32,
                                                            vp, u64, vp, u64, C.POINTER(Projection), C.POINTER(Projection),
                                                            C.POINTER(Projection), vp, u64, u64, vp, u64, u64, vp, u64, u64,
                                                            u32, u32, u32, u32, u32]),
    "tf_prefill_moe_reduce_token_major": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, u32, u32, u32]),
    "tf_int4_qmm": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, i32, i32, i32, i32]),
    "tf_prefill_int4_qmm": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, i32, i32, i32, i32]),
    "tf_embed_lookup_int4": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, C.c_float, u32]),
    "tf_prefill_embed_lookup_int4_block": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, C.c_float, u32]),
    "tf_logit_softcap_softmax": (i32, [vp, vp, vp, vp, u32, C.c_float, i32]),
    "tf_sample": (i32, [vp, vp, vp, vp, u32, C.c_float, u32, C.c_float, u64, u32]),
    "tf_sample_topk64": (i32, [vp, vp, vp, vp, u32, C.c_float, C.c_float, u64]),
    "tf_upload_packed_experts_layer": (i32, [vp, vp, C.c_char_p, u64, u32, C.POINTER(u32), vp]),
    "tf_upload_file_region": (i32, [vp, vp, C.c_char_p, u64, u64, vp]),
    "tf_lm_head_greedy_int4": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u32, u32, C.c_float, i32]),
    "tf_lm_head_logits_int4": (i32, [vp, vp, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, vp, u64, u32, u32, C.c_float,
                                     i32, i32]),
}

# measurement helpers of include/tf_bench.h: same library, not part of the drop-in surface
BENCH_EXPORTS = {
    "tf_bench_empty_launch": (i32, [vp, vp, u32, u32, vp, vp]),
    "tf_bench_stream_read": (i32, [vp, vp, vp, u64, vp]),
    "tf_bench_moe_decode_step_stages": None,     # the argument list of tf_moe_decode_step + stages, filled in below
}

BENCH_EXPORTS["tf_bench_moe_decode_step_stages"] = (i32, list(EXPORTS["tf_moe_decode_step"][1]) + [u32])

_lib = None


def load() -> C.CDLL:
    """Load the HIP library; raise if it has not been built (no fallback exists)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python turbo-fieldfare_amd/build.py` (hipcc, gfx950). "
            "There is no CPU fallback.")
    try:
        # callers allocate device memory and streams with PyTorch; loading it first makes both share one HIP runtime
        # (the dynamic loader resolves libamdhip64.so.7 to whichever copy is already mapped)
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = C.CDLL(LIB_PATH)
    for name, (restype, argtypes) in {**EXPORTS, **BENCH_EXPORTS}.items():
        fn = getattr(lib, name)      # AttributeError if the ABI and the library disagree
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def _p(t):
    """Device pointer of a torch tensor (or pass an int / None through)."""
    if t is None:
        return None
    if isinstance(t, int):
        return t
    return t.data_ptr()


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


class Context:
    """Owns a tf_ctx; methods mirror the C entry points one to one and raise TFError on a negative status."""

    def __init__(self, device: int = 0):
        self.lib = load()
        h = vp()
        rc = self.lib.tf_ctx_create(device, C.byref(h))
        if rc != TF_OK:
            raise TFError(rc, self.lib.tf_status_string(rc).decode())
        self.handle = h

    def close(self):
        if getattr(self, "handle", None):
            self.lib.tf_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def check(self, rc: int) -> int:
        if rc != TF_OK:
            raise TFError(rc, self.lib.tf_last_error(self.handle).decode())
        return rc

    def last_error(self) -> str:
        return self.lib.tf_last_error(self.handle).decode()

    def synchronize(self, stream=None):
        return self.check(self.lib.tf_stream_synchronize(self.handle, _stream() if stream is None else stream))

    def reserve(self, **limits) -> "ScratchLimits":
        """Raises the wrapper-scratch limits (tf_ctx_reserve; set-up time only: it may wait for the device) and returns them."""
        want = ScratchLimits(**limits)
        self.check(self.lib.tf_ctx_reserve(self.handle, C.byref(want)))
        return self.scratch_limits()

    def scratch_limits(self) -> "ScratchLimits":
        out = ScratchLimits()
        self.check(self.lib.tf_ctx_scratch_limits(self.handle, C.byref(out)))
        return out

    def set_step_timing(self, enabled: bool):
        return self.check(self.lib.tf_ctx_set_step_timing(self.handle, 1 if enabled else 0))

    def last_step_timing(self):
        """(router_us, phase1_us, phase2_us, empty_bracket_us) of the most recent tf_moe_decode_step; waits for it."""
        out = (C.c_float * 4)()
        self.check(self.lib.tf_ctx_last_step_timing(self.handle, out))
        return tuple(out)

    # ---- raw calls (return the status, do not raise) -----------------------------------------------------
    def call(self, name: str, *args) -> int:
        return getattr(self.lib, name)(self.handle, *args)

    # ---- conveniences over torch tensors --------------------------------------------------------------------
    def dequantize_int4(self, W, S, B, out, m, n, scale_dtype=TF_BF16, offsets=(0, 0, 0, 0), bits=4):
        fn = self.lib.tf_dequantize_int4_affine if bits == 4 else self.lib.tf_dequantize_int8_affine
        return self.check(fn(self.handle, _stream(), _p(W), offsets[0], _p(S), offsets[1], _p(B), offsets[2], _p(out),
                             offsets[3], m, n, scale_dtype))

    def dequant_int4_gemv(self, W, S, B, x, y, m, n, scale_dtype=TF_BF16, out_dtype=TF_FP16,
                          offsets=(0, 0, 0, 0, 0), bits=4, raise_on_error=True):
        fn = self.lib.tf_dequant_int4_gemv if bits == 4 else self.lib.tf_dequant_int8_gemv
        rc = fn(self.handle, _stream(), _p(W), offsets[0], _p(S), offsets[1], _p(B), offsets[2], _p(x), offsets[3],
                _p(y), offsets[4], m, n, scale_dtype, out_dtype)
        return self.check(rc) if raise_on_error else rc

    def gelu_mul_fp16(self, gate, up, out, count):
        return self.check(self.lib.tf_gelu_mul_fp16(self.handle, _stream(), _p(gate), 0, _p(up), 0, _p(out), 0, count))

    def rmsnorm_bf16w(self, x, w, out, d, eps, x_offset=0):
        return self.check(self.lib.tf_rmsnorm_bf16w(self.handle, _stream(), _p(x), x_offset, _p(w), 0, _p(out), 0, d, eps))

    def router_gemma4(self, W, S, B, hidden, eff, per_expert, out_idx, out_w, num_experts, d, top_k=8, raise_on_error=True):
        rc = self.lib.tf_router_gemma4(self.handle, _stream(), _p(W), 0, _p(S), 0, _p(B), 0, _p(hidden), _p(eff), 0,
                                       _p(per_expert), 0, _p(out_idx), _p(out_w), num_experts, d, top_k)
        return self.check(rc) if raise_on_error else rc

    def router_logits_ptr(self) -> int:
        return int(self.lib.tf_router_logits(self.handle))

    @staticmethod
    def routed_from_pointers(ptrs) -> RoutedBlobs:
        r = RoutedBlobs()
        for i, p in enumerate(ptrs):
            r.blobs[i] = p
        return r

    @staticmethod
    def routed_from_pool(pool, stride: int, indices, num_experts: int) -> RoutedBlobs:
        r = RoutedBlobs()
        r.pool = _p(pool)
        r.pool_stride = stride
        r.indices = _p(indices)
        r.num_experts = num_experts
        return r

    def moe_phase1(self, routed: RoutedBlobs, off: ExpertOffsets, x, acts, d, f, top_k=8, scale_dtype=TF_BF16,
                   active_slots=None, active_count=0, raise_on_error=True):
        if active_slots is None:
            rc = self.lib.tf_moe_phase1_gate_up_act(self.handle, _stream(), C.byref(routed), C.byref(off), _p(x), _p(acts),
                                                    d, f, top_k, scale_dtype)
        else:
            rc = self.lib.tf_moe_phase1_gate_up_act_subset(self.handle, _stream(), C.byref(routed), C.byref(off), _p(x),
                                                           _p(acts), _p(active_slots), active_count, d, f, top_k, scale_dtype)
        return self.check(rc) if raise_on_error else rc

    def moe_phase2(self, routed: RoutedBlobs, off: ExpertOffsets, acts, routing_w, residual, y, d, f, top_k=8,
                   scale_dtype=TF_BF16, raise_on_error=True):
        rc = self.lib.tf_moe_phase2_down_reduce(self.handle, _stream(), C.byref(routed), C.byref(off), _p(acts), _p(routing_w),
                                                _p(residual), _p(y), d, f, top_k, scale_dtype)
        return self.check(rc) if raise_on_error else rc

    def shared_expert_int4(self, x, gate: Projection, up: Projection, down: Projection, y, sg, su, sa, weight_bits=4,
                           scale_dtype=TF_BF16, raise_on_error=True, lengths=None):
        def nbytes(t):
            return t.numel() * t.element_size()
        ln = lengths or (nbytes(x), nbytes(y), nbytes(sg), nbytes(su), nbytes(sa))
        rc = self.lib.tf_shared_expert_int4(self.handle, _stream(), _p(x), 0, ln[0], C.byref(gate), C.byref(up), C.byref(down),
                                            _p(y), 0, ln[1], _p(sg), 0, ln[2], _p(su), 0, ln[3], _p(sa), 0, ln[4],
                                            weight_bits, scale_dtype)
        return self.check(rc) if raise_on_error else rc

    def prefill_shared_expert_block(self, x, gate: Projection, up: Projection, down: Projection, y, sg, su, sa, query_count, d,
                                    intermediate, x_stride=None, y_stride=None, x_offset=0, y_offset=0, weight_bits=4,
                                    scale_dtype=TF_BF16, raise_on_error=True):
        def nbytes(t):
            return t.numel() * t.element_size()
        rc = self.lib.tf_prefill_shared_expert_int4_block(self.handle, _stream(), _p(x), x_offset, _p(y), y_offset, C.byref(gate),
                                                          C.byref(up), C.byref(down), _p(sg), 0, nbytes(sg), _p(su), 0, nbytes(su),
                                                          _p(sa), 0, nbytes(sa), query_count, d, intermediate,
                                                          d if x_stride is None else x_stride, d if y_stride is None else y_stride,
                                                          weight_bits, scale_dtype)
        return self.check(rc) if raise_on_error else rc

    def attention_swa(self, q, k, v, out, head_dim, num_q_heads, num_kv_heads, seq_len, window, scale=0.0, ring_capacity=0,
                      offsets=(0, 0, 0, 0), raise_on_error=True):
        rc = self.lib.tf_attention_swa(self.handle, _stream(), _p(q), offsets[0], _p(k), offsets[1], _p(v), offsets[2], _p(out), offsets[3],
                                       head_dim, num_q_heads, num_kv_heads, seq_len, window, scale, ring_capacity)
        return self.check(rc) if raise_on_error else rc

    def attention_full(self, q, k, v, out, head_dim, num_q_heads, num_kv_heads, seq_len, scale=0.0, offsets=(0, 0, 0, 0),
                       raise_on_error=True):
        rc = self.lib.tf_attention_full(self.handle, _stream(), _p(q), offsets[0], _p(k), offsets[1], _p(v), offsets[2], _p(out), offsets[3],
                                        head_dim, num_q_heads, num_kv_heads, seq_len, scale)
        return self.check(rc) if raise_on_error else rc

    def lm_head_greedy(self, hidden, norm_w, W, S, B, out_token, d, vocab, eps=1e-6, scale_dtype=TF_BF16,
                       hidden_offset=0, weights_offset=0, raise_on_error=True):
        rc = self.lib.tf_lm_head_greedy_int4(self.handle, _stream(), _p(hidden), hidden_offset, _p(norm_w), 0, _p(W),
                                             weights_offset, _p(S), 0, _p(B), 0, _p(out_token), d, vocab, eps, scale_dtype)
        return self.check(rc) if raise_on_error else rc

    def lm_head_logits(self, hidden, norm_w, W, S, B, logits, d, vocab, eps=1e-6, scale_dtype=TF_BF16, out_dtype=TF_FP16):
        return self.check(self.lib.tf_lm_head_logits_int4(self.handle, _stream(), _p(hidden), 0, _p(norm_w), 0, _p(W), 0,
                                                          _p(S), 0, _p(B), 0, _p(logits), 0, d, vocab, eps, scale_dtype, out_dtype))


def projection(W, S, B, rows: int, cols: int, offsets=(0, 0, 0)) -> Projection:
    return Projection(_p(W), offsets[0], _p(S), offsets[1], _p(B), offsets[2], rows, cols)


# ---- host-side grouping (pure CPU functions of the library) ----------------------------------------------------------
def make_token_expert_pairs(indices, weights_f16_bits, query_count: int, top_k: int):
    """PrefillRouter.makeTokenExpertPairs over numpy arrays -> (PrefillPair * n)."""
    import numpy as np
    lib = load()
    idx = np.ascontiguousarray(indices, np.uint32)
    w = np.ascontiguousarray(weights_f16_bits, np.uint16)
    pairs = (PrefillPair * max(1, query_count * top_k))()
    rc = lib.tf_prefill_make_token_expert_pairs(idx.ctypes.data, w.ctypes.data, query_count, top_k, C.cast(pairs, vp))
    if rc != TF_OK:
        raise TFError(rc, "make_token_expert_pairs")
    return pairs


def group_token_expert_pairs(pairs, query_count: int, top_k: int, num_experts: int, tile_expert_count: int = 16,
                             expert_sort_keys=None):
    """PrefillMoEGrouping.groupTokenExpertPairs.  `pairs`: sequence of (token, expert, rank, weight_bits) or PrefillPair array.
    Returns a dict of python lists; raises TFError whose .status is one of the TF_ERR_GROUP_* codes."""
    lib = load()
    if not isinstance(pairs, C.Array):
        arr = (PrefillPair * max(1, len(pairs)))()
        for i, p in enumerate(pairs):
            arr[i] = PrefillPair(*p)
        n = len(pairs)
    else:
        arr, n = pairs, len(pairs)
    ne = max(num_experts, 1)
    cap = max(1, min(ne, max(n, 1)))
    sorted_pairs = (PrefillPair * max(1, n))()
    offs, cnts = (u32 * ne)(), (u32 * ne)()
    groups, tiles = (PrefillGroup * cap)(), (PrefillTile * cap)()
    ng, nt = u32(0), u32(0)
    keys, nkeys = None, 0
    if expert_sort_keys is not None:
        keys_arr = (u64 * len(expert_sort_keys))(*expert_sort_keys)
        keys, nkeys = C.cast(keys_arr, vp), len(expert_sort_keys)
    rc = lib.tf_prefill_group_token_expert_pairs(C.cast(arr, vp), n, query_count, top_k, num_experts, tile_expert_count, keys, nkeys,
                                                 C.cast(sorted_pairs, vp), C.cast(offs, vp), C.cast(cnts, vp), C.cast(groups, vp),
                                                 C.byref(ng), C.cast(tiles, vp), C.byref(nt))
    if rc != TF_OK:
        raise TFError(rc, GROUP_ERRORS.get(rc, "grouping failed"))
    return dict(
        sorted_pairs=[(p.token, p.expert, p.rank, p.weight_bits_and_reserved) for p in sorted_pairs[:n]],
        sorted_pairs_raw=sorted_pairs, n_pairs=n,
        per_expert_offsets=list(offs[:num_experts]), per_expert_counts=list(cnts[:num_experts]),
        groups=[(g.expert, g.pair_start, g.pair_count) for g in groups[:ng.value]], groups_raw=groups,
        tiles=[(t.group_start, t.group_count, t.pair_start, t.pair_count) for t in tiles[:nt.value]])
