"""ctypes/numpy binding of the CPU oracle (``libtf_oracle.so``).

TEST INFRASTRUCTURE ONLY.  Import this from ``tests/``, from the smoke check and
from the benchmark's CPU-baseline leg; never from the product package.  Each
wrapper is a thin numpy front for the C function of the same name in
``tf_oracle.h`` (which carries the reference file:line citations).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtf_oracle.so")
GROUP = 64


def build(force: bool = False) -> str:
    """Compile the oracle with g++ (``make -C oracle``)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-C", _HERE, "libtf_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load() -> C.CDLL:
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


lib = _load()

u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
u64p = np.ctypeslib.ndpointer(np.uint64, flags="C_CONTIGUOUS")
f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
i32 = C.c_int
i64 = C.c_int64


class ExpertOffsets(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "gate_W_off", "gate_s_off", "gate_b_off", "up_W_off", "up_s_off", "up_b_off",
        "down_W_off", "down_s_off", "down_b_off")]

    def as_tuple(self):
        return tuple(getattr(self, n) for n, _ in self._fields_)


PAIR_DTYPE = np.dtype([("token", "<u4"), ("expert", "<u4"), ("rank", "<u4"), ("weight_bits", "<u4")])
GROUP_DTYPE = np.dtype([("expert", "<u4"), ("pair_start", "<u4"), ("pair_count", "<u4")])
TILE_DTYPE = np.dtype([("group_start", "<u4"), ("group_count", "<u4"), ("pair_start", "<u4"), ("pair_count", "<u4")])


def _sig(name, restype, *argtypes):
    fn = getattr(lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_bf16_bits = _sig("tfo_bf16_bits", C.c_uint16, C.c_float)
_bf16_to_float = _sig("tfo_bf16_to_float", C.c_float, C.c_uint16)
_f16_bits = _sig("tfo_f16_bits", C.c_uint16, C.c_float)
_f16_to_float = _sig("tfo_f16_to_float", C.c_float, C.c_uint16)
_sm_next = _sig("tfo_splitmix64_next", C.c_uint64, C.POINTER(C.c_uint64))
_sm_uniform = _sig("tfo_splitmix64_uniform", C.c_float, C.POINTER(C.c_uint64), C.c_float, C.c_float)
_seed_key = _sig("tfo_seedtree_key", C.c_uint64, C.c_uint64, C.c_char_p)
_fill_uniform = _sig("tfo_fill_uniform", None, C.POINTER(C.c_uint64), C.c_float, C.c_float, f32p, i64)


def bf16_bits(x: float) -> int:
    return int(_bf16_bits(float(np.float32(x))))


def bf16_to_float(b: int) -> float:
    return float(_bf16_to_float(int(b)))


def f16_bits(x: float) -> int:
    return int(_f16_bits(float(np.float32(x))))


def f16_to_float(b: int) -> float:
    return float(_f16_to_float(int(b)))


def bf16_bits_array(x: np.ndarray) -> np.ndarray:
    """Vectorised Quantization.bf16Bits over an fp32 array (same integer formula)."""
    bits = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    lsb = (bits >> 16) & 1
    return (((bits + 0x7FFF + lsb) & 0xFFFFFFFF) >> 16).astype(np.uint16)


def bf16_array_to_float(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


class SplitMix64:
    """The reference's seeded stream (SplitMix64.swift)."""

    def __init__(self, seed: int):
        self._state = C.c_uint64(seed & 0xFFFFFFFFFFFFFFFF)

    @property
    def state(self) -> int:
        return int(self._state.value)

    def next(self) -> int:
        return int(_sm_next(C.byref(self._state)))

    def uniform(self, lo: float, hi: float) -> float:
        return float(_sm_uniform(C.byref(self._state), lo, hi))

    def uniform_array(self, lo: float, hi: float, n: int) -> np.ndarray:
        out = np.empty(int(n), np.float32)
        _fill_uniform(C.byref(self._state), lo, hi, out, int(n))
        return out


class SeedTree:
    """SeedTree.swift: root ^ FNV-1a(label) seeds a SplitMix64."""

    def __init__(self, root: int):
        self.root = root & 0xFFFFFFFFFFFFFFFF

    def key_state(self, label: str) -> int:
        return int(_seed_key(self.root, label.encode("utf-8")))

    def key(self, label: str) -> SplitMix64:
        return SplitMix64(self.key_state(label))


# ---- quantizer -----------------------------------------------------------------
for _n in ("tfo_quantize_int4_matrix", "tfo_quantize_int8_matrix"):
    _sig(_n, None, f32p, i32, i32, u8p, u16p, u16p)
for _n in ("tfo_dequantize_int4_matrix", "tfo_dequantize_int8_matrix"):
    _sig(_n, None, u8p, u16p, u16p, i32, i32, f32p)


def quantize_int4(w: np.ndarray):
    """[m, n] fp32 -> (packed [m, n/2] u8, scales [m, n/64] u16 bf16 bits, biases likewise)."""
    w = np.ascontiguousarray(np.atleast_2d(w), np.float32)
    m, n = w.shape
    assert n % GROUP == 0
    packed = np.zeros((m, n // 2), np.uint8)
    s = np.zeros((m, n // GROUP), np.uint16)
    b = np.zeros((m, n // GROUP), np.uint16)
    lib.tfo_quantize_int4_matrix(w, m, n, packed, s, b)
    return packed, s, b


def quantize_int8(w: np.ndarray):
    w = np.ascontiguousarray(np.atleast_2d(w), np.float32)
    m, n = w.shape
    assert n % GROUP == 0
    packed = np.zeros((m, n), np.uint8)
    s = np.zeros((m, n // GROUP), np.uint16)
    b = np.zeros((m, n // GROUP), np.uint16)
    lib.tfo_quantize_int8_matrix(w, m, n, packed, s, b)
    return packed, s, b


def dequantize_int4(packed, s, b) -> np.ndarray:
    packed = np.ascontiguousarray(np.atleast_2d(packed), np.uint8)
    m, n2 = packed.shape
    out = np.empty((m, n2 * 2), np.float32)
    lib.tfo_dequantize_int4_matrix(packed, np.ascontiguousarray(s, np.uint16), np.ascontiguousarray(b, np.uint16), m, n2 * 2, out)
    return out


def dequantize_int8(packed, s, b) -> np.ndarray:
    packed = np.ascontiguousarray(np.atleast_2d(packed), np.uint8)
    m, n = packed.shape
    out = np.empty((m, n), np.float32)
    lib.tfo_dequantize_int8_matrix(packed, np.ascontiguousarray(s, np.uint16), np.ascontiguousarray(b, np.uint16), m, n, out)
    return out


# ---- metrics --------------------------------------------------------------------
_rel = _sig("tfo_rel_error", C.c_float, f32p, f32p, i64)
_mad = _sig("tfo_max_abs_diff", C.c_float, f32p, f32p, i64)
_brel = _sig("tfo_bounded_rel", C.c_float, f32p, f32p, i64, C.c_float)


def _flat32(a):
    return np.ascontiguousarray(np.asarray(a, np.float32).ravel())


def rel_error(actual, reference) -> float:
    a, r = _flat32(actual), _flat32(reference)
    assert a.size == r.size
    return float(_rel(a, r, a.size))


def max_abs_diff(a, b) -> float:
    a, b = _flat32(a), _flat32(b)
    assert a.size == b.size
    return float(_mad(a, b, a.size))


def bounded_rel(actual, reference, abs_floor: float) -> float:
    a, r = _flat32(actual), _flat32(reference)
    return float(_brel(a, r, a.size, abs_floor))


class Tolerance:
    """Tolerances.swift:4-21."""
    identity = 1e-5
    fp16Reduction = 5e-3
    fp16ChainedReduction = 1e-2
    quantInt4 = 1.5e-3
    quantInt8 = 1e-3


# ---- GEMV -------------------------------------------------------------------------
_sig("tfo_int4_gemv_ref", None, u8p, u16p, u16p, f32p, f32p, i64, i32, i32)
_sig("tfo_int8_gemv_ref", None, u8p, u16p, u16p, f32p, f32p, i64, i32, i32)
_sig("tfo_int4_gemv_f64", None, u8p, u16p, u16p, f32p, f64p, i64, i32)
_sig("tfo_int8_gemv_f64", None, u8p, u16p, u16p, f32p, f64p, i64, i32)
_sig("tfo_k_int4_gemv", None, u8p, u16p, u16p, u16p, f32p, i64, i32)


def _wsb(W, S, B):
    return (np.ascontiguousarray(W, np.uint8), np.ascontiguousarray(S, np.uint16), np.ascontiguousarray(B, np.uint16))


def int4_gemv_ref(W, S, B, x, threads: int = 1) -> np.ndarray:
    W, S, B = _wsb(W, S, B)
    m, n = W.shape[0], W.shape[1] * 2
    y = np.empty(m, np.float32)
    lib.tfo_int4_gemv_ref(W, S, B, _flat32(x), y, m, n, threads)
    return y


def int8_gemv_ref(W, S, B, x, threads: int = 1) -> np.ndarray:
    W, S, B = _wsb(W, S, B)
    m, n = W.shape
    y = np.empty(m, np.float32)
    lib.tfo_int8_gemv_ref(W, S, B, _flat32(x), y, m, n, threads)
    return y


def int4_gemv_f64(W, S, B, x) -> np.ndarray:
    W, S, B = _wsb(W, S, B)
    m, n = W.shape[0], W.shape[1] * 2
    y = np.empty(m, np.float64)
    lib.tfo_int4_gemv_f64(W, S, B, _flat32(x), y, m, n)
    return y


def int8_gemv_f64(W, S, B, x) -> np.ndarray:
    W, S, B = _wsb(W, S, B)
    m, n = W.shape
    y = np.empty(m, np.float64)
    lib.tfo_int8_gemv_f64(W, S, B, _flat32(x), y, m, n)
    return y


def k_int4_gemv(W, S, B, x_f16_bits) -> np.ndarray:
    W, S, B = _wsb(W, S, B)
    m, n = W.shape[0], W.shape[1] * 2
    y = np.empty(m, np.float32)
    lib.tfo_k_int4_gemv(W, S, B, np.ascontiguousarray(x_f16_bits, np.uint16), y, m, n)
    return y


# ---- primitives ------------------------------------------------------------------------
_sig("tfo_gelu_tanh", None, f32p, f32p, i64)
_sig("tfo_rmsnorm_ref", None, f32p, f32p, C.c_float, f32p, i32)
_sig("tfo_k_gelu_mul_fp16", None, u16p, u16p, u16p, i32)
_sig("tfo_k_rmsnorm_bf16w", None, u16p, u16p, C.c_float, u16p, i32)
_sig("tfo_k_rmsnorm_rows", None, u16p, C.c_void_p, C.c_float, u16p, i32, i32, i32, i32)


def gelu_tanh(x) -> np.ndarray:
    x = _flat32(x)
    y = np.empty_like(x)
    lib.tfo_gelu_tanh(x, y, x.size)
    return y


def rmsnorm_ref(x, w, eps: float) -> np.ndarray:
    x, w = _flat32(x), _flat32(w)
    y = np.empty_like(x)
    lib.tfo_rmsnorm_ref(x, w, eps, y, x.size)
    return y


def k_gelu_mul_fp16(gate_bits, up_bits) -> np.ndarray:
    g = np.ascontiguousarray(gate_bits, np.uint16)
    u = np.ascontiguousarray(up_bits, np.uint16)
    out = np.empty_like(g)
    lib.tfo_k_gelu_mul_fp16(g, u, out, g.size)
    return out


def k_rmsnorm_rows(x_bits, w_bits, eps: float, tokens: int, heads: int, d: int, token_stride: int, out_bits=None) -> np.ndarray:
    """Row-grid norms in kernel order (w_bits None: no scale); `out_bits` supplies what lies between the rows (default: x)."""
    x = np.ascontiguousarray(x_bits, np.uint16)
    out = np.array(x if out_bits is None else out_bits, np.uint16, copy=True)
    w = None if w_bits is None else np.ascontiguousarray(w_bits, np.uint16)
    lib.tfo_k_rmsnorm_rows(x, None if w is None else w.ctypes.data_as(C.c_void_p), eps, out, tokens, heads, d, token_stride)
    return out


def k_rmsnorm_bf16w(x_bits, w_bits, eps: float) -> np.ndarray:
    x = np.ascontiguousarray(x_bits, np.uint16)
    out = np.empty_like(x)
    lib.tfo_k_rmsnorm_bf16w(x, np.ascontiguousarray(w_bits, np.uint16), eps, out, x.size)
    return out


_sig("tfo_k_post_attn_setup", None, u16p, u16p, u16p, u16p, u16p, C.c_float, u16p, u16p, u16p, i32)
_sig("tfo_k_layer_tail", None, u16p, u16p, u16p, u16p, u16p, C.c_float, C.c_float, i32)
_sig("tfo_layer_tail_ref", None, u16p, u16p, u16p, u16p, u16p, C.c_float, C.c_float, f32p, i32)


def _u16(a):
    return np.ascontiguousarray(a, np.uint16)


def k_post_attn_setup(hidden_bits, attn_bits, w_post_bits, w_pre_bits, w_pre2_bits, eps: float):
    """-> (hidden', dense_x, routed_x, router_x) as fp16 bit arrays (fused.metal:190-269)."""
    hidden = _u16(hidden_bits).copy()
    dense, routed, router = np.empty_like(hidden), np.empty_like(hidden), np.empty_like(hidden)
    lib.tfo_k_post_attn_setup(hidden, _u16(attn_bits), _u16(w_post_bits), _u16(w_pre_bits), _u16(w_pre2_bits), eps, dense, routed,
                              router, hidden.size)
    return hidden, dense, routed, router


def k_layer_tail(h2_bits, h1_bits, hidden_bits, w_postffn2_bits, w_postffn_bits, eps: float, layer_scalar: float) -> np.ndarray:
    hidden = _u16(hidden_bits).copy()
    lib.tfo_k_layer_tail(_u16(h2_bits), _u16(h1_bits), hidden, _u16(w_postffn2_bits), _u16(w_postffn_bits), eps, layer_scalar, hidden.size)
    return hidden


def layer_tail_ref(h2_bits, h1_bits, hidden_bits, w_postffn2_bits, w_postffn_bits, eps: float, layer_scalar: float) -> np.ndarray:
    hidden = _u16(hidden_bits)
    out = np.empty(hidden.size, np.float32)
    lib.tfo_layer_tail_ref(_u16(h2_bits), _u16(h1_bits), hidden, _u16(w_postffn2_bits), _u16(w_postffn_bits), eps, layer_scalar, out,
                           hidden.size)
    return out


# ---- neighbours of the output head --------------------------------------------------------
_sig("tfo_embed_lookup_int4", None, u8p, u16p, u16p, C.c_uint32, i32, C.c_float, f32p)
_sig("tfo_logit_softcap_softmax_ref", None, f32p, i32, C.c_float, f32p)
_sig("tfo_sampler_xorshift64", C.c_uint64, C.POINTER(C.c_uint64))
_sig("tfo_sampler_gumbel", C.c_float, C.c_uint64, C.c_uint32, C.c_uint32)
_sig("tfo_sample", C.c_uint32, u16p, C.c_uint32, C.c_float, C.c_uint32, C.c_float, C.c_uint64, C.c_uint32)
_sig("tfo_sample_topk64", C.c_uint32, u16p, C.c_uint32, C.c_float, C.c_float, C.c_uint64)


def embed_lookup_int4(W, S, B, token: int, out_scale: float) -> np.ndarray:
    W, S, B = _wsb(W, S, B)
    d = W.shape[1] * 2
    out = np.empty(d, np.float32)
    lib.tfo_embed_lookup_int4(W, S, B, token, d, out_scale, out)
    return out


def logit_softcap_softmax_ref(x, softcap: float) -> np.ndarray:
    x = _flat32(x)
    out = np.empty_like(x)
    lib.tfo_logit_softcap_softmax_ref(x, x.size, softcap, out)
    return out


def sampler_xorshift64(state: int):
    """-> (output, new state)"""
    s = C.c_uint64(state)
    out = lib.tfo_sampler_xorshift64(C.byref(s))
    return int(out), int(s.value)


def sampler_gumbel(seed: int, position: int, row: int) -> float:
    return float(lib.tfo_sampler_gumbel(seed, position, row))


def sample(probs_bits, temperature: float, top_k: int, top_p: float, seed: int, position: int = 0) -> int:
    p = np.ascontiguousarray(probs_bits, np.uint16)
    return int(lib.tfo_sample(p, p.size, temperature, top_k, top_p, seed, position))


def sample_topk64(probs_bits, temperature: float, top_p: float, seed: int) -> int:
    p = np.ascontiguousarray(probs_bits, np.uint16)
    return int(lib.tfo_sample_topk64(p, p.size, temperature, top_p, seed))


# ---- MoE ---------------------------------------------------------------------------------
_pp = C.POINTER(C.c_void_p)
_sig("tfo_moe_run_ffn", None, C.c_void_p, C.POINTER(ExpertOffsets), f32p, f32p, i32, i32)
_sig("tfo_moe_apply_streamed_routed", None, _pp, C.POINTER(ExpertOffsets), f32p, f32p, f32p, i32, f32p, i32, i32, i32)
_sig("tfo_router_reference", None, u8p, u16p, u16p, f32p, f32p, f32p, i32, i32, i32, u32p, f32p, C.c_void_p)
_sig("tfo_shared_expert_ref", None, u8p, u16p, u16p, u8p, u16p, u16p, u8p, u16p, u16p, f32p, f32p, i32, i32, i32)
_sig("tfo_k_router_logits", None, u8p, u16p, u16p, u16p, u16p, f32p, i32, i32)
_sig("tfo_k_prefill_router_logits", None, u8p, u16p, u16p, u16p, u16p, f32p, i32, i32)
_sig("tfo_k_router_topk", None, f32p, u16p, i32, i32, u32p, u16p)
_sig("tfo_k_moe_phase1", None, _pp, C.POINTER(ExpertOffsets), u16p, u16p, i32, i32, i32)
_sig("tfo_k_moe_phase2", None, _pp, C.POINTER(ExpertOffsets), u16p, u16p, u16p, u16p, i32, i32)


def make_blob(gate, up, down):
    """Pack one routed expert the way the reference's tests do: gate W,S,B, up W,S,B, down W,S,B
    back to back (MoEFusedFFNTests.swift:161-197).  gate/up/down are (packed, scales, biases)."""
    parts, offs, pos = [], [], 0
    for packed, s, b in (gate, up, down):
        for arr in (np.ascontiguousarray(packed, np.uint8), np.ascontiguousarray(s, "<u2"), np.ascontiguousarray(b, "<u2")):
            raw = arr.view(np.uint8).ravel()
            offs.append(pos)
            parts.append(raw)
            pos += raw.size
    return np.concatenate(parts), ExpertOffsets(*offs)


def _blob_ptrs(blobs):
    arr = (C.c_void_p * len(blobs))()
    keep = []
    for i, b in enumerate(blobs):
        b = np.ascontiguousarray(b, np.uint8)
        keep.append(b)
        arr[i] = b.ctypes.data
    return arr, keep


def moe_run_ffn(blob, off: ExpertOffsets, x, d: int, f: int) -> np.ndarray:
    blob = np.ascontiguousarray(blob, np.uint8)
    y = np.empty(d, np.float32)
    lib.tfo_moe_run_ffn(blob.ctypes.data, C.byref(off), _flat32(x), y, d, f)
    return y


def moe_apply_streamed_routed(blobs, off: ExpertOffsets, x, residual, routing_w, d: int, f: int, threads: int = 1) -> np.ndarray:
    ptrs, _keep = _blob_ptrs(blobs)
    y = np.empty(d, np.float32)
    lib.tfo_moe_apply_streamed_routed(ptrs, C.byref(off), _flat32(x), _flat32(residual), _flat32(routing_w),
                                      len(blobs), y, d, f, threads)
    return y


def router_reference(W, S, B, hidden, effective_scale, expert_scale, top_k: int = 8):
    W, S, B = _wsb(W, S, B)
    e, d = W.shape
    k = min(top_k, e)
    idx = np.zeros(k, np.uint32)
    wts = np.zeros(k, np.float32)
    logits = np.zeros(e, np.float32)
    lib.tfo_router_reference(W, S, B, _flat32(hidden), _flat32(effective_scale), _flat32(expert_scale), e, d, top_k,
                             idx, wts, logits.ctypes.data)
    return idx, wts, logits


def shared_expert_ref(gate, up, down, x, threads: int = 1) -> np.ndarray:
    gW, gS, gB = _wsb(*gate)
    uW, uS, uB = _wsb(*up)
    dW, dS, dB = _wsb(*down)
    f, d = gW.shape[0], gW.shape[1] * 2
    y = np.empty(d, np.float32)
    lib.tfo_shared_expert_ref(gW, gS, gB, uW, uS, uB, dW, dS, dB, _flat32(x), y, d, f, threads)
    return y


def k_router_logits(W, S, B, hidden_bits, eff_bits, prefill_order: bool = False) -> np.ndarray:
    W, S, B = _wsb(W, S, B)
    e, d = W.shape
    logits = np.empty(e, np.float32)
    fn = lib.tfo_k_prefill_router_logits if prefill_order else lib.tfo_k_router_logits
    fn(W, S, B, np.ascontiguousarray(hidden_bits, np.uint16), np.ascontiguousarray(eff_bits, np.uint16), logits, e, d)
    return logits


def k_router_topk(logits, per_expert_scale_bits, top_k: int = 8):
    logits = _flat32(logits)
    idx = np.zeros(top_k, np.uint32)
    w = np.zeros(top_k, np.uint16)
    lib.tfo_k_router_topk(logits, np.ascontiguousarray(per_expert_scale_bits, np.uint16), logits.size, top_k, idx, w)
    return idx, w


def k_moe_phase1(blobs, off: ExpertOffsets, x_bits, d: int, f: int) -> np.ndarray:
    ptrs, _keep = _blob_ptrs(blobs)
    acts = np.zeros(len(blobs) * f, np.uint16)
    lib.tfo_k_moe_phase1(ptrs, C.byref(off), np.ascontiguousarray(x_bits, np.uint16), acts, d, f, len(blobs))
    return acts


def k_moe_phase2(blobs, off: ExpertOffsets, acts_bits, routing_w_bits, residual_bits, d: int, f: int) -> np.ndarray:
    assert len(blobs) == 8
    ptrs, _keep = _blob_ptrs(blobs)
    y = np.zeros(d, np.uint16)
    lib.tfo_k_moe_phase2(ptrs, C.byref(off), np.ascontiguousarray(acts_bits, np.uint16),
                         np.ascontiguousarray(routing_w_bits, np.uint16), np.ascontiguousarray(residual_bits, np.uint16), y, d, f)
    return y


# ---- lm_head -----------------------------------------------------------------------------------
_sig("tfo_lm_head_cpu_greedy", C.c_uint32, u16p, u16p, u8p, u16p, u16p, i32, i64, C.c_float, C.c_void_p, i32)


def lm_head_cpu_greedy(hidden_bits, norm_bits, W, S, B, eps: float = 1e-6, threads: int = 1, want_logits: bool = False):
    W, S, B = _wsb(W, S, B)
    v, d = W.shape[0], W.shape[1] * 2
    logits = np.empty(v, np.float32) if want_logits else None
    tok = lib.tfo_lm_head_cpu_greedy(np.ascontiguousarray(hidden_bits, np.uint16), np.ascontiguousarray(norm_bits, np.uint16),
                                     W, S, B, d, v, eps, logits.ctypes.data if want_logits else None, threads)
    return (int(tok), logits) if want_logits else int(tok)


# ---- prefill -------------------------------------------------------------------------------------
_pairp = np.ctypeslib.ndpointer(PAIR_DTYPE, flags="C_CONTIGUOUS")
_sig("tfo_prefill_make_pairs", None, u32p, u16p, i32, i32, _pairp)
_sig("tfo_prefill_group_pairs", i32, _pairp, i64, i32, i32, i32, i32, C.c_void_p, i32, _pairp, u32p, u32p,
     np.ctypeslib.ndpointer(GROUP_DTYPE, flags="C_CONTIGUOUS"), C.POINTER(i32),
     np.ctypeslib.ndpointer(TILE_DTYPE, flags="C_CONTIGUOUS"), C.POINTER(i32))
_sig("tfo_prefill_route_partials", None, _pairp, i64, i32, u16p, i32, u8p, i64, C.POINTER(ExpertOffsets), i32, i32, i32,
     C.c_uint16, u16p, i32)
_sig("tfo_prefill_reduce_token_major", None, u16p, u16p, i32, i32, i32, u16p)
_sig("tfo_qmm_cpu_reference", None, u8p, u16p, u16p, u16p, i32, i32, i32, f32p, i32)
_sig("tfo_k_prefill_int4_row", C.c_float, u8p, u16p, u16p, u16p, i32, i32)
_sig("tfo_prefill_cpu_int4_dot", C.c_float, u8p, i64, i64, i64, i64, i32, i32, f32p)

GROUP_ERRORS = {
    1: "invalidQueryCount", 2: "invalidTopK", 3: "invalidNumExperts", 4: "invalidTileExpertCount",
    5: "pairCountMismatch", 6: "tokenOutOfRange", 7: "rankOutOfRange", 8: "expertOutOfRange",
    9: "duplicateTokenRank", 10: "expertSortKeyCountMismatch",
}


class GroupingError(ValueError):
    def __init__(self, code: int):
        super().__init__(GROUP_ERRORS.get(code, str(code)))
        self.code = code
        self.case = GROUP_ERRORS.get(code, str(code))


def make_pairs(indices, weights_f16_bits, query_count: int, top_k: int) -> np.ndarray:
    pairs = np.zeros(query_count * top_k, PAIR_DTYPE)
    lib.tfo_prefill_make_pairs(np.ascontiguousarray(indices, np.uint32), np.ascontiguousarray(weights_f16_bits, np.uint16),
                               query_count, top_k, pairs)
    return pairs


def pairs_from_tuples(tuples) -> np.ndarray:
    arr = np.zeros(len(tuples), PAIR_DTYPE)
    for i, (t, e, r, w) in enumerate(tuples):
        arr[i] = (t, e, r, w)
    return arr


def group_pairs(pairs: np.ndarray, query_count: int, top_k: int, num_experts: int, tile_expert_count: int = 16,
                expert_sort_keys=None):
    pairs = np.ascontiguousarray(pairs, PAIR_DTYPE)
    n = pairs.size
    cap = max(1, min(max(num_experts, 1), max(n, 1)))
    sorted_pairs = np.zeros(max(n, 1), PAIR_DTYPE)
    offs = np.zeros(max(num_experts, 1), np.uint32)
    cnts = np.zeros(max(num_experts, 1), np.uint32)
    groups = np.zeros(cap, GROUP_DTYPE)
    tiles = np.zeros(cap, TILE_DTYPE)
    ng, nt = i32(0), i32(0)
    keys, nkeys = None, 0
    if expert_sort_keys is not None:
        keys_arr = np.ascontiguousarray(expert_sort_keys, np.uint64)
        keys, nkeys = keys_arr.ctypes.data, keys_arr.size
    rc = lib.tfo_prefill_group_pairs(pairs if n else np.zeros(1, PAIR_DTYPE), n, query_count, top_k, num_experts,
                                     tile_expert_count, keys, nkeys, sorted_pairs, offs, cnts, groups, C.byref(ng),
                                     tiles, C.byref(nt))
    if rc != 0:
        raise GroupingError(rc)
    return dict(sorted_pairs=sorted_pairs[:n], per_expert_offsets=offs[:num_experts], per_expert_counts=cnts[:num_experts],
                groups=groups[:ng.value], tiles=tiles[:nt.value], query_count=query_count)


def prefill_route_partials(sorted_pairs, query_count, hidden_bits, hidden_stride, pool, pool_stride, off: ExpertOffsets,
                           top_k, d, f, fill_bits=0xD630, threads: int = 1) -> np.ndarray:
    sorted_pairs = np.ascontiguousarray(sorted_pairs, PAIR_DTYPE)
    out = np.zeros(query_count * top_k * d, np.uint16)
    lib.tfo_prefill_route_partials(sorted_pairs, sorted_pairs.size, query_count, np.ascontiguousarray(hidden_bits, np.uint16),
                                   hidden_stride, np.ascontiguousarray(pool, np.uint8), pool_stride, C.byref(off), top_k, d, f,
                                   fill_bits, out, threads)
    return out


def prefill_reduce_token_major(partials_bits, weights_bits, rows, top_k, d) -> np.ndarray:
    out = np.zeros(rows * d, np.uint16)
    lib.tfo_prefill_reduce_token_major(np.ascontiguousarray(partials_bits, np.uint16), np.ascontiguousarray(weights_bits, np.uint16),
                                       rows, top_k, d, out)
    return out


def qmm_cpu_reference(W, S, B, x_bits, m, n, k, threads: int = 1) -> np.ndarray:
    W, S, B = _wsb(W, S, B)
    out = np.zeros((m, n), np.float32)
    lib.tfo_qmm_cpu_reference(W, S, B, np.ascontiguousarray(x_bits, np.uint16), m, n, k, out, threads)
    return out


def k_prefill_int4_row(W, S, B, x_bits, row: int) -> float:
    W, S, B = _wsb(W, S, B)
    return float(lib.tfo_k_prefill_int4_row(W, S, B, np.ascontiguousarray(x_bits, np.uint16), row, W.shape[1] * 2))


# ---- fp16 helpers on arrays (numpy's float16 is IEEE RNE, checked against tfo_f16_bits in the tests) ----
def to_f16_bits(x) -> np.ndarray:
    return np.asarray(x, np.float32).astype(np.float16).view(np.uint16)


def from_f16_bits(b) -> np.ndarray:
    return np.asarray(b, np.uint16).view(np.float16).astype(np.float32)


# ---- decode attention ----------------------------------------------------------------------
_sig("tfo_attention_ref", None, f32p, f32p, f32p, i32, i32, i32, i32, i32, C.c_float, f32p)
_sig("tfo_k_attention_split", None, u16p, u16p, u16p, i32, i32, i32, i32, i32, i32, i32, C.c_float, i32, u16p)
_sig("tfo_attention_split_geometry", None, C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, i32, C.POINTER(C.c_int32))


def attention_ref(q, k, v, head_dim: int, num_q_heads: int, num_kv_heads: int, seq_len: int, window=None, scale=None) -> np.ndarray:
    """AttentionRef.apply: q [Hq, D], k / v [T, Hkv, D] as float32 -> [Hq * D] float32."""
    out = np.empty(num_q_heads * head_dim, np.float32)
    lib.tfo_attention_ref(_flat32(q), _flat32(k), _flat32(v), head_dim, num_q_heads, num_kv_heads, seq_len,
                          -1 if window is None else int(window), 0.0 if scale is None else float(scale), out)
    return out


def k_attention_split(q_bits, k_bits, v_bits, head_dim, num_q_heads, num_kv_heads, seq_len, kv_start, chunk_len, num_chunks, scale,
                      ring_capacity=0) -> np.ndarray:
    out = np.empty(num_q_heads * head_dim, np.uint16)
    lib.tfo_k_attention_split(_u16(q_bits), _u16(k_bits), _u16(v_bits), head_dim, num_q_heads, num_kv_heads, seq_len, kv_start,
                              chunk_len, num_chunks, float(scale), ring_capacity, out)
    return out


def attention_split_geometry(num_q_heads, num_kv_heads, seq_len, kv_start, prefer_gqa_swa: bool) -> dict:
    out = (C.c_int32 * 5)()
    lib.tfo_attention_split_geometry(num_q_heads, num_kv_heads, seq_len, kv_start, int(prefer_gqa_swa), out)
    return dict(effectiveLength=out[0], numChunks=out[1], chunkLength=out[2], partialThreadgroups=out[3], useSWAGroupedPartial=bool(out[4]))


# ---- RoPE and the Q/K/V epilogue -------------------------------------------------------------
_sig("tfo_rope_neox_ref", None, f32p, i32, i32, i32, i32, i32, C.c_float, f32p)
_sig("tfo_k_rope_neox", None, u16p, i32, i32, i32, i32, C.c_uint32, C.c_float)
_sig("tfo_k_fused_qkv_epilogue", None, u16p, u16p, u16p, u16p, u16p, i32, i32, i32, C.c_uint32, C.c_float, i32, C.c_float)


def rope_neox_ref(x, num_tokens, num_heads, head_dim, rotated_pairs, position, theta) -> np.ndarray:
    x = _flat32(x)
    out = np.empty_like(x)
    lib.tfo_rope_neox_ref(x, num_tokens, num_heads, head_dim, rotated_pairs, position, float(theta), out)
    return out


def k_rope_neox(bits, num_tokens, num_heads, head_dim, rotated_pairs, position, theta) -> np.ndarray:
    data = _u16(bits).copy()
    lib.tfo_k_rope_neox(data, num_tokens, num_heads, head_dim, rotated_pairs, position, float(theta))
    return data


def k_fused_qkv_epilogue(q_bits, k_bits, v_bits, q_weight_bits, k_weight_bits, head_dim, num_q_heads, num_kv_heads, position, theta,
                         rotated_pairs, eps):
    q, k, v = _u16(q_bits).copy(), _u16(k_bits).copy(), _u16(v_bits).copy()
    lib.tfo_k_fused_qkv_epilogue(q, k, v, _u16(q_weight_bits), _u16(k_weight_bits), head_dim, num_q_heads, num_kv_heads, position,
                                 float(theta), rotated_pairs, float(eps))
    return q, k, v


# ---- causal attention of a block of query tokens (prefill) ------------------------------------
_sig("tfo_prefill_attention_ref", None, f32p, f32p, f32p, i32, i32, i32, i32, i32, i32, i32, i32, i32, C.c_float, f32p)
_sig("tfo_k_prefill_attention", None, u16p, u16p, u16p, u16p, i32, i32, i32, i32, i32, i32, i32, i32, i32, i32, C.c_float, i32)


def prefill_attention_ref(q, k, v, start, chunk, head_dim, q_heads, kv_heads, kv_valid, window, q_stride, kv_stride, scale) -> np.ndarray:
    out = np.empty(chunk * q_heads * head_dim, np.float32)
    lib.tfo_prefill_attention_ref(_flat32(q), _flat32(k), _flat32(v), start, chunk, head_dim, q_heads, kv_heads, kv_valid, window, q_stride,
                                  kv_stride, float(scale), out)
    return out


def k_prefill_attention(q_bits, k_bits, v_bits, out_bits, start, chunk, head_dim, q_heads, kv_heads, kv_valid, window, q_stride, kv_stride,
                        o_stride, scale, ring_capacity=0) -> np.ndarray:
    out = _u16(out_bits).copy()
    lib.tfo_k_prefill_attention(_u16(q_bits), _u16(k_bits), _u16(v_bits), out, start, chunk, head_dim, q_heads, kv_heads, kv_valid, window,
                                q_stride, kv_stride, o_stride, float(scale), ring_capacity)
    return out
