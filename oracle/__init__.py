"""CPU oracle for the decode hot path: ctypes binding of libfk_oracle.so.

TEST INFRASTRUCTURE ONLY.  Importable from tests/, from the smoke check and
from the benchmark's cpu_baseline leg; the product package never imports it.

bf16 tensors are numpy uint16 arrays holding the bit patterns.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfk_oracle.so")


def build() -> str:
    """Compile the C restatement in place (gcc); returns the library path."""
    subprocess.check_call(["make", "-C", _HERE, "-B", "libfk_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load() -> C.CDLL:
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()

_u16p = C.POINTER(C.c_uint16)
_u32p = C.POINTER(C.c_uint32)
_f32p = C.POINTER(C.c_float)


class Weight(C.Structure):
    """Mirror of `fko_weight`: one [n, k] matrix, MLX-affine (bits 4/8) or dense bf16 (bits 16)."""

    _fields_ = [
        ("w", C.c_void_p),
        ("scales", _u16p),
        ("biases", _u16p),
        ("n", C.c_int64),
        ("k", C.c_int64),
        ("bits", C.c_int),
        ("group", C.c_int),
    ]


class Layer(C.Structure):
    _fields_ = [
        ("input_norm", _u16p),
        ("post_norm", _u16p),
        ("wq", Weight), ("wk", Weight), ("wv", Weight), ("wo", Weight),
        ("wgate", Weight), ("wup", Weight), ("wdown", Weight),
        ("bq", _u16p), ("bk", _u16p), ("bv", _u16p),
        ("q_norm", _u16p), ("k_norm", _u16p),
        ("cache_k", _u16p), ("cache_v", _u16p),
        ("ck_packed", _u32p), ("ck_scales", _u16p), ("ck_biases", _u16p),
        ("cv_packed", _u32p), ("cv_scales", _u16p), ("cv_biases", _u16p),
    ]


class Model(C.Structure):
    _fields_ = [
        ("n_layers", C.c_int64), ("hidden", C.c_int64), ("n_heads", C.c_int64), ("n_kv", C.c_int64),
        ("head_dim", C.c_int64), ("inter", C.c_int64), ("vocab", C.c_int64),
        ("eps", C.c_float), ("theta", C.c_float), ("attn_scale", C.c_float), ("embed_scale", C.c_float),
        ("swiglu_variant", C.c_int),
        ("capacity", C.c_uint32),
        ("embed", Weight),
        ("lm_head", Weight),
        ("final_norm", _u16p),
        ("layers", C.POINTER(Layer)),
        ("kv_bits", C.c_int), ("kv_group", C.c_int),
    ]


def _p(a: np.ndarray | None, ty):
    if a is None:
        return C.cast(None, ty)
    assert a.flags["C_CONTIGUOUS"], "oracle wants contiguous arrays"
    return a.ctypes.data_as(ty)


# ------------------------------------------------------------------ bf16 helpers

def f32_to_bf16(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    _lib.fko_f32_to_bf16(_p(a, _f32p), _p(out, _u16p), C.c_int64(a.size))
    return out


def bf16_to_f32(a: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.uint16)
    return (a.astype(np.uint32) << 16).view(np.float32)


def num_threads() -> int:
    return int(_lib.fko_num_threads())


def set_num_threads(n: int) -> None:
    _lib.fko_set_num_threads(C.c_int(n))


def set_accum_mode(mode: int) -> None:
    """Accumulation of every projection: 0 double (default), 1 fp32 per element in order, 2 fp32 qdot form
    per group (dense rows: 32 interleaved partial sums, pairwise tree)."""
    _lib.fko_set_accum_mode(C.c_int(mode))


def get_accum_mode() -> int:
    return int(_lib.fko_get_accum_mode())


def synth_fill(count: int, seed: int, mean: float, std: float, kind: int, row_len: int = 0, tau: float = 0.0,
               loud_rows: int = 0, loud_gain: float = 1.0) -> np.ndarray:
    """The GPU library's host-reproducible synthetic fill (fk_synth_fill_exact), bit for bit:
    kind 3 -> float32 array, kind 4 -> bf16 bit patterns (uint16)."""
    assert kind in (3, 4)
    out = np.empty(count, dtype=np.float32 if kind == 3 else np.uint16)
    _lib.fko_synth_fill(C.c_void_p(out.ctypes.data), C.c_int64(count), C.c_uint64(seed), C.c_float(mean), C.c_float(std),
                        C.c_int(kind), C.c_int64(row_len), C.c_float(tau), C.c_int64(loud_rows), C.c_float(loud_gain))
    return out


# ------------------------------------------------------------------ weights

class QWeight:
    """Host copy of one matrix; keeps the numpy arrays alive for the ctypes view."""

    def __init__(self, w, scales, biases, n, k, bits, group=64):
        self.w = np.ascontiguousarray(w)
        self.scales = None if scales is None else np.ascontiguousarray(scales, dtype=np.uint16)
        self.biases = None if biases is None else np.ascontiguousarray(biases, dtype=np.uint16)
        self.n, self.k, self.bits, self.group = int(n), int(k), int(bits), int(group)

    @property
    def c(self) -> Weight:
        return Weight(self.w.ctypes.data, _p(self.scales, _u16p), _p(self.biases, _u16p),
                      self.n, self.k, self.bits, self.group)

    @property
    def nbytes(self) -> int:
        b = self.w.nbytes
        if self.scales is not None:
            b += self.scales.nbytes + self.biases.nbytes
        return b


def quantize(w: np.ndarray, bits: int = 4, group: int = 64) -> QWeight:
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, k = w.shape
    packed = np.empty((n, k * bits // 32), dtype=np.uint32)
    scales = np.empty((n, k // group), dtype=np.uint16)
    biases = np.empty((n, k // group), dtype=np.uint16)
    _lib.fko_quantize_affine(_p(w, _f32p), C.c_int64(n), C.c_int64(k), C.c_int(bits), C.c_int(group),
                             _p(packed, _u32p), _p(scales, _u16p), _p(biases, _u16p))
    return QWeight(packed, scales, biases, n, k, bits, group)


def dense(w_bf16: np.ndarray) -> QWeight:
    n, k = w_bf16.shape
    return QWeight(np.ascontiguousarray(w_bf16, dtype=np.uint16), None, None, n, k, 16, 0)


def unpack_codes(W: QWeight) -> np.ndarray:
    out = np.empty((W.n, W.k), dtype=np.uint8)
    _lib.fko_unpack_codes(_p(W.w, _u32p), C.c_int64(W.n), C.c_int64(W.k), C.c_int(W.bits),
                          out.ctypes.data_as(C.POINTER(C.c_uint8)))
    return out


def dequantize(W: QWeight) -> np.ndarray:
    if W.bits == 16:
        return bf16_to_f32(W.w)
    out = np.empty((W.n, W.k), dtype=np.float32)
    _lib.fko_dequantize(_p(W.w, _u32p), _p(W.scales, _u16p), _p(W.biases, _u16p), C.c_int64(W.n),
                        C.c_int64(W.k), C.c_int(W.bits), C.c_int(W.group), _p(out, _f32p))
    return out


def dequantize_rows(W: QWeight, r0: int, r1: int) -> np.ndarray:
    """Rows [r0, r1) of dequantize(W) without materialising the whole matrix."""
    if W.bits == 16:
        return bf16_to_f32(W.w[r0:r1])
    sub = QWeight(W.w[r0:r1], W.scales[r0:r1], W.biases[r0:r1], r1 - r0, W.k, W.bits, W.group)
    return dequantize(sub)


# ------------------------------------------------------------------ operators

def linear_acc(W: QWeight, x: np.ndarray) -> np.ndarray:
    acc = np.empty(W.n, dtype=np.float32)
    _lib.fko_linear_acc(C.byref(W.c), _p(x, _u16p), _p(acc, _f32p))
    return acc


def qgemv(W: QWeight, x: np.ndarray, bias: np.ndarray | None = None) -> np.ndarray:
    y = np.empty(W.n, dtype=np.uint16)
    _lib.fko_qgemv(C.byref(W.c), _p(x, _u16p), _p(bias, _u16p), _p(y, _u16p))
    return y


def linear_residual(W: QWeight, x, res, res2=None) -> np.ndarray:
    y = np.empty(W.n, dtype=np.uint16)
    _lib.fko_linear_residual(C.byref(W.c), _p(x, _u16p), _p(res, _u16p), _p(res2, _u16p), _p(y, _u16p))
    return y


def rmsnorm(x, w, eps: float) -> np.ndarray:
    y = np.empty(x.shape, dtype=np.uint16)
    _lib.fko_rmsnorm(_p(x, _u16p), _p(w, _u16p), C.c_int64(x.size), C.c_float(eps), _p(y, _u16p))
    return y


def rmsnorm_qkv(x, norm_w, eps, Wq, Wk, Wv, bq=None, bk=None, bv=None):
    q = np.empty(Wq.n, dtype=np.uint16)
    k = np.empty(Wk.n, dtype=np.uint16)
    v = np.empty(Wv.n, dtype=np.uint16)
    _lib.fko_rmsnorm_qkv(_p(x, _u16p), _p(norm_w, _u16p), C.c_float(eps), C.byref(Wq.c), C.byref(Wk.c),
                         C.byref(Wv.c), _p(bq, _u16p), _p(bk, _u16p), _p(bv, _u16p), _p(q, _u16p),
                         _p(k, _u16p), _p(v, _u16p))
    return q, k, v


_lib.fko_swiglu_scalar.restype = C.c_uint16


def swiglu_scalar(g: float, u: float, variant: int) -> int:
    return int(_lib.fko_swiglu_scalar(C.c_float(g), C.c_float(u), C.c_int(variant)))


def gateup_swiglu(x, norm_w, eps, Wg, Wu, variant=0) -> np.ndarray:
    out = np.empty(Wg.n, dtype=np.uint16)
    _lib.fko_gateup_swiglu(_p(x, _u16p), _p(norm_w, _u16p), C.c_float(eps), C.byref(Wg.c), C.byref(Wu.c),
                           C.c_int(variant), _p(out, _u16p))
    return out


def rope_q(q, n_heads, head_dim, rope_dims, theta, pos) -> np.ndarray:
    q = np.array(q, dtype=np.uint16, copy=True)
    _lib.fko_rope_q(_p(q, _u16p), C.c_int64(n_heads), C.c_int64(head_dim), C.c_int64(rope_dims),
                    C.c_float(theta), C.c_uint32(pos))
    return q


def rope_kv_store(k, v, n_kv, head_dim, rope_dims, theta, pos, write_offset, capacity, cache_k, cache_v):
    _lib.fko_rope_kv_store(_p(k, _u16p), _p(v, _u16p), C.c_int64(n_kv), C.c_int64(head_dim),
                           C.c_int64(rope_dims), C.c_float(theta), C.c_uint32(pos), C.c_uint32(write_offset),
                           C.c_uint32(capacity), _p(cache_k, _u16p), _p(cache_v, _u16p))


def headnorm_rope(x, w, n_heads, head_dim, rope_dims, eps, theta, pos) -> np.ndarray:
    x = np.array(x, dtype=np.uint16, copy=True)
    _lib.fko_headnorm_rope(_p(x, _u16p), _p(w, _u16p), C.c_int64(n_heads), C.c_int64(head_dim),
                           C.c_int64(rope_dims), C.c_float(eps), C.c_float(theta), C.c_uint32(pos))
    return x


def kv_store(k, v, n_kv, k_dim, v_dim, write_offset, capacity, cache_k, cache_v):
    _lib.fko_kv_store(_p(k, _u16p), _p(v, _u16p), C.c_int64(n_kv), C.c_int64(k_dim), C.c_int64(v_dim),
                      C.c_uint32(write_offset), C.c_uint32(capacity), _p(cache_k, _u16p), _p(cache_v, _u16p))


def sdpa_decode(q, cache_k, cache_v, n_heads, n_kv, qk_dim, v_dim, kv_len, capacity, scale) -> np.ndarray:
    out = np.empty(n_heads * v_dim, dtype=np.uint16)
    _lib.fko_sdpa_decode(_p(q, _u16p), _p(cache_k, _u16p), _p(cache_v, _u16p), C.c_int64(n_heads),
                         C.c_int64(n_kv), C.c_int64(qk_dim), C.c_int64(v_dim), C.c_uint32(kv_len),
                         C.c_uint32(capacity), C.c_float(scale), _p(out, _u16p))
    return out


def sdpa_decode_split_q(q, n_heads, q0_dim, q1_dim, rope_dims, traditional, theta, cache_k, cache_v, n_kv, v_dim,
                        kv_len, capacity, scale) -> np.ndarray:
    """q: packed [n_heads, q0_dim + q1_dim]; Q1's first rope_dims are rotated at kv_len - 1 in fp32."""
    q = np.ascontiguousarray(q, dtype=np.uint16).reshape(-1)
    out = np.empty(n_heads * v_dim, dtype=np.uint16)
    stride = q0_dim + q1_dim
    _lib.fko_sdpa_decode_split_q(_p(q, _u16p), C.c_int64(stride), _p(q[q0_dim:], _u16p), C.c_int64(stride),
                                 C.c_int64(q0_dim), C.c_int64(q1_dim), C.c_int64(rope_dims), C.c_int(int(traditional)),
                                 C.c_float(theta), _p(cache_k, _u16p), _p(cache_v, _u16p), C.c_int64(n_heads),
                                 C.c_int64(n_kv), C.c_int64(v_dim), C.c_uint32(kv_len), C.c_uint32(capacity),
                                 C.c_float(scale), _p(out, _u16p))
    return out


def kv_store_split(k0, k0_stride, k1, k1_heads, v, v_stride, n_kv, k0_dim, k1_dim, v_dim, rope_dims, traditional, theta,
                   pos, write_offset, capacity, cache_k, cache_v):
    """k0 / v: flat uint16 arrays whose head rows start k0_stride / v_stride elements apart."""
    _lib.fko_kv_store_split(_p(k0, _u16p), C.c_int64(k0_stride), _p(k1, _u16p), C.c_int64(k1_heads), _p(v, _u16p),
                            C.c_int64(v_stride), C.c_int64(n_kv), C.c_int64(k0_dim), C.c_int64(k1_dim), C.c_int64(v_dim),
                            C.c_int64(rope_dims), C.c_int(int(traditional)), C.c_float(theta), C.c_uint32(pos),
                            C.c_uint32(write_offset), C.c_uint32(capacity), _p(cache_k, _u16p), _p(cache_v, _u16p))


def softmax_topk_route(logits, top_k, scale):
    """logits bf16 [rows, row_n]; scale: one bf16 value or bf16 [rows, top_k].  Returns (idx u32, weight bf16)."""
    logits = np.ascontiguousarray(logits, dtype=np.uint16)
    rows, row_n = (1, logits.size) if logits.ndim == 1 else logits.shape
    scale = np.ascontiguousarray(scale, dtype=np.uint16).reshape(-1)
    idx, weight = np.empty(rows * top_k, np.uint32), np.empty(rows * top_k, np.uint16)
    _lib.fko_softmax_topk_route(_p(logits, _u16p), C.c_int64(rows), C.c_int64(row_n), C.c_int64(top_k), _p(scale, _u16p),
                                C.c_int(int(scale.size > 1)), _p(idx, C.POINTER(C.c_uint32)), _p(weight, _u16p))
    return idx.reshape(rows, top_k), weight.reshape(rows, top_k)


def sdpa_prefill(q, cache_k, cache_v, rows, n_heads, n_kv, dim, kv_len, capacity, scale) -> np.ndarray:
    """Causal attention of `rows` rows; kv_len counts them (row r sees kv_len - rows + r + 1 positions)."""
    out = np.empty(rows * n_heads * dim, dtype=np.uint16)
    _lib.fko_sdpa_prefill(_p(q, _u16p), _p(cache_k, _u16p), _p(cache_v, _u16p), C.c_int64(rows), C.c_int64(n_heads),
                          C.c_int64(n_kv), C.c_int64(dim), C.c_uint32(kv_len), C.c_uint32(capacity), C.c_float(scale),
                          _p(out, _u16p))
    return out


def embed_lookup(E: QWeight, token: int, out_scale: float = 1.0) -> np.ndarray:
    x = np.empty(E.k, dtype=np.uint16)
    _lib.fko_embed_lookup(C.byref(E.c), C.c_uint32(token), C.c_float(out_scale), _p(x, _u16p))
    return x


def final_rmsnorm_lm_head(x, norm_w, eps, W: QWeight) -> np.ndarray:
    logits = np.empty(W.n, dtype=np.uint16)
    _lib.fko_final_rmsnorm_lm_head(_p(x, _u16p), _p(norm_w, _u16p), C.c_float(eps), C.byref(W.c),
                                   _p(logits, _u16p))
    return logits


_lib.fko_argmax.restype = C.c_uint32
_lib.fko_top2_margin.restype = C.c_float
_lib.fko_decoder_step.restype = C.c_uint32


def argmax(logits) -> int:
    return int(_lib.fko_argmax(_p(logits, _u16p), C.c_int64(logits.size)))


def top2_margin(logits) -> float:
    return float(_lib.fko_top2_margin(_p(logits, _u16p), C.c_int64(logits.size)))


def decoder_step(model: Model, token: int, offset: int, logits: np.ndarray | None = None):
    margin = C.c_float(0.0)
    nxt = _lib.fko_decoder_step(C.byref(model), C.c_uint32(token), C.c_uint32(offset), _p(logits, _u16p),
                                C.byref(margin))
    return int(nxt), float(margin.value)


# ------------------------------------------------------------------ MoE / multi-row

class StackedWeight(QWeight):
    """Expert-stacked MLX-affine weights: w [E, O, K*bits/32], scales / biases [E, O, K/group]."""

    def __init__(self, experts):
        first = experts[0]
        dense_kind = first.scales is None
        super().__init__(np.stack([e.w for e in experts]),
                         None if dense_kind else np.stack([e.scales for e in experts]),
                         None if dense_kind else np.stack([e.biases for e in experts]),
                         first.n, first.k, first.bits, first.group)
        self.n_experts = len(experts)

    def expert(self, e: int) -> QWeight:
        if self.scales is None:
            return QWeight(self.w[e], None, None, self.n, self.k, self.bits, self.group)
        return QWeight(self.w[e], self.scales[e], self.biases[e], self.n, self.k, self.bits, self.group)


def routed_qmv_swiglu(x, Wg: StackedWeight, Wu: StackedWeight, row_idx, expert_idx, route_weight=None) -> np.ndarray:
    n_routes = int(expert_idx.size)
    out = np.empty((n_routes, Wg.n), dtype=np.uint16)
    _lib.fko_routed_qmv_swiglu(_p(x, _u16p), C.byref(Wg.c), C.byref(Wu.c), C.c_int64(Wg.n_experts),
                               _p(row_idx, _u32p), _p(expert_idx, _u32p), _p(route_weight, _u16p),
                               C.c_int64(n_routes), _p(out, _u16p))
    return out


def routed_qmv_reduce(h, Wd: StackedWeight, expert_idx, route_weight, residual_extra, n_tokens, top_k,
                      row_idx=None, shared_x=None, Wshared: QWeight = None) -> np.ndarray:
    out = np.empty((n_tokens, Wd.n), dtype=np.uint16)
    _lib.fko_routed_qmv_reduce(_p(h, _u16p), C.byref(Wd.c), C.c_int64(Wd.n_experts), _p(row_idx, _u32p),
                               _p(expert_idx, _u32p), _p(route_weight, _u16p), _p(shared_x, _u16p),
                               C.byref(Wshared.c) if Wshared is not None else None, _p(residual_extra, _u16p),
                               C.c_int64(n_tokens), C.c_int64(top_k), _p(out, _u16p))
    return out


def qgemm(W: QWeight, x: np.ndarray, bias=None) -> np.ndarray:
    m = x.shape[0]
    y = np.empty((m, W.n), dtype=np.uint16)
    _lib.fko_qgemm(C.byref(W.c), _p(x, _u16p), C.c_int64(m), _p(bias, _u16p), _p(y, _u16p))
    return y


def qgemm_bf16w(W: QWeight, x: np.ndarray, bias=None, want_acc: bool = False):
    """Multi-row matmul with every dequantised weight rounded to bf16 first (the reference's
    large-M form).  Returns y, or (y, unrounded fp32 sums) with want_acc."""
    m = x.shape[0]
    y = np.empty((m, W.n), dtype=np.uint16)
    acc = np.empty((m, W.n), dtype=np.float32) if want_acc else None
    _lib.fko_qgemm_bf16w(C.byref(W.c), _p(x, _u16p), C.c_int64(m), _p(bias, _u16p), _p(y, _u16p), _p(acc, _f32p))
    return (y, acc) if want_acc else y


# ------------------------------------------------------------------ quantised KV cache

class QuantCache:
    """K or V cache in the mlx-lm QuantizedKVCache layout: packed [n_kv, capacity, D*bits/32],
    scales / biases [n_kv, capacity, D/group]."""

    def __init__(self, n_kv: int, capacity: int, dim: int, bits: int, group: int = 64):
        self.n_kv, self.capacity, self.dim, self.bits, self.group = n_kv, capacity, dim, bits, group
        self.packed = np.zeros((n_kv, capacity, dim * bits // 32), np.uint32)
        self.scales = np.zeros((n_kv, capacity, dim // group), np.uint16)
        self.biases = np.zeros((n_kv, capacity, dim // group), np.uint16)

    def dequantize(self) -> np.ndarray:
        flat = QWeight(self.packed.reshape(-1, self.packed.shape[-1]), self.scales.reshape(-1, self.scales.shape[-1]),
                       self.biases.reshape(-1, self.biases.shape[-1]), self.n_kv * self.capacity, self.dim, self.bits, self.group)
        return dequantize(flat).reshape(self.n_kv, self.capacity, self.dim)


def rope_kv_store_quant(k, v, k_norm, n_kv, head_dim, rope_dims, theta, eps, pos, write_offset, K: QuantCache, V: QuantCache):
    _lib.fko_rope_kv_store_quant(_p(k, _u16p), _p(v, _u16p), _p(k_norm, _u16p), C.c_int64(n_kv), C.c_int64(head_dim),
                                 C.c_int64(rope_dims), C.c_float(theta), C.c_float(eps), C.c_uint32(pos),
                                 C.c_uint32(write_offset), C.c_uint32(K.capacity), C.c_int(K.bits), C.c_int(K.group),
                                 _p(K.packed, _u32p), _p(K.scales, _u16p), _p(K.biases, _u16p),
                                 _p(V.packed, _u32p), _p(V.scales, _u16p), _p(V.biases, _u16p))


def sdpa_decode_quant(q, K: QuantCache, V: QuantCache, n_heads, kv_len, scale) -> np.ndarray:
    out = np.empty(n_heads * V.dim, dtype=np.uint16)
    _lib.fko_sdpa_decode_quant(_p(q, _u16p), _p(K.packed, _u32p), _p(K.scales, _u16p), _p(K.biases, _u16p),
                               _p(V.packed, _u32p), _p(V.scales, _u16p), _p(V.biases, _u16p), C.c_int64(n_heads),
                               C.c_int64(K.n_kv), C.c_int64(K.dim), C.c_int64(V.dim), C.c_uint32(kv_len),
                               C.c_uint32(K.capacity), C.c_int(K.bits), C.c_int(K.group), C.c_float(scale), _p(out, _u16p))
    return out
