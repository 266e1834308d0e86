"""ctypes binding of libfusekit_hip.so (the C ABI in include/fusekit_hip.h).

Mirrors how the reference's Python runtime talks to `_fusekit_runtime_native`
(reference python/fusekit_runtime/dispatch.py -> python_runtime/src/lib.rs):
Python owns no arithmetic, only pointers and sizes.  bf16 tensors travel as
numpy uint16 bit patterns.  Loading fails loudly when the library is missing;
there is no fallback path.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("FUSEKIT_HIP_LIB") or os.path.join(_HERE, "libfusekit_hip.so")

FK_OK, FK_ERR_INVALID, FK_ERR_IO, FK_ERR_NOT_FOUND, FK_ERR_HIP, FK_ERR_UNSUPPORTED = range(6)


class FusekitError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"[fk_status {status}] {message}")
        self.status = status


class InvalidArgument(FusekitError, ValueError):
    """FK_ERR_INVALID: what the reference raises as PyValueError."""


def _load() -> C.CDLL:
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(hipcc, gfx950). fusekit_amd has no CPU fallback."
        )
    return C.CDLL(LIB_PATH)


lib = _load()
lib.fk_last_error.restype = C.c_char_p
lib.fk_version.restype = C.c_char_p


def check(status: int) -> None:
    if status != FK_OK:
        msg = lib.fk_last_error().decode("utf-8", "replace")
        if status == FK_ERR_INVALID:
            raise InvalidArgument(status, msg)
        raise FusekitError(status, msg)


def version() -> str:
    return lib.fk_version().decode()


class DeviceProps(C.Structure):
    _fields_ = [
        ("name", C.c_char * 128), ("arch", C.c_char * 32), ("compute_units", C.c_int), ("wavefront", C.c_int),
        ("lds_bytes_per_block", C.c_int), ("l2_bytes", C.c_int), ("hbm_bytes", C.c_uint64), ("clock_khz", C.c_int),
    ]


class Target(C.Structure):
    """fk_target: the gfx950 entry of the reference's ChipModel / Budgets table."""
    _fields_ = [("arch", C.c_char * 32), ("from_device", C.c_uint32), ("compute_units", C.c_uint32),
                ("xcds", C.c_uint32), ("wave_size", C.c_uint32), ("simds_per_cu", C.c_uint32),
                ("vgprs_per_lane", C.c_uint32), ("lds_bytes_per_cu", C.c_uint32), ("workgroup_threads", C.c_uint32),
                ("gemm_min_rows", C.c_uint32), ("gemm_rows_per_pass", C.c_uint32), ("hbm_bytes", C.c_uint64),
                ("hbm_peak_bytes_per_s", C.c_double), ("mfma_bf16_peak_flops", C.c_double)]


def target_describe() -> Target:
    t = Target()
    check(lib.fk_target_describe(C.byref(t)))
    return t


def device_props() -> DeviceProps:
    p = DeviceProps()
    check(lib.fk_device_props_get(C.byref(p)))
    return p


def mem_info():
    """(free, total) device memory in bytes."""
    a, b = C.c_size_t(), C.c_size_t()
    check(lib.fk_mem_info(C.byref(a), C.byref(b)))
    return a.value, b.value


def has_device() -> bool:
    p = DeviceProps()
    return lib.fk_device_props_get(C.byref(p)) == FK_OK


class Weight(C.Structure):
    """`fk_weight`."""

    _fields_ = [
        ("w", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p),
        ("n", C.c_uint32), ("k", C.c_uint32), ("bits", C.c_uint32), ("group", C.c_uint32),
    ]


class DeviceBuffer:
    """One device allocation owned through fk_alloc / fk_free."""

    def __init__(self, nbytes: int):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        check(lib.fk_alloc(C.c_size_t(max(self.nbytes, 1)), C.byref(p)))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        if a.nbytes:
            check(lib.fk_upload(C.c_void_p(b.ptr), a.ctypes.data_as(C.c_void_p), C.c_size_t(a.nbytes)))
        return b

    def upload(self, a: np.ndarray, offset: int = 0) -> None:
        a = np.ascontiguousarray(a)
        assert offset + a.nbytes <= self.nbytes
        check(lib.fk_upload(C.c_void_p(self.ptr + offset), a.ctypes.data_as(C.c_void_p), C.c_size_t(a.nbytes)))

    def to_numpy(self, dtype, shape=None, offset: int = 0) -> np.ndarray:
        dtype = np.dtype(dtype)
        if shape is None:
            shape = ((self.nbytes - offset) // dtype.itemsize,)
        out = np.empty(shape, dtype=dtype)
        assert offset + out.nbytes <= self.nbytes
        if out.nbytes:
            check(lib.fk_download(out.ctypes.data_as(C.c_void_p), C.c_void_p(self.ptr + offset),
                                  C.c_size_t(out.nbytes)))
        return out

    def free(self) -> None:
        if getattr(self, "ptr", None):
            lib.fk_free(C.c_void_p(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class DeviceWeight:
    """A weight matrix resident in HBM (packed + scales + biases, or dense bf16)."""

    def __init__(self, w: np.ndarray, scales, biases, n: int, k: int, bits: int, group: int = 64):
        self.n, self.k, self.bits, self.group = int(n), int(k), int(bits), int(group)
        self.w = DeviceBuffer.from_numpy(w)
        self.scales = None if scales is None else DeviceBuffer.from_numpy(np.asarray(scales, dtype=np.uint16))
        self.biases = None if biases is None else DeviceBuffer.from_numpy(np.asarray(biases, dtype=np.uint16))

    @property
    def c(self) -> Weight:
        return Weight(self.w.ptr, self.scales.ptr if self.scales else None,
                      self.biases.ptr if self.biases else None, self.n, self.k, self.bits, self.group)

    @property
    def nbytes(self) -> int:
        return self.w.nbytes + (self.scales.nbytes + self.biases.nbytes if self.scales else 0)


def _ptr(b) -> C.c_void_p:
    if b is None:
        return C.c_void_p(None)
    if isinstance(b, DeviceBuffer):
        return C.c_void_p(b.ptr)
    return C.c_void_p(int(b))


# ---------------------------------------------------------------- operators

def qgemv(W: DeviceWeight, x, bias, y, stream=None) -> None:
    check(lib.fk_qgemv(C.byref(W.c), _ptr(x), _ptr(bias), _ptr(y), _ptr(stream)))


def linear_residual(W: DeviceWeight, x, res, res2, y, stream=None) -> None:
    check(lib.fk_linear_residual(C.byref(W.c), _ptr(x), _ptr(res), _ptr(res2), _ptr(y), _ptr(stream)))


def rmsnorm_qkv(x, norm_w, eps, Wq, Wk, Wv, bq, bk, bv, q, k, v, stream=None) -> None:
    check(lib.fk_rmsnorm_qkv(_ptr(x), _ptr(norm_w), C.c_float(eps), C.byref(Wq.c), C.byref(Wk.c), C.byref(Wv.c),
                             _ptr(bq), _ptr(bk), _ptr(bv), _ptr(q), _ptr(k), _ptr(v), _ptr(stream)))


def gateup_swiglu_rows(x, rows, norm_w, eps, Wg, Wu, variant, out, stream=None) -> None:
    """fk_gateup_swiglu_rows: RMSNorm + gate / up + SwiGLU of 2..8 token rows in one launch."""
    check(lib.fk_gateup_swiglu_rows(_ptr(x), C.c_uint32(rows), _ptr(norm_w), C.c_float(eps), C.byref(Wg.c), C.byref(Wu.c),
                                    C.c_int(variant), _ptr(out), _ptr(stream)))


def rmsnorm_qkv_rows(x, rows, x_row_stride, norm_w, eps, Wq, Wk, Wv, q, q_row_stride, k=None, k_row_stride=0, v=None,
                     v_row_stride=0, stream=None) -> None:
    """fk_rmsnorm_qkv_rows: RMSNorm + one to three projections of 2..8 token rows in one launch."""
    wk = C.byref(Wk.c) if Wk is not None else None
    wv = C.byref(Wv.c) if Wv is not None else None
    check(lib.fk_rmsnorm_qkv_rows(_ptr(x), C.c_uint32(rows), C.c_uint32(x_row_stride), _ptr(norm_w), C.c_float(eps),
                                  C.byref(Wq.c), wk, wv, _ptr(q), C.c_uint32(q_row_stride), _ptr(k), C.c_uint32(k_row_stride),
                                  _ptr(v), C.c_uint32(v_row_stride), _ptr(stream)))


def gateup_swiglu(x, norm_w, eps, Wg, Wu, variant, out, stream=None) -> None:
    check(lib.fk_gateup_swiglu(_ptr(x), _ptr(norm_w), C.c_float(eps), C.byref(Wg.c), C.byref(Wu.c),
                               C.c_int(variant), _ptr(out), _ptr(stream)))


def routed_qmv_swiglu(x, n_x_rows, Wg, Wu, n_experts, row_idx, expert_idx, route_weight, n_routes, out0,
                      stream=None) -> None:
    """Wg / Wu: DeviceWeight whose arrays are stacked [E, n, ...] and whose n, k describe one expert."""
    check(lib.fk_routed_qmv_swiglu(_ptr(x), C.c_uint32(n_x_rows), C.byref(Wg.c), C.byref(Wu.c),
                                   C.c_uint32(n_experts), _ptr(row_idx), _ptr(expert_idx), _ptr(route_weight),
                                   C.c_uint32(n_routes), _ptr(out0), _ptr(stream)))


def routed_qmv_swiglu_shared(x, Wg, Wu, n_experts, expert_idx, route_weight, n_routes, out0, Sg, Su, shared_out,
                             stream=None) -> None:
    """One token: the routed gate/up + SwiGLU with the shared experts' pair as further routes of the same launch."""
    check(lib.fk_routed_qmv_swiglu_shared(_ptr(x), C.byref(Wg.c), C.byref(Wu.c), C.c_uint32(n_experts), _ptr(expert_idx),
                                          _ptr(route_weight), C.c_uint32(n_routes), _ptr(out0), C.byref(Sg.c), C.byref(Su.c),
                                          _ptr(shared_out), _ptr(stream)))


def routed_qmv_swiglu_routing(x, Wg, Wu, n_experts, logits, scale, top_k, apply_weight, idx_out, weight_out, out0, Sg=None,
                              Su=None, shared_out=None, stream=None) -> None:
    """One token: the routed (+ shared) gate/up launch ranking the router logits itself (fk_routed_qmv_swiglu_routing)."""
    check(lib.fk_routed_qmv_swiglu_routing(_ptr(x), C.byref(Wg.c), C.byref(Wu.c), C.c_uint32(n_experts), _ptr(logits), _ptr(scale),
                                           C.c_uint32(top_k), C.c_int(int(apply_weight)), _ptr(idx_out), _ptr(weight_out),
                                           _ptr(out0), C.byref(Sg.c) if Sg is not None else None,
                                           C.byref(Su.c) if Su is not None else None, _ptr(shared_out), _ptr(stream)))


lib.fk_routed_reduce_workspace_bytes.restype = C.c_size_t


lib.fk_routed_reduce_workspace_bytes_shared.restype = C.c_size_t


def routed_reduce_workspace_bytes(n_tokens, top_k, out_dim, shared_k=0, group=64) -> int:
    """shared_k: input width of a shared expert (several tokens then also need the multi-row matmul's workspace)."""
    return int(lib.fk_routed_reduce_workspace_bytes_shared(C.c_uint32(n_tokens), C.c_uint32(top_k), C.c_uint32(out_dim),
                                                           C.c_uint32(shared_k), C.c_uint32(group)))


def routed_qmv_reduce(h, n_h_rows, Wd, n_experts, row_idx, expert_idx, route_weight, shared_x, W_shared,
                      residual_extra, n_tokens, top_k, out, workspace, stream=None) -> None:
    check(lib.fk_routed_qmv_reduce(_ptr(h), C.c_uint32(n_h_rows), C.byref(Wd.c), C.c_uint32(n_experts),
                                   _ptr(row_idx), _ptr(expert_idx), _ptr(route_weight), _ptr(shared_x),
                                   C.byref(W_shared.c) if W_shared is not None else None, _ptr(residual_extra),
                                   C.c_uint32(n_tokens), C.c_uint32(top_k), _ptr(out), _ptr(workspace),
                                   _ptr(stream)))


def routed_qmv_swiglu_ordered(x, n_x_rows, Wg, Wu, n_experts, row_idx, expert_idx, route_weight, n_routes, order, out0,
                              stream=None) -> None:
    """fk_routed_qmv_swiglu with the routes served in `order` (fk_route_order): same results, shared slices read once."""
    check(lib.fk_routed_qmv_swiglu_ordered(_ptr(x), C.c_uint32(n_x_rows), C.byref(Wg.c), C.byref(Wu.c), C.c_uint32(n_experts),
                                           _ptr(row_idx), _ptr(expert_idx), _ptr(route_weight), C.c_uint32(n_routes), _ptr(order),
                                           _ptr(out0), _ptr(stream)))


def routed_qmv_reduce_ordered(h, n_h_rows, Wd, n_experts, row_idx, expert_idx, route_weight, shared_x, W_shared,
                              residual_extra, n_tokens, top_k, order, out, workspace, stream=None) -> None:
    check(lib.fk_routed_qmv_reduce_ordered(_ptr(h), C.c_uint32(n_h_rows), C.byref(Wd.c), C.c_uint32(n_experts),
                                           _ptr(row_idx), _ptr(expert_idx), _ptr(route_weight), _ptr(shared_x),
                                           C.byref(W_shared.c) if W_shared is not None else None, _ptr(residual_extra),
                                           C.c_uint32(n_tokens), C.c_uint32(top_k), _ptr(order), _ptr(out), _ptr(workspace),
                                           _ptr(stream)))


def set_routed_fused_reduce(on: bool) -> None:
    lib.fk_set_routed_fused_reduce(C.c_int(int(on)))


def qgemm_workspace_bytes(m, n, k, group=64) -> int:
    out = C.c_size_t(0)
    check(lib.fk_qgemm_workspace_bytes(C.c_uint32(m), C.c_uint32(n), C.c_uint32(k), C.c_uint32(group), C.byref(out)))
    return int(out.value)


def qgemm(W, x, m, bias, residual, y, workspace, stream=None) -> None:
    check(lib.fk_qgemm(C.byref(W.c), _ptr(x), C.c_uint32(m), _ptr(bias), _ptr(residual), _ptr(y), _ptr(workspace),
                       _ptr(stream)))


def qgemm_fanout(Ws, x, m, biases, ys, workspace, stream=None) -> None:
    """One to three matrices over the same activation rows (q / k / v of a prompt pass); workspace:
    qgemm_workspace_bytes(m, sum of n, k, group)."""
    n = len(Ws)
    w_arr = (C.POINTER(type(Ws[0].c)) * n)(*[C.pointer(W.c) for W in Ws])
    y_arr = (C.c_void_p * n)(*[_ptr(y).value for y in ys])
    b_arr = None if biases is None else (C.c_void_p * n)(*[_ptr(b).value for b in biases])
    check(lib.fk_qgemm_fanout(w_arr, C.c_uint32(n), _ptr(x), C.c_uint32(m), b_arr, y_arr, _ptr(workspace), _ptr(stream)))


def qgemm_swiglu(Wg, Wu, x, m, variant, out, workspace, stream=None) -> None:
    check(lib.fk_qgemm_swiglu(C.byref(Wg.c), C.byref(Wu.c), _ptr(x), C.c_uint32(m), C.c_int(variant), _ptr(out),
                              _ptr(workspace), _ptr(stream)))


def final_rmsnorm_lm_head(x, norm_w, eps, W, logits, stream=None) -> None:
    check(lib.fk_final_rmsnorm_lm_head(_ptr(x), _ptr(norm_w), C.c_float(eps), C.byref(W.c), _ptr(logits),
                                       _ptr(stream)))


HEAD_ARGMAX_WORKSPACE_BYTES = 32776


def final_rmsnorm_lm_head_argmax(x, norm_w, eps, W, logits, next_token, history, hist_counter, hist_capacity, workspace,
                                 stream=None) -> None:
    """The LM head that also selects the greedy token (one launch); UnsupportedError unless gemv_form(...) == 1."""
    check(lib.fk_final_rmsnorm_lm_head_argmax(_ptr(x), _ptr(norm_w), C.c_float(eps), C.byref(W.c), _ptr(logits),
                                              _ptr(next_token), _ptr(history), _ptr(hist_counter),
                                              C.c_uint32(hist_capacity), _ptr(workspace), _ptr(stream)))


def rope_q_decode(q, q_norm, n_heads, head_dim, rope_dims, theta, eps=0.0, d_offset=None, offset=0, stream=None):
    check(lib.fk_rope_q_decode(_ptr(q), _ptr(q_norm), C.c_uint32(n_heads), C.c_uint32(head_dim),
                               C.c_uint32(rope_dims), C.c_float(theta), C.c_float(eps), _ptr(d_offset),
                               C.c_uint32(offset), _ptr(stream)))


def rope_kv_cache_store_decode(k, v, k_norm, n_kv, k_dim, v_dim, rope_dims, theta, eps, d_offset, offset,
                               d_write_offset, write_offset, capacity, cache_k, cache_v, stream=None):
    check(lib.fk_rope_kv_cache_store_decode(
        _ptr(k), _ptr(v), _ptr(k_norm), C.c_uint32(n_kv), C.c_uint32(k_dim), C.c_uint32(v_dim),
        C.c_uint32(rope_dims), C.c_float(theta), C.c_float(eps), _ptr(d_offset), C.c_uint32(offset),
        _ptr(d_write_offset), C.c_uint32(write_offset), C.c_uint32(capacity), _ptr(cache_k), _ptr(cache_v),
        _ptr(stream)))


def kv_cache_store_split_decode(q, n_heads, q0_dim, q1_dim, k0, k0_stride, k1, k1_heads, v, v_stride, n_kv, k0_dim,
                                k1_dim, v_dim, rope_dims, traditional, theta, d_offset, offset, d_write_offset,
                                write_offset, capacity, cache_k, cache_v, stream=None):
    """Cache K row = [K0 | rope(K1)], V row; with a query also rope(Q1) in place (fk_kv_cache_store_split_decode)."""
    check(lib.fk_kv_cache_store_split_decode(
        _ptr(q), C.c_uint32(n_heads), C.c_uint32(q0_dim), C.c_uint32(q1_dim), _ptr(k0), C.c_uint32(k0_stride), _ptr(k1),
        C.c_uint32(k1_heads), _ptr(v), C.c_uint32(v_stride), C.c_uint32(n_kv), C.c_uint32(k0_dim), C.c_uint32(k1_dim),
        C.c_uint32(v_dim), C.c_uint32(rope_dims), C.c_int(int(traditional)), C.c_float(theta), _ptr(d_offset),
        C.c_uint32(offset), _ptr(d_write_offset), C.c_uint32(write_offset), C.c_uint32(capacity), _ptr(cache_k),
        _ptr(cache_v), _ptr(stream)))


def split_store_sdpa_decode(q, n_heads, q0_dim, q1_dim, k0, k0_stride, k1, k1_heads, v, v_stride, n_kv, v_dim, rope_dims,
                            traditional, theta, rope_tab, cache_k, cache_v, out, d_kv_len, kv_len, max_len, capacity, scale,
                            partials, counters, stream=None):
    """Split-key cache store + attention of a layer in one launch (fk_split_store_sdpa_decode)."""
    check(lib.fk_split_store_sdpa_decode(
        _ptr(q), C.c_uint32(n_heads), C.c_uint32(q0_dim), C.c_uint32(q1_dim), _ptr(k0), C.c_uint32(k0_stride), _ptr(k1),
        C.c_uint32(k1_heads), _ptr(v), C.c_uint32(v_stride), C.c_uint32(n_kv), C.c_uint32(v_dim), C.c_uint32(rope_dims),
        C.c_int(int(traditional)), C.c_float(theta), _ptr(rope_tab), _ptr(cache_k), _ptr(cache_v), _ptr(out), _ptr(d_kv_len),
        C.c_uint32(kv_len), C.c_uint32(max_len), C.c_uint32(capacity), C.c_float(scale), _ptr(partials), _ptr(counters),
        _ptr(stream)))


def softmax_topk_route(logits, scale, scale_per_route, rows, row_n, top_k, idx, weight, stream=None):
    check(lib.fk_softmax_topk_route(_ptr(logits), _ptr(scale), C.c_int(int(scale_per_route)), C.c_uint32(rows),
                                    C.c_uint32(row_n), C.c_uint32(top_k), _ptr(idx), _ptr(weight), _ptr(stream)))


def moe_router(x, norm_w, eps, w, scale, hidden, experts, top_k, xn, logits, idx, weight, workspace, rows=1, stream=None):
    """RMSNorm + router projection (bf16 weights) + softmax top-k route in one launch (fk_moe_router);
    workspace: zeros(4 * rows * (experts + 1)), reusable by launches that do not overlap."""
    check(lib.fk_moe_router(_ptr(x), _ptr(norm_w), C.c_float(eps), _ptr(w), _ptr(scale), C.c_uint32(hidden),
                            C.c_uint32(experts), C.c_uint32(top_k), _ptr(xn), _ptr(logits), _ptr(idx), _ptr(weight),
                            _ptr(workspace), C.c_uint32(rows), _ptr(stream)))


def kv_cache_store_split_rows(q, n_heads, q0_dim, q1_dim, k0, k0_stride, k0_row_stride, k1, k1_heads, k1_row_stride, v, v_stride,
                              v_row_stride, n_kv, k0_dim, k1_dim, v_dim, rope_dims, traditional, theta, rows, offset, capacity,
                              cache_k, cache_v, stream=None):
    check(lib.fk_kv_cache_store_split_rows(
        _ptr(q), C.c_uint32(n_heads), C.c_uint32(q0_dim), C.c_uint32(q1_dim), _ptr(k0), C.c_uint32(k0_stride),
        C.c_uint32(k0_row_stride), _ptr(k1), C.c_uint32(k1_heads), C.c_uint32(k1_row_stride), _ptr(v), C.c_uint32(v_stride),
        C.c_uint32(v_row_stride), C.c_uint32(n_kv), C.c_uint32(k0_dim), C.c_uint32(k1_dim), C.c_uint32(v_dim),
        C.c_uint32(rope_dims), C.c_int(int(traditional)), C.c_float(theta), C.c_uint32(rows), C.c_uint32(offset),
        C.c_uint32(capacity), _ptr(cache_k), _ptr(cache_v), _ptr(stream)))


def qkv_rope_store_decode(q, k, v, q_norm, k_norm, n_heads, n_kv, head_dim, rope_dims, theta, eps, d_offset,
                          offset, capacity, cache_k, cache_v, stream=None):
    check(lib.fk_qkv_rope_store_decode(
        _ptr(q), _ptr(k), _ptr(v), _ptr(q_norm), _ptr(k_norm), C.c_uint32(n_heads), C.c_uint32(n_kv),
        C.c_uint32(head_dim), C.c_uint32(rope_dims), C.c_float(theta), C.c_float(eps), _ptr(d_offset),
        C.c_uint32(offset), C.c_uint32(capacity), _ptr(cache_k), _ptr(cache_v), _ptr(stream)))


def sdpa_workspace_bytes(n_heads, n_kv, qk_dim, v_dim, max_len):
    pb, cb = C.c_size_t(), C.c_size_t()
    check(lib.fk_sdpa_workspace_bytes(C.c_uint32(n_heads), C.c_uint32(n_kv), C.c_uint32(qk_dim), C.c_uint32(v_dim),
                                      C.c_uint32(max_len), C.byref(pb), C.byref(cb)))
    return int(pb.value), int(cb.value)


def sdpa_decode(q, cache_k, cache_v, out, d_kv_len, kv_len, max_len, n_heads, n_kv, qk_dim, v_dim, capacity,
                scale, partials, counters, stream=None):
    check(lib.fk_sdpa_decode(_ptr(q), _ptr(cache_k), _ptr(cache_v), _ptr(out), _ptr(d_kv_len),
                             C.c_uint32(kv_len), C.c_uint32(max_len), C.c_uint32(n_heads), C.c_uint32(n_kv),
                             C.c_uint32(qk_dim), C.c_uint32(v_dim), C.c_uint32(capacity), C.c_float(scale),
                             _ptr(partials), _ptr(counters), _ptr(stream)))


def sdpa_decode_static(q, cache_k, cache_v, out, d_kv_len, kv_len, max_len, n_heads, n_kv, qk_dim, v_dim, capacity,
                       scale, stream=None):
    """fk_sdpa_decode with the split-K workspace in the library's static device array: allocates nothing."""
    check(lib.fk_sdpa_decode_static(_ptr(q), _ptr(cache_k), _ptr(cache_v), _ptr(out), _ptr(d_kv_len),
                                    C.c_uint32(kv_len), C.c_uint32(max_len), C.c_uint32(n_heads), C.c_uint32(n_kv),
                                    C.c_uint32(qk_dim), C.c_uint32(v_dim), C.c_uint32(capacity), C.c_float(scale),
                                    _ptr(stream)))


class _KvQuantCache(C.Structure):
    _fields_ = [("packed", C.c_void_p), ("scales", C.c_void_p), ("biases", C.c_void_p)]


class QuantKvCache:
    """One K or V cache in the quantised layout, resident in HBM."""

    def __init__(self, n_kv: int, capacity: int, dim: int, bits: int, group: int = 64, zero: bool = True):
        self.n_kv, self.capacity, self.dim, self.bits, self.group = n_kv, capacity, dim, bits, group
        alloc = zeros if zero else DeviceBuffer
        self.packed = alloc(n_kv * capacity * dim * bits // 8)
        self.scales = alloc(n_kv * capacity * (dim // group) * 2)
        self.biases = alloc(n_kv * capacity * (dim // group) * 2)

    @property
    def c(self) -> _KvQuantCache:
        return _KvQuantCache(self.packed.ptr, self.scales.ptr, self.biases.ptr)

    @property
    def nbytes(self) -> int:
        return self.packed.nbytes + self.scales.nbytes + self.biases.nbytes


def kv_cache_dequant(cache: "QuantKvCache", rows: int, out, out_capacity: int, stream=None):
    """Rows [0, rows) of a quantised cache as bf16 [n_kv, out_capacity, dim]."""
    check(lib.fk_kv_cache_dequant(C.byref(cache.c), C.c_uint32(cache.n_kv), C.c_uint32(cache.dim), C.c_uint32(cache.capacity),
                                  C.c_uint32(cache.bits), C.c_uint32(cache.group), C.c_uint32(rows), _ptr(out),
                                  C.c_uint32(out_capacity), _ptr(stream)))


def kv_cache_store_quant(k, v, k_norm, n_kv, head_dim, rope_dims, theta, eps, d_offset, offset, rows, K: QuantKvCache,
                         V: QuantKvCache, stream=None):
    check(lib.fk_kv_cache_store_quant(_ptr(k), _ptr(v), _ptr(k_norm), C.c_uint32(n_kv), C.c_uint32(head_dim),
                                      C.c_uint32(rope_dims), C.c_float(theta), C.c_float(eps), _ptr(d_offset),
                                      C.c_uint32(offset), C.c_uint32(rows), C.c_uint32(K.capacity), C.c_uint32(K.bits),
                                      C.c_uint32(K.group), C.byref(K.c), C.byref(V.c), _ptr(stream)))


def sdpa_decode_quant(q, K: QuantKvCache, V: QuantKvCache, out, d_kv_len, kv_len, max_len, rows, n_heads, scale,
                      partials, counters, stream=None):
    check(lib.fk_sdpa_decode_quant(_ptr(q), C.byref(K.c), C.byref(V.c), _ptr(out), _ptr(d_kv_len), C.c_uint32(kv_len),
                                   C.c_uint32(max_len), C.c_uint32(rows), C.c_uint32(n_heads), C.c_uint32(K.n_kv),
                                   C.c_uint32(K.dim), C.c_uint32(V.dim), C.c_uint32(K.capacity), C.c_uint32(K.bits),
                                   C.c_uint32(K.group), C.c_float(scale), _ptr(partials), _ptr(counters), _ptr(stream)))


def rmsnorm_rows(x, w, eps, rows, hidden, y, stream=None):
    check(lib.fk_rmsnorm_rows(_ptr(x), _ptr(w), C.c_float(eps), C.c_uint32(rows), C.c_uint32(hidden), _ptr(y), _ptr(stream)))


def embed_lookup_rows(E, d_tokens, rows, out_scale, x, stream=None):
    check(lib.fk_embed_lookup_rows(C.byref(E.c), _ptr(d_tokens), C.c_uint32(rows), C.c_float(out_scale), _ptr(x),
                                   _ptr(stream)))


def qkv_rope_store_rows(q, k, v, q_norm, k_norm, n_heads, n_kv, head_dim, rope_dims, theta, eps, rows, offset,
                        capacity, cache_k, cache_v, stream=None, rope_tab=None):
    check(lib.fk_qkv_rope_store_rows(
        _ptr(q), _ptr(k), _ptr(v), _ptr(q_norm), _ptr(k_norm), C.c_uint32(n_heads), C.c_uint32(n_kv),
        C.c_uint32(head_dim), C.c_uint32(rope_dims), C.c_float(theta), C.c_float(eps), C.c_uint32(rows),
        C.c_uint32(offset), C.c_uint32(capacity), _ptr(cache_k), _ptr(cache_v), _ptr(rope_tab), _ptr(stream)))


def rope_table_rows(tab, rope_dims, theta, offset, rows, stream=None):
    """(cos, sin) of every rotary pair at positions offset .. offset + rows - 1, [rows][rope_dims/2][2] fp32."""
    check(lib.fk_rope_table_rows(_ptr(tab), C.c_uint32(rope_dims), C.c_float(theta), C.c_uint32(offset), C.c_uint32(rows),
                                 _ptr(stream)))


def sdpa_decode_rows(q, cache_k, cache_v, out, rows, kv_len, n_heads, n_kv, qk_dim, v_dim, capacity, scale, partials,
                     counters, stream=None):
    check(lib.fk_sdpa_decode_rows(_ptr(q), _ptr(cache_k), _ptr(cache_v), _ptr(out), C.c_uint32(rows), C.c_uint32(kv_len),
                                  C.c_uint32(n_heads), C.c_uint32(n_kv), C.c_uint32(qk_dim), C.c_uint32(v_dim),
                                  C.c_uint32(capacity), C.c_float(scale), _ptr(partials), _ptr(counters), _ptr(stream)))


def sdpa_prefill(q, cache_k, cache_v, out, rows, kv_len, n_heads, n_kv, head_dim, capacity, scale, stream=None):
    """Causal attention of a group of rows on the matrix cores; kv_len counts the group's rows."""
    check(lib.fk_sdpa_prefill(_ptr(q), _ptr(cache_k), _ptr(cache_v), _ptr(out), C.c_uint32(rows), C.c_uint32(kv_len),
                              C.c_uint32(n_heads), C.c_uint32(n_kv), C.c_uint32(head_dim), C.c_uint32(capacity),
                              C.c_float(scale), _ptr(stream)))


def gemm_library_available() -> bool:
    return bool(lib.fk_gemm_library_available())


def dequantize_bf16(W: DeviceWeight, stream=None) -> DeviceWeight:
    """The bf16 copy of a quantised matrix (fk_dequantize_bf16) as a bits-16 DeviceWeight."""
    D = DeviceWeight.__new__(DeviceWeight)
    D.n, D.k, D.bits, D.group, D.scales, D.biases = W.n, W.k, 16, 0, None, None
    D.w = DeviceBuffer(W.n * W.k * 2)
    check(lib.fk_dequantize_bf16(C.byref(W.c), _ptr(D.w), _ptr(stream)))
    return D


GEMM_LIBRARY_ROWS_DEFAULT = 1024  # fk_set_gemm_library_rows' default


def set_gemm_library_rows(rows: int):
    """Row count from which qgemm / qgemm_swiglu take the dequantise + library-GEMM route (0: never)."""
    check(lib.fk_set_gemm_library_rows(C.c_uint32(rows)))


def embed_lookup_decode(E, d_token, token, out_scale, x, stream=None):
    check(lib.fk_embed_lookup_decode(C.byref(E.c), _ptr(d_token), C.c_uint32(token), C.c_float(out_scale),
                                     _ptr(x), _ptr(stream)))


ARGMAX_WORKSPACE_BYTES = 1288


def argmax_logits_decode(logits, n, next_token, history, hist_counter, hist_capacity, workspace, stream=None):
    check(lib.fk_argmax_logits_decode(_ptr(logits), C.c_uint32(n), _ptr(next_token), _ptr(history),
                                      _ptr(hist_counter), C.c_uint32(hist_capacity), _ptr(workspace),
                                      _ptr(stream)))


def step_init(step_counter, offset, kv_len, stream=None):
    check(lib.fk_step_init(_ptr(step_counter), _ptr(offset), _ptr(kv_len), _ptr(stream)))


def step_init_rope(step_counter, offset, kv_len, rope_tab, rope_dims, theta, stream=None):
    check(lib.fk_step_init_rope(_ptr(step_counter), _ptr(offset), _ptr(kv_len), _ptr(rope_tab), C.c_uint32(rope_dims),
                                C.c_float(theta), _ptr(stream)))


def rope_store_sdpa_decode(q, k, v, q_norm, k_norm, cache_k, cache_v, out, d_kv_len, kv_len, max_len, n_heads, n_kv,
                           head_dim, rope_dims, theta, eps, capacity, scale, rope_tab, partials, counters, stream=None):
    check(lib.fk_rope_store_sdpa_decode(
        _ptr(q), _ptr(k), _ptr(v), _ptr(q_norm), _ptr(k_norm), _ptr(cache_k), _ptr(cache_v), _ptr(out), _ptr(d_kv_len),
        C.c_uint32(kv_len), C.c_uint32(max_len), C.c_uint32(n_heads), C.c_uint32(n_kv), C.c_uint32(head_dim),
        C.c_uint32(rope_dims), C.c_float(theta), C.c_float(eps), C.c_uint32(capacity), C.c_float(scale), _ptr(rope_tab),
        _ptr(partials), _ptr(counters), _ptr(stream)))


def xcd_layer_supported(hidden, inter, n_heads, n_kv, head_dim, capacity, bits, group) -> bool:
    """Can a layer of this shape run as two XCD-resident launches (fk_xcd_layer_supported)?"""
    return lib.fk_xcd_layer_supported(C.c_uint32(hidden), C.c_uint32(inter), C.c_uint32(n_heads), C.c_uint32(n_kv),
                                      C.c_uint32(head_dim), C.c_uint32(capacity), C.c_uint32(bits), C.c_uint32(group)) == 0


def xcd_workspace_bytes(n_heads, head_dim):
    """(bytes of the control block, bytes of the attention partial rows)."""
    a, b = C.c_size_t(), C.c_size_t()
    check(lib.fk_xcd_workspace_bytes(C.c_uint32(n_heads), C.c_uint32(head_dim), C.byref(a), C.byref(b)))
    return a.value, b.value


lib.fk_xcd_sum_row_bytes.restype = C.c_size_t


def xcd_sum_row_bytes(hidden: int) -> int:
    return int(lib.fk_xcd_sum_row_bytes(C.c_uint32(hidden)))


def xcd_moe_supported(hidden, inter, shared_inter, experts, top_k, bits, group) -> bool:
    """Can the expert block of a layer of this shape run as one XCD-resident launch (fk_xcd_moe_supported)?"""
    return lib.fk_xcd_moe_supported(C.c_uint32(hidden), C.c_uint32(inter), C.c_uint32(shared_inter), C.c_uint32(experts),
                                    C.c_uint32(top_k), C.c_uint32(bits), C.c_uint32(group)) == FK_OK


def xcd_mla_supported(hidden, n_heads, rank, rope_dim, nope_dim, v_dim, capacity, bits, group) -> bool:
    """Can the attention half of a layer with low-rank keys run as one XCD-resident launch (fk_xcd_mla_supported)?"""
    u = C.c_uint32
    return lib.fk_xcd_mla_supported(u(hidden), u(n_heads), u(rank), u(rope_dim), u(nope_dim), u(v_dim), u(capacity), u(bits),
                                    u(group)) == FK_OK


def xcd_mla_workspace_bytes(n_heads, rank, rope_dim, v_dim):
    """(bytes of the `kva` slot, bytes of the attention partial rows) of fusekit_xcd_mla_block."""
    a, b = C.c_size_t(), C.c_size_t()
    check(lib.fk_xcd_mla_workspace_bytes(C.c_uint32(n_heads), C.c_uint32(rank), C.c_uint32(rope_dim), C.c_uint32(v_dim),
                                         C.byref(a), C.byref(b)))
    return a.value, b.value


lib.fk_xcd_moe_scratch_bytes.restype = C.c_size_t


def xcd_moe_scratch_bytes(inter: int) -> int:
    return int(lib.fk_xcd_moe_scratch_bytes(C.c_uint32(inter)))


def xcd_kslice_meta(src: "DeviceBuffer", n: int, groups: int, stream=None) -> "DeviceBuffer":
    """The per-XCD re-laid-out copy of a scale or bias array [n, groups] (fk_xcd_kslice_meta)."""
    dst = DeviceBuffer(n * groups * 2)
    check(lib.fk_xcd_kslice_meta(_ptr(src), C.c_uint32(n), C.c_uint32(groups), _ptr(dst), _ptr(stream)))
    return dst


def xcd_sum_index(hidden: int):
    """Index of element e of a hidden-wide vector inside a sum row (numpy array of hidden indices)."""
    import numpy as np
    e = np.arange(hidden, dtype=np.int64)
    t = e >> 3
    return ((((t >> 6) * 4 + ((e & 7) >> 1)) * 64 + (t & 63)) << 1) | (e & 1)


def xcd_check(workspace, stream=None) -> None:
    check(lib.fk_xcd_check(_ptr(workspace), _ptr(stream)))


def copy(dst, src, nbytes, stream=None):
    check(lib.fk_copy(_ptr(dst), _ptr(src), C.c_size_t(nbytes), _ptr(stream)))


def route_order(expert_idx, n_routes: int, n_experts: int, order, stream=None) -> None:
    """order[position] = route, the routes sorted by expert index, stable (fk_route_order)."""
    check(lib.fk_route_order(_ptr(expert_idx), C.c_uint32(n_routes), C.c_uint32(n_experts), _ptr(order), _ptr(stream)))


lib.fk_read_reduce_out_bytes.restype = C.c_size_t


def read_reduce_out_bytes() -> int:
    return int(lib.fk_read_reduce_out_bytes())


def read_reduce(src, nbytes, out, stream=None):
    """XOR of nbytes read with plain 16-byte loads, one word per workgroup into `out` (fk_read_reduce)."""
    check(lib.fk_read_reduce(_ptr(src), C.c_size_t(nbytes), _ptr(out), C.c_size_t(out.nbytes), _ptr(stream)))


def fill_u32(buf, value, count, stream=None):
    check(lib.fk_fill_u32(_ptr(buf), C.c_uint32(value), C.c_size_t(count), _ptr(stream)))


def zeros(nbytes: int) -> DeviceBuffer:
    b = DeviceBuffer(nbytes)
    b.upload(np.zeros(nbytes, dtype=np.uint8))
    return b


def set_gemv_policy(rows_per_tile: int = 0, grid_blocks: int = 0) -> None:
    check(lib.fk_set_gemv_policy(C.c_uint32(rows_per_tile), C.c_uint32(grid_blocks)))


def gemv_form(n: int, k: int, bits: int, group: int = 64) -> int:
    """1 when a plain GEMV over an [n, k] matrix runs the row-group kernel form, 0 for the flat stream."""
    return int(lib.fk_gemv_form(C.c_uint32(n), C.c_uint32(k), C.c_uint32(bits), C.c_uint32(group)))


def set_qgemm_wide(enabled: bool) -> None:
    check(lib.fk_set_qgemm_wide(C.c_int(1 if enabled else 0)))


def set_gemv_flat_only(flat_only: bool) -> None:
    check(lib.fk_set_gemv_flat_only(C.c_int(1 if flat_only else 0)))


def sync(stream=None) -> None:
    check(lib.fk_stream_sync(_ptr(stream)))


class Event:
    def __init__(self):
        p = C.c_void_p()
        check(lib.fk_event_create(C.byref(p)))
        self.ptr = p.value

    def record(self, stream=None) -> None:
        check(lib.fk_event_record(C.c_void_p(self.ptr), _ptr(stream)))

    def elapsed_ms_until(self, stop: "Event") -> float:
        ms = C.c_float()
        check(lib.fk_event_elapsed_ms(C.c_void_p(self.ptr), C.c_void_p(stop.ptr), C.byref(ms)))
        return float(ms.value)

    def __del__(self):
        try:
            if self.ptr:
                lib.fk_event_destroy(C.c_void_p(self.ptr))
        except Exception:
            pass
