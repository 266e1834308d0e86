"""Dispatcher: host-side mirror of the reference's use of `_fusekit_runtime_native`.

The reference's Python `Dispatcher` (python/fusekit_runtime/dispatch.py:279) resolves
bindings to raw pointers, calls `build_icb` once and then replays it per token through
`decode_chunk_*`.  This class does the same against the C ABI: `build_graph` encodes a
list of dispatches as one hipGraph, `decode_chunk` replays it with the argmax fed back
on the GPU, `decode_host_loop` feeds forced tokens (a prompt).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import native
from .native import DeviceBuffer, check, lib

FK_CHUNK = 64  # tokens per native chunk, reference dispatch.py:1103


class _Arg(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("nbytes", C.c_size_t)]


class _Param(C.Structure):
    _fields_ = [("key", C.c_char_p), ("value", C.c_double)]


class _Dispatch(C.Structure):
    _fields_ = [("kernel", C.c_char_p), ("args", C.POINTER(_Arg)), ("n_args", C.c_uint32),
                ("params", C.POINTER(_Param)), ("n_params", C.c_uint32)]


class _BindingUpdate(C.Structure):
    _fields_ = [("cmd_idx", C.c_uint32), ("slot", C.c_uint32), ("ptr", C.c_void_p), ("nbytes", C.c_size_t)]


class LaunchGeometry(C.Structure):
    """fk_launch_geometry: kernels, grid / threadgroup / LDS of each, read-write bits per slot."""
    _fields_ = [("n_kernels", C.c_uint32), ("grid", (C.c_uint32 * 3) * 4), ("threadgroup", (C.c_uint32 * 3) * 4),
                ("lds_bytes", C.c_uint32 * 4), ("n_slots", C.c_uint32), ("slot_access", C.c_uint8 * 32)]


class _Uniforms(C.Structure):
    _fields_ = [("token", C.c_void_p), ("step_counter", C.c_void_p), ("hist_counter", C.c_void_p),
                ("history", C.c_void_p), ("hist_capacity", C.c_uint32)]


@dataclass
class Dispatch:
    """One kernel launch: family-prefixed name, (pointer, nbytes) per slot, scalar parameters."""
    kernel: str
    args: List[Tuple[int, int]]
    params: Dict[str, float] = field(default_factory=dict)


def _marshal(dispatches: Sequence[Dispatch]):
    keep = []
    arr = (_Dispatch * len(dispatches))()
    for i, d in enumerate(dispatches):
        args = (_Arg * len(d.args))(*[_Arg(p, n) for p, n in d.args])
        keys = [k.encode() for k in d.params]
        params = (_Param * max(len(keys), 1))(*[_Param(k, float(v)) for k, v in zip(keys, d.params.values())])
        name = d.kernel.encode()
        keep.append((args, keys, params, name))
        arr[i] = _Dispatch(name, args, len(d.args), params, len(keys))
    return arr, keep


def arg(buf: DeviceBuffer, nbytes: Optional[int] = None, offset: int = 0) -> Tuple[int, int]:
    return (buf.ptr + offset, buf.nbytes - offset if nbytes is None else nbytes)


class Dispatcher:
    def __init__(self, code_object_path: Optional[str] = None, task_graph_path: Optional[str] = None):
        h = C.c_uint64()
        check(lib.fk_load_dispatcher(code_object_path.encode() if code_object_path else None,
                                     task_graph_path.encode() if task_graph_path else None, C.byref(h)))
        self.handle = h

    def kernel_names(self) -> List[str]:
        names = C.POINTER(C.c_char_p)()
        n = C.c_size_t()
        check(lib.fk_kernel_names(self.handle, C.byref(names), C.byref(n)))
        return [names[i].decode() for i in range(n.value)]

    def plan_geometry(self, d: Dispatch) -> LaunchGeometry:
        arr, keep = _marshal([d])
        g = LaunchGeometry()
        check(lib.fk_plan_geometry(self.handle, C.byref(arr[0]), C.byref(g)))
        return g

    def dispatch_kernel(self, d: Dispatch) -> float:
        return self.dispatch_batch([d])

    def dispatch_batch(self, ds: Sequence[Dispatch]) -> float:
        arr, keep = _marshal(ds)
        sec = C.c_double()
        check(lib.fk_dispatch_batch(self.handle, arr, C.c_size_t(len(ds)), C.byref(sec)))
        return sec.value

    def build_graph(self, ds: Sequence[Dispatch], barriers: Optional[Sequence[bool]] = None) -> int:
        arr, keep = _marshal(ds)
        gid = C.c_uint32()
        b = None
        if barriers is not None:
            b = (C.c_uint8 * len(ds))(*[1 if x else 0 for x in barriers])
        check(lib.fk_build_graph(self.handle, arr, C.c_size_t(len(ds)), b, C.byref(gid)))
        return gid.value

    def build_decode_graph(self, ds: Sequence[Dispatch], persistent: bool = True, spin_limit: int = 0) -> int:
        """The decode pipeline as one graph; persistent=True runs it as ONE whole-token kernel."""
        arr, keep = _marshal(ds)
        gid = C.c_uint32()
        check(lib.fk_build_decode_graph(self.handle, arr, C.c_size_t(len(ds)), C.c_int(1 if persistent else 0),
                                        C.c_uint32(spin_limit), C.byref(gid)))
        return gid.value

    def graph_launch_shape(self, gid: int) -> Tuple[bool, int, int]:
        p, g, l = C.c_uint32(), C.c_uint32(), C.c_uint32()
        check(lib.fk_graph_launch_shape(self.handle, C.c_uint32(gid), C.byref(p), C.byref(g), C.byref(l)))
        return bool(p.value), g.value, l.value

    def graph_phase_trace(self, gid: int) -> List[float]:
        """Seconds per phase of the last launch of a persistent decode graph."""
        n = C.c_uint32()
        buf = (C.c_double * 4096)()
        check(lib.fk_graph_phase_trace(self.handle, C.c_uint32(gid), buf, 4096, C.byref(n)))
        return [buf[i] for i in range(min(n.value, 4096))]

    def graph_info(self, gid: int) -> Tuple[int, int]:
        n, e = C.c_uint32(), C.c_uint32()
        check(lib.fk_graph_info(self.handle, C.c_uint32(gid), C.byref(n), C.byref(e)))
        return n.value, e.value

    def node_deps(self, gid: int, node: int) -> List[int]:
        buf = (C.c_uint32 * 64)()
        n = C.c_uint32()
        check(lib.fk_graph_node_deps(self.handle, C.c_uint32(gid), C.c_uint32(node), buf, 64, C.byref(n)))
        return [buf[i] for i in range(min(n.value, 64))]

    def update_graph_bindings(self, gid: int, updates: Sequence[Tuple[int, int, int, int]]) -> None:
        arr = (_BindingUpdate * max(len(updates), 1))(*[_BindingUpdate(*u) for u in updates])
        check(lib.fk_update_graph_bindings(self.handle, C.c_uint32(gid), arr, C.c_size_t(len(updates))))

    def execute_graph(self, gid: int, repeat: int = 1) -> float:
        sec = C.c_double()
        if repeat == 1:
            check(lib.fk_execute_graph(self.handle, C.c_uint32(gid), C.byref(sec)))
        else:
            check(lib.fk_execute_graph_repeat(self.handle, C.c_uint32(gid), C.c_uint32(repeat), C.byref(sec)))
        return sec.value

    def execute_graph_range(self, gid: int, start: int, end: int) -> float:
        sec = C.c_double()
        check(lib.fk_execute_graph_range(self.handle, C.c_uint32(gid), C.c_uint32(start), C.c_uint32(end),
                                         C.byref(sec)))
        return sec.value

    def profile_graph_nodes(self, gid: int) -> List[float]:
        n, _ = self.graph_info(gid)
        out = (C.c_double * n)()
        check(lib.fk_profile_graph_nodes(self.handle, C.c_uint32(gid), out, C.c_size_t(n)))
        return list(out)

    def submit_graph_async(self, gid: int) -> None:
        check(lib.fk_submit_graph_async(self.handle, C.c_uint32(gid)))

    def wait_pending(self) -> float:
        sec = C.c_double()
        check(lib.fk_wait_pending(self.handle, C.byref(sec)))
        return sec.value

    def decode_chunk(self, gid: int, uniforms: _Uniforms, start_offset: int, seed_token: int, count: int):
        out = (C.c_uint32 * count)()
        sec = C.c_double()
        check(lib.fk_decode_chunk(self.handle, C.c_uint32(gid), C.byref(uniforms), C.c_uint32(start_offset),
                                  C.c_uint32(seed_token), C.c_uint32(count), out, C.byref(sec)))
        return list(out), sec.value

    def decode_host_loop(self, gid: int, uniforms: _Uniforms, start_offset: int, tokens: Sequence[int]):
        n = len(tokens)
        tin = (C.c_uint32 * n)(*tokens)
        out = (C.c_uint32 * n)()
        sec = C.c_double()
        check(lib.fk_decode_chunk_host_loop(self.handle, C.c_uint32(gid), C.byref(uniforms),
                                            C.c_uint32(start_offset), tin, C.c_uint32(n), out, C.byref(sec)))
        return list(out), sec.value


def make_uniforms(token: DeviceBuffer, step_counter: DeviceBuffer, hist_counter: DeviceBuffer,
                  history: DeviceBuffer) -> _Uniforms:
    return _Uniforms(token.ptr, step_counter.ptr, hist_counter.ptr, history.ptr, history.nbytes // 4)
