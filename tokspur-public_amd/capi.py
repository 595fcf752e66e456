"""ctypes binding of the C ABI in include/tokspur_hip.h.

The library must have been built (python -m build step or __graft_entry__.build()); loading fails
loudly when libtokspur_hip.so is missing — there is no fallback path of any kind. `Device` wraps
torch tensors as device buffers and calls every device entry point on torch's current stream.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtokspur_hip.so")

OK, ERR_FORMAT, ERR_HIP = 0, 1, 2
ERRBIT_NONFINITE, ERRBIT_INDEX = 1, 4
LAYOUT_GGUF, LAYOUT_Q8_LANES_V1, LAYOUT_PLANAR_V3 = 0, 1, 3
u8p = C.POINTER(C.c_uint8)


class FormatError(RuntimeError):
    """A host-side refusal: what the engine reports as tokspur::FormatError."""


class HipError(RuntimeError):
    pass


class PlanarSpec(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("source_type", "columns", "rows", "blocks_per_row")] + \
               [(n, C.c_uint64) for n in ("source_row_bytes", "planar_row_bytes", "source_expert_bytes",
                                          "planar_expert_bytes", "qs_offset", "qh_offset", "sm_offset", "dm_offset")]


class GroupedMmPlan(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in ("columns", "rows", "row_bytes", "experts", "selected", "tokens",
                                          "broadcast", "maximum_tasks")] + \
               [(n, C.c_uint64) for n in ("expert_stride_bytes", "input_stride_bytes", "output_stride_bytes",
                                          "matrix_bytes", "indices_bytes", "input_bytes", "output_bytes",
                                          "token_map_bytes", "counts_bytes", "tasks_bytes")] + \
               [("grid_x", C.c_uint32), ("grid_y", C.c_uint32)]


_dll = None


def dll():
    global _dll
    if _dll is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with __graft_entry__.build() — there is no fallback")
        _dll = C.CDLL(LIB_PATH)
        _dll.tsp_last_error.restype = C.c_char_p
        _dll.tsp_abi_version.restype = C.c_uint32
    return _dll


def check(status):
    if status == OK:
        return
    message = dll().tsp_last_error().decode()
    raise (FormatError if status == ERR_FORMAT else HipError)(message)


def _np_u8(a):
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint8
    return a


# ------------------------------------------------------------------ host functions

def encoding(t):
    e, b = C.c_uint32(), C.c_uint32()
    check(dll().tsp_encoding(C.c_uint32(t), C.byref(e), C.byref(b)))
    return e.value, b.value


def make_expert_spec(source_type, columns, rows):
    s = PlanarSpec()
    check(dll().tsp_make_expert_spec(C.c_uint32(source_type), C.c_uint32(columns), C.c_uint32(rows), C.byref(s)))
    return s


def pack_sm16(s12):
    s12 = _np_u8(s12)
    out = np.empty(16, dtype=np.uint8)
    dll().tsp_pack_sm16(s12.ctypes.data_as(u8p), out.ctypes.data_as(u8p))
    return out


def unpack_sm16(sm):
    sm = _np_u8(sm)
    out = np.empty(12, dtype=np.uint8)
    check(dll().tsp_unpack_sm16(sm.ctypes.data_as(u8p), out.ctypes.data_as(u8p)))
    return out


def pack_expert(spec, gguf):
    gguf = _np_u8(gguf)
    out = np.zeros(spec.planar_expert_bytes, dtype=np.uint8)
    check(dll().tsp_pack_expert_planar_v3(C.byref(spec), gguf.ctypes.data_as(u8p), C.c_uint64(gguf.size),
                                          out.ctypes.data_as(u8p), C.c_uint64(out.size)))
    return out


def unpack_expert(spec, planar):
    planar = _np_u8(planar)
    out = np.zeros(spec.source_expert_bytes, dtype=np.uint8)
    check(dll().tsp_unpack_expert_planar_v3(C.byref(spec), planar.ctypes.data_as(u8p), C.c_uint64(planar.size),
                                            out.ctypes.data_as(u8p), C.c_uint64(out.size)))
    return out


def pack_experts(spec, gguf_stack, experts):
    """[experts] contiguous planar experts (the layout of a down-projection tensor)."""
    gguf_stack = _np_u8(gguf_stack)
    sb = spec.source_expert_bytes
    return np.concatenate([pack_expert(spec, gguf_stack[e * sb:(e + 1) * sb]) for e in range(experts)])


def pack_coloc_half(spec, gate, up, experts, half):
    gate, up = _np_u8(gate), _np_u8(up)
    out = np.zeros((experts // 2) * 2 * spec.planar_expert_bytes, dtype=np.uint8)
    check(dll().tsp_pack_coloc_half(C.byref(spec), gate.ctypes.data_as(u8p), up.ctypes.data_as(u8p), C.c_uint32(experts),
                                    C.c_uint32(half), out.ctypes.data_as(u8p), C.c_uint64(out.size)))
    return out


def q8_lanes_quant_offset(columns, block, index):
    o = C.c_uint64()
    check(dll().tsp_q8_lanes_quant_offset(C.c_uint32(columns), C.c_uint32(block), C.c_uint32(index), C.byref(o)))
    return o.value


def q8_lanes_pack_rows(columns, original):
    original = _np_u8(original)
    out = np.empty_like(original)
    check(dll().tsp_q8_lanes_pack_rows(C.c_uint32(columns), original.ctypes.data_as(u8p), out.ctypes.data_as(u8p), C.c_uint64(original.size)))
    return out


def q8_lanes_unpack_rows(columns, packed):
    packed = _np_u8(packed)
    out = np.empty_like(packed)
    check(dll().tsp_q8_lanes_unpack_rows(C.c_uint32(columns), packed.ctypes.data_as(u8p), out.ctypes.data_as(u8p), C.c_uint64(packed.size)))
    return out


def grouped_mm_plan(t, layout, columns, rows, experts, selected, tokens, in_stride, out_stride, broadcast, allow_2k=False):
    p = GroupedMmPlan()
    check(dll().tsp_grouped_mm_plan(C.c_uint32(t), C.c_uint32(layout), C.c_uint32(columns), C.c_uint32(rows), C.c_uint32(experts),
                                    C.c_uint32(selected), C.c_uint32(tokens), C.c_uint64(in_stride), C.c_uint64(out_stride),
                                    C.c_int(bool(broadcast)), C.c_int(bool(allow_2k)), C.byref(p)))
    return p


def dense_mm_q8_plan(layout, columns, rows, tokens, in_stride, out_stride, allow_2k=False):
    p = GroupedMmPlan()
    check(dll().tsp_dense_mm_q8_plan(C.c_uint32(layout), C.c_uint32(columns), C.c_uint32(rows), C.c_uint32(tokens),
                                     C.c_uint64(in_stride), C.c_uint64(out_stride), C.c_int(bool(allow_2k)), C.byref(p)))
    return p


def moe_mm_many_bytes(channels, hidden, experts, selected, capacity, allow_2k=False):
    views = (C.c_uint64 * 13)()
    total = C.c_uint64()
    check(dll().tsp_moe_mm_many_bytes(C.c_uint32(channels), C.c_uint32(hidden), C.c_uint32(experts), C.c_uint32(selected),
                                      C.c_uint32(capacity), C.c_int(bool(allow_2k)), views, C.byref(total)))
    return list(views), total.value


def q8_many_width(remaining):
    w = C.c_uint32()
    check(dll().tsp_q8_many_width(C.c_uint32(remaining), C.byref(w)))
    return w.value


def q8_many_chunks(rows):
    w = C.c_uint32()
    check(dll().tsp_q8_many_chunks(C.c_uint32(rows), C.byref(w)))
    return w.value


# ------------------------------------------------------------------ device side

class Device:
    """Device buffers are torch tensors on cuda:0; kernels run on torch's current stream."""

    def __init__(self):
        import torch
        self.torch = torch
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU: the HIP path cannot run and there is no CPU fallback")
        self.dev = torch.device("cuda", torch.cuda.current_device())
        self.err = torch.zeros(1, dtype=torch.int32, device=self.dev)
        dll()

    # -- memory
    def upload(self, a):
        a = np.ascontiguousarray(a)
        if a.dtype == np.uint32:
            return self.torch.from_numpy(a.view(np.int32)).to(self.dev)
        if a.dtype == np.uint16:
            return self.torch.from_numpy(a.view(np.int16)).to(self.dev)
        return self.torch.from_numpy(a).to(self.dev)

    def empty(self, shape, dtype="float32"):
        return self.torch.empty(shape, dtype=getattr(self.torch, dtype), device=self.dev)

    def zeros(self, shape, dtype="float32"):
        return self.torch.zeros(shape, dtype=getattr(self.torch, dtype), device=self.dev)

    def full(self, shape, value, dtype="float32"):
        return self.torch.full(shape, value, dtype=getattr(self.torch, dtype), device=self.dev)

    @staticmethod
    def ptr(t):
        return C.c_void_p(t.data_ptr()) if t is not None else None

    @staticmethod
    def nbytes(t):
        return t.numel() * t.element_size()

    def stream(self):
        return C.c_void_p(self.torch.cuda.current_stream().cuda_stream)

    def sync(self):
        self.torch.cuda.synchronize()

    def clear_error(self):
        self.err.zero_()

    def error(self):
        """Reads and clears the sticky error word (synchronises)."""
        value = int(self.err.item()) & 0xFFFFFFFF
        self.err.zero_()
        return value

    # -- operators
    def dequantize(self, t, blocks, nelem):
        out = self.empty(nelem)
        check(dll().tsp_dequantize(C.c_uint32(t), self.ptr(blocks), C.c_uint64(self.nbytes(blocks)), self.ptr(out),
                                   C.c_uint64(nelem), self.ptr(self.err), self.stream()))
        return out

    def dequantize_planar(self, spec, planar):
        out = self.empty(spec.rows * spec.columns)
        check(dll().tsp_dequantize_planar(C.byref(spec), self.ptr(planar), self.ptr(out), self.ptr(self.err), self.stream()))
        return out

    def gemv(self, t, matrix, x, columns, rows, layout=LAYOUT_GGUF, y=None, matrix_bytes=None):
        y = self.empty(rows) if y is None else y
        nbytes = self.nbytes(matrix) if matrix_bytes is None else matrix_bytes
        check(dll().tsp_gemv(C.c_uint32(t), C.c_uint32(layout), self.ptr(matrix), C.c_uint64(nbytes), self.ptr(x), self.ptr(y),
                             C.c_uint32(columns), C.c_uint32(rows), self.ptr(self.err), self.stream()))
        return y

    def gemv_rows(self, t, matrix, x, y, count, columns, rows, x_stride, y_stride, layout=LAYOUT_GGUF):
        check(dll().tsp_gemv_rows(C.c_uint32(t), C.c_uint32(layout), self.ptr(matrix), C.c_uint64(self.nbytes(matrix)), self.ptr(x),
                                  C.c_uint64(x_stride), self.ptr(y), C.c_uint64(y_stride), C.c_uint32(count), C.c_uint32(columns),
                                  C.c_uint32(rows), self.ptr(self.err), self.stream()))
        return y

    def q8_matvec_many(self, matrix, x, columns, rows, width, layout=LAYOUT_GGUF, y=None):
        y = self.empty((width, rows)) if y is None else y
        check(dll().tsp_q8_matvec_many(C.c_uint32(layout), self.ptr(matrix), C.c_uint64(self.nbytes(matrix)), self.ptr(x), self.ptr(y),
                                       C.c_uint32(columns), C.c_uint32(rows), C.c_uint32(width), self.ptr(self.err), self.stream()))
        return y

    def routed_gemv(self, t, matrices, ids, x, columns, rows, experts, selected, broadcast):
        y = self.empty((selected, rows))
        check(dll().tsp_routed_gemv(C.c_uint32(t), self.ptr(matrices), C.c_uint64(self.nbytes(matrices)), self.ptr(ids), self.ptr(x),
                                    self.ptr(y), C.c_uint32(columns), C.c_uint32(rows), C.c_uint32(experts), C.c_uint32(selected),
                                    C.c_int(bool(broadcast)), self.ptr(self.err), self.stream()))
        return y
