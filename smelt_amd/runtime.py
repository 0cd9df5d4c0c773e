"""ctypes binding of the C-ABI in include/smelt_hip.h (thin; all logic lives in the library).

There is no CPU fallback: every call goes to libsmelt_hip.so and the gfx950 code object, and
loading fails loudly if either file has not been built.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(HERE, "lib")
HOST_LIB = os.path.join(LIB_DIR, "libsmelt_hip.so")
HSACO = os.path.join(LIB_DIR, "smelt_kernels.hsaco")
MATVEC_AUTO, MATVEC_MATRIX_CORE, MATVEC_VECTOR = 0, 1, 2


def code_objects() -> list[str]:
    """Every gfx950 code object of the build (smelt_kernels*.hsaco), in load order."""
    import glob
    return sorted(glob.glob(os.path.join(LIB_DIR, "smelt_kernels*.hsaco")))

ACT_F16, ACT_BF16 = 0, 1
SLOT_CUR, SLOT_ALT = -1, -2
STYLE_THREADGROUPS, STYLE_THREADS = 0, 1
GRID_LITERAL, GRID_SEQ_LEN, GRID_SEQ_LEN_MUL, GRID_SEQ_LEN_CEIL_DIV = 0, 1, 2, 3
CONST_U32, CONST_F32, CONST_POSITION, CONST_POSITION_PLUS1, CONST_SEQ_LEN = 0, 1, 2, 3, 4


class SmeltHipError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"smelt_hip error {code}: {message}")
        self.code = code
        self.message = message


class BufferRecord(C.Structure):
    _fields_ = [("slot", C.c_int16), ("binding_index", C.c_uint8), ("offset_kind", C.c_uint8),
                ("_pad", C.c_uint32), ("offset", C.c_uint64)]


class ConstantRecord(C.Structure):
    _fields_ = [("kind", C.c_uint8), ("binding_index", C.c_uint8), ("pad", C.c_uint16),
                ("value", C.c_uint32)]


class DispatchRecord(C.Structure):
    _fields_ = [("op_kind", C.c_uint8), ("_pad0", C.c_uint8), ("pipeline", C.c_uint16),
                ("style", C.c_uint8), ("buffer_count", C.c_uint8), ("constant_count", C.c_uint8),
                ("_pad1", C.c_uint8), ("min_seq_len", C.c_uint16), ("_pad2", C.c_uint16),
                ("grid_w", C.c_uint32), ("grid_h", C.c_uint32), ("grid_d", C.c_uint32),
                ("tg_w", C.c_uint32), ("tg_h", C.c_uint32), ("tg_d", C.c_uint32),
                ("_pad3", C.c_uint32),
                ("buffers", BufferRecord * 16), ("constants", ConstantRecord * 8)]


assert C.sizeof(BufferRecord) == 16 and C.sizeof(ConstantRecord) == 8
assert C.sizeof(DispatchRecord) == 360


def make_record(pipeline: int, buffers, constants, grid, tg, style=STYLE_THREADGROUPS,
                grid_kinds=(0, 0, 0), min_seq_len=0) -> DispatchRecord:
    """buffers: (slot, binding_index, offset[, offset_kind]); constants: (binding_index, value
    [, kind]) where a float value is stored as its IEEE bits with kind 1."""
    r = DispatchRecord()
    r.op_kind = 0
    r.pipeline = pipeline
    r.style = style | (grid_kinds[0] << 2) | (grid_kinds[1] << 4) | (grid_kinds[2] << 6)
    r.buffer_count = len(buffers)
    r.constant_count = len(constants)
    r.min_seq_len = min_seq_len
    r.grid_w, r.grid_h, r.grid_d = grid
    r.tg_w, r.tg_h, r.tg_d = tg
    for i, b in enumerate(buffers):
        r.buffers[i].slot, r.buffers[i].binding_index, r.buffers[i].offset = b[0], b[1], b[2]
        r.buffers[i].offset_kind = b[3] if len(b) > 3 else 0
    for i, c in enumerate(constants):
        idx, val = c[0], c[1]
        kind = c[2] if len(c) > 2 else (CONST_F32 if isinstance(val, float) else CONST_U32)
        if isinstance(val, float):
            val = int(np.float32(val).view(np.uint32))
        r.constants[i].binding_index, r.constants[i].value, r.constants[i].kind = idx, val, kind
    return r


def swap_record() -> DispatchRecord:
    r = DispatchRecord()
    r.op_kind = 1
    return r


_lib = None


def load_library() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    for path in (HOST_LIB, HSACO):
        if not os.path.exists(path):
            raise FileNotFoundError(
                f"{path} is missing: build the HIP extension first (python -m smelt_amd.build); "
                "this backend has no CPU fallback")
    lib = C.CDLL(HOST_LIB)
    vp, i32, u32, sz = C.c_void_p, C.c_int, C.c_uint32, C.c_size_t
    rp = C.POINTER(DispatchRecord)
    sig = {
        "smelt_hip_context_create": (i32, [i32, C.POINTER(vp)]),
        "smelt_hip_context_destroy": (None, [vp]),
        "smelt_hip_last_error": (C.c_char_p, [vp]),
        "smelt_hip_set_activation_dtype": (i32, [vp, i32]),
        "smelt_hip_set_matvec_engine": (i32, [vp, i32]),
        "smelt_hip_module_load": (i32, [vp, vp, sz]),
        "smelt_hip_module_load_file": (i32, [vp, C.c_char_p]),
        "smelt_hip_pipeline_create": (i32, [vp, C.c_char_p, i32, C.POINTER(u32)]),
        "smelt_hip_pipeline_count": (i32, [vp]),
        "smelt_hip_pipeline_is_ready": (i32, [vp, u32]),
        "smelt_hip_buffer_alloc": (i32, [vp, i32, sz]),
        "smelt_hip_buffer_write": (i32, [vp, i32, sz, vp, sz]),
        "smelt_hip_buffer_read": (i32, [vp, i32, sz, vp, sz]),
        "smelt_hip_buffer_size": (i32, [vp, i32, C.POINTER(sz)]),
        "smelt_hip_weights_upload": (i32, [vp, i32, vp, sz]),
        "smelt_hip_set_cache_seq_capacity": (i32, [vp, u32]),
        "smelt_hip_dispatch_table_count": (i32, [sz, C.POINTER(sz)]),
        "smelt_hip_encode_decode_record": (i32, [vp, rp, i32, i32, C.c_int32]),
        "smelt_hip_encode_prefill_record": (i32, [vp, rp, i32, i32, C.c_int32, C.c_int32]),
        "smelt_hip_encode_prefill_record_static_scratch": (i32, [vp, rp, i32, i32, C.c_int32, C.c_int32]),
        "smelt_hip_interpret_decode_table": (i32, [vp, rp, sz, i32, i32, C.c_int32]),
        "smelt_hip_interpret_prefill_table": (i32, [vp, rp, sz, i32, i32, C.c_int32, C.c_int32]),
        "smelt_hip_submit": (i32, [vp]),
        "smelt_hip_wait": (i32, [vp]),
        "smelt_hip_last_gpu_ns": (i32, [vp, C.POINTER(C.c_uint64)]),
        "smelt_hip_benchmark_record": (i32, [vp, rp, i32, i32, i32, C.c_int32, C.c_int32, i32, i32,
                                             C.POINTER(C.c_float)]),
        "smelt_hip_graph_capture_decode": (i32, [vp, rp, sz, i32, i32, C.c_int32, C.POINTER(vp)]),
        "smelt_hip_graph_capture_prefill": (i32, [vp, rp, sz, i32, i32, C.c_int32, C.c_int32,
                                                  C.POINTER(vp)]),
        "smelt_hip_graph_launch": (i32, [vp, vp]),
        "smelt_hip_graph_destroy": (None, [vp, vp]),
        "smelt_hip_graph_time": (i32, [vp, vp, i32, C.POINTER(C.c_float)]),
        "smelt_hip_device_info": (i32, [vp, C.c_char_p, sz, C.POINTER(i32), C.POINTER(sz),
                                        C.POINTER(sz)]),
        "smelt_hip_memory_info": (i32, [vp, C.POINTER(sz), C.POINTER(sz)]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def exported_symbols() -> list[str]:
    """Function names the headers under include/ declare (parsed from the header text)."""
    import re
    names = set()
    inc = os.path.join(os.path.dirname(HERE), "include")
    for hdr in sorted(os.listdir(inc)):
        if hdr.endswith(".h"):
            text = open(os.path.join(inc, hdr)).read()
            text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
            names.update(re.findall(r"\b(smelt_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


class Context:
    """One device context: code object, pipeline table, slot buffers, one stream."""

    def __init__(self, device: int = 0, act_dtype: int = ACT_F16, load_module: bool = True):
        self.lib = load_library()
        h = C.c_void_p()
        rc = self.lib.smelt_hip_context_create(device, C.byref(h))
        if rc != 0:
            raise SmeltHipError(rc, (self.lib.smelt_hip_last_error(None) or b"").decode())
        self.h = h
        self._pipelines: dict[str, int] = {}
        self.check(self.lib.smelt_hip_set_activation_dtype(self.h, act_dtype))
        if load_module:
            self.check(self.lib.smelt_hip_module_load_file(self.h, LIB_DIR.encode()))

    def set_matvec_engine(self, engine: int) -> None:
        self.check(self.lib.smelt_hip_set_matvec_engine(self.h, engine))

    def close(self) -> None:
        if getattr(self, "h", None):
            self.lib.smelt_hip_context_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def check(self, rc: int) -> int:
        if rc < 0:
            raise SmeltHipError(rc, (self.lib.smelt_hip_last_error(self.h) or b"").decode())
        return rc

    # -- pipelines -----------------------------------------------------------------------
    def pipeline(self, entry: str, allow_missing: bool = False) -> int:
        if entry in self._pipelines:
            return self._pipelines[entry]
        idx = C.c_uint32()
        self.check(self.lib.smelt_hip_pipeline_create(self.h, entry.encode(), int(allow_missing),
                                                      C.byref(idx)))
        self._pipelines[entry] = idx.value
        return idx.value

    def pipeline_ready(self, index: int) -> bool:
        return self.check(self.lib.smelt_hip_pipeline_is_ready(self.h, index)) == 1

    # -- buffers -------------------------------------------------------------------------
    def alloc(self, slot: int, nbytes: int) -> None:
        self.check(self.lib.smelt_hip_buffer_alloc(self.h, slot, nbytes))

    def upload_weights(self, slot: int, data: np.ndarray) -> None:
        data = np.ascontiguousarray(data)
        self.check(self.lib.smelt_hip_weights_upload(self.h, slot, data.ctypes.data, data.nbytes))

    def write(self, slot: int, data: np.ndarray, offset: int = 0) -> None:
        data = np.ascontiguousarray(data)
        self.check(self.lib.smelt_hip_buffer_write(self.h, slot, offset, data.ctypes.data, data.nbytes))

    def put(self, slot: int, data: np.ndarray) -> None:
        """Allocate `slot` to the size of `data` and copy it in."""
        data = np.ascontiguousarray(data)
        self.alloc(slot, max(data.nbytes, 1))
        self.write(slot, data)

    def read(self, slot: int, dtype, count: int, offset: int = 0) -> np.ndarray:
        out = np.zeros(count, dtype=dtype)
        self.check(self.lib.smelt_hip_buffer_read(self.h, slot, offset, out.ctypes.data, out.nbytes))
        return out

    # -- dispatch ------------------------------------------------------------------------
    def encode_decode(self, rec: DispatchRecord, cur=0, alt=1, position=0) -> int:
        return self.check(self.lib.smelt_hip_encode_decode_record(self.h, C.byref(rec), cur, alt, position))

    def encode_prefill(self, rec: DispatchRecord, cur=0, alt=1, seq_len=1, start_pos=0) -> int:
        return self.check(self.lib.smelt_hip_encode_prefill_record(self.h, C.byref(rec), cur, alt,
                                                                   seq_len, start_pos))

    def encode_prefill_static_scratch(self, rec: DispatchRecord, cur=0, alt=1, seq_len=1, start_pos=0) -> int:
        """encode_prefill with the split-K scratch in the library's file-scope device array."""
        return self.check(self.lib.smelt_hip_encode_prefill_record_static_scratch(
            self.h, C.byref(rec), cur, alt, seq_len, start_pos))

    @staticmethod
    def table(records) -> C.Array:
        arr = (DispatchRecord * len(records))()
        for i, r in enumerate(records):
            arr[i] = r
        return arr

    def interpret_decode(self, table, cur=0, alt=1, position=0) -> int:
        return self.check(self.lib.smelt_hip_interpret_decode_table(self.h, table, len(table), cur, alt, position))

    def interpret_prefill(self, table, cur=0, alt=1, seq_len=1, start_pos=0) -> int:
        return self.check(self.lib.smelt_hip_interpret_prefill_table(self.h, table, len(table), cur,
                                                                     alt, seq_len, start_pos))

    def submit(self) -> None:
        self.check(self.lib.smelt_hip_submit(self.h))

    def wait(self) -> None:
        self.check(self.lib.smelt_hip_wait(self.h))

    def last_gpu_ns(self) -> int:
        v = C.c_uint64()
        self.check(self.lib.smelt_hip_last_gpu_ns(self.h, C.byref(v)))
        return v.value

    def benchmark_record(self, rec, warmup=20, iters=200, prefill=False, a=0, b=0, cur=0, alt=1) -> np.ndarray:
        out = np.zeros(iters, np.float32)
        self.check(self.lib.smelt_hip_benchmark_record(
            self.h, C.byref(rec), cur, alt, int(prefill), a, b, warmup, iters,
            out.ctypes.data_as(C.POINTER(C.c_float))))
        return out

    def capture_decode(self, table, cur=0, alt=1, position=0):
        g = C.c_void_p()
        n = self.check(self.lib.smelt_hip_graph_capture_decode(self.h, table, len(table), cur, alt,
                                                               position, C.byref(g)))
        return g, n

    def capture_prefill(self, table, cur=0, alt=1, seq_len=1, start_pos=0):
        g = C.c_void_p()
        n = self.check(self.lib.smelt_hip_graph_capture_prefill(self.h, table, len(table), cur, alt,
                                                                seq_len, start_pos, C.byref(g)))
        return g, n

    def graph_launch(self, g) -> int:
        return self.check(self.lib.smelt_hip_graph_launch(self.h, g))

    def graph_time(self, g, iters: int) -> float:
        v = C.c_float()
        self.check(self.lib.smelt_hip_graph_time(self.h, g, iters, C.byref(v)))
        return float(v.value)

    def graph_destroy(self, g) -> None:
        self.lib.smelt_hip_graph_destroy(self.h, g)

    def memory_info(self) -> tuple[int, int]:
        """(free, total) device bytes as hipMemGetInfo reports them."""
        free, total = C.c_size_t(), C.c_size_t()
        self.check(self.lib.smelt_hip_memory_info(self.h, C.byref(free), C.byref(total)))
        return free.value, total.value

    def device_info(self) -> dict:
        name = C.create_string_buffer(256)
        cu, lds, hbm = C.c_int(), C.c_size_t(), C.c_size_t()
        self.check(self.lib.smelt_hip_device_info(self.h, name, 256, C.byref(cu), C.byref(lds), C.byref(hbm)))
        return {"name": name.value.decode(), "compute_units": cu.value, "lds_per_block": lds.value,
                "hbm_bytes": hbm.value}
