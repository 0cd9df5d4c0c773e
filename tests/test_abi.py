"""CPU-side checks of the C-ABI library: it loads, exports every symbol the header declares,
agrees with the record strides the reference pins, and refuses to run without a GPU."""
import ctypes as C
import os

import pytest

from smelt_amd import runtime as rt


def test_library_loads_and_exports_every_declared_symbol():
    lib = rt.load_library()
    names = rt.exported_symbols()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), n


def test_record_strides_match_the_reference_table_format():
    # DispatchTableTests.swift:12-31: strides 16 / 8 / 360
    assert C.sizeof(rt.BufferRecord) == 16
    assert C.sizeof(rt.ConstantRecord) == 8
    assert C.sizeof(rt.DispatchRecord) == 360
    assert rt.DispatchRecord.pipeline.offset == 2
    assert rt.DispatchRecord.style.offset == 4
    assert rt.DispatchRecord.min_seq_len.offset == 8
    assert rt.DispatchRecord.grid_w.offset == 12
    assert rt.DispatchRecord.tg_d.offset == 32
    assert rt.DispatchRecord.buffers.offset == 40
    assert rt.DispatchRecord.constants.offset == 296


def test_dispatch_table_size_must_be_a_multiple_of_the_stride():
    lib = rt.load_library()
    n = C.c_size_t()
    assert lib.smelt_hip_dispatch_table_count(360 * 7, C.byref(n)) == 0 and n.value == 7
    assert lib.smelt_hip_dispatch_table_count(360 * 7 + 8, C.byref(n)) == -3
    assert b"not a multiple of dispatch stride 360" in lib.smelt_hip_last_error(None)


def test_no_gpu_means_a_loud_error_not_a_fallback():
    import subprocess, sys
    # run in a child so a box that does have a GPU is unaffected by the hidden device
    code = ("import os; os.environ['HIP_VISIBLE_DEVICES']='-1'; os.environ['ROCR_VISIBLE_DEVICES']='-1';"
            "from smelt_amd import runtime as rt\n"
            "try:\n    rt.Context()\n    print('CREATED')\n"
            "except rt.SmeltHipError as e:\n    print('ERR', e.code)\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True, timeout=120)
    assert "ERR -8" in out.stdout, out.stdout + out.stderr
