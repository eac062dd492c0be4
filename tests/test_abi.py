"""No-GPU checks of the C ABI: the library loads, exports every symbol include/candy_hip.h
declares (and the binding knows each of them), and argument validation that needs no device
behaves like candy's CPU backend (errors, not crashes)."""
import ctypes
import os
import re

import pytest

from candy_amd import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "candy_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(candy_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = ctypes.CDLL(hip.LIB_PATH)
    names = _declared_symbols()
    assert len(names) >= 40
    for n in names:
        assert hasattr(L, n), f"{n} is declared in candy_hip.h but not exported"


def test_binding_covers_exactly_the_header():
    assert sorted(hip.SIGNATURES) == _declared_symbols()


def test_header_documents_exactly_the_options_the_library_accepts():
    # candy_hip_set_option's table in the header (one "key" default meaning line per switch) against the table the
    # runtime looks keys up in: an undocumented switch or a documented one that does not exist fails here
    header = open(os.path.join(ROOT, "include", "candy_hip.h")).read()
    documented = set(re.findall(r'^ \*\s+"([a-z0-9_.]+)"\s+-?\d+\s', header, flags=re.M))
    runtime = open(os.path.join(ROOT, "candy_amd", "csrc", "runtime.hip")).read()
    accepted = set(re.findall(r'\{"([a-z0-9_.]+)", &candy::Options::', runtime))
    assert len(accepted) >= 15
    assert documented == accepted, (sorted(documented - accepted), sorted(accepted - documented))


def test_format_tables():
    L = hip.lib()
    assert [L.candy_hip_block_bytes(f) for f in (hip.Q4_0, hip.Q8_0, hip.Q4_K, hip.Q6_K, hip.Q4_0_GGML)] == [18, 34, 144, 210, 18]
    assert [L.candy_hip_block_elems(f) for f in (hip.Q4_0, hip.Q8_0, hip.Q4_K, hip.Q6_K)] == [32, 32, 256, 256]
    # the reference's other formats, by ggml type id (Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K, Q8_K) and Q4_1 in ggml order
    assert [L.candy_hip_block_bytes(f) for f in (3, 6, 7, 10, 11, 13, 15, 103)] == [20, 22, 24, 84, 110, 176, 292, 20]
    assert [L.candy_hip_block_elems(f) for f in (3, 6, 7, 10, 11, 13, 15, 103)] == [32, 32, 32, 256, 256, 256, 256, 32]
    assert L.candy_hip_block_bytes(9) == 0 and L.candy_hip_block_bytes(16) == 0
    # sizes the hot-path shapes must have
    assert L.candy_hip_qweight_bytes(hip.Q4_K, 4096, 11008) == 25362432
    assert L.candy_hip_qweight_bytes(hip.Q8_0, 32000, 4096) == 139264000
    assert L.candy_hip_qweight_bytes(hip.Q6_K, 32000, 4096) == 107520000
    assert L.candy_hip_qweight_bytes(hip.Q4_0, 4096, 4096) == 9437184
    assert L.candy_hip_qweight_bytes(hip.Q4_K, 16, 100) == 0  # cols not a multiple of the block


def test_nil_and_shape_errors_do_not_need_a_device():
    L = hip.lib()
    assert L.candy_hip_device_count(None) == 1
    assert b"nil" in L.candy_hip_last_error()
    out = ctypes.c_void_p()
    # nil device handle
    assert L.candy_hip_qtensor_upload(None, hip.Q4_K, 4, 256, None, 4 * 144, ctypes.byref(out)) == 1
    assert L.candy_hip_synchronize(None) == 1
    assert L.candy_hip_qmatmul(None, None, None, 1, None) == 1
    assert b"nil" in L.candy_hip_last_error()
    assert L.candy_hip_quantize_q8_0(None, None, 1, 33, None) == 1
    assert b"multiple of the block size" in L.candy_hip_last_error()
    assert L.candy_hip_dequantize_blocks(None, 77, None, 1, None) == 1
    assert b"unknown quantized format" in L.candy_hip_last_error()
    assert L.candy_hip_matmul_f32(None, None, None, None, 1, 0, 1, 1, 0) == 1
    assert b"invalid matrix dimensions" in L.candy_hip_last_error()  # cpu/storage.go:877-879


@pytest.mark.skipif(hip.device_count() > 0, reason="only meaningful without a GPU")
def test_open_fails_loudly_without_a_gpu():
    with pytest.raises(hip.CandyHipError):
        hip.Device(0)


def test_product_code_never_touches_the_oracle():
    # the oracle is test infrastructure: nothing under candy_amd/ or include/ may mention it
    bad = []
    for base in ("candy_amd", "include"):
        for dp, _, files in os.walk(os.path.join(ROOT, base)):
            if "build" in dp.split(os.sep):
                continue
            for f in files:
                if f.endswith((".py", ".hip", ".h", ".hpp", ".cpp", ".go", "Makefile")):
                    t = open(os.path.join(dp, f), errors="ignore").read()
                    if re.search(r"candy_oracle|from oracle|import oracle|liboracle", t):
                        bad.append(os.path.join(dp, f))
    assert not bad, bad
