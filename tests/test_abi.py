"""CPU-side checks of the C-ABI library: it loads, exports every declared symbol, and the
device-free entry points (type registry, error text, init failure) behave like the reference's."""
import ctypes as C
import os
import re

import pytest

from axonml_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    return _lib.load_library()


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "axq.h")).read()
    return sorted(set(re.findall(r"AXQ_API\s+[\w\s\*]+?\b(axq_\w+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    names = declared_symbols()
    assert len(names) >= 40
    for n in names:
        assert hasattr(lib, n), f"libaxq.so does not export {n}"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names


def test_type_registry_matches_reference(lib):
    # types.rs:45-78
    table = {0: ("Q8_0", 32, 34, 8), 1: ("Q4_0", 32, 18, 4), 2: ("Q4_1", 32, 20, 4), 3: ("Q5_0", 32, 22, 5),
             4: ("Q5_1", 32, 24, 5), 5: ("F16", 1, 2, 16), 6: ("F32", 1, 4, 32), 7: ("Q4_K", 256, 144, 4),
             8: ("Q6_K", 256, 210, 6), 9: ("Q5_K", 256, 176, 5)}
    for t, (name, bs, bb, bits) in table.items():
        assert lib.axq_type_name(t).decode() == name
        assert lib.axq_type_block_size(t) == bs
        assert lib.axq_type_bytes_per_block(t) == bb
        assert lib.axq_type_bits_per_value(t) == bits
        assert lib.axq_type_is_block_quantized(t) == (0 if name in ("F16", "F32") else 1)
    assert lib.axq_type_name(42) is None and lib.axq_type_block_size(42) == 0


def test_from_str_aliases(lib):
    # types.rs:94-105 and its test :356-363
    for s, t in [("Q8_0", 0), ("INT8", 0), ("q8", 0), ("Q4", 1), ("int4", 1), ("Q4_1", 2), ("Q5", 3), ("Q5_1", 4),
                 ("F16", 5), ("half", 5), ("FLOAT16", 5), ("F32", 6), ("float", 6), ("Q4_K", 7), ("Q6_K", 8), ("q6k", 8), ("Q5_K", 9), ("Q5K", 9)]:
        assert lib.axq_type_from_str(s.encode()) == t
    assert lib.axq_type_from_str(b"invalid") == -1


def test_block_counts(lib):
    assert lib.axq_num_blocks(0, 8) == 1 and lib.axq_num_blocks(1, 64) == 2  # quantize.rs:294-313
    assert lib.axq_packed_bytes(7, 14336 * 4096) == 33030144
    assert lib.axq_packed_bytes(0, 4096 * 4096) == 17825792
    assert lib.axq_packed_bytes(1, 11008 * 4096) == 25362432
    assert lib.axq_packed_bytes(2, 11008 * 4096) == 28180480


def test_status_strings_follow_quant_error_display(lib):
    assert lib.axq_status_str(0).decode() == "ok"
    assert lib.axq_status_str(-2).decode().startswith("Invalid quantization type")  # error.rs:21
    assert lib.axq_status_str(-4).decode().startswith("Data length mismatch")  # error.rs:34
    assert lib.axq_status_str(-20).decode() == "Device not found"


def test_null_arguments_are_errors_not_crashes(lib):
    assert lib.axq_init(0, None) == -30
    assert lib.axq_synchronize(None) == -30
    assert lib.axq_quantize(None, 0, None, 0, None, 0) == -30
    assert lib.axq_weight_info(None, None, None, None, None) == -30
    lib.axq_destroy(None)
    lib.axq_weight_free(None, None)


def test_init_without_gpu_fails_loudly(lib):
    import torch

    if torch.cuda.device_count() > 0:
        pytest.skip("a GPU is present")
    h = C.c_void_p()
    st = lib.axq_init(0, C.byref(h))
    assert st == -20 and not h.value
    assert b"HIP device" in lib.axq_last_error(None)
