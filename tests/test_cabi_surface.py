"""Host-side checks that need no GPU: the C ABI library loads and exports every symbol the header declares."""
import os
import re

from mor_amd import _cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mor_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mor_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    L = _cabi.lib()
    names = declared_symbols()
    assert len(names) >= 12
    for n in names:
        assert hasattr(L, n), n
    assert sorted(_cabi.SIGNATURES) == names


def test_version_and_workspace_sizes():
    L = _cabi.lib()
    assert b"gfx950" in L.mor_version()
    assert L.mor_workspace_bytes(_cabi.OP_FAKE_QUANTIZE, 128, 128, 1, 32) == 0
    small = L.mor_workspace_bytes(_cabi.OP_BLOCK_SCALING, 256, 256, 128, 128)
    big = L.mor_workspace_bytes(_cabi.OP_CHANNEL_SCALING, 256, 256, 1, 32)
    assert 0 < small < big and big - small == (256 * 8 - 4) * 4
    assert L.mor_workspace_bytes(_cabi.OP_E8MX, 256, 256, 128, 128) == small - 4 * 4


def test_argument_errors_are_reported_without_a_gpu():
    """Argument validation happens before any HIP call, so it can be exercised on the CPU."""
    L = _cabi.lib()
    assert L.mor_fake_quantize(None, None, None, 16, 16, 4, 4, 0.0, 1, 1, 0, None) == -1
    assert b"NULL" in L.mor_last_error()
    assert L.mor_fake_quantize(1, 1, 1, 0, 16, 4, 4, 0.0, 1, 1, 0, None) == -1
    assert b"positive" in L.mor_last_error()
    assert L.mor_block_scaling(1, 1, 1, 1, 1, 1, 100, 256, 128, 128, 0.045, 1, 0, 1, 1 << 20, 0, None) == -1
    assert b"divide" in L.mor_last_error()
    assert L.mor_block_scaling(1, 1, 1, 1, 1, 1, 256, 256, 128, 128, 0.045, 1, 0, None, 0, 0, None) == -2
    assert L.mor_e8mx(1, 1, 16, 16, 4, 4, 7, 1, 1, 64, 0, None) == -1
    assert L.mor_quant_dequant(1, 1, 16, 9, None) == -1


def test_batch_entry_rejects_bad_arguments_without_a_gpu():
    """argument checks run before any device call"""
    from mor_amd import _cabi
    from mor_amd.batch import TensorDesc
    import ctypes as C
    L = _cabi.lib()
    assert L.mor_fake_quantize_batch(None, 3, 0, None) != 0
    assert b"descriptor" in L.mor_last_error()
    assert L.mor_fake_quantize_batch(None, -1, 0, None) != 0
    assert L.mor_fake_quantize_batch(None, 0, 0, None) == 0            # an empty list is no work
    d = (TensorDesc * 1)()
    d[0].input, d[0].output, d[0].meta = 256, 256, 256                 # (never dereferenced: the shape is rejected first)
    d[0].rows, d[0].cols, d[0].block_rows, d[0].block_cols = 4, 0, 1, 32
    assert L.mor_fake_quantize_batch(d, 1, 0, None) != 0
    assert b"positive" in L.mor_last_error()
    assert C.sizeof(TensorDesc) == 80


def test_tile_code_entries_reject_bad_arguments_without_a_gpu():
    """argument checks of mor_mor_quantize / mor_mor_dequantize run before any device call"""
    from mor_amd import _cabi
    L = _cabi.lib()
    assert L.mor_mor_quantize(256, 512, 768, 1024, 128, 200, 0.0, 1, None) == -1 and b"multiples of 128" in L.mor_last_error()
    assert L.mor_mor_quantize(256, 512, 768, 1024, 128, 256, 0.0, 4, None) == -1 and b"mode" in L.mor_last_error()
    assert L.mor_mor_quantize(256, 256, 768, 1024, 128, 256, 0.0, 1, None) == -1 and b"different" in L.mor_last_error()
    assert L.mor_mor_quantize(256, 520, 768, 1024, 128, 256, 0.0, 1, None) == -1 and b"aligned" in L.mor_last_error()
    assert L.mor_mor_quantize(256, 512, None, 1024, 128, 256, 0.0, 1, None) == -1
    assert L.mor_mor_dequantize(512, 768, 1024, 256, 100, 256, None) == -1
    assert L.mor_mor_dequantize(512, None, 1024, 256, 128, 256, None) == -1
    assert L.mor_mor_transpose(512, 768, 1024, 1536, 2048, 2560, 0, 4, None) == -1 and b"tile grid" in L.mor_last_error()
    assert L.mor_mor_transpose(512, 768, 1024, 512, 2048, 2560, 2, 4, None) == -1 and b"different" in L.mor_last_error()
    assert L.mor_mor_transpose(512, 768, 1024, 1544, 2048, 2560, 2, 4, None) == -1 and b"aligned" in L.mor_last_error()
    assert L.mor_mor_transpose(512, None, 1024, 1536, 2048, 2560, 2, 4, None) == -1
    # a tile row's chunk offsets are 32-bit: tensors of 2^27 columns and more are refused
    assert L.mor_mor_quantize(256, 512, 768, 1024, 128, 1 << 27, 0.0, 1, None) == -1 and b"columns" in L.mor_last_error()
    assert L.mor_fake_quantize_dual_tiles(256, 512, 768, 1024, 1280, 128, 1 << 27, 0.0, 1, 1, None) == -1 and b"2^27" in L.mor_last_error()
