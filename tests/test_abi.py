"""The C-ABI library: it loads without a GPU, exports every symbol the header declares, and rejects bad
arguments with the documented codes before touching the device."""
import ctypes as C
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


def _declared():
    text = (ROOT / "include" / "bergson_amd.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bgx_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from bergson_amd import _lib

    lib = _lib.load()
    names = _declared()
    assert "bgx_collect_seq" in names and "bgx_scan" in names and len(names) >= 9
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes bindings and header disagree"
    assert lib.bgx_abi_version() == _lib.ABI_VERSION == 12


def test_module_desc_layout_matches_header():
    from bergson_amd._lib import ModuleDesc

    # 8 pointers, 5 int64, 2 int32
    assert C.sizeof(ModuleDesc) == 8 * 8 + 5 * 8 + 2 * 4
    assert ModuleDesc.out_col.offset == 8 * 8 + 4 * 8 and ModuleDesc.I.offset == 8 * 8 + 5 * 8


def test_block_desc_layout_matches_header():
    from bergson_amd._lib import BlockDesc

    # pointer, int64, 2 int32
    assert C.sizeof(BlockDesc) == 24 and BlockDesc.col0.offset == 8 and BlockDesc.dim.offset == 16


def test_precond_argument_errors_before_any_launch():
    from bergson_amd import _lib

    lib = _lib.load()
    assert lib.bgx_precond_workspace_bytes(48) >= 48 * 24
    descs = (_lib.BlockDesc * 1)()
    rc = lib.bgx_block_gemm(None, 0, 8, None, 0, 8, 4, descs, 1, None, 0, None)
    assert rc == -1 and b"null" in lib.bgx_last_error()
    rc = lib.bgx_gram_accumulate(C.c_void_p(256), 7, 8, 4, descs, 1, C.c_void_p(256), 1 << 20, None)
    assert rc != 0 and b"dtype" in lib.bgx_last_error()
    rc = lib.bgx_block_gemm(C.c_void_p(256), 0, 8, C.c_void_p(256), 0, 8, 4, descs, 1, C.c_void_p(512), 1 << 20, None)
    assert rc != 0 and b"out" in lib.bgx_last_error()


def test_workspace_sizes():
    from bergson_amd import _lib

    lib = _lib.load()
    # head (descriptors + 1025 int32 item ranges of the persistent workgroups) rounded to 256 B
    # + one fp32 p*p partial per (module, sequence, 64-token tile)
    # + one int64 per module (its place in the fragment table), rounded to 256 B
    head = -(-(-(-(48 * 112 + 1025 * 4) // 8) * 8 + 48 * 8) // 256) * 256
    assert lib.bgx_collect_workspace_bytes(48, 2, 2048, 16) == head + 48 * 2 * 32 * 256 * 4
    assert lib.bgx_collect_workspace_bytes(0, 2, 64, 16) == 0
    # with the modules known: + 1 KB per k-step of I + O for the fragment table (bf16: 32 features per k-step)
    descs = (_lib.ModuleDesc * 2)()
    for d, (I, O) in zip(descs, [(4096, 14336), (4096, 1024)]):
        d.I, d.O = I, O
    base = lib.bgx_collect_workspace_bytes(2, 2, 2048, 16)
    # the table (32 bytes per column of a and g) and, behind it, the list of items: one per 64 tokens and module
    # and, at p = 8 or 16, 128 bytes per module and token for the two-step per-token rows
    up = lambda x: -(-x // 256) * 256
    tokens = 2 * 2 * 2048 * 128
    assert (lib.bgx_collect_workspace_bytes_for(descs, 2, 2, 2048, 16, 2)
            == up(up(up(base) + (4096 + 14336 + 4096 + 1024) * 32) + 2 * 2 * (2048 // 64) * 4) + tokens)
    descs[1].O = 1000   # a width the streamed kernel cannot take: no table
    assert lib.bgx_collect_workspace_bytes_for(descs, 2, 2, 2048, 16, 2) == up(base) + tokens
    base32 = lib.bgx_collect_workspace_bytes(2, 2, 2048, 32)
    assert lib.bgx_collect_workspace_bytes_for(descs, 2, 2, 2048, 32, 2) == up(base32)   # p = 32: neither
    descs[1].O = 1024   # p = 32, 64: the table holds two, four blocks of 16 projection columns; the tokens' projections
    for p, blocks in ((32, 2), (48, 4), (50, 4), (64, 4)):   # are 128 bytes per block (p a multiple of 8 only)
        basep = lib.bgx_collect_workspace_bytes(2, 2, 2048, p)
        assert (lib.bgx_collect_workspace_bytes_for(descs, 2, 2, 2048, p, 2)
                == up(up(up(basep) + (4096 + 14336 + 4096 + 1024) * 32 * blocks) + 2 * 2 * (2048 // 64) * 4)
                + (tokens * blocks if p % 8 == 0 else 0))
    small = lib.bgx_scan_workspace_bytes(8, 10, 1024)
    assert small >= 8 * 10 * 8 + 8 * 1024 * 8
    assert lib.bgx_scan_workspace_bytes(1024, 100, 0) >= 1024 * 65536 * 8
    # the few-queries kernel's table: 1 KB per block of 16 queries and k-step (32 elements at 16 bits, 16 at fp32)
    base = lib.bgx_scan_workspace_bytes(20, 100, 0)
    padded = -(-base // 256) * 256
    assert lib.bgx_scan_workspace_bytes_for(20, 100, 0, 12288, 1) == padded + 2 * (12288 // 32) * 1024
    assert lib.bgx_scan_workspace_bytes_for(20, 100, 0, 12288, 0) == padded + 2 * (12288 // 16) * 1024
    base33 = -(-lib.bgx_scan_workspace_bytes(33, 100, 0) // 256) * 256
    assert lib.bgx_scan_workspace_bytes_for(33, 100, 0, 12288, 1) == base33 + 3 * (12288 // 32) * 1024   # three blocks
    base96 = -(-lib.bgx_scan_workspace_bytes(96, 100, 0) // 256) * 256
    assert lib.bgx_scan_workspace_bytes_for(96, 100, 0, 12288, 1) == base96 + 6 * (12288 // 32) * 1024   # six: the most
    assert lib.bgx_scan_workspace_bytes_for(97, 100, 0, 12288, 1) == -(-lib.bgx_scan_workspace_bytes(97, 100, 0) // 256) * 256
    assert lib.bgx_scan_workspace_bytes_for(20, 100, 0, 12288 + 32, 1) == padded   # not two k-steps: no table
    # per-sequence rows through the weight-shaped gradient: p * p fp32 values per sequence and 64 x 64 tile, and
    # per group of 16 tiles
    tiles = (3072 // 64) * (768 // 64)
    assert lib.bgx_collect_seq_weight_workspace_bytes(4, 768, 3072, 16) == 4 * (tiles + tiles // 16) * 256 * 4
    assert lib.bgx_collect_seq_weight_workspace_bytes(1, 70, 61, 7) == up(1 * (2 * 1 + 1) * 49 * 4)
    assert lib.bgx_collect_seq_weight_workspace_bytes(0, 64, 64, 16) == 0


def test_argument_errors_before_any_launch():
    from bergson_amd import _lib

    lib = _lib.load()
    descs = (_lib.ModuleDesc * 1)()
    rc = lib.bgx_collect_seq(descs, 1, 1, 8, 16, 2, None, None, None, 256, 2, 0.0, 0.0, None, 0, None)
    assert rc == -1 and b"null" in lib.bgx_last_error()
    rc = lib.bgx_collect_seq(descs, 1, 1, 8, 65, 2, None, None, C.c_void_p(256), 256, 2, 0.0, 0.0, C.c_void_p(256), 0, None)
    assert rc == -3 and b"p=65" in lib.bgx_last_error()
    rc = lib.bgx_collect_seq(descs, 1, 1, 8, 16, 7, None, None, C.c_void_p(256), 256, 2, 0.0, 0.0, C.c_void_p(256), 0, None)
    assert rc == -2
    rc = lib.bgx_collect_seq(descs, 1, 1, 8, 16, 2, None, None, C.c_void_p(256), 256, 2, 0.0, 0.0, C.c_void_p(256), 16, None)
    assert rc == -4 and b"workspace" in lib.bgx_last_error()
    rc = lib.bgx_collect_tok(descs, 1, 1, 8, 16, 2, None, None, C.c_void_p(256), 256, 2, 0.0, 0.0, C.c_void_p(256), 1 << 20, None)
    assert rc == -1 and b"lengths" in lib.bgx_last_error()
    rc = lib.bgx_scan(None, 10, 8, 8, 1, None, 2, 1.0, 1, 1, 0, None, None, None, None, None, None, None, 0, 0, None)
    assert rc == -1
    rc = lib.bgx_scan(C.c_void_p(256), 10, 8, 8, 1, C.c_void_p(256), 2, 1.0, 1, 11, 0, C.c_void_p(256), C.c_void_p(256),
                      None, None, None, None, C.c_void_p(256), 1 << 30, 0, None)
    assert rc == -3 and b"k=11" in lib.bgx_last_error()
    P = C.c_void_p(256)
    seq_weight = lambda p, dtype, ws, ws_bytes: lib.bgx_collect_seq_weight(
        P, P, 64 * 8, 64, 64 * 8, 64, 2, 8, 64, 64, p, dtype, None, None, P, P, P, 64, None, None, None, None, P, 1024,
        0, 2, 0.0, 0.0, ws, ws_bytes, None)
    assert seq_weight(33, 2, P, 1 << 20) == -3 and b"p=33" in lib.bgx_last_error()
    assert seq_weight(16, 0, P, 1 << 20) == -2 and b"16-bit" in lib.bgx_last_error()
    assert seq_weight(16, 2, P, 16) == -4 and b"workspace" in lib.bgx_last_error()
    assert seq_weight(16, 2, None, 0) == -4
    rc = lib.bgx_unit_normalize_rows(None, 1, 1, 1, 0, None)
    assert rc == -1
    with pytest.raises(_lib.BergsonAmdError, match="code -1"):
        _lib.check(rc, "bgx_unit_normalize_rows")
