"""The C-ABI library: loads, exports every symbol the header declares, rejects bad arguments.

No compute call is made here (no GPU): every call below returns from the argument checks,
before the library touches the HIP runtime.
"""
import ctypes
import os
import re

import pytest

from pytorch_block_sparse_amd import native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "pbs_hip.h")

OK, ERR_NULL, ERR_SHAPE, ERR_DTYPE, ERR_ALIGN, ERR_WS, ERR_LARGE = 0, -1, -2, -3, -4, -5, -6


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(native.LIB_PATH):
        pytest.skip("libpbs_hip.so is not built")
    return native.load()


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pbs_\w+)\s*\(", text)))


def test_header_symbols_are_exported(lib):
    declared = _declared_symbols()
    assert len(declared) >= 8
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in pbs_hip.h but not exported"
    assert set(declared) == set(native.EXPORTED_SYMBOLS)


def test_version_and_error_strings(lib):
    text = open(HEADER).read()
    assert lib.pbs_abi_version() == int(re.search(r"#define PBS_ABI_VERSION (\d+)", text).group(1))
    assert native.error_string(0) == "ok"
    for code in (ERR_NULL, ERR_SHAPE, ERR_DTYPE, ERR_ALIGN, ERR_WS, ERR_LARGE):
        assert native.error_string(code).startswith("pbs:")
    for name, code in re.findall(r"#define (PBS_ERR_\w+) \((-\d+)\)", text):
        assert native.error_string(int(code)) != "pbs: unknown error code", name


def test_matmul_argument_checks(lib):
    p = ctypes.c_void_p(0x1000)  # never dereferenced: the checks fail first
    null = ctypes.c_void_p(0)
    f = lib.pbs_blocksparse_matmul
    assert f(p, p, p, null, p, 4, 64, 64, 1, 1, 7, null) == ERR_DTYPE
    assert f(p, p, p, null, p, 4, 65, 64, 1, 1, 0, null) == ERR_SHAPE
    assert f(p, p, p, null, p, 4, 64, 33, 1, 1, 0, null) == ERR_SHAPE
    assert f(p, p, p, null, p, -1, 64, 64, 1, 1, 0, null) == ERR_SHAPE
    assert f(p, p, p, null, p, 4, 64, 64, 5, 1, 0, null) == ERR_LARGE      # more blocks than positions
    assert f(p, p, p, null, p, 0, 64, 64, 1, 1, 0, null) == OK             # no tokens: nothing to do
    assert f(null, p, p, null, p, 4, 64, 64, 1, 1, 0, null) == ERR_NULL
    assert f(p, p, null, null, p, 4, 64, 64, 1, 1, 0, null) == ERR_NULL    # the plan is required
    assert f(ctypes.c_void_p(0x1004), p, p, null, p, 4, 64, 64, 1, 1, 1, null) == ERR_ALIGN


def test_matmul_workspace_entry_point(lib):
    p = ctypes.c_void_p(0x1000)
    null = ctypes.c_void_p(0)
    f = lib.pbs_blocksparse_matmul_ws
    assert f(p, p, p, null, p, 4, 64, 64, 1, 1, 7, null, 0, null) == ERR_DTYPE
    assert f(p, p, p, null, p, 4, 65, 64, 1, 1, 0, null, 0, null) == ERR_SHAPE
    assert f(p, p, p, null, p, 0, 64, 64, 1, 1, 1, null, 0, null) == OK
    assert f(p, p, null, null, p, 4, 64, 64, 1, 1, 1, p, 1 << 20, null) == ERR_NULL
    ws = lib.pbs_blocksparse_matmul_workspace_bytes
    # the transposed copy of the blocks, 2 KB each: bf16, forward direction, large and dense enough
    assert ws(16384, 4096, 4096, 8192, 1, 1) == 8192 * 2048
    assert ws(16384, 4096, 4096, 8192, 0, 1) == 0      # the input gradient reads the data as stored
    assert ws(16384, 4096, 4096, 8192, 1, 0) == 0      # fp32
    assert ws(16384, 4096, 4096, 400, 1, 1) == 400 * 2048   # 3 blocks per column of a result of 4096 columns: still that kernel
    assert ws(16384, 4096, 4096, 128, 1, 1) == 0       # 1 block per column
    assert ws(16384, 1024, 4096, 512, 1, 1) == 0       # a result of 1024 columns at 16 blocks per column
    assert ws(16384, 2048, 512, 640, 1, 1) == 0        # a short contraction below 16 blocks per column
    assert ws(16384, 2048, 512, 1024, 1, 1) == 1024 * 2048   # ... and at 16
    assert ws(256, 4096, 4096, 8192, 1, 1) == 0        # too few tiles
    assert ws(16384, 4096, 8192, 16384, 1, 1) == 0     # contraction too long for the kernel's lists
    assert ws(16384, 4096, 4096, 0, 1, 1) == 0 and ws(0, 4096, 4096, 8192, 1, 1) == 0


def test_plan_argument_checks(lib):
    p = ctypes.c_void_p(0x1000)
    null = ctypes.c_void_p(0)
    nbytes = lib.pbs_blocksparse_matmul_plan_bytes(4096, 4096)
    # narrow plans: groups of 8, 7, 6 and 5 block columns (128 columns -> 16, 19, 22, 26 groups), 64-byte
    # records per k-block, each with the table of the block column in every one of a group's 8 places
    narrow = sum(g * (128 + 2) * 16 * 4 for g in (16, 19, 22, 26))
    slots = sum((g * 8 * 4 + 63) // 64 * 64 for g in (16, 19, 22, 26))   # each table padded to 64 bytes
    wide = 8 * (64 + 2) * 64 * 4 + 256 * 4     # 8 groups of 16, 256-byte records per k-pair, progress table
    # one column per wave: the column table of 8 groups of 16, per group a header of 64 ints, 64 k-pairs and 16 lists
    # of up to 128 two-word items, then the table 0, 1, 2, ... of 16384 ints
    column = 8 * 16 * 4 + (8 * (64 + 64 + 16 * 2 * 128) + 16384) * 4
    assert nbytes == narrow + wide + slots + column
    # contraction sizes that are not a multiple of 64 have no k-pair plans
    assert lib.pbs_blocksparse_matmul_plan_bytes(64, 96) == 4 * (1 * (3 + 2) * 16 * 4 + 64)
    # nor does the column kernel serve contractions whose lists would not fit its LDS area
    assert (lib.pbs_blocksparse_matmul_plan_bytes(512, 8192) - lib.pbs_blocksparse_matmul_plan_bytes(512, 8192 - 32)
            < lib.pbs_blocksparse_matmul_plan_bytes(512, 4096) - lib.pbs_blocksparse_matmul_plan_bytes(512, 4096 - 32))
    assert lib.pbs_blocksparse_matmul_plan_bytes(100, 64) == 0
    f = lib.pbs_blocksparse_matmul_plan
    assert f(p, p, 64, 100, 1, p, 1 << 20, null) == ERR_SHAPE
    assert f(null, p, 64, 64, 1, p, 1 << 20, null) == ERR_NULL
    assert f(p, p, 64, 64, 1, p, 16, null) == ERR_WS


def test_back_argument_checks(lib):
    p = ctypes.c_void_p(0x1000)
    null = ctypes.c_void_p(0)
    f = lib.pbs_blocksparse_matmul_back
    assert f(p, p, p, p, p, 8, 64, 64, 1, 9, null, 0, null) == ERR_DTYPE
    assert f(p, p, p, p, p, 8, 64, 60, 1, 0, null, 0, null) == ERR_SHAPE
    assert f(p, p, p, p, p, 8, 64, 64, 0, 0, null, 0, null) == OK           # no blocks: nothing to do
    assert f(p, p, null, p, p, 8, 64, 64, 1, 0, null, 0, null) == ERR_NULL
    assert f(ctypes.c_void_p(0x1008), p, p, p, p, 8, 64, 64, 1, 0, null, 0, null) == ERR_ALIGN
    ws = lib.pbs_blocksparse_matmul_back_workspace_bytes
    assert ws(0, 64, 64, 1, 0) == 0 and ws(16384, 4096, 4096, 4096, 5) == 0
    need = ws(16384, 4096, 4096, 4096, 1)
    assert need > 0 and need % (4096 * 1024 * 4) == 0
    # the token range is split but no workspace is given
    assert f(p, p, p, p, p, 16384, 4096, 4096, 4096, 1, null, 0, null) == ERR_WS


def test_build_indices_argument_checks(lib):
    p = ctypes.c_void_p(0x1000)
    null = ctypes.c_void_p(0)
    f = lib.pbs_build_indices
    assert f(p, null, 0, 4, 0, p, p, p, p, p, p, null) == ERR_SHAPE
    assert f(p, null, 4, 4, 17, p, p, p, p, p, p, null) == ERR_SHAPE
    assert f(null, null, 4, 4, 2, p, p, p, p, p, p, null) == ERR_NULL
    assert f(p, null, 4, 4, 2, null, p, p, p, p, p, null) == ERR_NULL


def test_reference_side_binding_matches_the_header(lib):
    """include/pbs_hip_ctypes.py is the binding a maintainer of the reference would use: its prototypes must be
    those the package's own binding declares, and its error path must raise on a rejected call."""
    import importlib.util

    spec = importlib.util.spec_from_file_location("pbs_hip_ctypes", os.path.join(ROOT, "include", "pbs_hip_ctypes.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    for name, (restype, argtypes) in mod.PROTOTYPES.items():
        assert name in native._PROTOTYPES, name
        r2, a2 = native._PROTOTYPES[name]
        assert restype is r2 and list(argtypes) == list(a2), name
    b = mod.PbsHip(native.LIB_PATH)
    assert b.lib.pbs_abi_version() == lib.pbs_abi_version()
    with pytest.raises(RuntimeError, match="pbs:"):
        b._check(b.lib.pbs_blocksparse_matmul(None, None, None, None, None, 4, 64, 64, 1, 1, 0, None), "matmul")
