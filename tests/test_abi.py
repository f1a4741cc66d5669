"""The C ABI library loads and exports every symbol include/megray_vrank.h declares; host-only
entry points agree with the oracle.  No compute calls, no GPU."""
import ctypes
import os
import re

import pytest

import oracle as orc

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "megray_vrank.h")


@pytest.fixture(scope="module")
def lib():
    from megray_amd import _lib
    return _lib.load()


def declared_symbols():
    text = open(HEADER).read()
    return re.findall(r"MRV_API\s+[\w\s\*]+?\b(mrv_\w+)\s*\(", text)


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ("mrv_reduce", "mrv_all_reduce", "mrv_reduce_scatter", "mrv_all_gather", "mrv_all_to_all",
                 "mrv_scatter", "mrv_gather", "mrv_broadcast", "mrv_describe", "mrv_fold_order",
                 "mrv_chunk_partition", "mrv_dtype_size", "mrv_last_error", "mrv_abi_version"):
        assert must in names
    assert len(names) == len(set(names))


def test_library_exports_every_declared_symbol(lib):
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in megray_vrank.h but not exported"


def test_cxx_api_symbols_are_exported(lib):
    # MegRay::get_dtype_size(MegRay::DType), the mangled C++ symbol a C++ caller links against
    assert hasattr(lib, "_ZN6MegRay14get_dtype_sizeENS_5DTypeE")


def test_abi_version_and_dtype_sizes(lib):
    assert lib.mrv_abi_version() >= 1
    for dtype in range(10):
        assert lib.mrv_dtype_size(dtype) == orc.dtype_size(dtype)
    for bad in (-1, 10, 99):
        assert lib.mrv_dtype_size(bad) == 0
        assert lib.mrv_last_error() == b"unknown dtype"  # src/core/common.cpp:35-36


def test_chunk_partition_matches_oracle():
    import megray_amd as mr
    for nchunks in range(1, 33):
        for length in list(range(0, 70)) + [2 ** 28, 2 ** 28 + 5, 2 ** 33 + 7]:
            assert mr.chunk_partition(length, nchunks) == tuple(orc.chunk_partition(length, nchunks))


def test_fold_order_matches_oracle():
    import megray_amd as mr
    for nranks in range(1, 33):
        for coll in (orc.COLL_ALL_REDUCE, orc.COLL_REDUCE_SCATTER):
            for order in (orc.ORDER_UCX, orc.ORDER_SHM, orc.ORDER_RANK0):
                nchunks = orc.fold_order(coll, order, nranks, 0)[2]
                for chunk in range(nchunks):
                    ranks, new_wins, nch, owner = mr.fold_order(coll, order, nranks, chunk)
                    assert (ranks, new_wins, nch) == orc.fold_order(coll, order, nranks, chunk)
                    assert 0 <= owner < nranks
                with pytest.raises(mr.MegRayError):
                    mr.fold_order(coll, order, nranks, nchunks)
    with pytest.raises(mr.MegRayError):
        mr.fold_order(0, 0, 33, 0)
    with pytest.raises(mr.MegRayError):
        mr.fold_order(0, 5, 4, 0)


def test_missing_library_fails_loudly(monkeypatch):
    from megray_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmegray_vrank.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()


def test_product_never_imports_the_oracle():
    """The shipped package must not reference the CPU oracle in any way."""
    pkg = os.path.join(ROOT, "megray_amd")
    for dirpath, _, files in os.walk(pkg):
        for name in files:
            if name.endswith((".py", ".cpp", ".h", ".hip")):
                text = open(os.path.join(dirpath, name)).read()
                assert "import oracle" not in text and "megray_oracle" not in text, name


def test_no_kernel_spills_or_hogs_registers():
    """The build records every kernel's resources.  A kernel that needs scratch memory (register spills,
    run-time indexed arrays) or more than 128 vector registers halves the wavefronts a CU can hold and
    has cost a third of the throughput before; the kernels are written so that none does."""
    import json
    import os

    from megray_amd import build
    if not os.path.exists(build.RESOURCES_PATH):
        pytest.skip("the library was not built in this tree (kernel_resources.json is a build product)")
    with open(build.RESOURCES_PATH) as f:
        kernels = json.load(f)
    assert len(kernels) > 100
    for name, res in kernels.items():
        assert res["scratch"] == 0, f"{name} uses {res['scratch']} bytes of scratch per lane"
        assert res["vgprs"] <= 128, f"{name} uses {res['vgprs']} vector registers"
        assert res["lds"] <= 40 * 1024, f"{name} uses {res['lds']} bytes of LDS"


def test_device_code_has_no_packed_fp32_instructions(tmp_path):
    """The fp32 and fp64 folds must be chains of single IEEE operations: the build switches the packed
    fp32 instructions off, and the generated gfx950 code of the fp32 kernels shows none."""
    import shutil
    import subprocess

    from megray_amd import build
    if not shutil.which(build.HIPCC) and not os.path.exists(build.HIPCC):
        pytest.skip("no hipcc here")
    out = tmp_path / "fold_f32.s"
    cmd = ([build.HIPCC] + build.COMMON_FLAGS + ["-x", "hip"] + build.DEVICE_FLAGS +
           ["--cuda-device-only", "-S", os.path.join(build.CSRC, "vrank_fold_f32.hip"), "-o", str(out)])
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr[-2000:]
    text = out.read_text()
    assert text.count("v_add_f32") > 100, "the fp32 kernels are not in this file"
    for bad in ("v_pk_add_f32", "v_pk_mul_f32", "v_pk_fma_f32"):
        assert bad not in text, f"{bad} in the generated code"


def test_python_wrappers_reject_lists_of_different_lengths():
    """The library indexes both per-rank arrays up to nranks: the Python mirror refuses a call whose two lists
    differ in length before anything reaches the C side, and pads the root-only forms it builds itself."""
    import megray_amd as mr
    with pytest.raises(mr.MegRayError, match="one of each per rank"):
        mr.all_reduce([0x1000, 0x2000, 0x3000], [0x4000, 0x5000], 4, mr.DType.FLOAT32, mr.ReduceOp.SUM)
    with pytest.raises(mr.MegRayError, match="one of each per rank"):
        mr.all_to_all([0x1000], [0x4000, 0x5000], 4, mr.DType.UINT8)
    # describe() with a shorter list: the missing ranks' entries are null, not read past the end
    runs, _, _ = mr.describe(mr.Collective.GATHER, [0x100000, 0x200000, 0x300000], [None, 0x900000], 16,
                             mr.DType.UINT8, root=1)
    assert len(runs) == 3 and all(r["out_first"] == 1 for r in runs)


def test_the_header_is_plain_c_and_the_python_binding_lays_the_run_record_out_the_same_way(tmp_path):
    """megray_vrank.h is what a foreign binding reads: it must compile as C99 on its own, and the ctypes mirror of
    mrv_plan_run must agree with the compiler field by field."""
    import subprocess

    from megray_amd import _lib

    fields = [name for name, _ in _lib.PlanRun._fields_]
    prints = "\n".join(f'    printf("{f} %zu\\n", offsetof(mrv_plan_run, {f}));' for f in fields)
    src = tmp_path / "layout.c"
    src.write_text(f'#include <stddef.h>\n#include <stdio.h>\n#include "megray_vrank.h"\nint main(void) {{\n'
                   f'    printf("sizeof %zu\\n", sizeof(mrv_plan_run));\n{prints}\n    return 0;\n}}\n')
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", f"-I{os.path.join(ROOT, 'include')}",
                    str(src), "-o", str(exe)], check=True, capture_output=True, text=True)
    lines = dict(line.split() for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    assert int(lines["sizeof"]) == ctypes.sizeof(_lib.PlanRun)
    for f in fields:
        assert int(lines[f]) == getattr(_lib.PlanRun, f).offset, f
