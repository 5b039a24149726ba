"""CPU-only checks of the C ABI: the library loads, exports every function the
header declares, the ctypes mirrors have the C struct sizes, and argument
validation fails cleanly (no GPU work is issued by any of these calls)."""

import ctypes
import re
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "ssm_amd.h"


def _lib():
    from ssm_amd import _lib as L
    return L


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    names = re.findall(r"\b(ssm_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_header_declares_functions():
    names = declared_functions()
    assert "ssm_scan_fwd" in names and "ssm_scan_bwd" in names and "ssm_ssd_chunk_scan" in names
    assert len(names) >= 20


def test_library_exports_every_declared_function():
    lib = _lib().load()
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, f"declared in ssm_amd.h but not exported: {missing}"


def test_binding_covers_every_declared_function():
    L = _lib()
    bound = set(L.ENTRY_POINTS) | set(L.PLAIN_SYMBOLS)
    missing = [n for n in declared_functions() if n not in bound]
    assert not missing, f"declared in ssm_amd.h but not bound in _lib.py: {missing}"


def test_ctypes_struct_sizes_match_the_header(tmp_path):
    L = _lib()
    structs = {cls.__name__: cls for cls in L.ENTRY_POINTS.values()}
    cname = {"ScanFwdArgs": "ssm_scan_fwd_args", "ScanBwdArgs": "ssm_scan_bwd_args",
             "StateStepArgs": "ssm_state_step_args", "DscanFwdArgs": "ssm_dscan_fwd_args",
             "Conv1dFwdArgs": "ssm_conv1d_fwd_args", "Conv1dBwdArgs": "ssm_conv1d_bwd_args",
             "NormFwdArgs": "ssm_norm_fwd_args", "NormBwdArgs": "ssm_norm_bwd_args",
             "SsdCumsumArgs": "ssm_ssd_cumsum_args", "SsdBmmArgs": "ssm_ssd_bmm_args",
             "SsdChunkStateArgs": "ssm_ssd_chunk_state_args",
             "SsdStatePassingArgs": "ssm_ssd_state_passing_args",
             "SsdChunkScanArgs": "ssm_ssd_chunk_scan_args", "DecodeStepArgs": "ssm_decode_step_args",
             "SsdCombinedArgs": "ssm_ssd_combined_args",
             "StateStepBwdArgs": "ssm_state_step_bwd_args",
             "DscanBwdArgs": "ssm_dscan_bwd_args",
             "SsdChunkStateVarlenArgs": "ssm_ssd_chunk_state_varlen_args",
             "Mamba2DecodeArgs": "ssm_mamba2_decode_args", "Conv1dUpdateArgs": "ssm_conv1d_update_args",
             "SsdBwdGateArgs": "ssm_ssd_bwd_gate_args", "SsdBwdDxArgs": "ssm_ssd_bwd_dx_args",
             "SsdBwdDbArgs": "ssm_ssd_bwd_db_args", "SsdBwdDcbArgs": "ssm_ssd_bwd_dcb_args",
             "SsdBwdStatesArgs": "ssm_ssd_bwd_states_args", "SsdScaleRowsArgs": "ssm_ssd_scale_rows_args",
             "SsdBwdDtArgs": "ssm_ssd_bwd_dt_args", "SsdBwdPrepArgs": "ssm_ssd_bwd_prep_args",
             "F64ScanArgs": "ssm_f64_scan_args", "F64StepArgs": "ssm_f64_step_args",
             "F64DscanArgs": "ssm_f64_dscan_args", "F64ConvArgs": "ssm_f64_conv_args",
             "F64NormArgs": "ssm_f64_norm_args", "RowsToBclArgs": "ssm_rows_to_bcl_args"}
    assert set(structs) <= set(cname), set(structs) - set(cname)
    src = tmp_path / "sizes.c"
    lines = ['#include <stdio.h>', f'#include "{HEADER}"', "int main(void) {"]
    for py, c in cname.items():
        if py in structs:
            lines.append(f'  printf("{py} %zu\\n", sizeof({c}));')
    lines += ["  return 0;", "}"]
    src.write_text("\n".join(lines))
    exe = tmp_path / "sizes"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    for line in out.splitlines():
        name, size = line.split()
        assert ctypes.sizeof(structs[name]) == int(size), name


def test_header_is_valid_c_and_cpp(tmp_path):
    for flags, ext in ((["-std=c99"], "c"), (["-std=c++17", "-x", "c++"], "cc")):
        src = tmp_path / f"inc.{ext}"
        src.write_text(f'#include "{HEADER}"\nint main(void) {{ return 0; }}\n')
        subprocess.run(["gcc", *flags, "-Wall", "-Werror", "-fsyntax-only", str(src)], check=True)


def test_abi_version_and_status_strings():
    lib = _lib().load()
    assert lib.ssm_amd_abi_version() == _lib().ABI_VERSION
    assert lib.ssm_amd_status_string(0) == b"ok"
    assert b"NULL" in lib.ssm_amd_status_string(-1)
    assert lib.ssm_amd_status_string(-99) == b"unknown status"
    assert lib.ssm_scan_chunk_len() == 512


@pytest.mark.parametrize("name", sorted(n for n in ["ssm_scan_fwd", "ssm_scan_bwd", "ssm_state_step",
                                                    "ssm_dscan_fwd", "ssm_conv1d_fwd", "ssm_conv1d_bwd",
                                                    "ssm_norm_fwd", "ssm_norm_bwd", "ssm_ssd_chunk_cumsum",
                                                    "ssm_ssd_bmm_chunk", "ssm_ssd_chunk_state",
                                                    "ssm_ssd_state_passing", "ssm_ssd_chunk_scan"]))
def test_null_arguments_are_rejected_without_touching_a_device(name):
    L = _lib()
    lib = L.load()
    fn = getattr(lib, name)
    assert fn(None, None) == -1                       # NULL args struct
    zeroed = L.ENTRY_POINTS[name]()
    rc = fn(ctypes.byref(zeroed), None)               # all pointers NULL, all sizes 0
    assert rc in (-1, -2), rc
    assert lib.ssm_amd_last_error() != b""


def test_shape_and_dtype_errors_come_back_as_status_codes():
    L = _lib()
    lib = L.load()
    buf = (ctypes.c_float * 64)()
    p = ctypes.addressof(buf)
    a = L.ScanFwdArgs(u=p, delta=p, A=p, Bproj=p, Cproj=p, out=p, batch=1, dim=2, seqlen=4, nstate=0)
    assert lib.ssm_scan_fwd(ctypes.byref(a), None) == -2            # bad shape
    a.nstate = 1000
    assert lib.ssm_scan_fwd(ctypes.byref(a), None) == -6            # too large
    a.nstate = 2
    a.io_dtype = 7
    assert lib.ssm_scan_fwd(ctypes.byref(a), None) == -3            # bad dtype
    a.io_dtype = 0
    a.b_kind = 9
    assert lib.ssm_scan_fwd(ctypes.byref(a), None) == -4            # bad kind
    a.b_kind, a.c_kind, a.b_groups, a.c_groups = 2, 2, 3, 1
    assert lib.ssm_scan_fwd(ctypes.byref(a), None) == -2            # groups do not divide dim
    a.b_groups = 1
    a.u = p + 2
    assert lib.ssm_scan_fwd(ctypes.byref(a), None) == -5            # misaligned pointer
    assert lib.ssm_conv1d_bwd_workspace_bytes(8, 1536, 4) == 8 * 32 * 1536 * 5 * 4    # per (batch row, time segment)
    assert lib.ssm_conv1d_bwd_workspace_bytes(0, 1, 1) == 0
    assert lib.ssm_scan_bwd_workspace_bytes(8, 1536, 2048, 16, 2, 2, 1, 1) > 0
    assert lib.ssm_scan_bwd_workspace_bytes(8, 1536, 2048, 16, 2, 2, 7, 1) == 0


def test_views_of_rows_are_checked_before_anything_is_launched():
    """The convolution's rows-in layout and the transposing copy say what they do not take, as status codes."""
    L = _lib()
    lib = L.load()
    buf = (ctypes.c_float * 4096)()
    p = ctypes.addressof(buf)
    p += (-p) % 16
    conv = dict(x=p, weight=p, y=p, batch=2, channels=8, seqlen=16, width=4, io_dtype=0, layout=L.LAYOUT_ROWS_TO_BCL,
                activation=1, x_batch_stride=16 * 8, x_row_stride=8)
    a = L.Conv1dFwdArgs(**conv)
    a.channels = 6
    assert lib.ssm_conv1d_fwd(ctypes.byref(a), None) == -2          # channels not a multiple of 4
    assert b"(B,C,L) copy" in lib.ssm_amd_last_error()
    a = L.Conv1dFwdArgs(**dict(conv, width=7))
    assert lib.ssm_conv1d_fwd(ctypes.byref(a), None) == -2          # wider than the vector kernels take
    a = L.Conv1dFwdArgs(**dict(conv, x_row_stride=6))
    assert lib.ssm_conv1d_fwd(ctypes.byref(a), None) == -2          # rows overlap
    a = L.Conv1dFwdArgs(**dict(conv, x_batch_stride=8))
    assert lib.ssm_conv1d_fwd(ctypes.byref(a), None) == -2          # batch entries overlap
    a = L.Conv1dFwdArgs(**dict(conv, x=p + 4))
    assert lib.ssm_conv1d_fwd(ctypes.byref(a), None) == -5          # x off a boundary of four elements
    a = L.Conv1dFwdArgs(**dict(conv, layout=L.LAYOUT_BCL))
    assert lib.ssm_conv1d_fwd(ctypes.byref(a), None) == -4          # strides with another layout
    assert lib.ssm_conv1d_fwd(ctypes.byref(L.Conv1dFwdArgs(**dict(conv, layout=3))), None) == -4
    t = dict(src=p, dst=p + 8192, src_batch_stride=16 * 8, src_row_stride=8, batch=2, channels=8, seqlen=16, element_size=4)
    assert lib.ssm_rows_to_bcl(ctypes.byref(L.RowsToBclArgs(**dict(t, element_size=8))), None) == -3
    assert lib.ssm_rows_to_bcl(ctypes.byref(L.RowsToBclArgs(**dict(t, channels=6))), None) == -2
    assert lib.ssm_rows_to_bcl(ctypes.byref(L.RowsToBclArgs(**dict(t, src_row_stride=4))), None) == -2
    assert lib.ssm_rows_to_bcl(ctypes.byref(L.RowsToBclArgs(**dict(t, src=p + 4))), None) == -5
    assert lib.ssm_rows_to_bcl(ctypes.byref(L.RowsToBclArgs(**dict(t, dst=None))), None) == -1


def test_shipped_library_has_no_test_hooks_and_the_hooks_build_does():
    """Kernel selectors and the record of kernels taken exist in the -DSSM_TEST_HOOKS build only
    (include/ssm_amd_testing.h): the shipped library rejects a non-zero ``reserved`` field and does not export
    ``ssm_ssd_mfma_launches``; the hooks build exports everything the header declares plus that."""
    L = _lib()
    lib, hooks = L.load(), L.load_test_hooks()
    assert not hasattr(lib, "ssm_ssd_mfma_launches")
    assert hooks.ssm_ssd_mfma_launches() == 0
    missing = [n for n in declared_functions() if not hasattr(hooks, n)]
    assert not missing, missing
    buf = (ctypes.c_float * 64)()
    p = ctypes.addressof(buf)
    a = L.ScanFwdArgs(u=p, delta=p, A=p, Bproj=p, Cproj=p, out=p, batch=1, dim=2, seqlen=4, nstate=2, reserved=808)
    assert lib.ssm_scan_fwd(ctypes.byref(a), None) == -4
    assert b"reserved" in lib.ssm_amd_last_error()
    for name in ("ssm_scan_bwd", "ssm_dscan_bwd", "ssm_ssd_bmm_chunk", "ssm_ssd_chunk_state", "ssm_ssd_chunk_scan"):
        args = L.ENTRY_POINTS[name]()
        for field, ctype in args._fields_:
            if ctype is ctypes.c_void_p:
                setattr(args, field, p)            # past the NULL checks; the reserved check comes before any use
        args.reserved = 1
        assert getattr(lib, name)(ctypes.byref(args), None) == -4, name
        assert b"reserved" in lib.ssm_amd_last_error(), name
    with L.test_hooks_build() as inside:
        assert inside is hooks and L.load() is hooks
    assert L.load() is lib


def test_missing_library_fails_loudly(tmp_path):
    code = ("import os, sys; os.environ['SSM_AMD_LIB'] = r'%s'; sys.path.insert(0, r'%s');\n"
            "from ssm_amd import _lib\n"
            "try:\n    _lib.load()\nexcept _lib.BackendUnavailable as e:\n    print('UNAVAILABLE'); sys.exit(0)\n"
            "sys.exit(1)\n") % (tmp_path / "nope.so", ROOT)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True)
    assert out.returncode == 0 and "UNAVAILABLE" in out.stdout, out.stderr
