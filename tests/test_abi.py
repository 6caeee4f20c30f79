"""The C ABI as a contract: the shared library loads without a GPU, exports every function that
include/triton_amd.h declares, the ctypes mirror has the same argument counts, struct field order and struct
sizes as the header (checked with gcc), and invalid descriptors come back as status codes with a message.
CPU only; no kernel is launched."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

from triton_amd import _native as nt

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "triton_amd.h")


def _strip_comments(text):
    return re.sub(r"/\*.*?\*/", "", text, flags=re.S)


def _declared_functions():
    text = _strip_comments(open(HEADER).read())
    out = {}
    for m in re.finditer(r"^(?:const\s+char\s*\*|int32_t|int64_t)\s+(tk_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.M | re.S):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args in ("", "void") else args.count(",") + 1
    return out


def _declared_struct_fields(name):
    text = _strip_comments(open(HEADER).read())
    body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (name, name), text, flags=re.S).group(1)
    fields = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        first, *rest = decl.split(",")
        fields.append(re.search(r"(\w+)\s*$", first).group(1))
        fields += [re.search(r"(\w+)\s*$", r).group(1) for r in rest]
    return fields


def test_header_declares_what_the_binding_lists():
    declared = _declared_functions()
    assert len(declared) >= 11
    assert set(declared) == set(nt.SIGNATURES), "include/triton_amd.h and _native.SIGNATURES disagree"
    for name, n_args in declared.items():
        assert len(nt.SIGNATURES[name][1]) == n_args, name


def test_library_exports_every_declared_symbol():
    lib = nt.lib()
    for name in _declared_functions():
        assert hasattr(lib, name), f"{name} not exported"
    out = subprocess.run(["nm", "-D", "--defined-only", nt.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line}
    assert set(_declared_functions()) <= exported
    assert lib.tk_version() >= 100


def test_struct_field_order_matches_header():
    assert _declared_struct_fields("tk_route_desc") == [f[0] for f in nt.RouteDesc._fields_]
    assert _declared_struct_fields("tk_gemm_desc") == [f[0] for f in nt.GemmDesc._fields_]
    assert _declared_struct_fields("tk_ragged_k_desc") == [f[0] for f in nt.RaggedKDesc._fields_]
    assert _declared_struct_fields("tk_decode_layer_desc") == [f[0] for f in nt.DecodeLayerDesc._fields_]


def test_header_is_plain_c_and_struct_sizes_match(tmp_path):
    src = tmp_path / "probe.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "triton_amd.h"\n'
                   'int main(void){printf("%zu %zu %zu %zu %zu %zu %zu\\n", sizeof(tk_route_desc), sizeof(tk_gemm_desc),'
                   ' offsetof(tk_gemm_desc, y), offsetof(tk_route_desc, workspace), sizeof(tk_ragged_k_desc),'
                   ' sizeof(tk_decode_layer_desc), offsetof(tk_decode_layer_desc, workspace));return 0;}\n')
    exe = tmp_path / "probe"
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)],
                   check=True)
    sizes = [int(v) for v in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()]
    assert sizes == [ctypes.sizeof(nt.RouteDesc), ctypes.sizeof(nt.GemmDesc), nt.GemmDesc.y.offset, nt.RouteDesc.workspace.offset,
                     ctypes.sizeof(nt.RaggedKDesc), ctypes.sizeof(nt.DecodeLayerDesc), nt.DecodeLayerDesc.workspace.offset]


def test_enum_values_match_header():
    text = _strip_comments(open(HEADER).read())

    def enum(name):
        body = re.search(r"enum %s \{(.*?)\}" % name, text, flags=re.S).group(1)
        return {m.group(1): int(m.group(2)) for m in re.finditer(r"(TK_\w+)\s*=\s*(\d+)", body)}

    dt = enum("tk_dtype")
    for k in ("TK_F32", "TK_BF16", "TK_F16", "TK_E4M3", "TK_E5M2", "TK_E2M1", "TK_U8", "TK_I16", "TK_I32"):
        assert dt[k] == getattr(nt, k)
    st = enum("tk_status")
    assert (st["TK_OK"], st["TK_ERR_INVALID"], st["TK_ERR_UNSUPPORTED"], st["TK_ERR_LAUNCH"]) == (0, 1, 2, 3)
    act = enum("tk_activation")
    assert (act["TK_ACT_NONE"], act["TK_ACT_SWIGLU"]) == (nt.TK_ACT_NONE, nt.TK_ACT_SWIGLU)


def test_invalid_descriptors_return_status_and_message():
    lib = nt.lib()
    d = nt.GemmDesc()  # all NULL / zero: an empty problem is fine
    assert lib.tk_moe_gemm(ctypes.byref(d), None) == nt.TK_OK
    d.M, d.N, d.K, d.grid_m = 16, 16, 32, 1  # sizes without operands
    assert lib.tk_moe_gemm(ctypes.byref(d), None) == nt.TK_ERR_INVALID
    assert "null operand" in nt.last_error()
    assert nt.last_error()
    with pytest.raises(ValueError):
        nt.check(lib.tk_moe_gemm(ctypes.byref(d), None))
    r = nt.RouteDesc()
    r.n_experts, r.k, r.n_tokens = 4096, 2, 1
    status = lib.tk_route(ctypes.byref(r), None)
    assert status in (nt.TK_ERR_INVALID, nt.TK_ERR_UNSUPPORTED) and nt.last_error()
    assert lib.tk_mx_downcast(None, nt.TK_BF16, 1, 33, 1, 0, 33, 1, 1, None, None, nt.TK_E2M1, 0, None) != nt.TK_OK
    assert lib.tk_route_workspace_bytes(4096, 128) > 0


def test_gather_without_x_rows_is_refused_by_the_prefill_tiled_kernels():
    """The prefill kernels for tiled MXFP4 weights address x with 32-bit offsets; with a gather the extent of x cannot
    be derived from M, so a descriptor that leaves x_rows at 0 is refused before any launch (fake, aligned pointers)."""
    lib = nt.lib()
    d = nt.GemmDesc()
    d.x, d.w, d.y, d.w_mx_scale, d.gather_indx = 0x1000, 0x2000, 0x3000, 0x4000, 0x5000
    d.x_dtype, d.w_dtype, d.y_dtype, d.w_layout = nt.TK_BF16, nt.TK_E2M1, nt.TK_BF16, nt.TK_W_TILED
    d.M, d.N, d.K, d.grid_m, d.block_m, d.n_slices = 256, 256, 256, 2, 128, 1
    d.x_stride_m, d.y_stride_m = 256, 256
    d.w_stride_e, d.ws_stride_e = 8 * 2 * 2048, 8 * 2 * 128
    d.x_rows = 0
    assert lib.tk_moe_gemm(ctypes.byref(d), None) == nt.TK_ERR_INVALID
    assert "x_rows is required" in nt.last_error()


def test_status_to_exception_mapping():
    with pytest.raises(ValueError):
        nt.check(nt.TK_ERR_INVALID, "bad")
    with pytest.raises(NotImplementedError):
        nt.check(nt.TK_ERR_UNSUPPORTED, "nope")
    with pytest.raises(RuntimeError):
        nt.check(nt.TK_ERR_LAUNCH, "launch")
    nt.check(nt.TK_OK)


def test_missing_library_is_a_hard_error():
    code = ("import triton_amd._native as nt, sys\n"
            "nt.LIB_PATH = '/nonexistent/libtriton_amd.so'\n"
            "try:\n    nt.lib()\nexcept nt.NativeLibraryMissing as e:\n    print('MISSING'); sys.exit(0)\nsys.exit(1)\n")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=ROOT)
    assert out.returncode == 0 and "MISSING" in out.stdout, out.stderr
