"""CPU-only checks of the C ABI: exported symbols, struct layout, code generation + offline build."""
import ctypes as C
import re
import os

import numpy as np
import pytest

from charmnumeric_amd import _lib as L
from charmnumeric_amd.astbuild import AstBuilder
from tests import helpers as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_declared_symbol_is_exported():
    header = open(os.path.join(ROOT, "include", "cnhip.h")).read()
    declared = set(re.findall(r"\b(cnh_[a-z0-9_]+)\s*\(", header))
    declared -= {"cnh_kernel"}
    executor = open(os.path.join(ROOT, "include", "cnexec.h")).read()
    executor = re.sub(r"/\*.*?\*/", "", executor, flags=re.S)       # comments mention cnx_ names too
    declared |= set(re.findall(r"\b(cnx_[a-z0-9_]+)\s*\(", executor))
    fixtures = open(os.path.join(ROOT, "include", "cnbench.h")).read()          # benchmark fixtures
    fixtures = re.sub(r"/\*.*?\*/", "", fixtures, flags=re.S)
    declared |= set(re.findall(r"\b(cn[hx]_[a-z0-9_]+)\s*\(", fixtures))
    assert declared, "no declarations found"
    for name in sorted(declared):
        assert hasattr(L.lib, name), f"{name} declared in a header but not exported"
    assert declared == set(L.EXPORTS), declared ^ set(L.EXPORTS)


def test_struct_layouts_match_header():
    assert C.sizeof(L.Region) == 44
    assert C.sizeof(L.AstNode) == 192
    assert L.AstNode.scalar.offset == 48
    assert L.AstNode.operand_regions.offset == 56
    assert L.AstNode.region.offset == 144
    assert C.sizeof(L.Memref) == 72
    assert C.sizeof(L.Tiled) == 88 and L.Tiled.pitch.offset == 64
    assert C.sizeof(L.GemmJob) == 72 and L.GemmJob.C.offset == 56
    assert C.sizeof(L.GemvPanel) == 32 and L.GemvPanel.xoff.offset == 24
    assert C.sizeof(L.Decomp) == 40 and L.Decomp.tile.offset == 32


def test_scalar_conversion():
    buf = np.zeros(1, np.int64)
    L.check(L.lib.cnh_scalar_to_dtype(L.I32, -3.9, buf.ctypes.data))
    assert buf.view(np.int32)[0] == -3  # truncation toward zero, like (int32_t)double
    L.check(L.lib.cnh_scalar_to_dtype(L.F32, 0.1, buf.ctypes.data))
    assert buf.view(np.float32)[0] == np.float32(0.1)


@pytest.mark.parametrize("variant", ["flat", "nd", "tiles", "slide", "direct", "directr"])
def test_generated_source_builds_for_gfx950(variant):
    """hipRTC cross-compiles the generated source without a GPU."""
    ast = H.ast_jacobi2d(64) if variant in ("tiles", "slide", "direct", "directr") else H.ast_c1(L.F64)
    nd = 2 if variant in ("tiles", "slide", "direct", "directr") else 1
    k = H.compile_group(ast, L.F64, nd)
    src = H.kernel_source(k, variant)
    assert "group_eval" in src and "fma" not in src
    L.check(L.lib.cnh_kernel_build(k, variant.encode()))
    L.check(L.lib.cnh_kernel_release(k))


def test_signature_follows_upstream_argument_order():
    # leaf uses x, y, x, y -> 4 input memrefs, 0 scalars, 1 output
    k = H.compile_group(H.ast_c1(L.F64), L.F64, 1)
    a, b, c = C.c_int(), C.c_int(), C.c_int()
    L.check(L.lib.cnh_kernel_signature(k, C.byref(a), C.byref(b), C.byref(c)))
    assert (a.value, b.value, c.value) == (4, 0, 1)
    src = H.kernel_source(k, "flat")
    assert "#define NL 2" in src  # identical (array, region) uses are loaded once
    # jacobi: 4 shifted uses of u, SET_REGION target is not an input
    k2 = H.compile_group(H.ast_jacobi2d(64), L.F64, 2)
    L.check(L.lib.cnh_kernel_signature(k2, C.byref(a), C.byref(b), C.byref(c)))
    assert (a.value, b.value, c.value) == (4, 0, 1)
    # broadcast leaves are deduplicated by name
    bld = AstBuilder(L.F64, 1)
    x, al = bld.leaf(0), bld.broadcast(9)
    t = bld.binary(L.OP_MUL, 100, al, x)
    bld.binary(L.OP_ADD, 2, t, bld.broadcast(9), is_temp=False)
    k3 = H.compile_group(bld.finish(), L.F64, 1)
    L.check(L.lib.cnh_kernel_signature(k3, C.byref(a), C.byref(b), C.byref(c)))
    assert (a.value, b.value, c.value) == (1, 1, 1)


def test_compile_cache_by_key():
    k1 = H.compile_group(H.ast_c1(L.F64), L.F64, 1, key=0xABCDEF)
    k2 = H.compile_group(H.ast_c1(L.F64), L.F64, 1, key=0xABCDEF)
    assert k1.value == k2.value
    L.check(L.lib.cnh_kernel_release(k1))
    L.check(L.lib.cnh_kernel_release(k2))


def test_two_groups_under_one_key_stay_apart():
    """The cache key is a hash of the AST: a kernel found by key is reused only when it was compiled
    from that very AST; another group under the same key gets a kernel of its own."""
    k1 = H.compile_group(H.ast_c1(L.F64), L.F64, 1, key=0x5150)
    other = AstBuilder(L.F64, 1)
    other.binary(L.OP_MUL, 10, other.leaf(0), other.scalar(3.0), is_temp=False)
    ast2 = other.finish()
    k2 = H.compile_group(ast2, L.F64, 1, key=0x5150)
    assert k1.value != k2.value
    same, c1 = H.ast_c1(L.F64), H.ast_c1(L.F64)
    assert L.lib.cnh_kernel_matches(k1, C.byref(same), L.F64, 1) == 1
    assert L.lib.cnh_kernel_matches(k2, C.byref(c1), L.F64, 1) == 0
    assert L.lib.cnh_kernel_matches(k2, C.byref(ast2), L.F64, 1) == 1
    assert L.lib.cnh_kernel_matches(k2, C.byref(ast2), L.F32, 1) == 0       # another element type
    assert "0x1.8p+1" in H.kernel_source(k2, "prelude")          # times three, not the first group
    L.check(L.lib.cnh_kernel_release(k1))
    L.check(L.lib.cnh_kernel_release(k2))


def test_literals_that_vary_share_one_code_object():
    """A literal that is no small multiple of a quarter is a launch parameter: two groups that
    differ only in it generate the same text and share the code object (built here for gfx950
    without a GPU); small literals stay in the source."""
    def scaled(c):
        b = AstBuilder(L.F64, 1)
        t = b.binary(L.OP_MUL, 100, b.leaf(0), b.scalar(c))
        b.binary(L.OP_ADD, 10, t, b.scalar(0.5), is_temp=False)
        return b.finish()

    ks = [H.compile_group(scaled(c), L.F64, 1) for c in (0.1234, 0.777, 1e-3)]
    assert len({k.value for k in ks}) == 3                   # three kernels (they carry their values) ...
    before = L.lib.cnh_code_objects()
    for k in ks:
        L.check(L.lib.cnh_kernel_build(k, b"flat"))
    assert L.lib.cnh_code_objects() == before + 1            # ... one code object
    src = [H.kernel_source(k, "flat") for k in ks]
    assert src[0] == src[1] == src[2] and "s[NS + 0]" in src[0] and "0x1p-1" in src[0]
    assert "0x1.f9" not in src[0]                            # 0.1234 is not in the text
    k4 = H.compile_group(scaled(2.5), L.F64, 1)              # a small multiple of a quarter stays
    assert "0x1.4p+1" in H.kernel_source(k4, "flat")
    for k in ks + [k4]:
        L.check(L.lib.cnh_kernel_release(k))


def test_uncompilable_groups_report_an_error():
    b = AstBuilder(L.I64, 1)
    b.unary(L.OP_EXP, 2, b.leaf(0), is_temp=False)
    k = C.c_void_p()
    assert L.lib.cnh_compile_group(C.byref(b.finish()), L.I64, 1, 0, C.byref(k)) < 0
    assert b"integer" in L.lib.cnh_last_error()
    b = AstBuilder(L.F64, 1)
    n = b._new(5, L.OP_MATMUL)
    b._roots.append(n)
    assert L.lib.cnh_compile_group(C.byref(b.finish()), L.F64, 1, 0, C.byref(k)) < 0


def test_slide_variant_builds_for_3d_and_is_refused_for_other_groups():
    k = H.compile_group(H.ast_jacobi3d(32), L.F64, 3)
    L.check(L.lib.cnh_kernel_build(k, b"slide"))
    L.check(L.lib.cnh_kernel_build(k, b"direct"))
    src = H.kernel_source(k, "slide")
    assert "SL_SHIFT[NLA][3] = {{-1, 0, 0}, {1, 0, 0}, {0, -1, 0}, {0, 1, 0}, {0, 0, -1}, {0, 0, 1}}" in src
    k1 = H.compile_group(H.ast_c1(L.F64), L.F64, 1)
    assert L.lib.cnh_kernel_build(k1, b"slide") < 0


def test_code_objects_kept_on_disk_are_loaded_by_the_next_process(tmp_path):
    """CHARMNUMERIC_KERNEL_CACHE: the first process compiles and writes one file per code object,
    the second loads it (no compile); a damaged file is ignored."""
    import subprocess
    import sys

    prog = (
        "import ctypes as C\n"
        "from charmnumeric_amd import _lib as L\n"
        "from tests import helpers as H\n"
        "k = H.compile_group(H.ast_jacobi2d(64), L.F64, 2)\n"
        "L.check(L.lib.cnh_kernel_build(k, b'tiles'))\n"
        "print(L.lib.cnh_code_objects(), L.lib.cnh_code_objects_from_disk())\n"
    )
    env = dict(os.environ, CHARMNUMERIC_KERNEL_CACHE=str(tmp_path), PYTHONPATH=os.getcwd())
    run = lambda: subprocess.run([sys.executable, "-c", prog], env=env, capture_output=True, text=True, check=True).stdout.split()
    assert run() == ["1", "0"]
    files = list(tmp_path.iterdir())
    assert len(files) == 1 and files[0].name.startswith("cnh-gfx950-") and files[0].stat().st_size > 1000
    assert run() == ["1", "1"]
    data = bytearray(files[0].read_bytes())
    data[40] ^= 0xFF                                   # inside the stored text: no longer this group's
    files[0].write_bytes(bytes(data))
    assert run() == ["1", "0"]
    assert run() == ["1", "1"]                         # rewritten by the process that had to compile
