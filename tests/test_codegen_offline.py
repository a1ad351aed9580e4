"""Generated kernel variants built for gfx950 with hipRTC on a machine without a GPU."""
import pytest

from charmnumeric_amd import _lib as L
from tests import helpers as H


@pytest.mark.parametrize("make,nd", [(H.ast_jacobi2d, 2), (H.ast_jacobi3d, 3), (H.ast_poisson2d, 2),
                                     (H.ast_poisson3d, 3)])
@pytest.mark.parametrize("variant", ["tiles", "direct", "slide"])
def test_stencil_variants_build(make, nd, variant):
    k = H.compile_group(make(64), L.F64, nd)
    two_arrays = make in (H.ast_poisson2d, H.ast_poisson3d)
    if variant == "slide" and two_arrays:
        # the LDS sliding window is for one array only
        assert L.lib.cnh_kernel_build(k, variant.encode()) != 0
        return
    L.check(L.lib.cnh_kernel_build(k, variant.encode()))
    assert L.lib.cnh_kernel_variants_loaded(k, variant.encode()) == 1
    src = H.kernel_source(k, variant)
    if variant == "direct":
        assert ("#define DR_NOTH 1" in src) == two_arrays


@pytest.mark.parametrize("dt", [L.F32, L.I32, L.I64])
def test_register_window_kernel_builds_for_other_element_types(dt):
    k = H.compile_group(H.ast_jacobi2d(64, dtype=dt, coef=2.0), dt, 2)
    L.check(L.lib.cnh_kernel_build(k, b"direct"))
    k3 = H.compile_group(H.ast_jacobi3d(32, dtype=dt, coef=2.0), dt, 3)
    L.check(L.lib.cnh_kernel_build(k3, b"direct"))


def test_register_window_kernel_for_a_sweep_from_one_array_into_another():
    """out[1:-1,1:-1] = coef*(shifted reads of u): the window array is u, the launch writes the
    assigned elements of out only."""
    from charmnumeric_amd.astbuild import AstBuilder
    n = 64
    b = AstBuilder(L.F64, 2)
    u, out = b.leaf(0), b.leaf(1)
    mid = ((1, 1), (n - 1, n - 1), (1, 1))
    t1 = b.binary(L.OP_ADD, 100, u, u, ((0, 1), (n - 2, n - 1), (1, 1)), ((2, 1), (n, n - 1), (1, 1)))
    t2 = b.binary(L.OP_ADD, 101, t1, u, None, ((1, 0), (n - 1, n - 2), (1, 1)))
    t3 = b.binary(L.OP_ADD, 102, t2, u, None, ((1, 2), (n - 1, n), (1, 1)))
    t4 = b.binary(L.OP_MUL, 103, b.scalar(0.25), t3)
    b.set_region(104, out, t4, mid)
    k = H.compile_group(b.finish(), L.F64, 2)
    L.check(L.lib.cnh_kernel_build(k, b"direct"))
    src = H.kernel_source(k, "direct")
    assert "#define DR_MASKED 1" in src and "#define DR_NOTH 0" in src
    k2 = H.compile_group(H.ast_jacobi2d(64), L.F64, 2)
    L.check(L.lib.cnh_kernel_build(k2, b"direct"))
    assert "#define DR_MASKED 0" in H.kernel_source(k2, "direct")
