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
