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


def _red_black_roots(b, phi, g, n, starts):
    """phi[r0:-1:2, c0:-1:2] = 0.25 * (up + down + left + right - g[same]) for every (r0, c0)."""
    for j, (r0, c0) in enumerate(starts):
        def reg(dr, dc):
            return ((r0 + dr, c0 + dc), (n - 1 + dr, n - 1 + dc), (2, 2))
        base = 100 + 10 * j
        t1 = b.binary(L.OP_ADD, base, phi, phi, reg(-1, 0), reg(1, 0))
        t2 = b.binary(L.OP_ADD, base + 1, t1, phi, None, reg(0, -1))
        t3 = b.binary(L.OP_ADD, base + 2, t2, phi, None, reg(0, 1))
        t4 = b.binary(L.OP_SUB, base + 3, t3, g, None, reg(0, 0))
        t5 = b.binary(L.OP_MUL, base + 4, b.scalar(0.25), t4)
        b.set_region(base + 5, phi, t5, reg(0, 0))


def test_which_groups_qualify_for_the_lattice_sweep():
    """cnh_kernel_lattice: 0 for a unit-step sweep; 2 (in place) for one step-2 lattice whose
    shifted reads miss it and for the two lattices of one colour; 1 (second buffer only) when a
    shifted read of one root meets a point another assigns (red and black in one group)."""
    from charmnumeric_amd.astbuild import AstBuilder
    n = 64
    assert L.lib.cnh_kernel_lattice(H.compile_group(H.ast_jacobi2d(n), L.F64, 2)) == 0
    for starts, want in (([(1, 1)], 2), ([(1, 1), (2, 2)], 2), ([(1, 1), (1, 2)], 1)):
        b = AstBuilder(L.F64, 2)
        _red_black_roots(b, b.leaf(0), b.leaf(1), n, starts)
        k = H.compile_group(b.finish(), L.F64, 2)
        assert L.lib.cnh_kernel_lattice(k) == want, (starts, want)
        L.check(L.lib.cnh_kernel_build(k, b"direct"))
        src = H.kernel_source(k, "direct")
        assert f"#define DR_NROOTS {len(starts)}" in src and "#define DR_TAIL_OK 0" in src


def test_scatter_kernels_exist_for_two_to_four_assigned_lattices():
    """The gather variant of a group with several SET_REGION roots carries the scatter entry points
    (one lane evaluates every root at a lattice index); a single root does not, five are refused."""
    from charmnumeric_amd.astbuild import AstBuilder

    def group(roots):
        b = AstBuilder(L.F64, 2)
        fine, coarse = b.leaf(0), b.leaf(1)
        for j in range(roots):
            r0, c0 = 1 + j // 2, 1 + j % 2 + 2 * (j // 4)
            t = b.binary(L.OP_MUL, 100 + 2 * j, b.scalar(0.5), coarse, None, ((0, 0), (8, 8), (1, 1)))
            b.set_region(101 + 2 * j, fine, t, ((r0, c0), (r0 + 16, c0 + 16), (2, 2)))
        return H.compile_group(b.finish(), L.F64, 2)

    for roots in (1, 2, 4):
        k = group(roots)
        L.check(L.lib.cnh_kernel_build(k, b"tiles"))
        src = H.kernel_source(k, "tiles")
        assert f"#define NO {roots}" in src and "grp_scatter" in src and "grp_block" in src
    assert L.lib.cnh_kernel_build(group(5), b"tiles") != 0


def test_the_boundary_column_rule_of_the_whole_array_kernel():
    """DR_TAIL_OK: an in-place style sweep whose every output row holds its right-hand neighbour
    pair may copy the columns beyond its last wavefront; a sweep into another array never copies."""
    k = H.compile_group(H.ast_jacobi2d(64), L.F64, 2)
    L.check(L.lib.cnh_kernel_build(k, b"direct"))
    assert "#define DR_TAIL_OK 1" in H.kernel_source(k, "direct")
    k3 = H.compile_group(H.ast_jacobi3d(32), L.F64, 3)
    L.check(L.lib.cnh_kernel_build(k3, b"direct"))
    assert "#define DR_TAIL_OK 1" in H.kernel_source(k3, "direct")


@pytest.mark.parametrize("blocks", [1, 2, 4])
def test_product_kernel_with_a_groups_statements_builds(blocks):
    """The matrix-core product kernel with the gate statements of an LSTM step appended (one launch
    per step): its text is the ahead-of-time kernel's, compiled at run time with the group."""
    import bench
    k = H.compile_group(bench.lstm_fused_ast(L, False, True), L.F64, 2)
    variant = b"product%d" % blocks
    L.check(L.lib.cnh_kernel_build(k, variant))
    src = H.kernel_source(k, variant.decode())
    assert "#define CN_EPI_Q %d" % blocks in src and "grp_product" in src and "cn_tanh_f64" in src
    assert L.lib.cnh_kernel_build(k, b"product3") != 0
    # the other two forms of the product kernel (grids of more than one tile per CU)
    for form in (b"e", b"f"):
        L.check(L.lib.cnh_kernel_build(k, variant + form))
    assert L.lib.cnh_kernel_build(k, variant + b"x") != 0
    # other element types keep their two launches
    k32 = H.compile_group(H.ast_jacobi2d(64, dtype=L.F32, coef=2.0), L.F32, 2)
    assert L.lib.cnh_kernel_build(k32, b"product4") != 0
