"""Host-side logic: irreps algebra, Clebsch-Gordan tensors, coefficient tables and their packing."""

import itertools
import math

import numpy as np
import pytest

from e3j_amd import Convolution, O3Irrep, O3Space, ScalarMixing, TensorProduct
from e3j_amd.clebsch_gordan import (change_basis_real_to_complex, clebsch_gordan,
                                    su2_clebsch_gordan)
from e3j_amd.coef import Coef, Coef4D, resolve_val_dtype
from e3j_amd.sparse import narrow_index_dtype, sparse_coo
from e3j_amd.tensor_product import block_sort_permutation
from tests import helpers as H


# --- spaces ------------------------------------------------------------------
def test_irrep_parse_and_products():
    ir = O3Irrep("1o")
    assert (ir.l, ir.p, ir.dim, str(ir)) == (1, -1, 3, "1o")
    assert O3Irrep(2) == O3Irrep("2e") == O3Irrep(2, 1)
    assert [str(i) for _, i in O3Irrep("1o") * O3Irrep("1o")] == ["0e", "1e", "2e"]
    assert [str(i) for _, i in O3Irrep("3e") * O3Irrep("1o")] == ["2o", "3o", "4o"]
    assert (8 * O3Irrep("1o")).dim == 24
    with pytest.raises(ValueError):
        O3Irrep("1x")


def test_space_parse_dim_slices():
    space = O3Space("16x0e + 8x1o+8x2e")
    assert space.dim == 16 + 24 + 40 and space.num_irreps == 32 and space.l_max == 2
    assert space == O3Space([(16, "0e"), (8, (1, -1)), (8, 2, 1)])
    assert [(s.start, s.stop) for s in space.slices()] == [(0, 16), (16, 40), (40, 80)]
    assert str(O3Space("0e+1o")) == "1x0e + 1x1o"


def test_sort_order_natural_parity_first():
    """Increasing degree; within a degree p = (-1)^l first (src/e3j/spaces/o3.py:110-116)."""
    space = O3Space("1e + 2e + 0o + 1o + 0e + 2o")
    assert str(space.sort()) == "1x0e + 1x0o + 1x1o + 1x1e + 1x2e + 1x2o"
    assert str(O3Space("1o + 0e + 1o + 0e").regroup()) == "2x0e + 2x1o"
    _, inv = O3Space("1o + 0e + 1o").sort(return_inverse=True)
    assert inv.tolist() == [1, 0, 2]  # stable


def test_otimes_selection_rules_and_filter():
    full = O3Space.otimes("0e+1o", "0e+1o", None)
    assert str(full) == "1x0e + 1x1o + 1x1o + 1x0e + 1x1e + 1x2e"
    kept = O3Space.otimes("0e+1o", "0e+1o", "0e+1o")
    assert str(kept) == "1x0e + 1x1o + 1x1o + 1x0e"
    assert str(O3Space.otimes("0e+1o", "0e+1o", "0e+1o", sort=True)) == "2x0e + 2x1o"
    with pytest.raises(ValueError, match="multiplicities 1"):
        O3Space.otimes("0e", "0e", "2x0e")


def test_block_sort_permutation():
    sigma, sigma_inv, target = block_sort_permutation(O3Space("1o + 0e + 1o + 0e"))
    assert sigma.tolist() == [3, 7, 0, 1, 2, 4, 5, 6]
    assert sigma_inv[sigma].tolist() == list(range(8))
    assert str(target) == "2x0e + 2x1o"


# --- Clebsch-Gordan tensors ----------------------------------------------------
def test_su2_coefficients_match_sympy():
    from sympy import S
    from sympy.physics.quantum.cg import CG
    for j1, j2 in itertools.product(range(3), repeat=2):
        for j3 in range(abs(j1 - j2), j1 + j2 + 1):
            c = su2_clebsch_gordan(j1, j2, j3)
            for m1, m2 in itertools.product(range(-j1, j1 + 1), range(-j2, j2 + 1)):
                m3 = m1 + m2
                if abs(m3) > j3:
                    continue
                want = float(CG(S(j1), S(m1), S(j2), S(m2), S(j3), S(m3)).doit())
                assert abs(c[j1 + m1, j2 + m2, j3 + m3] - want) < 1e-12


def test_change_of_basis_is_unitary():
    for l in range(5):
        q = change_basis_real_to_complex(l)
        np.testing.assert_allclose(q.conj().T @ q, np.eye(2 * l + 1), atol=1e-14)


def test_cg_unit_norm_and_reference_value():
    """|C(0; 1, 1)| = delta_ij / sqrt(3): the one value the reference's files hold
    (tests/test_power_expansion.py:157-158)."""
    np.testing.assert_allclose(np.abs(clebsch_gordan(0, 1, 1)[0]), np.eye(3) / math.sqrt(3), atol=1e-14)
    for l1, l2, l3 in itertools.product(range(4), repeat=3):
        if abs(l2 - l3) <= l1 <= l2 + l3:
            assert abs(np.linalg.norm(clebsch_gordan(l1, l2, l3)) - 1.0) < 1e-13


def test_cg_special_cases():
    # l (x) 0 -> l is the identity / sqrt(2l+1)
    for l in range(4):
        np.testing.assert_allclose(clebsch_gordan(l, l, 0)[:, :, 0], np.eye(2 * l + 1) / math.sqrt(2 * l + 1),
                                   atol=1e-14)
    # 1 (x) 1 -> 1 is the cross product (Levi-Civita / sqrt 6), in any cyclic relabelling of the axes
    eps = np.zeros((3, 3, 3))
    for a, b, c in ((0, 1, 2), (1, 2, 0), (2, 0, 1)):
        eps[a, b, c], eps[a, c, b] = 1.0, -1.0
    np.testing.assert_allclose(clebsch_gordan(1, 1, 1), eps / math.sqrt(6), atol=1e-14)


def test_cg_orthogonality_between_paths():
    """sum_{m1 m2} C^{l}_{m m1 m2} C^{l'}_{m' m1 m2} = delta_{ll'} delta_{mm'} / (2l+1)."""
    l1, l2 = 2, 3
    for la, lb in itertools.product(range(abs(l1 - l2), l1 + l2 + 1), repeat=2):
        ca, cb = clebsch_gordan(la, l1, l2), clebsch_gordan(lb, l1, l2)
        gram = np.einsum("ajk,bjk->ab", ca, cb)
        want = np.eye(2 * la + 1) / (2 * la + 1) if la == lb else np.zeros_like(gram)
        np.testing.assert_allclose(gram, want, atol=1e-13)


def _wigner_d(l, rot):
    """D^l(R) in the harmonics basis of this package, from Y^l(R r) = D^l(R) Y^l(r)."""
    import torch
    from e3j_amd.harmonics import Harmonics
    pts = torch.randn(4 * (2 * l + 1), 3, dtype=torch.float64, generator=torch.Generator().manual_seed(l))
    pts = pts / pts.norm(dim=-1, keepdim=True)
    sh = Harmonics(l)(pts)[:, l * l:]
    sh_rot = Harmonics(l)(pts @ torch.as_tensor(rot).T)[:, l * l:]
    return np.linalg.lstsq(sh.numpy(), sh_rot.numpy(), rcond=None)[0].T


def test_cg_is_equivariant():
    """C (D^l1 x) (D^l2 y) = D^l0 C x y for a random rotation (tests/test_tensor_product.py:151-156)."""
    from scipy.spatial.transform import Rotation
    rot = Rotation.from_rotvec([0.3, -1.1, 0.7]).as_matrix()
    rng = np.random.default_rng(0)
    for l0, l1, l2 in ((1, 1, 1), (2, 1, 1), (1, 2, 3), (3, 3, 2), (0, 2, 2)):
        c = clebsch_gordan(l0, l1, l2)
        x, y = rng.normal(size=2 * l1 + 1), rng.normal(size=2 * l2 + 1)
        d0, d1, d2 = _wigner_d(l0, rot), _wigner_d(l1, rot), _wigner_d(l2, rot)
        lhs = np.einsum("ijk,j,k->i", c, d1 @ x, d2 @ y)
        rhs = d0 @ np.einsum("ijk,j,k->i", c, x, y)
        np.testing.assert_allclose(lhs, rhs, atol=1e-9)


# --- coefficient tables ----------------------------------------------------------
SIGNATURES = [
    # x irreps, y irreps, output filter, paths, Z, X, Y, nnz, distinct (z, x) pairs
    ("0e+1o", "0e+1o+2e", "0e+1o+2e", 7, 21, 4, 9, 37, 35),
    ("0e+1o+2e", "0e+1o+2e+3o", "0e+1o+2e", 13, 43, 9, 16, 125, 109),
    ("0e+1o+2e", "0e+1o+2e+3o", "0e+1o+2e+3o", 17, 71, 9, 16, 215, 187),
    ("0e+1o+2e+3o", "0e+1o+2e+3o", "0e+1o+2e+3o", 23, 99, 16, 16, 353, 311),
]


@pytest.mark.parametrize("xs, ys, out, S, Z, X, Y, nnz, pairs", SIGNATURES)
def test_table_counts(xs, ys, out, S, Z, X, Y, nnz, pairs):
    """Sizes from the irreps selection rules alone (independent count)."""
    tp = TensorProduct((xs, ys), out, normalization="SQRT_DIM_OUT")
    c = tp.coef
    assert (tp.target.dim, tp.source[0].dim, tp.source[1].dim) == (Z, X, Y)
    assert ScalarMixing(tp.target).num_irreps == S
    assert c.nnz == nnz and c.shape == (Z, X, Y) and c.indices.dtype == np.uint8
    assert len({(int(i), int(j)) for i, j, _ in c.indices}) == pairs
    # independent path count: allowed (lx, ly, lo) triples
    keep = {(ir.l, ir.p) for _, ir in O3Space(out)}
    count = sum(1 for (_, a), (_, b) in itertools.product(O3Space(xs), O3Space(ys))
                for l in range(abs(a.l - b.l), a.l + b.l + 1) if (l, a.p * b.p) in keep)
    assert count == S


def test_table_is_sorted_regrouped_and_matches_dense_blocks():
    tp = TensorProduct(("0e+1o", "0e+1o"), "0e+1o", normalization="SQRT_DIM_OUT")
    assert str(tp.target) == "2x0e + 2x1o"          # regrouped e3nn order
    dense = tp.coef.todense()
    # output rows: [0e from 0x0, 0e from 1x1, 1o from 0x1, 1o from 1x0]
    np.testing.assert_allclose(dense[0, 0, 0], 1.0, atol=1e-7)
    np.testing.assert_allclose(dense[1, 1:, 1:], np.sqrt(1) * clebsch_gordan(0, 1, 1)[0], atol=1e-7)
    np.testing.assert_allclose(dense[2:5, 0, 1:], np.sqrt(3) * clebsch_gordan(1, 0, 1)[:, 0, :], atol=1e-7)
    np.testing.assert_allclose(dense[5:8, 1:, 0], np.sqrt(3) * clebsch_gordan(1, 1, 0)[:, :, 0], atol=1e-7)
    # lexicographic, coalesced
    keys = np.ravel_multi_index(tuple(tp.indices.astype(np.int64).T), tp.shape)
    assert np.all(np.diff(keys) > 0)


def test_multiplicities_tile_the_table():
    """k0 = k1 * m2 + k2 (src/e3j/core/tensor_product.py:248-266)."""
    one = TensorProduct(("1o", "1o"), "0e").coef.todense()
    two = TensorProduct(("2x1o", "3x1o"), "0e").coef.todense()
    assert two.shape == (6, 6, 9)
    for k1, k2 in itertools.product(range(2), range(3)):
        np.testing.assert_array_equal(two[k1 * 3 + k2, 3 * k1:3 * k1 + 3, 3 * k2:3 * k2 + 3], one[0])


def test_sparse_coo_coalesce():
    c = sparse_coo([1.0, 2.0, -2.0, 3.0], [[1, 0], [0, 1], [0, 1], [1, 0]], (2, 2))
    assert c.indices.tolist() == [[1, 0]] and c.data.tolist() == [4.0]
    assert narrow_index_dtype((255, 3)) == np.uint8 and narrow_index_dtype((256,)) == np.int32
    with pytest.raises(ValueError, match="Out of bounds"):
        sparse_coo([1.0], [[2, 0]], (2, 2))


def test_sparse_coo_sums_duplicates_in_the_value_dtype():
    """Duplicates are added one after another in float32 and dropped when that sum is exactly zero
    (`src/e3j/utils/sparse.py:116-124`): 1e8 + 1 - 1e8 is 0 in float32 and 1 in float64."""
    vals = [1e8, 2.5, 1.0, -1e8, 0.1, 0.2, 0.3]
    idx = [[3, 1], [0, 2], [3, 1], [3, 1], [1, 1], [1, 1], [1, 1]]
    c = sparse_coo(vals, idx, (4, 3))
    assert c.data.dtype == np.float32
    assert c.indices.tolist() == [[0, 2], [1, 1]]          # (3, 1) cancels in float32
    want = np.float32(0.1) + np.float32(0.2)                 # left to right, rounded at every step
    want = np.float32(want + np.float32(0.3))
    assert c.data.tobytes() == np.array([2.5, want], np.float32).tobytes()
    # literal restatement of the rule on random duplicates: sort stably, add runs sequentially
    rng = np.random.default_rng(5)
    idx = rng.integers(0, 4, size=(200, 3))
    vals = rng.normal(size=200).astype(np.float32)
    c = sparse_coo(vals, idx, (4, 4, 4))
    sums = {}
    for v, row in zip(vals, map(tuple, idx.tolist())):
        sums[row] = np.float32(sums.get(row, np.float32(0)) + v)
    rows = sorted(r for r, v in sums.items() if v != 0)
    assert c.indices.tolist() == [list(r) for r in rows]
    assert c.data.tobytes() == np.array([sums[r] for r in rows], np.float32).tobytes()


def test_sparse_coo_shapes_beyond_int64_positions():
    """A shape whose number of elements does not fit int64 is coalesced by comparing coordinate
    rows (the reference switches to a lexicographic sort there, `src/e3j/utils/sparse.py:104-113`)."""
    big = 2 ** 31 - 1
    idx = [[5, 1, big - 1], [0, 7, 3], [5, 1, big - 1], [0, 7, 2]]
    c = sparse_coo([1.0, 2.0, 3.0, 4.0], idx, (big, big, big))
    assert c.indices.dtype == np.int32
    assert c.indices.tolist() == [[0, 7, 2], [0, 7, 3], [5, 1, big - 1]]
    assert c.data.tolist() == [4.0, 2.0, 4.0]


def test_mix_indices():
    assert ScalarMixing("2x0e + 1x1o + 1x2e").mix_indices.tolist() == [0, 1, 2, 2, 2, 3, 3, 3, 3, 3]


# --- Convolution module (host side) ------------------------------------------------
def test_convolution_coef_invariants():
    """tests/test_convolution.py:117-151."""
    module = Convolution(("0e+1o+2e", "0e+1o+2e+3o"), "0e+1o+2e", graph_ordering="RECEIVER")
    coef = module.coef
    assert isinstance(coef, Coef4D) and coef.rank == 4 and coef.idx.shape == (len(coef), 4)
    bounds = (module.target.dim, module.source[0].dim, module.source[1].dim, module.source[2].dim)
    assert np.dtype(coef.idx.dtype) == np.dtype(coef.idx_dtype) == narrow_index_dtype(bounds)
    assert (coef.idx.max(axis=0) < np.array(bounds)).all()
    np.testing.assert_array_equal(coef.idx[:, 3], module._mix.mix_indices[coef.idx[:, 0]])
    unpacked = Coef4D.unpack(coef.pack(), val_dtype=coef.val_dtype)
    assert np.dtype(unpacked.idx.dtype) == np.dtype(coef.idx_dtype)
    np.testing.assert_array_equal(unpacked.val, coef.val.astype(np.float32))
    assert str(module.source[2]) == "13x0e"


def test_avg_num_neighbors_scales_coefficients():
    """tests/test_convolution.py:169-184."""
    a = Convolution(("0e+1o", "0e+1o"), None, graph_ordering="RECEIVER")
    b = Convolution(("0e+1o", "0e+1o"), None, graph_ordering="RECEIVER", avg_num_neighbors=4.0)
    np.testing.assert_allclose(b.coef.val, a.coef.val / 4.0, rtol=1e-7)
    np.testing.assert_array_equal(b.coef.idx, a.coef.idx)
    assert b.y_parity.tolist() == [1.0, -1.0, -1.0, -1.0]


# --- packed wire format (tests/test_ops/test_coef.py:30-46,67-83) ----------------------
COEF_ITEMSIZE = [("float32", "int32", 16), ("float32", "uint8", 8), ("float64", "int32", 32),
                 ("float64", "uint8", 16), ("float16", "int32", 16), ("float16", "uint8", 8)]
COEF4D_ITEMSIZE = [("float32", "int32", 32), ("float32", "uint8", 8), ("float64", "int32", 32),
                   ("float64", "uint8", 16), ("float16", "int32", 32), ("float16", "uint8", 8)]


@pytest.mark.parametrize("cls, table", [(Coef, COEF_ITEMSIZE), (Coef4D, COEF4D_ITEMSIZE)])
def test_packed_sizes_and_offsets(cls, table):
    for val_dtype, idx_dtype, itemsize in table:
        dt = cls._numpy_dtype(val_dtype, idx_dtype)
        assert dt.itemsize == itemsize
        assert dt.fields["val"][1] == 0
        stride = np.dtype(idx_dtype).itemsize
        base = -(-np.dtype(val_dtype).itemsize // stride) * stride
        for n, name in enumerate(cls.index_names):
            assert dt.fields[name][1] == base + n * stride


@pytest.mark.parametrize("val_dtype, idx_dtype", [(v, i) for v, i, _ in COEF4D_ITEMSIZE])
def test_pack_unpack_round_trip(val_dtype, idx_dtype):
    val = np.array([1.0, -0.5, 3.14], dtype=val_dtype)
    idx = np.array([[0, 1, 2, 0], [3, 0, 1, 1], [7, 2, 5, 2]], dtype=idx_dtype)
    c = Coef4D(val, idx, val_dtype, idx_dtype)
    packed = c.pack()
    assert packed.dtype == np.dtype(idx_dtype)
    assert packed.shape == (3, c.dtype.itemsize // np.dtype(idx_dtype).itemsize)
    back = Coef4D.unpack(packed, val_dtype)
    np.testing.assert_array_equal(back.val, val)
    np.testing.assert_array_equal(back.idx, idx)
    assert len(Coef4D.unpack(packed[:0], val_dtype)) == 0


def test_transpose_is_stable_sort_by_new_first_column():
    c = Coef4D(np.array([1.0, 2.0, 3.0, 4.0]), np.array([[0, 2, 0, 0], [0, 1, 1, 0], [1, 2, 2, 1], [1, 0, 0, 1]]))
    t = c.transpose((1, 0, 2, 3))
    assert t.idx[:, 0].tolist() == [0, 1, 2, 2]
    assert t.val.tolist() == [4.0, 2.0, 1.0, 3.0]
    assert t.idx[2].tolist() == [2, 0, 0, 0] and t.idx[3].tolist() == [2, 1, 2, 1]


def test_resolve_val_dtype():
    assert resolve_val_dtype(np.float32) == "float32"
    with pytest.raises(TypeError, match="Cast the operands"):
        resolve_val_dtype(np.int32)


def test_energy_model_forces_are_the_energy_gradient():
    """The end-to-end model on the host with the dense form of the operator: central differences
    of the energy along a random direction equal -F.direction (pins the reference the GPU
    energy and forces are compared with)."""
    import torch
    from e3j_amd import workloads as W
    from tests import helpers as H
    w = W.config5(0.02)
    host = w.to("cpu", torch.float64)
    conv = H.dense_convolve(w.model)
    args = (host.node_features, host.sender, host.receiver, host.shift, conv)
    _, forces = w.model.energy_and_forces(host.positions, *args)
    direction = torch.from_numpy(np.random.default_rng(0).standard_normal(tuple(host.positions.shape)))
    h = 1e-5
    slope = (w.model.energy(host.positions + h * direction, *args)
             - w.model.energy(host.positions - h * direction, *args)) / (2 * h)
    torch.testing.assert_close(slope, -(forces * direction).sum(), rtol=1e-6, atol=1e-8)
    # translation invariance of a periodic cell: no net force
    assert float(forces.sum(0).abs().max()) < 1e-12


def test_run_time_signature_compiles_and_registers():
    """A table the library was not built for: the generator's output compiles against the
    installed kernel templates, loads next to the library and is found by the signature
    lookup (hipcc cross-compiles, so this runs without a GPU)."""
    import ctypes
    from e3j_amd import _lib, jit
    module = Convolution(("0e+1o", "0e+1o"), "0e+1o", graph_ordering="RECEIVER")
    c = module.coef
    dims = (4, 4, module.params.num_out, module.params.num_scalars)
    lib = _lib.load()
    packed = module._packed_coef("float32")
    scale, flip = ctypes.c_float(0), ctypes.c_uint32(0)

    def find(channels, layout):
        return lib.e3j_amd_find_signature(packed.ctypes.data, 1, _lib.F32, packed.shape[0], *dims, channels,
                                          layout, ctypes.byref(scale), ctypes.byref(flip))
    ids = jit.register(np.asarray(c.val, np.float32), np.asarray(c.idx, np.int64), dims, 64)
    assert len(ids) == 2 and ids == jit.register(np.asarray(c.val, np.float32), np.asarray(c.idx, np.int64), dims, 64)
    assert find(64, 1) == ids[0] and find(64, 0) == ids[1] and scale.value == 1.0
    assert b"run-time table" in lib.e3j_amd_signature_name(ids[0])
    assert find(128, 1) == -1                                     # another channel count: not built
    # 25 y components (harmonics up to l = 4): the dy sums are reduced sixteen at a time
    big = Convolution(("0e+1o", "0e+1o+2e+3o+4e"), "0e+1o", graph_ordering="RECEIVER")
    cb = big.coef
    assert len(jit.register(np.asarray(cb.val, np.float32), np.asarray(cb.idx, np.int64),
                            (4, 25, big.params.num_out, big.params.num_scalars), 64)) == 2
    # more than 255 output coordinates: outside the templates, served table-driven
    rng = np.random.default_rng(0)
    idx, val, mix = H.random_table(rng, 400, 4, 5, 300, 7)
    idx4 = np.concatenate([idx, mix[idx[:, 0]][:, None]], axis=1).astype(np.int64)
    assert jit.register(np.asarray(val, np.float32), idx4, (4, 5, 300, 7), 64) == []


def test_run_time_tensor_product_signature_compiles_and_registers():
    """The tensor-product generator's output for a table outside the built-in ones compiles,
    loads and is found by the lookup, in both layouts (no GPU needed)."""
    import ctypes
    from e3j_amd import TensorProduct, _lib, jit
    tp = TensorProduct(("0e+1o", "0e+1o"), None)
    val, idx = np.asarray(tp.values, np.float32), np.asarray(tp.indices, np.int64)
    Z, X, Y = tp.shape
    lib = _lib.load()
    packed = tp.packed_coef("float32")
    scale = ctypes.c_float(0)

    def find(channels, kind, layout):
        return lib.e3j_amd_tp_find_signature(packed.ctypes.data, packed.dtype.itemsize, _lib.F32, packed.shape[0],
                                             X, Y, Z, channels, kind, layout, ctypes.byref(scale))
    assert find(64, 0, 1) == -1
    ids = jit.register_tp(val, idx, tp.shape, 64)
    assert len(ids) == 3 and ids == jit.register_tp(val, idx, tp.shape, 64)
    assert [find(64, kind, 1) for kind in (0, 1, 2)] == ids and scale.value == 1.0
    assert b"run-time table" in lib.e3j_amd_tp_signature_name(ids[0])
    assert find(128, 0, 1) == -1 and find(64, 0, 0) == -1       # other channel count / layout: not built
    lead = jit.register_tp(val, idx, tp.shape, 0)               # leading layout: any multiple of 4 channels
    assert len(lead) == 3 and find(20, 0, 0) == lead[0] and find(128, 2, 0) == lead[2]
    big = TensorProduct(("0e+1o", "0e+1o+2e+3o+4e"), "0e+1o")   # 25 y components: sums reduced 16 at a time
    assert len(jit.register_tp(np.asarray(big.values, np.float32), np.asarray(big.indices, np.int64),
                               big.shape, 64)) == 3
    idx, val, _ = H.random_table(np.random.default_rng(0), 400, 4, 5, 300, 7)   # 300 outputs: outside the templates
    assert jit.register_tp(np.asarray(val, np.float32), idx.astype(np.int64), (300, 4, 5), 64) == []


def test_build_reads_the_assembly_for_dpp_operands_written_too_late():
    """The planned kernels use `v_fmac_f32_dpp` through inline assembly, which the compiler's hazard
    pass does not see: the build scans the assembly for a DPP operand written by a vector
    instruction fewer than two wait states earlier."""
    from e3j_amd.build import dpp_read_hazards
    fine = """
        ds_read2_b32 v[2:3], v193 offset1:16
        s_waitcnt lgkmcnt(0)
        v_mov_b32_e32 v40, v0
        v_fmac_f32_dpp v32, v2, v16 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf
        v_fmac_f32_dpp v33, v3, v16 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf
    """
    assert dpp_read_hazards(fine) == []
    late = """
        v_mov_b32_e32 v2, v7
        v_fmac_f32_dpp v32, v2, v16 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf
    """
    assert len(dpp_read_hazards(late)) == 1
    spaced = """
        v_mov_b32_e32 v2, v7
        s_nop 1
        v_fmac_f32_dpp v32, v2, v16 quad_perm:[0,0,0,0] row_mask:0xf bank_mask:0xf
    """
    assert dpp_read_hazards(spaced) == []
    pair = """
        v_mov_b64_e32 v[2:3], v[8:9]
        v_add_f32_e32 v9, v9, v9
        v_fmac_f32_dpp v32, v3, v16 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf
    """
    assert len(dpp_read_hazards(pair)) == 1
