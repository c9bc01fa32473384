"""SpMM on the MI355X through the C ABI, against the oracle, the golden
fixtures, and (at full size) an fp64 recomputation on the host.

Tolerance for fp32 (and fp64) values: relative Frobenius error <= 1e-5 against
an fp64 recomputation.  Integer results are bit-exact.  The sparsity
structure of the operands is read-only and C is dense, so "structure bit-exact"
means here: shape (M, N), every element written, rows without entries zero.
"""
import numpy as np
import pytest
import scipy.sparse
import torch

from conftest import random_csr
from gpu_util import dev, hip_spmm, host
from scorch_amd import scorch_ops_hip as H
from scorch_amd import workloads

pytestmark = pytest.mark.gpu

TOL = 1e-5
# every kernel that can serve a product is pinned in turn (scorch_ops_hip.SPMM_PATH)
PATHS = ["rows", "merge", "merge_unplanned", "tiled"]
SPMM_F32_CASES = ["spmm_square95", "spmm_dispatch32", "spmm_rect", "spmm_wide300", "spmm_emptyrows",
                  "spmm_n1", "spmm_longrow", "spmm_allzero", "spmm_diag_literal"]


@pytest.mark.parametrize("name", SPMM_F32_CASES)
def test_golden_f32(golden, oracle, name):
    c = golden.case(name)
    got = hip_spmm(c["row_ptr"], c["col_idx"], c["vals"], c["B"])
    ref64 = oracle.spmm_fp64(c["row_ptr"], c["col_idx"], c["vals"], c["B"])
    assert got.shape == c["C_v2"].shape and got.dtype == np.float32
    assert oracle.rel_fro(got, ref64) <= TOL
    np.testing.assert_allclose(got, c["C_v2"], rtol=1e-4, atol=1e-5)   # the reference's own output
    empty = np.diff(c["row_ptr"]) == 0
    assert not got[empty].any()


def test_golden_diag_literal_exact(golden):
    c = golden.case("spmm_diag_literal")
    assert np.array_equal(hip_spmm(c["row_ptr"], c["col_idx"], c["vals"], c["B"]), c["C_v2"])


def test_golden_f64(golden, oracle):
    c = golden.case("spmm_f64")
    got = hip_spmm(c["row_ptr"], c["col_idx"], c["vals"], c["B"])
    assert got.dtype == np.float64
    np.testing.assert_allclose(got, c["C_typed"], rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("name", ["spmm_i32", "spmm_i64", "spmm_i32_wrap"])
def test_golden_integer_bit_exact(golden, name):
    c = golden.case(name)
    got = hip_spmm(c["row_ptr"], c["col_idx"], c["vals"], c["B"])
    assert got.dtype == c["C_typed"].dtype and np.array_equal(got, c["C_typed"])


@pytest.mark.parametrize("relu", [False, True])
def test_golden_bias_act(golden, oracle, relu):
    c = golden.case("spmm_bias")
    got = hip_spmm(c["row_ptr"], c["col_idx"], c["vals"], c["B"], bias=c["bias"], relu=relu)
    np.testing.assert_allclose(got, c["C_bias_relu" if relu else "C_bias"], rtol=1e-4, atol=1e-5)


# N chosen to hit every vector width and tile count: 1 lane, odd, < 64, = 64,
# between tiles, 2-wide vectors (128), partial second tile (192), 4-wide (256+), many tiles
@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("N", [1, 3, 17, 48, 64, 70, 96, 100, 128, 130, 192, 256, 300, 512, 1028])
def test_widths_against_oracle(oracle, N, path):
    rng = np.random.default_rng(N)
    rp, ci, v = random_csr(rng, 333, 217, 0.06, empty_rows=(0, 100, 332))
    B = rng.standard_normal((217, N)).astype(np.float32)
    got = hip_spmm(rp, ci, v, B, path=path)
    assert oracle.rel_fro(got, oracle.spmm_fp64(rp, ci, v, B)) <= TOL
    np.testing.assert_allclose(got, oracle.spmm_csr_f32_v2(rp, ci, v, B), rtol=1e-4, atol=1e-5)


def row_length_cases():
    rng = np.random.default_rng(99)
    cases = {}
    # one row only, longer than several chunks
    cases["single_long_row"] = (np.array([0, 3000], np.int32), rng.integers(0, 500, 3000).astype(np.int32))
    # many empty rows, then entries, then empty rows (chunks made of markers only)
    lens = np.zeros(5000, np.int64); lens[2500:2510] = 40
    cases["mostly_empty"] = lens
    # every row one entry (markers == nonzeros)
    cases["one_per_row"] = np.ones(3000, np.int64)
    # rows exactly at chunk size boundaries
    cases["chunk_aligned"] = np.array([255, 1, 256, 0, 511, 257, 128, 128], np.int64)
    # power-law in miniature
    z = np.minimum(rng.zipf(1.7, 2000), 4000); cases["power_law"] = z.astype(np.int64)
    # last row long, first row long
    cases["long_ends"] = np.array([1500] + [2] * 300 + [1700], np.int64)
    out = {}
    for name, spec in cases.items():
        if isinstance(spec, tuple):
            out[name] = spec
            continue
        rp = np.concatenate([[0], np.cumsum(spec)]).astype(np.int32)
        out[name] = (rp, rng.integers(0, 500, int(rp[-1])).astype(np.int32))
    return out


ROW_CASES = row_length_cases()


@pytest.mark.parametrize("path", PATHS + ["auto"])
@pytest.mark.parametrize("name", sorted(ROW_CASES))
@pytest.mark.parametrize("N", [32, 128, 260])
def test_row_length_distributions(oracle, name, N, path):
    rp, ci = ROW_CASES[name]          # columns unsorted and repeating: allowed
    rng = np.random.default_rng(len(name) + N)
    v = rng.uniform(-1, 1, ci.size).astype(np.float32)
    B = rng.standard_normal((500, N)).astype(np.float32)
    got = hip_spmm(rp, ci, v, B, path=path)
    ref64 = oracle.spmm_fp64(rp, ci, v, B)
    assert oracle.rel_fro(got, ref64) <= TOL
    assert not got[np.diff(rp) == 0].any()


@pytest.mark.parametrize("path", PATHS)
@pytest.mark.parametrize("name", ["power_law", "long_ends", "mostly_empty"])
@pytest.mark.parametrize("relu", [False, True])
def test_bias_act_on_split_rows(oracle, name, relu, path):
    rp, ci = ROW_CASES[name]
    rng = np.random.default_rng(7)
    v = rng.uniform(-1, 1, ci.size).astype(np.float32)
    B = rng.standard_normal((500, 128)).astype(np.float32)
    bias = rng.standard_normal(128).astype(np.float32)
    got = hip_spmm(rp, ci, v, B, bias=bias, relu=relu, path=path)
    ref = oracle.spmm_fp64(rp, ci, v, B) + bias.astype(np.float64)
    if relu:
        ref = np.maximum(ref, 0)
        assert (got >= 0).all()
    assert oracle.rel_fro(got, ref) <= TOL
    np.testing.assert_allclose(got, oracle.spmm_csr_bias_act_f32(rp, ci, v, B, bias, relu), rtol=1e-4,
                               atol=2e-5)


@pytest.mark.parametrize("path", ["rows", "merge", "merge_unplanned"])
@pytest.mark.parametrize("dtype", [np.float64, np.int32, np.int64])
@pytest.mark.parametrize("N", [5, 64, 128, 200])
def test_other_dtypes_against_oracle(oracle, dtype, N, path):
    rp, ci = ROW_CASES["power_law"]
    rng = np.random.default_rng(N)
    if np.issubdtype(dtype, np.integer):
        v = rng.integers(-2 ** 20, 2 ** 20, ci.size).astype(dtype)
        B = rng.integers(-2 ** 20, 2 ** 20, (500, N)).astype(dtype)
    else:
        v = rng.uniform(-1, 1, ci.size).astype(dtype)
        B = rng.standard_normal((500, N)).astype(dtype)
    got = hip_spmm(rp, ci, v, B, path=path)
    want = oracle.spmm_csr_typed(rp, ci, v, B)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(got, want)        # wraps identically (int32 products overflow here)
    else:
        np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)


def test_closed_forms(oracle):
    rng = np.random.default_rng(1)
    B = rng.standard_normal((700, 128)).astype(np.float32)
    ident = hip_spmm(np.arange(701, dtype=np.int32), np.arange(700, dtype=np.int32), np.ones(700, np.float32), B)
    assert np.array_equal(ident, B)
    perm = rng.integers(0, 700, 2000).astype(np.int32)
    gathered = hip_spmm(np.arange(2001, dtype=np.int32), perm, np.ones(2000, np.float32), B)
    assert np.array_equal(gathered, B[perm])
    zero = hip_spmm(np.zeros(11, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32), B[:, :6].copy())
    assert zero.shape == (10, 6) and not zero.any()


def test_runs_are_bit_reproducible_and_inputs_untouched():
    w = workloads.gcn_powerlaw(M=20000, N=128, seed=3, max_degree=5000)
    rp, ci, v, B = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"]), dev(w["B"]).reshape(-1)
    args = ([20000, 128], [20000, 20000], [[], [rp, ci]], v, [20000, 128], [[], []], B)
    first = H.spmm_csr_float_v2(*args).storage.value.clone()
    for _ in range(3):
        again = H.spmm_csr_float_v2(*args).storage.value
        assert torch.equal(first, again)
    assert np.array_equal(host(rp), w["row_ptr"]) and np.array_equal(host(ci), w["col_idx"])
    assert np.array_equal(host(v), w["vals"]) and np.array_equal(host(B).reshape(-1, 128), w["B"])


def test_output_needs_no_zero_fill():
    # poison the allocator's recycled block, then check every element was written
    w = workloads.gcn_powerlaw(M=5000, N=64, seed=4, max_degree=900)
    junk = torch.full((5000 * 64,), float("nan"), device="cuda")
    del junk
    got = hip_spmm(w["row_ptr"], w["col_idx"], w["vals"], w["B"])
    assert np.isfinite(got).all()


def test_output_beyond_two_to_the_31_elements():
    """M * N = 2^31 + 3072 elements of C: the reference keeps this count in an int
    (csrc/spmm.h:113); here every offset is 64-bit.  One unit entry per row makes
    C a row gather of B, checked bit for bit on the device."""
    M, K, N = (1 << 21) + 3, 512, 1024
    g = torch.Generator(device="cuda").manual_seed(5)
    B = torch.randn(K, N, device="cuda", generator=g)
    col = torch.randint(0, K, (M,), device="cuda", generator=g, dtype=torch.int32)
    rp = torch.arange(M + 1, device="cuda", dtype=torch.int32)
    out = H.spmm_csr_float_v2([M, N], [M, K], [[], [rp, col]], torch.ones(M, device="cuda"), [K, N],
                              [[], []], B.reshape(-1)).storage.value.reshape(M, N)
    for r0 in range(0, M, 1 << 19):  # compare in slabs to bound the extra memory
        r1 = min(M, r0 + (1 << 19))
        assert torch.equal(out[r0:r1], B[col[r0:r1].long()])
    assert torch.equal(out[M - 1], B[col[M - 1].long()])


def test_dense_operand_beyond_two_to_the_31_elements():
    """K * N > 2^31: rows of B past the 8 GiB mark are gathered with 64-bit offsets."""
    M, K, N = 4096, (1 << 21) + 5, 1024
    g = torch.Generator(device="cuda").manual_seed(6)
    B = torch.empty(K, N, device="cuda")
    B[:, :] = torch.arange(K, device="cuda", dtype=torch.float32)[:, None]  # row k holds k
    B[K - 4096:, :] += torch.randn(4096, N, device="cuda", generator=g)
    col = torch.randint(K - 4096, K, (M, 2), device="cuda", generator=g, dtype=torch.int32)
    col[:, 0] = torch.randint(0, 4096, (M,), device="cuda", generator=g, dtype=torch.int32)
    col, _ = torch.sort(col, dim=1)
    rp = torch.arange(0, 2 * M + 1, 2, device="cuda", dtype=torch.int32)
    vals = torch.ones(2 * M, device="cuda")
    out = H.spmm_csr_float_v2([M, N], [M, K], [[], [rp, col.reshape(-1).contiguous()]], vals, [K, N],
                              [[], []], B.reshape(-1)).storage.value.reshape(M, N)
    want = B[col[:, 0].long()] + B[col[:, 1].long()]
    assert torch.equal(out, want)


@pytest.mark.parametrize("N", [4, 64, 128, 256])
def test_operands_at_odd_element_offsets(oracle, N):
    """Dense and value operands that are only 4-byte aligned (views one element
    into their buffers): the kernels must fall back to narrower loads, not fault
    or read the wrong elements."""
    rng = np.random.default_rng(40 + N)
    rp, ci, v = random_csr(rng, 300, 200, 0.05, dtype=np.float32)
    B = rng.standard_normal((200, N)).astype(np.float32)
    big_b = torch.empty(200 * N + 1, device="cuda")
    big_v = torch.empty(v.size + 1, device="cuda")
    b_view, v_view = big_b[1:], big_v[1:]
    b_view.copy_(dev(B).reshape(-1))
    v_view.copy_(dev(v))
    assert b_view.data_ptr() % 16 == 4 and v_view.data_ptr() % 8 == 4
    out = H.spmm_csr_float_v2([300, N], [300, 200], [[], [dev(rp), dev(ci)]], v_view, [200, N], [[], []],
                              b_view).storage.value
    got = host(out).reshape(300, N)
    assert oracle.rel_fro(got, oracle.spmm_fp64(rp, ci, v, B)) <= TOL
    bias = rng.standard_normal(N).astype(np.float32)
    big_bias = torch.empty(N + 1, device="cuda")
    big_bias[1:].copy_(dev(bias))
    fused = H.spmm_csr_bias_relu_float([300, N], [300, 200], [[], [dev(rp), dev(ci)]], v_view, [200, N],
                                       [[], []], b_view, big_bias[1:]).storage.value
    want = np.maximum(oracle.spmm_fp64(rp, ci, v, B) + bias, 0)
    assert oracle.rel_fro(host(fused).reshape(300, N), want) <= TOL


def test_uniform_workload_reference_size(oracle):
    """4096 x 4096 at 1 % density, N = 64: the reference's own CPU-runnable case."""
    w = workloads.spmm_uniform()
    got = hip_spmm(w["row_ptr"], w["col_idx"], w["vals"], w["B"])
    assert oracle.rel_fro(got, oracle.spmm_fp64(w["row_ptr"], w["col_idx"], w["vals"], w["B"])) <= TOL
    np.testing.assert_allclose(got, oracle.spmm_csr_f32_v2(w["row_ptr"], w["col_idx"], w["vals"], w["B"]),
                               rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("path", ["merge", "tiled", "rows"])
@pytest.mark.parametrize("M", [1024, 4096])
def test_sae_decoder_workload(oracle, M, path):
    """Sparse-autoencoder decoder shape (32 entries per row, K = 16,384, N = 4096): at a quarter of the
    rows, and at the full 4096 rows that `bench.py --workload sae_decoder` times (the work split
    depends on the size, so the two take different chunk sizes)."""
    w = workloads.sae_decoder(M=M)
    assert w["K"] == 16_384 and w["N"] == 4096 and w["col_idx"].size == 32 * M
    got = hip_spmm(w["row_ptr"], w["col_idx"], w["vals"], w["B"], path=path)
    assert oracle.rel_fro(got, oracle.spmm_fp64(w["row_ptr"], w["col_idx"], w["vals"], w["B"])) <= TOL


def test_power_law_medium_against_oracle(oracle):
    w = workloads.gcn_powerlaw(M=1 << 16, N=128, seed=11, max_degree=20000)
    got = hip_spmm(w["row_ptr"], w["col_idx"], w["vals"], w["B"])
    assert oracle.rel_fro(got, oracle.spmm_fp64(w["row_ptr"], w["col_idx"], w["vals"], w["B"])) <= TOL
    np.testing.assert_allclose(got, oracle.spmm_csr_f32_v2(w["row_ptr"], w["col_idx"], w["vals"], w["B"]),
                               rtol=1e-4, atol=1e-5)


def test_power_law_full_size_properties():
    """The 1,048,576-row, N = 128 workload.  Size-independent checks:
    fp64 recomputation (scipy on the host), linearity in B, and the row sums
    of A recovered from a column of ones."""
    w = workloads.gcn_powerlaw()
    M, N = w["M"], w["N"]
    rp, ci, v = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"])
    B = dev(w["B"])

    def run(Bmat):
        return H.spmm_csr_float_v2([M, N], [M, M], [[], [rp, ci]], v, [M, N], [[], []],
                                   Bmat.reshape(-1)).storage.value.view(M, N)

    C = run(B)
    # (fp64 on the host: the GPU's vendor routine behind torch.sparse.mm / torch.mv has returned NaN
    # for long rows when its uninitialised scratch memory happened to hold NaN)
    A64 = scipy.sparse.csr_matrix((w["vals"].astype(np.float64), w["col_idx"], w["row_ptr"]), shape=(M, M))
    ref64 = torch.from_numpy(A64 @ w["B"].astype(np.float64)).cuda()
    err = (torch.linalg.norm(C.double() - ref64) / torch.linalg.norm(ref64)).item()
    assert err <= TOL, err
    del ref64

    ones = torch.ones_like(B)
    row_sums = torch.zeros(M, dtype=torch.float64, device="cuda")
    rows = torch.repeat_interleave(torch.arange(M, device="cuda"), (rp[1:] - rp[:-1]).long())
    row_sums.index_add_(0, rows, v.double())
    Cones = run(ones)
    assert torch.allclose(Cones[:, 0].double(), row_sums, rtol=1e-5, atol=1e-6)
    assert torch.equal(Cones[:, 0], Cones[:, N - 1])

    B2 = torch.roll(B, 1, dims=0)
    lin = run(B + B2) - (C + run(B2))
    assert (torch.linalg.norm(lin.double()) / torch.linalg.norm(C.double())).item() <= 1e-5


# ---- SpMV shares the merge-path split -----------------------------------------------------------
@pytest.mark.parametrize("name", sorted(ROW_CASES))
@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int64])
def test_spmv_row_length_distributions(oracle, name, dtype):
    from gpu_util import hip_spmv
    rp, ci = ROW_CASES[name]
    rng = np.random.default_rng(len(name))
    if np.issubdtype(dtype, np.integer):
        v = rng.integers(-1000, 1000, ci.size).astype(dtype)
        x = rng.integers(-1000, 1000, 500).astype(dtype)
    else:
        v = rng.uniform(-1, 1, ci.size).astype(dtype)
        x = rng.standard_normal(500).astype(dtype)
    got = hip_spmv(rp, ci, v, x)
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(got, oracle.spmv_csr_typed(rp, ci, v, x))
    else:
        ref64 = oracle.spmm_fp64(rp, ci, v, x.reshape(-1, 1)).reshape(-1)
        assert oracle.rel_fro(got, ref64) <= (TOL if dtype == np.float32 else 1e-13)
    assert not got[np.diff(rp) == 0].any()


@pytest.mark.parametrize("scale", [1, 7])
@pytest.mark.parametrize("dtype", [np.float32, np.float64, np.int64])
def test_spmv_rows_spread_over_many_wavefronts(oracle, dtype, scale):
    """Rows whose carries form long runs (a row of 40,000 entries spans ~80 wavefronts, one of
    600,000 over a thousand), next to ordinary ones and at both ends of the matrix.  Seven times
    that size the matrix is past 4 M merged items, where a wavefront takes 1024 of them."""
    from gpu_util import hip_spmv
    rng = np.random.default_rng(5)
    lens = rng.integers(0, 6, 300)
    lens[[0, 57, 58, 299]] = np.array([40_000, 600_000, 17_000, 33_000]) * scale
    K = 700_000 * scale
    assert scale == 1 or lens.sum() + lens.size >= 4 << 20
    rp = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ci = np.concatenate([np.sort(rng.choice(K, int(n), replace=False)) for n in lens]).astype(np.int32)
    if np.issubdtype(dtype, np.integer):
        v, x = rng.integers(-1000, 1000, ci.size).astype(dtype), rng.integers(-1000, 1000, K).astype(dtype)
    else:
        v, x = rng.uniform(-1, 1, ci.size).astype(dtype), rng.standard_normal(K).astype(dtype)
    got = hip_spmv(rp, ci, v, x)
    assert np.array_equal(got, hip_spmv(rp, ci, v, x))
    if np.issubdtype(dtype, np.integer):
        assert np.array_equal(got, oracle.spmv_csr_typed(rp, ci, v, x))
    else:
        ref64 = oracle.spmm_fp64(rp, ci, v, x.reshape(-1, 1)).reshape(-1)
        # (fp64 against fp64 summed in another order: rounding grows with the square root of a
        # row's length, 2e-13 for the row of 4.2 M entries)
        assert oracle.rel_fro(got, ref64) <= (TOL if dtype == np.float32 else 1e-13 * scale)


def test_spmv_full_size_and_reproducible():
    w = workloads.gcn_powerlaw(N=1)
    M = w["M"]
    rp, ci, v, x = dev(w["row_ptr"]), dev(w["col_idx"]), dev(w["vals"]), dev(w["B"]).reshape(-1)
    call = lambda: H.prebuilt_spmv_csr_f32([M], [M, M], [[], [rp, ci]], v, [M], [[]], x).storage.value
    y = call()
    assert torch.equal(y, call())
    A64 = scipy.sparse.csr_matrix((w["vals"].astype(np.float64), w["col_idx"], w["row_ptr"]), shape=(M, M))
    ref = torch.from_numpy(A64 @ w["B"].reshape(-1).astype(np.float64)).cuda()
    assert (torch.linalg.norm(y.double() - ref) / torch.linalg.norm(ref)).item() <= TOL


# ---- A in coordinate form (the reference's spmm_coo_float) ------------------------------
def hip_spmm_coo(row_idx, col_idx, vals, B, n_rows):
    out = H.spmm_coo_float([n_rows, B.shape[1]], [n_rows, B.shape[0]], [[dev(row_idx)], [dev(col_idx)]], dev(vals),
                           list(B.shape), [[], []], dev(B).reshape(-1))
    assert out.storage.index.mode_indices == [[], []]
    return host(out.storage.value).reshape(n_rows, B.shape[1])


@pytest.mark.parametrize("name", ["spmm_coo", "spmm_coo_unsorted"])
def test_golden_coordinate_operand(golden, name):
    c = golden.case(name)
    got = hip_spmm_coo(c["row_idx"], c["col_idx"], c["vals"], c["B"], int(c["n_rows"]))
    np.testing.assert_allclose(got, c["C"], rtol=1e-4, atol=1e-5)  # the reference's own output


def test_coordinate_operand_in_any_order_with_repeats(oracle):
    rng = np.random.default_rng(71)
    rp, ci, v = random_csr(rng, 3000, 2000, 0.004, empty_rows=(0, 2999))
    r = np.repeat(np.arange(3000, dtype=np.int32), np.diff(rp))
    B = rng.standard_normal((2000, 96)).astype(np.float32)
    ref64 = oracle.spmm_fp64(rp, ci, v, B)
    assert oracle.rel_fro(hip_spmm_coo(r, ci, v, B, 3000), ref64) <= TOL
    order = rng.permutation(r.size)  # shuffled, every entry twice
    got = hip_spmm_coo(np.tile(r[order], 2), np.tile(ci[order], 2), np.tile(v[order], 2), B, 3000)
    assert oracle.rel_fro(got, 2 * ref64) <= TOL


def test_coordinate_operand_checks_row_range():
    B = np.ones((4, 8), np.float32)
    with pytest.raises(ValueError, match="outside"):
        hip_spmm_coo(np.array([0, 5], np.int32), np.array([1, 1], np.int32), np.ones(2, np.float32), B, 4)


def test_coordinate_row_pointer(oracle):
    rng = np.random.default_rng(72)
    rows = np.sort(rng.integers(0, 50_000, 400_000)).astype(np.int32)
    pos = H.coo_row_ptr(dev(rows), 50_000)
    assert np.array_equal(host(pos), np.searchsorted(rows, np.arange(50_001)).astype(np.int32))
    # far more rows than entries, and no entries at all
    few = np.array([7, 7, 999_999], np.int32)
    assert np.array_equal(host(H.coo_row_ptr(dev(few), 1_000_000)),
                          np.searchsorted(few, np.arange(1_000_001)).astype(np.int32))
    assert not host(H.coo_row_ptr(dev(np.zeros(0, np.int32)), 9)).any()
    assert H.coo_row_ptr(dev(np.array([3, 2], np.int32)), 9) is None      # descending
    assert H.coo_row_ptr(dev(np.array([3, 9], np.int32)), 9) is None      # out of range
    assert H.coo_row_ptr(dev(np.array([-1, 2], np.int32)), 9) is None


def test_every_spmm_name_the_reference_binds_runs_the_device_kernel(golden):
    """reference: csrc/ops.cpp:107-164 (the fp32 CSR x dense names, with their tile arguments)"""
    c = golden.case("spmm_rect")
    M, (K, N) = c["row_ptr"].size - 1, c["B"].shape
    args = ([M, N], [M, K], [[], [dev(c["row_ptr"]), dev(c["col_idx"])]], dev(c["vals"]), [K, N], [[], []],
            dev(c["B"]).reshape(-1))
    expect = host(H.spmm_csr_float_v2(*args).storage.value)
    names = ["spmm_csr_float", "prebuilt_spmm_csr_f32"] + ["spmm_csr_float_" + v for v in H.SPMM_CSR_FLOAT_VARIANTS]
    assert len(names) == 15
    for name in names:
        assert np.array_equal(host(getattr(H, name)(*args).storage.value), expect), name
    for name in ("spmm_csr_float_v2", "spmm_csr_float_turbo", "spmm_csr_float_apex"):
        assert np.array_equal(host(getattr(H, name)(*args, tile_size=128).storage.value), expect)
    tiled = H.spmm_csr_float_tiled_i_k(*args, i_tile_size=64, k_tile_size=32)
    assert np.array_equal(host(tiled.storage.value), expect)


def test_direct_calls_on_a_large_square_like_the_references_perf_test():
    """reference: tests/test_scorch/test_perf_large.py:15-35,52-73 -- n = 1024, 95 % sparse, seed 7,
    the native symbols called directly with STensor parts, checked against torch.sparse.mm."""
    import scorch_amd as scorch
    generator = torch.Generator().manual_seed(7)
    n = 1024
    a_dense = torch.rand((n, n), generator=generator, dtype=torch.float32)
    b_dense = torch.rand((n, n), generator=generator, dtype=torch.float32)
    a_dense = a_dense * (torch.rand((n, n), generator=generator) > 0.95)
    reference = torch.sparse.mm(a_dense.to_sparse_csr(), b_dense)
    a = scorch.STensor.from_torch(a_dense, "A").to_sparse("ds").to("cuda")
    b = scorch.STensor.from_torch(b_dense, "B").to("cuda")
    args = [[n, n]]
    for tensor in (a, b):
        args += [list(tensor.shape), tensor.index.mode_indices, tensor.values]
    for name in ("spmm_csr_float_untiled", "spmm_csr_float", "spmm_csr_float_optimized", "spmm_csr_float_turbo",
                 "spmm_csr_float_ultra", "spmm_csr_float_apex", "spmm_csr_float_tiled_i_k", "spmm_csr_float_v2"):
        result = getattr(H, name)(*args).storage.value
        assert torch.allclose(result.cpu().view_as(reference), reference, atol=1e-3, rtol=1e-3), name
    out = scorch.matmul(a, b)
    assert torch.allclose(out.cpu(), reference, atol=1e-3, rtol=1e-3)
