"""The C-ABI library without a GPU: it loads, exports every symbol that
include/scorch_hip.h and include/scorch_hip_unstable.h declare, and rejects bad
arguments on the host before launching anything.  No compute call is made here."""
import ctypes
import os
import re

import pytest

from scorch_amd import native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "scorch_hip.h")                    # the stable surface
UNSTABLE_HEADER = os.path.join(ROOT, "include", "scorch_hip_unstable.h")  # the steps underneath
HEADERS = (HEADER, UNSTABLE_HEADER)


def declared_symbols(headers=HEADERS):
    names = []
    for header in headers:
        text = open(header).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"SCORCH_HIP_API[^;(]*?\b(scorch_hip_\w+)\s*\(", text)
    assert len(names) == len(set(names)), "a function is declared twice"
    return sorted(names)


@pytest.fixture(scope="module")
def L():
    return native.lib()


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for required in ["scorch_hip_spmm_csr_f32", "scorch_hip_spmm_csr_workspace_bytes",
                     "scorch_hip_sddmm_csr_f32", "scorch_hip_sddmm_coo_f32",
                     "scorch_hip_spmm_csr_bias_act_f32", "scorch_hip_last_error"]:
        assert required in names
    assert len(names) >= 16


def test_the_stable_header_holds_no_plan_step():
    """One call per operation and the plan handle in scorch_hip.h; inspection, boundaries, entry
    lists, block descriptions, work-item lists, pinned kernels and timing aids in the other."""
    stable = declared_symbols((HEADER,))
    unstable = declared_symbols((UNSTABLE_HEADER,))
    step = re.compile(r"inspect|bounds|planned|_rows_|tiled|lists|listed|known_rows|split|blocked|block_|batched|"
                      r"timing|timed|attn_blocksparse_f32|values_differ|list_values")
    assert [n for n in stable if step.search(n)] == []
    assert [n for n in unstable if not step.search(n)] == []
    assert len(stable) <= 40
    for name in ("create", "destroy", "info", "prepare"):
        assert "scorch_hip_csr_plan_" + name in stable
    for name in ("spmm", "sddmm", "softmax"):
        assert f"scorch_hip_{name}_csr_plan_f32" in stable


def test_library_exports_every_declared_symbol(L):
    for name in declared_symbols():
        assert hasattr(L, name), f"{name} is declared in a header but not exported"


def test_binding_table_matches_header(L):
    assert sorted(native.SIGNATURES) == declared_symbols()


def test_abi_version(L):
    m = re.search(r"#define SCORCH_HIP_ABI_VERSION (\d+)", open(HEADER).read())
    assert L.scorch_hip_abi_version() == int(m.group(1))


def test_workspace_bytes_formula(L):
    f = L.scorch_hip_spmm_csr_workspace_bytes
    assert f(-1, 0, 4, 4) == 0 and f(4, 4, 4, 0) == 0
    small = f(10, 100, 128, 4)
    assert small > 0 and small % 256 == 0
    # grows with the amount of work and with the row width
    assert f(1 << 20, 17_000_000, 128, 4) > f(1 << 20, 17_000_000, 64, 4) > small
    assert f(10, 100, 128, 8) > small


NULL = None
FAKE = ctypes.c_void_p(0x1000)  # never dereferenced: validation fails first


def spmm(L, M=4, K=4, N=4, nnz=4, row_ptr=FAKE, col=FAKE, vals=FAKE, B=FAKE, C=FAKE, ws=FAKE, ws_bytes=1 << 30):
    return L.scorch_hip_spmm_csr_f32(M, K, N, nnz, row_ptr, col, vals, B, C, ws, ws_bytes, NULL)


def test_spmm_rejects_bad_arguments(L):
    assert spmm(L, M=-1) == native.EINVAL
    assert b"negative" in L.scorch_hip_last_error()
    assert spmm(L, row_ptr=NULL) == native.EINVAL
    assert spmm(L, col=NULL) == native.EINVAL
    assert spmm(L, C=NULL) == native.EINVAL
    assert spmm(L, B=NULL) == native.EINVAL
    assert spmm(L, M=0, K=0, nnz=3) == native.EINVAL
    assert spmm(L, M=1 << 31) == native.EUNSUPPORTED
    assert spmm(L, nnz=1 << 31) == native.EUNSUPPORTED
    assert spmm(L, row_ptr=ctypes.c_void_p(0x1001)) == native.EINVAL  # misaligned
    assert spmm(L, ws=NULL) == native.EWORKSPACE
    assert spmm(L, ws_bytes=16) == native.EWORKSPACE
    assert b"workspace" in L.scorch_hip_last_error()
    assert spmm(L, ws=ctypes.c_void_p(0x1010)) == native.EINVAL  # not 256-byte aligned


def test_static_scratch_spmm_rejects_sizes_beyond_its_buffer(L):
    f = L.scorch_hip_spmm_csr_f32_static
    limit = int(re.search(r"#define SCORCH_HIP_STATIC_SCRATCH_BYTES \(\(size_t\)(\d+) << 20\)",
                          open(HEADER).read()).group(1)) << 20
    assert L.scorch_hip_spmm_csr_workspace_bytes(1 << 20, 60_000_000, 512, 4) > limit
    assert f(1 << 20, 1 << 20, 512, 60_000_000, FAKE, FAKE, FAKE, FAKE, FAKE, NULL) == native.EWORKSPACE
    assert b"static buffer" in L.scorch_hip_last_error()
    assert f(-1, 4, 4, 4, FAKE, FAKE, FAKE, FAKE, FAKE, NULL) == native.EINVAL
    # the headline product fits
    assert L.scorch_hip_spmm_csr_workspace_bytes(1 << 20, 17_825_865, 128, 4) <= limit


def test_spmm_empty_output_is_a_no_op(L):
    assert spmm(L, M=0, nnz=0, C=NULL, ws=NULL) == native.OK
    assert spmm(L, N=0, C=NULL, ws=NULL) == native.OK


def test_bias_act_rejects_unknown_activation_and_null_bias(L):
    f = L.scorch_hip_spmm_csr_bias_act_f32
    assert f(4, 4, 4, 4, FAKE, FAKE, FAKE, FAKE, FAKE, 7, FAKE, FAKE, 1 << 30, NULL) == native.EINVAL
    assert b"activation" in L.scorch_hip_last_error()
    assert f(4, 4, 4, 4, FAKE, FAKE, FAKE, FAKE, NULL, 1, FAKE, FAKE, 1 << 30, NULL) == native.EINVAL


def test_sddmm_rejects_bad_arguments(L):
    csr, coo = L.scorch_hip_sddmm_csr_f32, L.scorch_hip_sddmm_coo_f32
    assert csr(-1, 4, 4, 4, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, NULL, NULL) == native.EINVAL
    assert csr(4, 4, 4, 4, NULL, FAKE, FAKE, FAKE, FAKE, FAKE, NULL, NULL) == native.EINVAL
    assert csr(4, 4, 4, 4, FAKE, FAKE, FAKE, NULL, FAKE, FAKE, NULL, NULL) == native.EINVAL
    assert csr(0, 0, 4, 4, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, NULL, NULL) == native.EINVAL
    assert coo(4, 4, 4, 4, NULL, FAKE, FAKE, FAKE, FAKE, FAKE, NULL) == native.EINVAL
    assert coo(4, 4, 4, 4, FAKE, FAKE, FAKE, FAKE, FAKE, NULL, NULL) == native.EINVAL
    assert coo(4, 4, 4, 0, NULL, NULL, NULL, NULL, NULL, NULL, NULL) == native.OK  # nothing to do
    assert coo(4, 4, 4, 1 << 31, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, NULL) == native.EUNSUPPORTED


def test_spmv_softmax_rows_reject_bad_arguments(L):
    assert L.scorch_hip_spmv_csr_f64(4, 4, 4, FAKE, FAKE, FAKE, FAKE, NULL, FAKE, 1 << 20, NULL) == native.EINVAL
    assert L.scorch_hip_spmv_csr_i32(-4, 4, 4, FAKE, FAKE, FAKE, FAKE, FAKE, FAKE, 1 << 20, NULL) == native.EINVAL
    assert L.scorch_hip_spmv_csr_i64(0, 4, 0, FAKE, NULL, NULL, NULL, NULL, NULL, 0, NULL) == native.OK
    assert L.scorch_hip_spmv_csr_f32(4, 4, 4, FAKE, FAKE, FAKE, FAKE, FAKE, NULL, 0, NULL) == native.EWORKSPACE
    assert L.scorch_hip_spmv_csr_workspace_bytes(1000, 5000, 4) % 256 == 0
    assert L.scorch_hip_softmax_csr_f32(4, 4, NULL, FAKE, 1.0, FAKE, NULL, 0, NULL) == native.EINVAL
    assert L.scorch_hip_softmax_csr_f32(4, 4, FAKE, NULL, 1.0, FAKE, NULL, 0, NULL) == native.EINVAL
    # rows longer than 4096 entries are possible from nnz = 4097 on: a workspace is needed then
    assert L.scorch_hip_softmax_csr_workspace_bytes(4, 4096) == 0
    assert L.scorch_hip_softmax_csr_workspace_bytes(4, 4097) == 512
    assert L.scorch_hip_softmax_csr_workspace_bytes(1 << 20, 16_384) == 256 + 256
    # from 16,385 entries on a row can be long enough to be served in stretches (if it holds a large part
    # of the entries of all rows beyond 4096: at most 100 rows do; from 65,537 on in any case): three more
    # arrays (3 such rows at most, 7 + 3 stretches of 8192 or more; then 259 + 100 rows, 2,075 + 359 stretches)
    assert L.scorch_hip_softmax_csr_workspace_bytes(1 << 20, 60_000) == 256 + 256 + 256 + 2 * 256
    assert L.scorch_hip_softmax_csr_workspace_bytes(1 << 20, 17_000_000) == 256 + 16640 + 5888 + 2 * 19712
    assert L.scorch_hip_softmax_csr_f32(4, 5000, FAKE, FAKE, 1.0, FAKE, NULL, 0, NULL) == native.EWORKSPACE
    assert L.scorch_hip_softmax_csr_f32(4, 5000, FAKE, FAKE, 1.0, FAKE, FAKE, 256, NULL) == native.EWORKSPACE
    assert L.scorch_hip_csr_row_indices(4, 4, FAKE, NULL, NULL) == native.EINVAL
    assert L.scorch_hip_csr_row_indices(0, 4, FAKE, FAKE, NULL) == native.EINVAL
    assert L.scorch_hip_coo_row_ptr(4, 4, FAKE, NULL, FAKE, NULL) == native.EINVAL
    assert L.scorch_hip_coo_row_ptr(4, 4, FAKE, FAKE, NULL, NULL) == native.EINVAL
    assert L.scorch_hip_coo_row_ptr(4, 4, NULL, FAKE, FAKE, NULL) == native.EINVAL
    assert L.scorch_hip_coo_row_ptr(-1, 0, NULL, FAKE, FAKE, NULL) == native.EINVAL


def test_check_raises_with_the_library_message(L):
    code = spmm(L, M=-3)
    with pytest.raises(native.ScorchHipError) as info:
        native.check(code)
    assert info.value.code == native.EINVAL and "M=-3" in str(info.value)


def test_attention_rejects_unsupported_shapes(L):
    f = L.scorch_hip_attn_blocksparse_bf16
    ok_args = dict(H=2, S=128, D=64, block=64, nblk=3)

    def call(H=2, S=128, D=64, block=64, nblk=3, brp=FAKE, bci=FAKE, q=FAKE, k=FAKE, v=FAKE, o=FAKE):
        return f(H, S, D, block, nblk, brp, bci, q, k, v, 0.125, o, NULL)

    assert call(D=96) == native.EUNSUPPORTED
    assert b"head dimension" in L.scorch_hip_last_error()
    assert call(block=32) == native.EUNSUPPORTED
    assert call(S=100) == native.EINVAL
    assert call(H=-1) == native.EINVAL
    assert call(brp=NULL) == native.EINVAL
    assert call(q=NULL) == native.EINVAL
    assert call(o=ctypes.c_void_p(0x1008)) == native.EINVAL      # not 16-byte aligned
    assert call(H=0, q=NULL, k=NULL, v=NULL, o=NULL) == native.OK

    g = L.scorch_hip_attn_blocksparse_masked_bf16

    def masked(D=32, nblk=3, bmi=FAKE, n_masks=1, masks=FAKE, q=FAKE):
        return g(2, 128, D, 64, nblk, FAKE, FAKE, bmi, n_masks, masks, q, FAKE, FAKE, 0.125, FAKE, NULL)

    assert masked(D=48) == native.EUNSUPPORTED
    assert masked(bmi=NULL) == native.EINVAL
    assert masked(masks=NULL) == native.EINVAL
    assert masked(masks=ctypes.c_void_p(0x1004)) == native.EINVAL  # not 8-byte aligned
    assert masked(n_masks=-1) == native.EINVAL
    assert masked(q=NULL) == native.EINVAL

    h = L.scorch_hip_attn_blocksparse_split_bf16
    need = L.scorch_hip_attn_blocksparse_split_workspace_bytes(2, 3, 32)
    assert need == 2 * 3 * 64 * 36 * 4 and L.scorch_hip_attn_blocksparse_split_workspace_bytes(2, 0, 32) == 0

    def split(D=32, n_items=5, items=FAKE, n_split=1, rows=FAKE, n_slots=3, ws=FAKE, ws_bytes=need, q=FAKE, prio=0):
        return h(2, 128, D, 64, 4, n_items, items, 0, prio, n_split, rows, n_slots, FAKE, NULL, 0, NULL, q, FAKE, FAKE,
                 0.125, FAKE, ws, ws_bytes, NULL)

    assert split(D=48) == native.EUNSUPPORTED
    assert split(items=NULL) == native.EINVAL
    assert split(items=ctypes.c_void_p(0x1004)) == native.EINVAL   # not 16-byte aligned
    assert split(rows=NULL) == native.EINVAL
    assert split(ws=NULL) == native.EWORKSPACE
    assert split(ws_bytes=need - 1) == native.EWORKSPACE
    assert split(n_items=-1) == native.EINVAL
    assert split(prio=-1) == native.EINVAL
    assert split(q=NULL) == native.EINVAL
    assert split(n_items=0, items=NULL) == native.OK


def test_plan_handle_rejects_bad_arguments_on_the_host(L):
    handle = ctypes.c_void_p()
    ref = ctypes.byref(handle)
    index = (ctypes.c_int32 * 8)()
    at = ctypes.addressof(index)
    assert L.scorch_hip_csr_plan_create(4, 4, 0, at, NULL, None, None) == native.EINVAL
    assert b"plan is NULL" in L.scorch_hip_last_error()
    assert L.scorch_hip_csr_plan_create(-1, 4, 0, at, NULL, None, ref) == native.EINVAL
    assert L.scorch_hip_csr_plan_create(4, 4, 0, NULL, NULL, None, ref) == native.EINVAL
    assert L.scorch_hip_csr_plan_create(4, 4, 3, at, NULL, None, ref) == native.EINVAL
    assert L.scorch_hip_csr_plan_create(1 << 31, 4, 0, at, NULL, None, ref) == native.EUNSUPPORTED
    assert handle.value is None
    info = (ctypes.c_int64 * 8)()
    assert L.scorch_hip_csr_plan_info(None, info) == native.EINVAL
    assert L.scorch_hip_csr_plan_prepare(None, 0, 8, None) == native.EINVAL
    assert L.scorch_hip_spmm_csr_plan_f32(None, 8, at, at, None, 0, at, None) == native.EINVAL
    assert L.scorch_hip_sddmm_csr_plan_f32(None, 8, None, at, at, at, None, None) == native.EINVAL
    assert L.scorch_hip_softmax_csr_plan_f32(None, at, 1.0, at, None) == native.EINVAL
    assert L.scorch_hip_csr_plan_destroy(None) == native.OK
    assert L.scorch_hip_dense_plan_create(4, 4, at, None, None) == native.EINVAL
    assert L.scorch_hip_dense_plan_create(-1, 4, at, None, ref) == native.EINVAL
    assert L.scorch_hip_dense_plan_create(4, 4, NULL, None, ref) == native.EINVAL
    assert handle.value is None
    assert L.scorch_hip_dense_plan_update(None, None) == native.EINVAL
    assert L.scorch_hip_dense_plan_destroy(None) == native.OK
    assert L.scorch_hip_spmm_csr_plan_dense_f32(None, at, None, None, 0, at, None) == native.EINVAL


def test_header_is_plain_c_and_a_c_host_can_link(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 and as C++11, and a C program linked
    against the library reads the ABI version and a workspace size (no GPU involved)."""
    import os
    import shutil
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    gcc, gxx = shutil.which("gcc"), shutil.which("g++")
    if not gcc or not gxx:
        pytest.skip("no host compiler")
    for header in HEADERS:
        subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-x", "c", header], check=True)
        subprocess.run([gxx, "-std=c++11", "-Wall", "-Werror", "-fsyntax-only", "-x", "c++", header], check=True)
    src = tmp_path / "host.c"
    src.write_text(
        '#include <stdio.h>\n#include "scorch_hip.h"\n'
        "int main(void) {\n"
        '  printf("%d %zu\\n", scorch_hip_abi_version(),\n'
        "         scorch_hip_spmm_csr_workspace_bytes(1000, 5000, 64, 4));\n"
        "  return scorch_hip_last_error() == NULL;\n}\n")
    lib_dir = os.path.dirname(native.library_path())
    exe = tmp_path / "host"
    subprocess.run([gcc, "-std=c99", "-I", os.path.join(root, "include"), str(src), "-L", lib_dir,
                    "-l:libscorch_hip.so", "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib", "-o", str(exe)],
                   check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()
    assert int(out[0]) == native.lib().scorch_hip_abi_version()
    assert int(out[1]) == native.lib().scorch_hip_spmm_csr_workspace_bytes(1000, 5000, 64, 4)


def test_the_c_host_demo_builds(tmp_path):
    """The C99 host program of tests/host_c compiles and links against the library with gcc
    (it runs in the GPU tests)."""
    import shutil
    from scorch_amd import build
    if not shutil.which("gcc") or not os.path.exists("/opt/rocm/include/hip/hip_runtime_api.h"):
        pytest.skip("no gcc or no HIP headers")
    assert os.path.exists(build.build_host_demo())
