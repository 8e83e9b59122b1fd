"""The Linux stand-in for Apple's Accelerate (swift/honeycrisp-linux/Sources/Accelerate), the C
target that lets the reference's CPUBackend build off macOS: every symbol the reference calls,
with the operand order of its call site (BackendCPU.swift:284-2066, TensorElement.swift:262-338),
checked from Python through ctypes against numpy's IEEE single arithmetic (bit for bit), against
closed forms, and against the CPU oracle where both restate the same reference routine."""
import ctypes
import glob
import os
import shutil
import subprocess
import sys
from ctypes import POINTER, Structure, byref, c_char, c_float, c_int32, c_long, c_size_t, c_ulong, c_void_p

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHIM_DIR = os.path.join(ROOT, "swift", "honeycrisp-linux", "Sources", "Accelerate")
FP = POINTER(c_float)


def bundled_openblas():
    """OpenBLAS builds that ship inside the numpy / scipy wheels (symbols prefixed scipy_, the
    numpy one with 64-bit integers), if any."""
    found = []
    for mod in ("scipy", "numpy"):
        try:
            m = __import__(mod)
        except ImportError:
            continue
        libs = os.path.join(os.path.dirname(os.path.dirname(m.__file__)), mod + ".libs")
        found += sorted(glob.glob(os.path.join(libs, "libscipy_openblas*.so")))
    return found


@pytest.fixture(scope="session")
def shim_path(tmp_path_factory):
    out = tmp_path_factory.mktemp("accelerate") / "libAccelerateShim.so"
    subprocess.run(["gcc", "-O2", "-std=gnu11", "-fPIC", "-ffp-contract=off", "-fno-fast-math", "-Wall", "-Wextra",
                    "-Werror", "-shared", "-o", str(out), os.path.join(SHIM_DIR, "accelerate_shim.c"),
                    "-ldl", "-lm", "-lpthread"], check=True)
    return str(out)


class vImage_Buffer(Structure):
    _fields_ = [("data", c_void_p), ("height", c_ulong), ("width", c_ulong), ("rowBytes", c_size_t)]


def load(path, blas=None):
    """A private copy of the library (its BLAS binding happens once per loaded copy), bound to
    `blas`: a library path, "builtin", or None for the default search."""
    copy = path.replace(".so", "_%s.so" % (abs(hash(blas)) % 10**8))
    if not os.path.exists(copy):
        shutil.copy(path, copy)
    if blas is None:
        os.environ.pop("HC_ACCELERATE_BLAS", None)
    else:
        os.environ["HC_ACCELERATE_BLAS"] = blas
    lib = ctypes.CDLL(copy)
    lib.hc_accelerate_blas_backend.restype = ctypes.c_char_p
    backend = lib.hc_accelerate_blas_backend().decode()     # binds now, while the variable is set
    os.environ.pop("HC_ACCELERATE_BLAS", None)
    three = [FP, c_long, FP, c_long, FP, c_long, c_ulong]
    for name in ("vDSP_vadd", "vDSP_vmul", "vDSP_vsub", "vDSP_vdiv"):
        getattr(lib, name).argtypes = three
    for name in ("vDSP_vsadd", "vDSP_vsmul"):
        getattr(lib, name).argtypes = [FP, c_long, FP, FP, c_long, c_ulong]
    lib.vDSP_svdiv.argtypes = [FP, FP, c_long, FP, c_long, c_ulong]
    lib.vDSP_vsmsa.argtypes = [FP, c_long, FP, FP, FP, c_long, c_ulong]
    for name in ("vDSP_vma", "vDSP_vam"):
        getattr(lib, name).argtypes = [FP, c_long, FP, c_long, FP, c_long, FP, c_long, c_ulong]
    lib.vDSP_sve.argtypes = [FP, c_long, FP, c_ulong]
    lib.vDSP_mmul.argtypes = [FP, c_long, FP, c_long, FP, c_long, c_ulong, c_ulong, c_ulong]
    lib.vDSP_mtrans.argtypes = [FP, c_long, FP, c_long, c_ulong, c_ulong]
    for name in ("vImageConvert_PlanarFtoPlanar16F", "vImageConvert_Planar16FtoPlanarF"):
        getattr(lib, name).argtypes = [POINTER(vImage_Buffer), POINTER(vImage_Buffer), ctypes.c_uint32]
        getattr(lib, name).restype = c_long
    I = POINTER(c_int32)
    lib.sgeqrf_.argtypes = [I, I, FP, I, FP, FP, I, I]
    lib.sorgqr_.argtypes = [I, I, I, FP, I, FP, FP, I, I]
    lib.sgesvd_.argtypes = [POINTER(c_char), POINTER(c_char), I, I, FP, I, FP, FP, I, FP, I, FP, I, I]
    return lib, backend


@pytest.fixture(scope="session")
def shim(shim_path):
    return load(shim_path, "builtin")[0]


def fp(a):
    return a.ctypes.data_as(FP)


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


@pytest.fixture
def xy():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(1001) * 3).astype(np.float32)
    y = (rng.standard_normal(1001) + 2.5).astype(np.float32)
    x[:4] = [0.0, -0.0, np.inf, 1e-40]
    return x, y


def test_two_operand_forms_and_their_operand_order(shim, xy):
    x, y = xy
    n = x.size
    z = np.empty_like(x)
    # the reference calls vDSP_vsub(y, 1, x, 1, z, ...) and expects z = x - y (BackendCPU.swift:288-290)
    shim.vDSP_vsub(fp(y), 1, fp(x), 1, fp(z), 1, n)
    assert np.array_equal(bits(z), bits(x - y))
    shim.vDSP_vdiv(fp(y), 1, fp(x), 1, fp(z), 1, n)
    assert np.array_equal(bits(z), bits(x / y))
    shim.vDSP_vadd(fp(y), 1, fp(x), 1, fp(z), 1, n)
    assert np.array_equal(bits(z), bits(x + y))
    shim.vDSP_vmul(fp(y), 1, fp(x), 1, fp(z), 1, n)
    assert np.array_equal(bits(z), bits(x * y))
    # an asymmetric pair that a swapped implementation cannot pass
    a, b, out = np.float32([6.0]), np.float32([2.0]), np.float32([0.0])
    shim.vDSP_vsub(fp(b), 1, fp(a), 1, fp(out), 1, 1)
    assert out[0] == 4.0
    shim.vDSP_vdiv(fp(b), 1, fp(a), 1, fp(out), 1, 1)
    assert out[0] == 3.0


def test_scalar_forms(shim, xy):
    x, _ = xy
    n = x.size
    z = np.empty_like(x)
    s = np.float32([1.0 / 3.0])
    shim.vDSP_vsadd(fp(x), 1, fp(s), fp(z), 1, n)
    assert np.array_equal(bits(z), bits(x + s[0]))
    shim.vDSP_vsmul(fp(x), 1, fp(s), fp(z), 1, n)
    assert np.array_equal(bits(z), bits(x * s[0]))
    with np.errstate(divide="ignore"):
        want = s[0] / x
    shim.vDSP_svdiv(fp(s), fp(x), 1, fp(z), 1, n)
    assert np.array_equal(bits(z), bits(want))
    # vsmsa: x * m + a with two roundings (the reference's a - x is m = -1, BackendCPU.swift:384)
    m, a = np.float32([-1.0]), np.float32([0.1])
    shim.vDSP_vsmsa(fp(x), 1, fp(m), fp(a), fp(z), 1, n)
    assert np.array_equal(bits(z), bits((x * m[0]).astype(np.float32) + a[0]))
    m = np.float32([1.0000001])
    big = np.float32([16777216.0, 3.0000002]); out = np.empty_like(big)
    shim.vDSP_vsmsa(fp(big), 1, fp(m), fp(a), fp(out), 1, 2)
    assert np.array_equal(bits(out), bits((big * m[0]).astype(np.float32) + a[0]))   # not a fused multiply-add


def test_three_operand_forms(shim, xy):
    x, y = xy
    n = x.size
    rng = np.random.default_rng(6)
    c = rng.standard_normal(n).astype(np.float32)
    d = np.empty_like(x)
    finite = np.isfinite(x)
    shim.vDSP_vma(fp(x), 1, fp(y), 1, fp(c), 1, fp(d), 1, n)      # x * y + c
    assert np.array_equal(bits(d)[finite], bits((x * y).astype(np.float32) + c)[finite])
    shim.vDSP_vam(fp(x), 1, fp(y), 1, fp(c), 1, fp(d), 1, n)      # (x + y) * c
    assert np.array_equal(bits(d)[finite], bits((x + y).astype(np.float32) * c)[finite])


def test_strides_and_in_place_output(shim):
    rng = np.random.default_rng(7)
    a = rng.standard_normal(60).astype(np.float32)
    b = rng.standard_normal(60).astype(np.float32)
    c = np.zeros(60, np.float32)
    shim.vDSP_vadd(fp(a), 2, fp(b), 3, fp(c), 1, 20)
    assert np.array_equal(c[:20], a[::2][:20] + b[::3][:20]) and not c[20:].any()
    z = a.copy()
    shim.vDSP_vmul(fp(z), 1, fp(b), 1, fp(z), 1, 60)    # z = z * scales in place (BackendCPU.swift:680)
    assert np.array_equal(z, a * b)
    s = np.float32([2.5])
    z = a.copy()
    shim.vDSP_vsmul(fp(z), 1, fp(s), fp(z), 1, 60)      # (:668)
    assert np.array_equal(z, a * s[0])
    shim.vDSP_vadd(fp(a), 1, fp(b), 1, fp(c), 1, 0)     # n = 0 touches nothing


def test_sve_is_a_sequential_strided_sum(shim, oracle_backend):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((37, 11)).astype(np.float32)
    out = np.float32([0.0])
    for j in (0, 3, 10):
        shim.vDSP_sve(fp(x.reshape(-1)[j:]), 11, fp(out), 37)     # column j (BackendCPU.swift:802)
        acc = np.float32(0.0)
        for v in x[:, j]:
            acc = np.float32(acc + v)
        assert out[0] == acc
    # the oracle restates the same reduction with the same (sequential) order
    from honeycrisp_amd.descriptors import DType, ReduceDims, ReduceOp
    want = oracle_backend.reduce(oracle_backend.upload(x), ReduceOp.sum, ReduceDims(1, 37, 11), DType.float32)
    want = np.frombuffer(want.onCPU().tobytes(), np.float32)
    got = np.empty(11, np.float32)
    for j in range(11):
        shim.vDSP_sve(fp(x.reshape(-1)[j:]), 11, fp(got[j:]), 37)
    assert np.array_equal(got, want)
    ones = np.ones(1000, np.float32)
    shim.vDSP_sve(fp(ones), 1, fp(out), 1000)
    assert out[0] == 1000.0
    shim.vDSP_sve(fp(ones), 1, fp(out), 0)
    assert out[0] == 0.0


MMUL_SHAPES = [(1, 1, 1), (2, 4, 3), (3, 5, 7), (64, 32, 128), (127, 65, 1000), (5, 9, 0), (300, 257, 130)]


def check_mmul(lib, oracle_backend):
    from honeycrisp_amd.descriptors import DType
    rng = np.random.default_rng(9)
    # the reference's own known answer (BackendTests.swift:684-712): [2,3] x [3,4]
    a = np.float32([[1, 2, 3], [4, 5, 6]])
    b = np.ascontiguousarray(-np.arange(1, 13, dtype=np.float32).reshape(4, 3).T)
    c = np.empty((2, 4), np.float32)
    lib.vDSP_mmul(fp(a), 1, fp(b), 1, fp(c), 1, 2, 4, 3)
    assert c.reshape(-1).tolist() == [-14, -32, -50, -68, -32, -77, -122, -167]
    for (m, n, p) in MMUL_SHAPES:
        a = rng.standard_normal((m, p)).astype(np.float32)
        b = rng.standard_normal((p, n)).astype(np.float32)
        c = np.full((m, n), np.nan, np.float32)
        lib.vDSP_mmul(fp(a), 1, fp(b), 1, fp(c), 1, m, n, p)       # (rows, cols, inner), BackendCPU.swift:1256
        want = a.astype(np.float64) @ b.astype(np.float64)
        assert np.allclose(c, want, rtol=1e-4, atol=1e-4 * max(p, 1) ** 0.5)
        if p:
            ref = oracle_backend.matmul(oracle_backend.upload(a), False, oracle_backend.upload(b), False, False, m, p, n,
                                        DType.float32)
            ref = np.frombuffer(ref.onCPU().tobytes(), np.float32).reshape(m, n)
            assert np.allclose(c, ref, rtol=1e-4, atol=1e-4 * p ** 0.5)
    eye = np.eye(33, dtype=np.float32)
    a = rng.standard_normal((20, 33)).astype(np.float32)
    c = np.empty_like(a)
    lib.vDSP_mmul(fp(a), 1, fp(eye), 1, fp(c), 1, 20, 33, 33)
    assert np.array_equal(c, a)


def test_mmul_built_in(shim_path, oracle_backend):
    lib, backend = load(shim_path, "builtin")
    assert backend == "built-in"
    lib.hc_accelerate_blas_threads.restype = ctypes.c_int
    assert lib.hc_accelerate_blas_threads() == 1
    check_mmul(lib, oracle_backend)


@pytest.mark.parametrize("which", [0, 1])
def test_mmul_and_lapack_through_a_cblas_found_at_run_time(shim_path, oracle_backend, which):
    """vDSP_mmul -> cblas_sgemm(RowMajor, NoTrans, NoTrans, M, N, P, 1, A, P, B, N, 0, C, N), and
    the LAPACK entry points forwarded, through an OpenBLAS with 32-bit and with 64-bit integers."""
    libs = bundled_openblas()
    if len(libs) <= which:
        pytest.skip("no bundled OpenBLAS number %d in this environment" % which)
    lib, backend = load(shim_path, libs[which])
    assert backend.startswith(libs[which]) and "sgemm" in backend
    check_mmul(lib, oracle_backend)
    rng = np.random.default_rng(10)
    m, n = 7, 5
    a = rng.standard_normal((m, n)).astype(np.float32)
    col = np.asfortranarray(a).reshape(-1, order="F").copy()      # column-major storage, as the reference passes it
    tau = np.zeros(min(m, n), np.float32)
    mm, nn, lda, lwork, info = c_int32(m), c_int32(n), c_int32(m), c_int32(-1), c_int32(0)
    query = np.zeros(1, np.float32)
    lib.sgeqrf_(byref(mm), byref(nn), fp(col), byref(lda), fp(tau), fp(query), byref(lwork), byref(info))
    assert info.value == 0 and query[0] >= 1
    lwork = c_int32(int(query[0]))
    work = np.zeros(lwork.value, np.float32)
    lib.sgeqrf_(byref(mm), byref(nn), fp(col), byref(lda), fp(tau), fp(work), byref(lwork), byref(info))
    assert info.value == 0
    r = np.triu(col.reshape(n, m).T)[:n]
    kk = c_int32(n)
    lib.sorgqr_(byref(mm), byref(nn), byref(kk), fp(col), byref(lda), fp(tau), fp(work), byref(lwork), byref(info))
    assert info.value == 0
    q = col.reshape(n, m).T
    assert np.allclose(q @ r, a, atol=1e-5) and np.allclose(q.T @ q, np.eye(n), atol=1e-5)
    # SVD, jobu = jobvt = "S"
    col = np.asfortranarray(a).reshape(-1, order="F").copy()
    s, u, vt = np.zeros(n, np.float32), np.zeros(m * n, np.float32), np.zeros(n * n, np.float32)
    ldu, ldvt = c_int32(m), c_int32(n)
    job = (c_char * 1)(b"S")
    lwork = c_int32(-1)
    lib.sgesvd_(job, job, byref(mm), byref(nn), fp(col), byref(lda), fp(s), fp(u), byref(ldu), fp(vt), byref(ldvt),
                fp(query), byref(lwork), byref(info))
    lwork = c_int32(int(query[0]))
    work = np.zeros(lwork.value, np.float32)
    lib.sgesvd_(job, job, byref(mm), byref(nn), fp(col), byref(lda), fp(s), fp(u), byref(ldu), fp(vt), byref(ldvt),
                fp(work), byref(lwork), byref(info))
    assert info.value == 0
    assert np.allclose((u.reshape(n, m).T * s) @ vt.reshape(n, n).T, a, atol=1e-5)
    assert np.allclose(s, np.linalg.svd(a.astype(np.float64), compute_uv=False), atol=1e-5)


def test_lapack_without_a_library_reports_an_error_code(shim_path):
    lib, _ = load(shim_path, "builtin")
    a, tau, work = np.zeros(4, np.float32), np.zeros(2, np.float32), np.zeros(8, np.float32)
    two, lwork, info = c_int32(2), c_int32(8), c_int32(0)
    lib.sgeqrf_(byref(two), byref(two), fp(a), byref(two), fp(tau), fp(work), byref(lwork), byref(info))
    assert info.value != 0


def test_mtrans(shim):
    a = np.arange(15, dtype=np.float32).reshape(5, 3)       # A is N x M = 5 x 3
    c = np.empty((3, 5), np.float32)
    shim.vDSP_mtrans(fp(a), 1, fp(c), 1, 3, 5)              # C is M x N (BackendCPU.swift:2066)
    assert np.array_equal(c, a.T)


def convert_to_half(shim, x):
    out = np.empty(x.size, np.uint16)
    src = vImage_Buffer(x.ctypes.data, 1, x.size, x.size * 4)
    dst = vImage_Buffer(out.ctypes.data, 1, x.size, x.size * 2)
    assert shim.vImageConvert_PlanarFtoPlanar16F(byref(src), byref(dst), 0) == 0
    return out


def test_half_conversion_matches_ieee_round_to_nearest_even(shim, oracle_backend):
    # every binary16 pattern widens to the float numpy gives
    halfs = np.arange(65536, dtype=np.uint16)
    wide = np.empty(65536, np.float32)
    src = vImage_Buffer(halfs.ctypes.data, 1, 65536, 65536 * 2)
    dst = vImage_Buffer(wide.ctypes.data, 1, 65536, 65536 * 4)
    assert shim.vImageConvert_Planar16FtoPlanarF(byref(src), byref(dst), 0) == 0
    want = halfs.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(bits(wide)[~nan], bits(want)[~nan]) and np.isnan(wide[nan]).all()
    # and narrows back to itself
    back = convert_to_half(shim, wide)
    assert np.array_equal(back[~nan], halfs[~nan])
    # random floats of every magnitude, plus the boundaries: ties, overflow (65504 / 65520), the
    # subnormal range, signed zeros, infinities
    rng = np.random.default_rng(11)
    x = (rng.standard_normal(400000) * np.exp(rng.uniform(-20, 12, 400000))).astype(np.float32)
    special = np.float32([0.0, -0.0, np.inf, -np.inf, 65504.0, 65519.996, 65520.0, 65536.0, 1e9, -1e9, 5.9604645e-08,
                          2.9802322e-08, 2.98023224e-08 * 1.0000001, 6.1035156e-05, 6.0975552e-05, 1.0009766, 1.00048828125,
                          1.00146484375, 2049.0, 2051.0, -2050.999])
    x = np.concatenate([x, special, halfs.view(np.float16).astype(np.float32)[~nan]])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = convert_to_half(shim, x)
    assert np.array_equal(got, want)
    assert not np.isfinite(convert_to_half(shim, np.float32([1e9])).view(np.float16)[0])   # BackendTests.swift:81-83
    assert np.isnan(convert_to_half(shim, np.float32([np.nan])).view(np.float16)[0])
    # the oracle restates the same conversion (TensorElement.swift:262-338)
    ref = np.empty(x.size, np.uint16)
    oracle_backend.lib.ref_f32_to_f16_n(x.ctypes.data, ref.ctypes.data, x.size)
    assert np.array_equal(got, ref)
    # size mismatch is an error code, not a crash
    short = vImage_Buffer(wide.ctypes.data, 1, 10, 40)
    assert shim.vImageConvert_Planar16FtoPlanarF(byref(src), byref(short), 0) != 0


def test_header_declares_what_the_source_defines():
    """Every function the header declares is defined by the source and the other way round."""
    import re
    header = open(os.path.join(SHIM_DIR, "include", "Accelerate.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(vDSP_\w+|vImageConvert_\w+|s\w+_|hc_accelerate_\w+)\s*\(", header))
    source = re.sub(r"/\*.*?\*/", "", open(os.path.join(SHIM_DIR, "accelerate_shim.c")).read(), flags=re.S)
    defined = set(re.findall(r"^(?:void|vImage_Error|const char\*|int)\s+(\w+)\s*\(", source, flags=re.M))
    assert declared == defined, (declared ^ defined)
    used_by_reference = {"vDSP_vadd", "vDSP_vmul", "vDSP_vdiv", "vDSP_vsub", "vDSP_vsadd", "vDSP_vsmul", "vDSP_svdiv",
                         "vDSP_vsmsa", "vDSP_vma", "vDSP_vam", "vDSP_sve", "vDSP_mmul", "vDSP_mtrans",
                         "vImageConvert_PlanarFtoPlanar16F", "vImageConvert_Planar16FtoPlanarF", "sgeqrf_", "sorgqr_",
                         "sgesvd_"}
    assert used_by_reference <= declared
    for name in ("vDSP_Length", "vDSP_Stride", "vImage_Buffer", "kvImageNoError", "__LAPACK_int"):
        assert name in header
