"""The C-ABI library loads without a GPU and exports every entry point declared in include/xmk.h,
include/xmk_ffi.h.

No compute entry point is called here; argument validation that returns before any device work
(null descriptors, bad dtypes) is exercised because it must hold on a host without a GPU too."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", h) for h in ("xmk.h", "xmk_ffi.h")]
LIB = os.path.join(ROOT, "intel-extension-for-openxla_amd", "libxmk.so")


def declared_entry_points():
    text = "\n".join(open(h).read() for h in HEADERS)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    # function declarations at file scope: "<type> xmk_name(" not preceded by typedef
    names = re.findall(r"^\s*(?:const\s+)?[A-Za-z_][A-Za-z0-9_]*\s*\*?\s*(xmk_[a-z0-9_]+)\s*\(", text, flags=re.M)
    return sorted(set(names))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        pytest.fail(f"{LIB} is not built; run __graft_entry__.build()")
    return ctypes.CDLL(LIB)


def test_header_declares_the_expected_surface():
    names = declared_entry_points()
    for required in ("xmk_gemm", "xmk_fmha_fwd", "xmk_int4_gemm", "xmk_int4_dequant", "xmk_fp8_gemm",
                     "xmk_fmha_decode", "xmk_gptj_decode_step", "xmk_last_error", "xmk_version",
                     "xmk_ffi_cublas_gemm", "xmk_ffi_cublas_lt_matmul", "xmk_ffi_fmha_softmax",
                     "xmk_ffi_fmha_scale_bias_softmax", "xmk_ffi_int4_gemm", "xmk_ffi_cublas_lt_matmul_f8",
                     "xmk_ffi_targets", "xmk_ffi_register_all"):
        assert required in names, names


def test_every_declared_symbol_is_exported(lib):
    missing = [n for n in declared_entry_points() if not hasattr(lib, n)]
    assert not missing, f"declared in include/*.h but not exported: {missing}"


def test_version_and_error_strings(lib):
    lib.xmk_version.restype = ctypes.c_char_p
    lib.xmk_last_error.restype = ctypes.c_char_p
    assert lib.xmk_version().decode().strip() != ""
    assert isinstance(lib.xmk_last_error().decode(), str)


def test_null_arguments_are_rejected_before_any_device_work(lib):
    lib.xmk_last_error.restype = ctypes.c_char_p
    lib.xmk_gemm.restype = ctypes.c_int
    rc = lib.xmk_gemm(None, None)
    assert rc == 3  # XMK_INVALID_ARGUMENT
    assert lib.xmk_last_error().decode() != ""
    lib.xmk_fmha_fwd.restype = ctypes.c_int
    rc = lib.xmk_fmha_fwd(None, None, None, None, None, None, ctypes.c_int32(16), ctypes.c_uint32(1),
                          ctypes.c_uint32(1), ctypes.c_uint32(64), ctypes.c_uint32(1), ctypes.c_uint32(1),
                          ctypes.c_float(1.0), ctypes.c_int32(0), None)
    assert rc == 3


def test_decode_cache_workspace_covers_every_fill_level(lib):
    """The split plan of the decode attention is not monotonic in the number of keys; the workspace a
    cache is sized with must cover every fill level (e.g. 64 units: capacity 2050 plans 13 splits,
    2048 keys plan 16)."""
    lib.xmk_fmha_decode_workspace_bytes.restype = ctypes.c_size_t
    lib.xmk_fmha_decode_cache_workspace_bytes.restype = ctypes.c_size_t
    u32 = ctypes.c_uint32
    for units, cap in ((64, 2050), (64, 1087), (64, 1025), (64, 2048), (8, 4097), (300, 777), (1, 70000)):
        have = lib.xmk_fmha_decode_cache_workspace_bytes(u32(1), u32(units), u32(256), u32(cap))
        step = max(1, cap // 3000)
        worst = max(lib.xmk_fmha_decode_workspace_bytes(u32(1), u32(units), u32(256), u32(t))
                    for t in list(range(1, cap + 1, step)) + [cap])
        assert worst <= have, (units, cap, worst, have)
        assert have <= 4 * lib.xmk_fmha_decode_workspace_bytes(u32(1), u32(units), u32(256), u32(cap)) + 64 * 258 * 4
    # the closed form is exactly the maximum over all fill levels (scanned in full here), and it does not
    # walk the fill levels: the largest capacity a uint32 holds returns at once
    for units, cap in ((64, 2050), (64, 1000), (64, 5000), (64, 9000), (8, 4097), (300, 777), (1, 3000),
                       (1024, 700), (2000, 520), (3, 33), (1, 1)):
        have = lib.xmk_fmha_decode_cache_workspace_bytes(u32(1), u32(units), u32(256), u32(cap))
        worst = max(lib.xmk_fmha_decode_workspace_bytes(u32(1), u32(units), u32(256), u32(t)) for t in range(1, cap + 1))
        assert have == worst, (units, cap, worst, have)
    big = lib.xmk_fmha_decode_cache_workspace_bytes(u32(1), u32(64), u32(256), u32(0xFFFFFFFF))
    assert big == 64 * ((0xFFFFFFFF + 511) // 512) * 258 * 4


def test_shapes_beyond_32_bit_offsets_are_rejected_before_any_launch(lib):
    """The int4 kernel addresses its weights, and the GEMM tile loaders their operand rows, with 32-bit
    byte offsets; shapes past that must come back as XMK_INVALID_ARGUMENT from the host-side checks
    (no device is touched: this runs without a GPU)."""
    import importlib
    xmk = importlib.import_module("intel-extension-for-openxla_amd")
    lib.xmk_last_error.restype = ctypes.c_char_p
    fake = ctypes.c_void_p(0x10000)  # never dereferenced on the host
    i64 = ctypes.c_int64
    # 65536 x 65536 int4 weights pack into exactly 2 GiB
    rc = lib.xmk_int4_gemm(fake, fake, fake, fake, None, fake, i64(1), i64(65536), i64(65536), i64(128), None)
    assert rc == 3 and "2 GiB" in lib.xmk_last_error().decode()
    d = xmk.GemmDesc()
    m, n, k, ld = 64, 64, 64, 1 << 22
    d.lhs = xmk.Matrix(0x10000, 0, m, k, 0, ld)
    d.rhs = xmk.Matrix(0x10000, 0, k, n, 0, n)
    d.out = xmk.Matrix(0x10000, 0, m, n, 0, n)
    d.dtype_in = d.dtype_out = xmk.BF16
    d.batch_size, d.alpha, d.beta, d.epilogue = 1, 1.0, 0.0, xmk.EPI_DEFAULT
    assert lib.xmk_gemm(ctypes.byref(d), None) == 3 and "leading_dim_stride" in lib.xmk_last_error().decode()


def test_split_k_entry_point_validates_the_unsliced_descriptor(lib):
    """xmk_gemm_ws slices K before it calls the kernel; a reduction size that differs between the operands,
    or a leading dimension shorter than the row, must be reported as by xmk_gemm, not hidden by the
    slicing."""
    import importlib
    xmk = importlib.import_module("intel-extension-for-openxla_amd")
    lib.xmk_last_error.restype = ctypes.c_char_p
    lib.xmk_gemm_workspace_bytes.restype = ctypes.c_size_t
    m, n, k = 4, 4096, 16384
    d = xmk.GemmDesc()
    d.lhs = xmk.Matrix(0x10000, 0, m, k, 0, k)
    d.rhs = xmk.Matrix(0x10000, 0, k, n, 0, n)
    d.out = xmk.Matrix(0x10000, 0, m, n, 0, n)
    d.dtype_in = d.dtype_out = xmk.BF16
    d.batch_size, d.alpha, d.beta, d.epilogue = 1, 1.0, 0.0, xmk.EPI_DEFAULT
    need = lib.xmk_gemm_workspace_bytes(ctypes.byref(d))
    assert need > 0  # this shape does split
    ws = ctypes.c_void_p(0x20000)
    d.rhs.num_rows = k // 2  # rhs reduction size differs from the lhs one
    assert lib.xmk_gemm_ws(ctypes.byref(d), ws, ctypes.c_size_t(need), None) == 3
    assert "reduction sizes differ" in lib.xmk_last_error().decode()
    d.rhs.num_rows = k
    d.lhs.leading_dim_stride = k // 2  # shorter than the row
    assert lib.xmk_gemm_ws(ctypes.byref(d), ws, ctypes.c_size_t(need), None) == 3
    assert "leading_dim_stride" in lib.xmk_last_error().decode()
