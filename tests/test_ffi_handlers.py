"""XLA-FFI handlers against a fake host, without a GPU: registration, metadata queries, stage
filtering and every decoding error that is raised before any device work."""
import ctypes as C
import os

import pytest

import ffi_util as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "intel-extension-for-openxla_amd", "libxmk.so")

TARGETS = {
    "__cublas$gemm": "xmk_ffi_cublas_gemm",
    "__cublas$lt$matmul": "xmk_ffi_cublas_lt_matmul",
    "__cudnn$fmhaSoftmax": "xmk_ffi_fmha_softmax",
    "__cudnn$fmhaScaleBiasSoftmax": "xmk_ffi_fmha_scale_bias_softmax",
    "__cudnn$fmhaSoftmaxBackward": "xmk_ffi_fmha_softmax_backward",
    "__cudnn$fmhaScaleBiasSoftmaxBackward": "xmk_ffi_fmha_scale_bias_softmax_backward",
    "__xmk$int4_gemm": "xmk_ffi_int4_gemm",
    "__cublas$lt$matmul$f8": "xmk_ffi_cublas_lt_matmul_f8",
}


@pytest.fixture(scope="module")
def lib():
    l = C.CDLL(LIB)
    for name in TARGETS.values():
        getattr(l, name).restype = C.c_void_p
        getattr(l, name).argtypes = [C.POINTER(F.CallFrame)]
    return l


def test_target_table_and_registration(lib):
    class Target(C.Structure):
        _fields_ = [("target", C.c_char_p), ("handler", C.c_void_p)]
    lib.xmk_ffi_targets.restype = C.POINTER(Target)
    n = C.c_int32(0)
    table = lib.xmk_ffi_targets(C.byref(n))
    got = {table[i].target.decode(): table[i].handler for i in range(n.value)}
    assert set(got) == set(TARGETS)
    for target, sym in TARGETS.items():
        assert got[target] == C.cast(getattr(lib, sym), C.c_void_p).value
    host = F.FakeHost()
    lib.xmk_ffi_register_all.restype = C.c_void_p
    assert lib.xmk_ffi_register_all(C.byref(host.api), b"ROCM") is None
    assert {(name, plat) for name, plat, _ in host.registered} == {(t, "ROCM") for t in TARGETS}
    assert all(ptr == got[name] for name, _, ptr in host.registered)


@pytest.mark.parametrize("sym", sorted(TARGETS.values()))
def test_metadata_query_and_other_stages_do_nothing(lib, sym):
    host = F.FakeHost()
    f = host.frame([], [], {})
    md = F.Metadata(C.sizeof(F.Metadata), F.ApiVersion(C.sizeof(F.ApiVersion), None, -1, -1), 99)
    ext = F.MetadataExtension()
    ext.extension_base.struct_size = C.sizeof(F.MetadataExtension)
    ext.extension_base.type = 1
    ext.metadata = C.pointer(md)
    f.extension_start = C.cast(C.pointer(ext), C.POINTER(F.ExtBase))
    assert getattr(lib, sym)(C.byref(f)) is None
    assert (md.api_version.major_version, md.api_version.minor_version, md.traits) == (0, 1, 0)
    for stage in (0, 1, 2):  # instantiate / prepare / initialize: nothing to do, no error
        assert getattr(lib, sym)(C.byref(host.frame([], [], {}, stage=stage))) is None
    assert host.errors == []


def test_gemm_missing_operands_and_attributes(lib):
    host = F.FakeHost()
    attrs = F.gemm_attrs(8, 8, 8, F.BF16, F.BF16, epilogue=0)
    assert lib.xmk_ffi_cublas_lt_matmul(C.byref(host.frame([], [], attrs))) is not None
    assert host.errors[-1][0] == 3 and "operand 0" in host.errors[-1][1]
    bad = dict(attrs)
    del bad["lhs_num_rows"]
    buf = (F.BF16, 0x1000, [8, 8])
    assert lib.xmk_ffi_cublas_lt_matmul(C.byref(host.frame([buf, buf], [buf], bad))) is not None
    assert host.errors[-1][0] == 3 and "lhs_num_rows" in host.errors[-1][1]
    # unknown epilogue value -> Internal("Unsupported Epilogue."), as AsSYCLEpilogue
    attrs["epilogue"] = (F.S32, 42)
    assert lib.xmk_ffi_cublas_lt_matmul(C.byref(host.frame([buf, buf], [buf], attrs))) is not None
    assert host.errors[-1] == (13, "Unsupported Epilogue.")
    # a vector-bias epilogue needs operand 2
    attrs["epilogue"] = (F.S32, 1)
    assert lib.xmk_ffi_cublas_lt_matmul(C.byref(host.frame([buf, buf], [buf], attrs))) is not None
    assert "operand 2" in host.errors[-1][1]
    # auxiliary-output epilogues are rejected by the entry point like the reference does
    attrs["epilogue"] = (F.S32, 5)
    assert lib.xmk_ffi_cublas_lt_matmul(C.byref(host.frame([buf, buf], [buf, buf], attrs))) is not None
    assert host.errors[-1][0] == 12


def test_gemm_entry_point_errors_come_back_as_ffi_errors(lib):
    host = F.FakeHost()
    buf = (F.BF16, 0x1000, [8, 8])
    attrs = F.gemm_attrs(8, 8, 8, F.S32, F.BF16)  # unsupported dtype triple
    assert lib.xmk_ffi_cublas_gemm(C.byref(host.frame([buf, buf], [buf], attrs))) is not None
    code, msg = host.errors[-1]
    assert code in (3, 12, 13) and msg


def test_fmha_decoding_errors(lib):
    host = F.FakeHost()
    q = (F.BF16, 0x1000, [2, 4, 16, 64])
    kv = (F.BF16, 0x2000, [2, 4, 32, 64])
    out = (F.BF16, 0x3000, [2, 4, 16, 64])
    scratch = (6, 0x4000, [0])
    f = host.frame([q, kv, kv], [out, scratch], {"dropout_rate": (F.F64, 0.1)})
    assert lib.xmk_ffi_fmha_softmax(C.byref(f)) is not None
    assert host.errors[-1] == (12, "Unimplemented dropout")
    bad_kv = (F.BF16, 0x2000, [2, 4, 32, 32])
    assert lib.xmk_ffi_fmha_softmax(C.byref(host.frame([q, bad_kv, kv], [out, scratch], {}))) is not None
    assert "shapes" in host.errors[-1][1]
    assert lib.xmk_ffi_fmha_scale_bias_softmax(C.byref(host.frame([q, kv, kv], [out, scratch], {}))) is not None
    assert "operand 3" in host.errors[-1][1]
    f32q = (F.F32, 0x1000, [2, 4, 16, 64])
    f32kv = (F.F32, 0x2000, [2, 4, 32, 64])
    assert lib.xmk_ffi_fmha_softmax(C.byref(host.frame([f32q, f32kv, f32kv], [(F.F32, 0x3000, [2, 4, 16, 64]), scratch], {}))) is not None
    assert host.errors[-1] == (13, "Invalid MHA datatype")


def test_int4_and_f8_decoding_errors(lib):
    host = F.FakeHost()
    act = (F.F16, 0x1000, [4, 256])
    qw = (F.S32, 0x2000, [32, 64])
    sz = (F.F16, 0x3000, [2, 64])
    out = (F.F16, 0x4000, [4, 64])
    assert lib.xmk_ffi_int4_gemm(C.byref(host.frame([act, qw, sz, (F.F16, 0x3000, [4, 64])], [out], {}))) is not None
    assert "shapes" in host.errors[-1][1]
    assert lib.xmk_ffi_int4_gemm(C.byref(host.frame([act, (F.F32, 0x2000, [32, 64]), sz, sz], [out], {}))) is not None
    assert "qweight" in host.errors[-1][1]
    a = (F.F8E4M3FN, 0x1000, [64, 128])
    b = (F.F8E4M3FN, 0x2000, [64, 128])
    s = (F.F32, 0x3000, [])
    o = (F.BF16, 0x4000, [64, 64])
    attrs = F.gemm_attrs(64, 64, 128, F.F8E4M3FN, F.BF16, rhs_col_major=True, beta=1.0)
    assert lib.xmk_ffi_cublas_lt_matmul_f8(C.byref(host.frame([a, b, s, s], [o], attrs))) is not None
    assert host.errors[-1][0] == 12 and "beta" in host.errors[-1][1]
    attrs = F.gemm_attrs(64, 64, 128, F.F8E4M3FN, F.BF16, rhs_col_major=True)
    assert lib.xmk_ffi_cublas_lt_matmul_f8(C.byref(host.frame([a, b, s, s], [(F.F16, 0x4000, [64, 64])], attrs))) is not None
    assert "bf16" in host.errors[-1][1]
    # every operand is used or refused: a fifth operand alone fits neither (.., c_scale, d_scale) nor a bias
    # (the epilogue is DEFAULT); a bias operand needs epilogue BIAS and the other way round; GELU is not taken
    attrs = F.gemm_attrs(64, 64, 128, F.F8E4M3FN, F.BF16, rhs_col_major=True)
    assert lib.xmk_ffi_cublas_lt_matmul_f8(C.byref(host.frame([a, b, s, s, s], [o], attrs))) is not None
    assert host.errors[-1][0] == 3 and "operands do not fit" in host.errors[-1][1]
    bias = (F.BF16, 0x5000, [64])
    assert lib.xmk_ffi_cublas_lt_matmul_f8(C.byref(host.frame([a, b, s, s, s, s, bias], [o], attrs))) is not None
    assert host.errors[-1][0] == 3 and "operands do not fit" in host.errors[-1][1]
    attrs = F.gemm_attrs(64, 64, 128, F.F8E4M3FN, F.BF16, rhs_col_major=True, epilogue=1)
    assert lib.xmk_ffi_cublas_lt_matmul_f8(C.byref(host.frame([a, b, s, s, s, s], [o], attrs))) is not None
    assert host.errors[-1][0] == 3 and "operands do not fit" in host.errors[-1][1]
    assert lib.xmk_ffi_cublas_lt_matmul_f8(
        C.byref(host.frame([a, b, s, s, s, s, (F.F16, 0x5000, [64])], [o], attrs))) is not None
    assert "bias must be bf16" in host.errors[-1][1]
    assert lib.xmk_ffi_cublas_lt_matmul_f8(
        C.byref(host.frame([a, b, s, s, (F.F32, 0x6000, [2]), s, bias], [o], attrs))) is not None
    assert "f32 scalars" in host.errors[-1][1]
    attrs = F.gemm_attrs(64, 64, 128, F.F8E4M3FN, F.BF16, rhs_col_major=True, epilogue=4)
    assert lib.xmk_ffi_cublas_lt_matmul_f8(C.byref(host.frame([a, b, s, s], [o], attrs))) is not None
    assert host.errors[-1][0] == 12 and "epilogue" in host.errors[-1][1]
