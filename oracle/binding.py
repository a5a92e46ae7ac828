"""TEST INFRASTRUCTURE -- ctypes access to oracle/liboracle.so (and oracle/_ref/libqtip_ref.so where built).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_REF = {}

f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
u64p = np.ctypeslib.ndpointer(np.uint64, flags="C_CONTIGUOUS")
i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")


def build(force=False):
    so = os.path.join(HERE, "liboracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", HERE, "-B" if force else "-s", os.path.join(HERE, "liboracle.so")])
    return so


def lib():
    global _LIB
    if _LIB is not None:
        return _LIB
    L = C.CDLL(build())
    L.qo_f32_to_fp16.restype = C.c_uint16
    L.qo_f32_to_fp16.argtypes = [C.c_float]
    L.qo_fp16_to_f32.restype = C.c_float
    L.qo_fp16_to_f32.argtypes = [C.c_uint16]
    L.qo_round_fp16.restype = C.c_float
    L.qo_round_fp16.argtypes = [C.c_float]
    L.qo_f32_to_bf16.restype = C.c_uint16
    L.qo_f32_to_bf16.argtypes = [C.c_float]
    L.qo_bf16_to_f32.restype = C.c_float
    L.qo_bf16_to_f32.argtypes = [C.c_uint16]
    L.qo_rng.argtypes = [C.c_uint64, C.c_int, C.c_long, C.c_void_p, C.c_void_p]
    L.qo_build_codebook.argtypes = [f32p, f32p, f32p, u32p, C.POINTER(C.c_double)]
    L.qo_hyb_tlut_bits.restype = C.POINTER(C.c_uint32)
    L.qo_perm256.argtypes = [i32p, i32p]
    L.qo_had_K.argtypes = [C.c_int]
    L.qo_hadamard_rows.argtypes = [f64p, C.c_long, C.c_int, C.c_long, C.c_int]
    L.qo_hadamard_rows_f32.argtypes = [f32p, C.c_long, C.c_int, C.c_long, C.c_int]
    for name in ("qo_viterbi", "qo_viterbi_fast"):
        fn = getattr(L, name)
        fn.restype = C.c_double
        fn.argtypes = [f32p, f32p, f32p, C.c_int, u16p]
    L.qo_quantize_seq.restype = C.c_double
    L.qo_quantize_seq.argtypes = [f32p, f32p, f32p, u16p, f32p]
    L.qo_quantize_tiles.argtypes = [f32p, f32p, f32p, C.c_long, u16p, C.c_void_p, C.c_int, C.c_int]
    L.qo_decode_states.argtypes = [f32p, f32p, u16p, f32p]
    L.qo_path_cost.restype = C.c_double
    L.qo_path_cost.argtypes = [f32p, f32p, f32p, u16p]
    L.qo_pack_trellis.argtypes = [u16p, C.c_long, u16p]
    L.qo_unpack_trellis.argtypes = [u16p, C.c_long, u16p]
    L.qo_swizzle_for_kernel.argtypes = [u16p, C.c_int, C.c_int, u16p]
    L.qo_unswizzle_for_kernel.argtypes = [u16p, C.c_int, C.c_int, u16p]
    L.qo_cholesky.argtypes = [f64p, C.c_int]
    L.qo_block_ldl_to_L.argtypes = [f64p, C.c_int, f32p]
    for name in ("qo_ldlq", "qo_ldlq_naive"):
        getattr(L, name).argtypes = [f32p, f32p, f32p, f32p, C.c_int, C.c_int, f32p, u16p, C.c_int]
    L.qo_rotate_hessian.argtypes = [f32p, C.c_int, C.c_uint64, C.c_double, f32p, C.POINTER(C.c_double), f32p]
    L.qo_ldl_hessian.argtypes = [f32p, C.c_int, f32p]
    L.qo_proxy.restype = C.c_double
    L.qo_proxy.argtypes = [f32p, f32p, f32p, C.c_int, C.c_int, C.c_int]
    L.qo_quantize_group.argtypes = [f32p, C.c_int, C.POINTER(C.c_void_p), i32p, C.c_int, f32p, C.c_uint64, C.c_double,
                                    C.c_double, u16p, u16p, f32p, f32p, f64p, f64p, C.c_void_p, C.c_void_p,
                                    C.c_void_p, C.c_int]
    L.qo_f32_to_fp8e4m3.restype = C.c_uint8
    L.qo_f32_to_fp8e4m3.argtypes = [C.c_float]
    L.qo_fp8e4m3_to_f32.restype = C.c_float
    L.qo_fp8e4m3_to_f32.argtypes = [C.c_uint8]
    L.qo_nvfp4_quantize.argtypes = [f32p, C.c_int, C.c_int, u8p, u8p, C.POINTER(C.c_float)]
    L.qo_nvfp4_dequantize.argtypes = [u8p, u8p, C.c_float, C.c_int, C.c_int, f32p]
    L.qo_nvfp4_proxy_error.restype = C.c_double
    L.qo_nvfp4_proxy_error.argtypes = [f32p, f32p, C.c_int, C.c_int, C.c_void_p]
    L.qo_nvfp4_prepare.argtypes = [f32p, C.c_int, C.c_double, C.c_int, C.c_void_p, f32p]
    L.qo_nvfp4_blocks.argtypes = [f32p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_float, C.c_int, C.c_int, u8p, u8p]
    _LIB = L
    return L


def ref_lib(native=False):
    """The reference's own CPU core compiled in place (None when oracle/_ref was not built)."""
    name = "libqtip_ref_native.so" if native else "libqtip_ref.so"
    if name in _REF:
        return _REF[name]
    path = os.path.join(HERE, "_ref", name)
    if not os.path.exists(path):
        _REF[name] = None
        return None
    R = C.CDLL(path)
    R.ref_codebook.argtypes = [C.c_void_p] * 5
    R.ref_override_codebook.argtypes = [f32p, f32p, u32p, C.c_double]
    R.ref_perm256.argtypes = [i32p, i32p]
    R.ref_had_K.argtypes = [C.c_int]
    R.ref_hadamard_rows.argtypes = [f64p, C.c_long, C.c_int, C.c_long, C.c_int]
    R.ref_viterbi.restype = C.c_double
    R.ref_viterbi.argtypes = [f32p, C.c_int, u16p]
    R.ref_quantize_seq.restype = C.c_double
    R.ref_quantize_seq.argtypes = [f32p, u16p, f32p]
    R.ref_decode_states.argtypes = [u16p, f32p]
    R.ref_path_cost.restype = C.c_double
    R.ref_path_cost.argtypes = [f32p, u16p]
    R.ref_pack_trellis.argtypes = [u16p, C.c_long, u16p]
    R.ref_unpack_trellis.argtypes = [u16p, C.c_long, u16p]
    R.ref_swizzle.argtypes = [u16p, C.c_int, C.c_int, u16p]
    R.ref_unswizzle.argtypes = [u16p, C.c_int, C.c_int, u16p]
    R.ref_cholesky.argtypes = [f64p, C.c_int, C.c_int]
    R.ref_block_ldl.argtypes = [f64p, C.c_int, f32p, C.c_int]
    R.ref_f32_to_fp16.restype = C.c_uint16
    R.ref_f32_to_fp16.argtypes = [C.c_float]
    R.ref_fp16_to_f32.restype = C.c_float
    R.ref_fp16_to_f32.argtypes = [C.c_uint16]
    R.ref_f32_to_bf16.restype = C.c_uint16
    R.ref_f32_to_bf16.argtypes = [C.c_float]
    R.ref_rng.argtypes = [C.c_uint64, C.c_int, C.c_long, C.c_void_p, C.c_void_p]
    if hasattr(R, "ref_nvfp4_quantize"):
        R.ref_f32_to_fp8e4m3.restype = C.c_uint
        R.ref_f32_to_fp8e4m3.argtypes = [C.c_float]
        R.ref_nvfp4_quantize.restype = C.c_float
        R.ref_nvfp4_quantize.argtypes = [f32p, C.c_int, C.c_int, u8p, u8p]
        R.ref_nvfp4_dequantize.argtypes = [u8p, u8p, C.c_float, C.c_int, C.c_int, f32p]
        R.ref_nvfp4_proxy_error.restype = C.c_double
        R.ref_nvfp4_proxy_error.argtypes = [f32p, f32p, C.c_int, C.c_int, C.c_void_p]
    _REF[name] = R
    return R


# ---------------------------------------------------------------- numpy-level helpers
def hyb_tlut():
    bits = np.ctypeslib.as_array(lib().qo_hyb_tlut_bits(), shape=(1024,)).copy()
    return bits.view(np.float32).reshape(512, 2)


def synthetic_tlut(seed=1):
    """512x2 fp32 drawn N(0,1) from the splitmix stream and rescaled to unit rms."""
    v = rng_normal(seed, 1024).astype(np.float32).reshape(512, 2)
    rms = np.sqrt(np.mean(v.astype(np.float64) ** 2))
    return (v / np.float32(rms)).astype(np.float32)


class Codebook:
    def __init__(self, tlut=None):
        self.tlut = np.ascontiguousarray(hyb_tlut() if tlut is None else tlut, dtype=np.float32).reshape(512, 2)
        self.lut0 = np.zeros(65536, np.float32)
        self.lut1 = np.zeros(65536, np.float32)
        self.lut_h2 = np.zeros(65536, np.uint32)
        rms = C.c_double()
        lib().qo_build_codebook(self.tlut.reshape(-1), self.lut0, self.lut1, self.lut_h2, C.byref(rms))
        self.lut_rms = rms.value


def rng_next(seed, n):
    out = np.zeros(n, np.uint64)
    lib().qo_rng(seed, 0, n, None, out.ctypes.data)
    return out


def rng_normal(seed, n):
    out = np.zeros(n, np.float64)
    lib().qo_rng(seed, 2, n, out.ctypes.data, None)
    return out


def rng_sign(seed, n):
    out = np.zeros(n, np.float64)
    lib().qo_rng(seed, 3, n, out.ctypes.data, None)
    return out.astype(np.float32)


def perm256():
    p = np.zeros(256, np.int32)
    q = np.zeros(256, np.int32)
    lib().qo_perm256(p, q)
    return p, q


def quantize_tiles(cb, X, threads=0, fast=True, want_hat=False):
    X = np.ascontiguousarray(X, np.float32).reshape(-1, 256)
    B = X.shape[0]
    st = np.zeros((B, 128), np.uint16)
    hat = np.zeros((B, 256), np.float32) if want_hat else None
    lib().qo_quantize_tiles(cb.lut0, cb.lut1, X.reshape(-1), B, st.reshape(-1),
                            hat.ctypes.data if want_hat else None, threads, 1 if fast else 0)
    return (st, hat) if want_hat else st


def pack_trellis(states):
    states = np.ascontiguousarray(states, np.uint16).reshape(-1, 128)
    out = np.zeros((states.shape[0], 32), np.uint16)
    lib().qo_pack_trellis(states.reshape(-1), states.shape[0], out.reshape(-1))
    return out


def unpack_trellis(packed):
    packed = np.ascontiguousarray(packed, np.uint16).reshape(-1, 32)
    out = np.zeros((packed.shape[0], 128), np.uint16)
    lib().qo_unpack_trellis(packed.reshape(-1), packed.shape[0], out.reshape(-1))
    return out


def swizzle(packed, m, n):
    packed = np.ascontiguousarray(packed, np.uint16).reshape(-1)
    out = np.zeros_like(packed)
    assert lib().qo_swizzle_for_kernel(packed, m, n, out) == 0
    return out


def unswizzle(tr, m, n):
    tr = np.ascontiguousarray(tr, np.uint16).reshape(-1)
    out = np.zeros_like(tr)
    assert lib().qo_unswizzle_for_kernel(tr, m, n, out) == 0
    return out


def block_ldl(H64):
    A = np.array(H64, np.float64, order="C", copy=True)
    n = A.shape[0]
    L = np.zeros((n, n), np.float32)
    ok = lib().qo_block_ldl_to_L(A.reshape(-1), n, L.reshape(-1))
    return L if ok else None


def ldlq(cb, Wr, L, threads=0, naive=False):
    Wr = np.ascontiguousarray(Wr, np.float32)
    L = np.ascontiguousarray(L, np.float32)
    m, n = Wr.shape
    hat = np.zeros((m, n), np.float32)
    Q = np.zeros(((m // 16) * (n // 16), 128), np.uint16)
    fn = lib().qo_ldlq_naive if naive else lib().qo_ldlq
    rc = fn(cb.lut0, cb.lut1, Wr.reshape(-1), L.reshape(-1), m, n, hat.reshape(-1), Q.reshape(-1), threads)
    assert rc == 0, rc
    return hat, Q


def quantize_group(tlut, Ws, H, seed, sigma_reg=1e-2, scale_override=0.9, threads=0, want_debug=False):
    """CPU restatement of the whole group. Returns a dict of per-group outputs."""
    Ws = [np.ascontiguousarray(w, np.float32) for w in Ws]
    H = np.ascontiguousarray(H, np.float32)
    n = H.shape[0]
    ms = np.array([w.shape[0] for w in Ws], np.int32)
    mt = int(ms.sum())
    nlin = len(Ws)
    ptrs = (C.c_void_p * nlin)(*[w.ctypes.data for w in Ws])
    trellis = np.zeros((mt // 16) * (n // 16) * 32, np.uint16)
    su_bf16 = np.zeros(n, np.uint16)
    sv = np.zeros(mt, np.float32)
    wscale = np.zeros(nlin, np.float32)
    proxy = np.zeros(nlin, np.float64)
    prr = np.zeros(nlin, np.float64)
    Q = np.zeros(((mt // 16) * (n // 16), 128), np.uint16) if want_debug else None
    WT = np.zeros((n, mt), np.float32) if want_debug else None
    hT = np.zeros((n, mt), np.float32) if want_debug else None
    rc = lib().qo_quantize_group(np.ascontiguousarray(tlut, np.float32).reshape(-1), nlin, ptrs, ms, n, H.reshape(-1),
                                 seed, sigma_reg, scale_override, trellis, su_bf16, sv, wscale, proxy, prr,
                                 Q.ctypes.data if want_debug else None, WT.ctypes.data if want_debug else None,
                                 hT.ctypes.data if want_debug else None, threads)
    assert rc == 0, rc
    return dict(trellis=trellis, su_bf16=su_bf16, sv=sv, wscale=wscale, proxy=proxy, proxy_rot_reg=prr, Q=Q, WT=WT,
                hatWT=hT, m=ms, n=n)


# ---------------------------------------------------------------- NVFP4 fallback quantizer
def nvfp4_quantize(w):
    """nvfp4_quantize, src/nvfp4.cpp:12-55 -> (packed [m][n/2], scales [m][n/16], global)."""
    w = np.ascontiguousarray(w, np.float32)
    m, n = w.shape
    packed = np.zeros((m, n // 2), np.uint8)
    scales = np.zeros((m, n // 16), np.uint8)
    g = C.c_float()
    assert lib().qo_nvfp4_quantize(w.reshape(-1), m, n, packed.reshape(-1), scales.reshape(-1), C.byref(g)) == 0
    return packed, scales, g.value


def nvfp4_dequantize(packed, scales, g, m, n):
    out = np.zeros((m, n), np.float32)
    lib().qo_nvfp4_dequantize(np.ascontiguousarray(packed).reshape(-1), np.ascontiguousarray(scales).reshape(-1), g, m, n,
                              out.reshape(-1))
    return out


def nvfp4_proxy_error(w, what, H=None):
    m, n = w.shape
    Hp = None if H is None else np.ascontiguousarray(H, np.float32).ctypes.data
    return lib().qo_nvfp4_proxy_error(np.ascontiguousarray(w, np.float32).reshape(-1),
                                      np.ascontiguousarray(what, np.float32).reshape(-1), m, n, Hp)


def nvfp4_prepare(H, sigma_reg=1e-2, calibrate=True):
    """src/nvfp4_gpu.hip:181-207 -> (L or None, dw); None when H is not positive definite."""
    H = np.ascontiguousarray(H, np.float32)
    n = H.shape[0]
    L = np.zeros((n, n), np.float32) if calibrate else None
    dw = np.zeros(n, np.float32)
    rc = lib().qo_nvfp4_prepare(H.reshape(-1), n, sigma_reg, 1 if calibrate else 0, None if L is None else L.ctypes.data, dw)
    return None if rc else (L, dw)


def nvfp4_blocks(w, L, dw, g, calibrate, search):
    """The block loop of nvfp4_quantize_group (src/nvfp4_gpu.hip:217-228) -> (packed, scales)."""
    w = np.ascontiguousarray(w, np.float32)
    m, n = w.shape
    packed = np.zeros((m, n // 2), np.uint8)
    scales = np.zeros((m, n // 16), np.uint8)
    lib().qo_nvfp4_blocks(w.reshape(-1), m, n, None if L is None else L.ctypes.data, None if dw is None else dw.ctypes.data,
                          g, 1 if calibrate else 0, 1 if search else 0, packed.reshape(-1), scales.reshape(-1))
    return packed, scales
