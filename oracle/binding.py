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
    src = [os.path.join(HERE, f) for f in ("qtip_oracle.c", "qtip_oracle.h")]
    if force or not os.path.exists(so) or os.path.getmtime(so) < max(os.path.getmtime(f) for f in src):
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


def ref_gpu_lib():
    """The reference's own device path compiled for gfx950 (None when oracle/_ref was not built).  Its ref_gpu_*
    functions need a GPU, ref_ldlq does not; in a process that imports torch, import torch first (one HIP runtime per
    process)."""
    name = "libqtip_ref_gpu.so"
    if name in _REF:
        return _REF[name]
    path = os.path.join(HERE, "_ref", name)
    _REF[name] = C.CDLL(path) if os.path.exists(path) else None
    return _REF[name]


def ref_gpu_nvfp4_quantize_group(ws, n, H=None, scale_search=True, calibrate=True, sigma_reg=1e-2):
    """nvfp4_quantize_group of the reference itself (src/nvfp4_gpu.hip:174-243) -> ([(packed, scales, global)], used)."""
    R = ref_gpu_lib()
    ws = [np.ascontiguousarray(w, np.float32) for w in ws]
    k = len(ws)
    pk = [np.zeros((w.shape[0], n // 2), np.uint8) for w in ws]
    sc = [np.zeros((w.shape[0], n // 16), np.uint8) for w in ws]
    g = np.zeros(k, np.float32)
    wp = (C.c_void_p * k)(*[w.ctypes.data for w in ws])
    pp = (C.c_void_p * k)(*[a.ctypes.data for a in pk])
    sp = (C.c_void_p * k)(*[a.ctypes.data for a in sc])
    ms = (C.c_int * k)(*[w.shape[0] for w in ws])
    Hc = None if H is None else np.ascontiguousarray(H, np.float32)
    R.ref_gpu_nvfp4_quantize_group.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int,
                                               C.c_double, C.c_void_p, C.c_void_p, C.c_void_p]
    used = R.ref_gpu_nvfp4_quantize_group(k, wp, ms, n, None if Hc is None else Hc.ctypes.data, int(scale_search),
                                          int(calibrate), sigma_reg, pp, sp, g.ctypes.data)
    return [(pk[i], sc[i], float(g[i])) for i in range(k)], bool(used)


def ref_ldlq(Wr, L):
    """ldlq_ref of the reference's GPU test (tests/test_gpu.cpp:180-225; CPU code) -> (hatWr, Q)."""
    R = ref_gpu_lib()
    Wr = np.ascontiguousarray(Wr, np.float32)
    L = np.ascontiguousarray(L, np.float32)
    m, n = Wr.shape
    hat = np.zeros((m, n), np.float32)
    Q = np.zeros(((m // 16) * (n // 16), 128), np.uint16)
    R.ref_ldlq.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    R.ref_ldlq.restype = None
    R.ref_ldlq(Wr.ctypes.data, L.ctypes.data, m, n, hat.ctypes.data, Q.ctypes.data)
    return hat, Q


def ref_gpu_hadamard_rows(X, n, transpose):
    """k_hadamard_rows of the reference on the GPU (src/kernels.hip:293-313); X is rows x ld, returned transformed."""
    R = ref_gpu_lib()
    X = np.ascontiguousarray(X, np.float32).copy()
    rows, ld = X.shape
    R.ref_gpu_hadamard_rows.argtypes = [C.c_void_p, C.c_long, C.c_int, C.c_long, C.c_int]
    R.ref_gpu_hadamard_rows.restype = None
    R.ref_gpu_hadamard_rows(X.ctypes.data, rows, n, ld, int(transpose))
    return X


def ref_gpu_quantize_seqs(X):
    """The reference's device Viterbi, both passes (tests/test_gpu.cpp:67-88) -> (states [B][128], seconds)."""
    R = ref_gpu_lib()
    X = np.ascontiguousarray(X, np.float32).reshape(-1, 256)
    st = np.zeros((X.shape[0], 128), np.uint16)
    R.ref_gpu_quantize_seqs.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
    R.ref_gpu_quantize_seqs.restype = C.c_double
    secs = R.ref_gpu_quantize_seqs(X.ctypes.data, X.shape[0], st.ctypes.data)
    return st, secs


def ref_gpu_quantize_group(Ws, H, seed, sigma_reg=1e-2, scale_override=0.9, ldl_threads=16, want_hatW=False):
    """quantize_group of the reference itself on the GPU (src/quantizer.cpp:340-348): same keys as quantize_group
    below, per linear, plus its GroupTiming."""
    R = ref_gpu_lib()
    Ws = [np.ascontiguousarray(w, np.float32) for w in Ws]
    H = np.ascontiguousarray(H, np.float32)
    n = H.shape[0]
    k = len(Ws)
    ms = [w.shape[0] for w in Ws]
    tr = [np.zeros((m // 16) * (n // 16) * 32, np.uint16) for m in ms]
    su = [np.zeros(n, np.uint16) for _ in ms]
    sv = [np.zeros(m, np.float32) for m in ms]
    hw = [np.zeros((m, n), np.float32) for m in ms] if want_hatW else None
    wscale = np.zeros(k, np.float32)
    proxy = np.zeros(k)
    prr = np.zeros(k)
    tm = np.zeros(8)

    def arr(xs):
        return (C.c_void_p * k)(*[x.ctypes.data for x in xs])

    R.ref_gpu_quantize_group.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_uint64, C.c_double,
                                         C.c_double, C.c_int] + [C.c_void_p] * 8
    R.ref_gpu_quantize_group.restype = None
    R.ref_gpu_quantize_group(k, arr(Ws), (C.c_int * k)(*ms), n, H.ctypes.data, seed, sigma_reg, scale_override, ldl_threads,
                             arr(tr), arr(su), arr(sv), arr(hw) if want_hatW else None, wscale.ctypes.data,
                             proxy.ctypes.data, prr.ctypes.data, tm.ctypes.data)
    names = ("load", "rht", "ldl_cpu", "ldlq", "viterbi", "proxy", "pack", "total")
    return dict(trellis=tr, su_bf16=su, sv=sv, hatW=hw, wscale=wscale, proxy=proxy, proxy_rot_reg=prr,
                timing=dict(zip(names, tm)))


def ref_nvfp4_prepare(H, sigma_reg=1e-2):
    """L (unit lower, fp32) and dw = D of the regularised Hessian as the reference's host code makes them
    (src/nvfp4_gpu.hip:181-199), with the reference's own compiled cholesky_inplace."""
    R = ref_lib()
    H = np.ascontiguousarray(H, np.float32)
    n = H.shape[0]
    dsum = 0.0
    for i in range(n):
        dsum += float(H[i, i])
    creg = sigma_reg * dsum / n
    A = 0.5 * (H.astype(np.float64) + H.T.astype(np.float64))
    A[np.arange(n), np.arange(n)] += creg
    A = np.ascontiguousarray(np.tril(A))
    if R.ref_cholesky(A.reshape(-1), n, 16) != 1:
        raise ValueError("not positive definite")
    d = np.diag(A).copy()
    return np.tril(A / d[None, :], -1).astype(np.float32), (d * d).astype(np.float32)


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
