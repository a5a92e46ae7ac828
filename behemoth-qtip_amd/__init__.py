"""Python host side of the MI355X QTIP group quantizer.

A thin ctypes binding of libqtip_mi355.so (C ABI: include/qtip_mi355.h) plus a mirror of the reference's
operator interface for this path (src/quantizer.hpp:11-78 of the reference: QuantOpts, LinearIn, LinearOut,
GroupTiming, HessPrep, rotate_hessian, ldl_hessian, quantize_group, ldlq_gpu).  There is no CPU fallback:
importing works everywhere, but every compute call needs the HIP library and a gfx950 device and raises
otherwise.
"""
import ctypes as C
import os
import subprocess
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(CSRC, "libqtip_mi355.so")

QTIP_OK, QTIP_E_ARG, QTIP_E_HIP, QTIP_E_NOT_PD, QTIP_E_NOMEM = 0, -1, -2, -3, -4


NOALLOC_MAX_TILES = 4096  # QTIP_NOALLOC_MAX_TILES


class QtipError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("qtip error %d: %s" % (code, msg))
        self.code = code


def build(jobs=8):
    """Compile the HIP extension for gfx950 in-tree (hipcc cross-compiles without a GPU)."""
    subprocess.check_call(["make", "-C", CSRC, "-B", "-j%d" % jobs])
    return LIB_PATH


def _stream_handle(stream):
    if stream is None:
        import sys
        torch = sys.modules.get("torch")
        if torch is None or not torch.cuda.is_available():
            return None
        stream = torch.cuda.current_stream()
    h = getattr(stream, "cuda_stream", stream)
    return C.c_void_p(int(h)) if h else None


class _LinearInC(C.Structure):
    _fields_ = [("m", C.c_int), ("w_f32", C.c_void_p), ("w_bf16", C.c_void_p), ("w_fp8", C.c_void_p),
                ("scale_bf16", C.c_void_p), ("on_device", C.c_int)]


class _LinearOutC(C.Structure):
    _fields_ = [("trellis", C.c_void_p), ("su_bf16", C.c_void_p), ("sv", C.c_void_p), ("hatW", C.c_void_p),
                ("wscale", C.c_float), ("proxy", C.c_double), ("proxy_rot_reg", C.c_double), ("seconds", C.c_double)]


class _OptsC(C.Structure):
    _fields_ = [("sigma_reg", C.c_double), ("scale_override", C.c_double), ("ldl_threads", C.c_int),
                ("feedback", C.c_int), ("skip_proxy", C.c_int), ("ldl_device_updates", C.c_int),
                ("ldlq_chains", C.c_int), ("group_lanes", C.c_int)]


class _TimingC(C.Structure):
    _fields_ = [(k, C.c_double) for k in ("load", "rht", "ldl_cpu", "ldlq", "viterbi", "proxy", "pack", "total")]


_lib = None


def lib():
    """The loaded C-ABI library.  Raises if it has not been built: there is no other implementation."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise QtipError(QTIP_E_HIP, "%s is missing: build it with __graft_entry__.build() or make -C %s"
                        % (LIB_PATH, CSRC))
    # A process must hold ONE HIP runtime.  PyTorch-ROCm ships its own libamdhip64 and asks for it by the
    # unversioned name, so if this library (linked against libamdhip64.so.7) were loaded first, torch would
    # bring in a second runtime that finds no GPU.  Loaded after torch, the soname resolves to torch's copy.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    L = C.CDLL(LIB_PATH)
    vp, i, l, d, u64 = C.c_void_p, C.c_int, C.c_long, C.c_double, C.c_uint64
    L.qtip_last_error.restype = C.c_char_p
    L.qtip_create.argtypes = [i, C.POINTER(vp)]
    L.qtip_destroy.argtypes = [vp]
    L.qtip_destroy.restype = None
    L.qtip_stream.argtypes = [vp]
    L.qtip_stream.restype = vp
    L.qtip_synchronize.argtypes = [vp]
    L.qtip_set_tlut.argtypes = [vp, vp]
    L.qtip_lut_rms.argtypes = [vp]
    L.qtip_lut_rms.restype = d
    L.qtip_get_lut.argtypes = [vp, vp, vp]
    L.qtip_viterbi_tiles.argtypes = [vp, vp, l, vp, vp]
    L.qtip_viterbi_tiles_dev.argtypes = [vp, vp, l, vp, vp]
    L.qtip_viterbi_tiles_dev_noalloc.argtypes = [vp, vp, l, vp, vp]
    L.qtip_trim.argtypes = [vp, C.POINTER(C.c_ulonglong)]
    L.qtip_selftest_device_alloc_calls.restype = l
    L.qtip_set_viterbi_mode.argtypes = [vp, i, C.c_uint]
    L.qtip_viterbi_stats.argtypes = [vp, C.POINTER(C.c_ulonglong), C.POINTER(C.c_ulonglong), i]
    L.qtip_ldlq_default_chains.argtypes = [vp, C.POINTER(C.c_int)]
    L.qtip_stream_wait.argtypes = [vp, vp]
    L.qtip_stream_signal.argtypes = [vp, vp]
    L.qtip_device_lut.argtypes = [vp, C.POINTER(vp)]
    L.qtip_decode_states_dev.argtypes = [vp, vp, l, vp]
    L.qtip_hadamard_rows_dev.argtypes = [vp, vp, l, i, l, i]
    L.qtip_decode_trellis_dev.argtypes = [vp, vp, i, i, vp]
    L.qtip_dequantize_linear.argtypes = [vp, vp, vp, vp, C.c_float, i, i, vp, i]
    L.qtip_had_K.argtypes = [i]
    L.qtip_sign_vector.argtypes = [u64, l, vp]
    L.qtip_sign_vector.restype = None
    L.qtip_rotate_hessian.argtypes = [vp, vp, i, i, u64, d, vp, C.POINTER(d), vp]
    L.qtip_ldl_hessian.argtypes = [vp, i, i, vp]
    L.qtip_ldl_hessian_device_updates.argtypes = [vp, vp, i, i, vp]
    L.qtip_selftest_ldl_panel_handover.argtypes = [vp, i, i, vp]
    L.qtip_ldl_hessian_device_updates_dev.argtypes = [vp, vp, i, i, vp, vp]
    L.qtip_ldlq_dev.argtypes = [vp, vp, vp, l, l, vp, vp, i, C.POINTER(d)]
    L.qtip_prod_cache_bf16x3_dev.argtypes = [vp, i, l, vp, l, vp, vp, l, vp]
    L.qtip_default_opts.argtypes = [C.POINTER(_OptsC)]
    L.qtip_default_opts.restype = None
    L.qtip_quantize_group.argtypes = [vp, i, C.POINTER(_LinearInC), i, u64, vp, d, vp, vp, C.POINTER(_OptsC),
                                      C.POINTER(_LinearOutC), C.POINTER(_TimingC)]
    L.qtip_quantize_group_h.argtypes = [vp, i, C.POINTER(_LinearInC), i, vp, i, u64, C.POINTER(_OptsC),
                                        C.POINTER(_LinearOutC), C.POINTER(_TimingC)]
    L.qtip_hessian_accumulate_dev.argtypes = [vp, vp, l, i, vp]
    L.qtip_hessian_finish_dev.argtypes = [vp, vp, i, d]
    L.qtip_f32_to_fp8e4m3.restype = C.c_uint8
    L.qtip_f32_to_fp8e4m3.argtypes = [C.c_float]
    L.qtip_nvfp4_quantize.argtypes = [vp, i, i, vp, vp, C.POINTER(C.c_float)]
    L.qtip_nvfp4_dequantize.argtypes = [vp, vp, C.c_float, i, i, vp]
    L.qtip_nvfp4_proxy_error.argtypes = [vp, vp, i, i, vp, C.POINTER(d)]
    L.qtip_nvfp4_prepare.argtypes = [vp, i, d, i, i, vp, vp]
    L.qtip_nvfp4_prepare_device_updates.argtypes = [vp, vp, i, d, i, vp, vp]
    L.qtip_nvfp4_quantize_prepared.argtypes = [vp, i, vp, i, vp, vp, i]
    L.qtip_nvfp4_quantize_group.argtypes = [vp, i, vp, i, vp, C.POINTER(_Nvfp4OptsC), C.POINTER(i)]
    L.qtip_run_groups.argtypes = [vp, i, vp, C.POINTER(_OptsC), vp, vp]
    L.qtip_reserve_groups.argtypes = [vp, i]
    L.qtip_group_lanes.argtypes = [vp, i, vp, C.POINTER(_OptsC), C.POINTER(C.c_int)]
    L.qtip_selftest_group_lanes.argtypes = [i, i, i, i, i, C.POINTER(C.c_int)]
    L.qtip_st_create.argtypes = [C.POINTER(vp)]
    L.qtip_st_destroy.argtypes = [vp]
    L.qtip_st_destroy.restype = None
    L.qtip_st_add.argtypes = [vp, C.c_char_p, C.c_char_p, vp, i, vp, u64]
    L.qtip_st_add_qtip_linear.argtypes = [vp, C.c_char_p, vp, i, i, vp]
    L.qtip_st_write.argtypes = [vp, C.c_char_p, vp, i, C.POINTER(u64)]
    L.qtip_get_tlut_f16.argtypes = [vp, vp]
    L.qtip_pack_trellis.argtypes = [vp, l, vp]
    L.qtip_pack_trellis.restype = None
    L.qtip_unpack_trellis.argtypes = [vp, l, vp]
    L.qtip_unpack_trellis.restype = None
    L.qtip_swizzle_for_kernel.argtypes = [vp, i, i, vp]
    L.qtip_unswizzle_for_kernel.argtypes = [vp, i, i, vp]
    _lib = L
    return L


class _GroupC(C.Structure):
    _fields_ = [("nlin", C.c_int), ("lins", C.c_void_p), ("outs", C.c_void_p), ("n", C.c_int), ("H", C.c_void_p),
                ("h_on_device", C.c_int), ("seed", C.c_uint64)]


class _Nvfp4MatrixC(C.Structure):
    _fields_ = [("m", C.c_int), ("w", C.c_void_p), ("packed", C.c_void_p), ("scales", C.c_void_p), ("global_", C.c_float)]


class _Nvfp4OptsC(C.Structure):
    _fields_ = [("scale_search", C.c_int), ("calibrate", C.c_int), ("sigma_reg", C.c_double),
                ("factor_on_host", C.c_int)]


def _check(rc):
    if rc != 0:
        raise QtipError(rc, lib().qtip_last_error().decode("utf-8", "replace"))


def _ptr(a):
    """Address of a numpy array, a torch tensor (host or device) or a raw integer address."""
    if a is None:
        return None
    if isinstance(a, int):
        return a
    if isinstance(a, np.ndarray):
        assert a.flags["C_CONTIGUOUS"]
        return a.ctypes.data
    if hasattr(a, "data_ptr"):
        assert a.is_contiguous()
        if a.is_cuda:
            # the library works on a stream of its own: whatever torch has queued for this tensor (its fill, the
            # kernel that produced it) must have finished before the library touches it
            import torch
            torch.cuda.current_stream(a.device).synchronize()
        return a.data_ptr()
    raise TypeError(type(a))


# ---------------------------------------------------------------- mirror of src/quantizer.hpp
@dataclass
class QuantOpts:  # src/quantizer.hpp:11-19
    sigma_reg: float = 1e-2
    scale_override: float = 0.9
    vit_batch: int = 1024      # accepted for source compatibility; the tile kernel sizes its own workspace
    ldl_threads: int = 16
    share_su: bool = True      # False is refused, as in the reference (src/quantizer.cpp:209-211)
    want_hatW: bool = False
    feedback: int = 0          # 0: fp64 feedback (default), 1: fp32 feedback + bf16 hi/lo split MFMA
    skip_proxy: bool = False
    ldl_device_updates: bool = True    # the LDL's trailing updates run on the GPU (same L bit for bit); False: host alone
    ldlq_chains: int = 0       # independent chains of launches the tile rows are dealt to (0: the library's default: 3 where its side streams have hardware queues of their own, else 2: ldlq_default_chains())
    group_lanes: int = 0       # run_groups: groups run side by side on this many lanes (0: as many as fit the chip, 1 for large groups; 1: one after the other)


@dataclass
class LinearIn:  # src/quantizer.hpp:21-28; exactly one weight representation is set
    name: str
    m: int
    w_f32: Optional[object] = None
    w_bf16: Optional[object] = None
    w_fp8: Optional[object] = None
    scale_bf16: Optional[object] = None


@dataclass
class LinearOut:  # src/quantizer.hpp:30-43
    name: str = ""
    m: int = 0
    n: int = 0
    trellis: Optional[np.ndarray] = None
    su_bf16: Optional[np.ndarray] = None
    sv: Optional[np.ndarray] = None
    wscale: float = 0.0
    proxy: float = 0.0
    proxy_rot_reg: float = 0.0
    seconds: float = 0.0
    hatW: Optional[np.ndarray] = None


@dataclass
class GroupTiming:  # src/quantizer.hpp:45-47
    load: float = 0.0
    rht: float = 0.0
    ldl_cpu: float = 0.0
    ldlq: float = 0.0
    viterbi: float = 0.0
    proxy: float = 0.0
    pack: float = 0.0
    total: float = 0.0


@dataclass
class HessPrep:  # src/quantizer.hpp:51-59
    n: int = 0
    seed: int = 0
    su: Optional[np.ndarray] = None
    creg: float = 0.0
    HRr: Optional[np.ndarray] = None
    L: Optional[np.ndarray] = None
    t_rot: float = 0.0
    t_ldl: float = 0.0


def _is_device(a):
    return hasattr(a, "is_cuda") and a.is_cuda


class Quantizer:
    """One context: device, private stream, codebook (the reference's per-worker state)."""

    def __init__(self, device=0, tlut=None):
        self._h = C.c_void_p()
        _check(lib().qtip_create(device, C.byref(self._h)))
        if tlut is not None:
            self.set_tlut(tlut)

    def close(self):
        if self._h:
            lib().qtip_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def stream(self):
        return lib().qtip_stream(self._h)

    def synchronize(self):
        _check(lib().qtip_synchronize(self._h))

    def stream_wait(self, stream=None):
        """The context's stream waits for everything queued so far on `stream` (a hipStream_t as an integer, a
        torch.cuda.Stream, or None: torch's current stream if torch is loaded, else the null stream)."""
        _check(lib().qtip_stream_wait(self._h, _stream_handle(stream)))

    def stream_signal(self, stream=None):
        """`stream` waits for everything queued so far on the context's stream."""
        _check(lib().qtip_stream_signal(self._h, _stream_handle(stream)))

    def device_lut(self):
        """Device address of the 65536-entry fp16-pair table (device_lut(), src/quantizer.cpp:14-28)."""
        p = C.c_void_p()
        _check(lib().qtip_device_lut(self._h, C.byref(p)))
        return p.value

    def set_tlut(self, tlut):
        t = None if tlut is None else np.ascontiguousarray(tlut, np.float32).reshape(1024)
        _check(lib().qtip_set_tlut(self._h, _ptr(t)))

    @property
    def lut_rms(self):
        return lib().qtip_lut_rms(self._h)

    def lut(self):
        a = np.zeros(65536, np.float32)
        b = np.zeros(65536, np.float32)
        _check(lib().qtip_get_lut(self._h, _ptr(a), _ptr(b)))
        return a, b

    # ---- Viterbi of independent tiles
    def viterbi_tiles(self, X, want_states=True, want_packed=True):
        X = np.ascontiguousarray(X, np.float32).reshape(-1, 256)
        B = X.shape[0]
        st = np.zeros((B, 128), np.uint16) if want_states else None
        pk = np.zeros((B, 32), np.uint16) if want_packed else None
        _check(lib().qtip_viterbi_tiles(self._h, _ptr(X), B, _ptr(st), _ptr(pk)))
        return st, pk

    def trim(self):
        """Idle device memory the context keeps for reuse goes back to the runtime; returns the bytes released."""
        b = C.c_ulonglong(0)
        _check(lib().qtip_trim(self._h, C.byref(b)))
        return int(b.value)

    def set_viterbi_mode(self, mode=0, margin_units=0):
        """0: 32-bit metrics first, fp64 again where a traced decision is closer than margin_units (default 160)
        units of 2^-26; 1: fp64 metrics only; 2, 3: mode 0 with 256 / 512 threads per tile whatever the size of
        the launch (mode 0 picks 512 for launches of at most a third of the device's workgroup slots).  Same states
        in every mode."""
        _check(lib().qtip_set_viterbi_mode(self._h, int(mode), C.c_uint(int(margin_units))))

    def ldlq_default_chains(self):
        """What QuantOpts.ldlq_chains = 0 stands for in this context: 2 or 3."""
        n = C.c_int(0)
        _check(lib().qtip_ldlq_default_chains(self._h, C.byref(n)))
        return int(n.value)

    def viterbi_stats(self, reset=False):
        """(first passes, second passes) that mode 0 ran again on fp64 metrics."""
        a, b = C.c_ulonglong(0), C.c_ulonglong(0)
        _check(lib().qtip_viterbi_stats(self._h, C.byref(a), C.byref(b), 1 if reset else 0))
        return int(a.value), int(b.value)

    def viterbi_tiles_dev(self, dX, B, d_states=None, d_packed=None):
        _check(lib().qtip_viterbi_tiles_dev(self._h, _ptr(dX), B, _ptr(d_states), _ptr(d_packed)))

    def viterbi_tiles_dev_noalloc(self, dX, B, d_states=None, d_packed=None):
        """viterbi_tiles_dev on the library's fixed workspace: allocates nothing, B <= NOALLOC_MAX_TILES."""
        _check(lib().qtip_viterbi_tiles_dev_noalloc(self._h, _ptr(dX), B, _ptr(d_states), _ptr(d_packed)))

    def decode_states_dev(self, d_states, B, d_hat):
        _check(lib().qtip_decode_states_dev(self._h, _ptr(d_states), B, _ptr(d_hat)))

    def decode_trellis_dev(self, d_trellis, m, n, d_hatWr):
        """Kernel-layout trellis words (device) -> hatWr m x n fp32 (device); runtime/src/qtip.cpp:83-118."""
        _check(lib().qtip_decode_trellis_dev(self._h, _ptr(d_trellis), m, n, _ptr(d_hatWr)))

    def dequantize_linear(self, out: "LinearOut", hatW=None):
        """hatW (m x n fp32) of one quantized linear from its packed output; hatW may be a device tensor to fill."""
        m, n = out.m, out.n
        tr = np.ascontiguousarray(out.trellis, dtype=np.uint16)
        su = np.ascontiguousarray(out.su_bf16, dtype=np.uint16)
        sv = np.ascontiguousarray(out.sv, dtype=np.float32)
        if hatW is None:
            hatW = np.empty((m, n), np.float32)
        _check(lib().qtip_dequantize_linear(self._h, _ptr(tr), _ptr(su), _ptr(sv), float(out.wscale), m, n, _ptr(hatW),
                                            1 if _is_device(hatW) else 0))
        return hatW

    def hadamard_rows_dev(self, dX, rows, n, ld, transpose):
        _check(lib().qtip_hadamard_rows_dev(self._h, _ptr(dX), rows, n, ld, 1 if transpose else 0))

    # ---- the group path
    def rotate_hessian(self, H, n, seed, opt: QuantOpts = None) -> HessPrep:
        import time
        opt = opt or QuantOpts()
        t0 = time.time()
        hp = HessPrep(n=n, seed=seed)
        hp.su = np.zeros(n, np.float32)
        hp.HRr = np.zeros((n, n), np.float32)
        creg = C.c_double()
        if not _is_device(H):
            H = np.ascontiguousarray(H, np.float32)
        _check(lib().qtip_rotate_hessian(self._h, _ptr(H), 1 if _is_device(H) else 0, n, seed, opt.sigma_reg,
                                         _ptr(hp.su), C.byref(creg), _ptr(hp.HRr)))
        hp.creg = creg.value
        hp.t_rot = time.time() - t0
        return hp

    @staticmethod
    def ldl_hessian(hp: HessPrep, threads=16, tag=""):
        import time
        t0 = time.time()
        hp.L = np.zeros((hp.n, hp.n), np.float32)
        rc = lib().qtip_ldl_hessian(_ptr(hp.HRr), hp.n, threads, _ptr(hp.L))
        if rc != 0:
            hp.L = None
            _check(rc)
        hp.t_ldl = time.time() - t0

    def ldl_hessian_device_updates(self, hp: HessPrep, threads=16):
        """ldl_hessian with the trailing updates of the host's panels on the GPU; hp.L equals ldl_hessian's."""
        import time
        t0 = time.time()
        hp.L = np.zeros((hp.n, hp.n), np.float32)
        rc = lib().qtip_ldl_hessian_device_updates(self._h, _ptr(hp.HRr), hp.n, threads, _ptr(hp.L))
        if rc != 0:
            hp.L = None
            _check(rc)
        hp.t_ldl = time.time() - t0

    def ldl_hessian_device_resident(self, dHRr, n, L_host, dL=None, threads=16):
        """The same with the rotated Hessian on the device (dHRr, never written), as run_groups runs it: L goes to
        L_host (n x n fp32, page-locked when dL is given) and, column block by column block, to the device buffer
        dL.  Returns the seconds the call took."""
        import time
        t0 = time.time()
        _check(lib().qtip_ldl_hessian_device_updates_dev(self._h, _ptr(dHRr), n, threads, _ptr(L_host),
                                                         _ptr(dL) if dL is not None else None))
        return time.time() - t0

    def ldlq_dev(self, dWT, dL, n, m, d_hatWT, dQ, time_viterbi=False, feedback=0):
        vs = C.c_double()
        _check(lib().qtip_ldlq_dev(self._h, _ptr(dWT), _ptr(dL), n, m, _ptr(d_hatWT), _ptr(dQ), feedback,
                                   C.byref(vs) if time_viterbi else None))
        return vs.value

    def prod_cache_bf16x3_dev(self, N, K, dLrows, ldl, dWT, d_hatWT, ldw, dP):
        """P[128][N] = sum_k Lrows[k][r] (WT - hatWT)[k][j] in split-bf16 arithmetic (device fp32 tensors)."""
        _check(lib().qtip_prod_cache_bf16x3_dev(self._h, N, K, _ptr(dLrows), ldl, _ptr(dWT), _ptr(d_hatWT), ldw, _ptr(dP)))

    def _marshal(self, lins, n, opt):
        if not opt.share_su:
            raise QtipError(QTIP_E_ARG, "share_su=false not supported (one LDL per group)")
        cin = (_LinearInC * len(lins))()
        cout = (_LinearOutC * len(lins))()
        outs, keep = [], []
        for k, li in enumerate(lins):
            cin[k].m = li.m
            dev = 0
            for fld in ("w_f32", "w_bf16", "w_fp8", "scale_bf16"):
                v = getattr(li, fld)
                if v is not None:
                    if _is_device(v):
                        dev = 1
                    elif not isinstance(v, int):
                        v = np.ascontiguousarray(v)
                    keep.append(v)
                    setattr(cin[k], fld, _ptr(v))
            cin[k].on_device = dev
            o = LinearOut(name=li.name, m=li.m, n=n)
            o.trellis = np.zeros((li.m // 16) * (n // 16) * 32, np.uint16)
            o.su_bf16 = np.zeros(n, np.uint16)
            o.sv = np.zeros(li.m, np.float32)
            o.hatW = np.zeros((li.m, n), np.float32) if opt.want_hatW else None
            cout[k].trellis, cout[k].su_bf16, cout[k].sv = _ptr(o.trellis), _ptr(o.su_bf16), _ptr(o.sv)
            cout[k].hatW = _ptr(o.hatW)
            outs.append(o)
        co = _OptsC(opt.sigma_reg, opt.scale_override, opt.ldl_threads, opt.feedback, 1 if opt.skip_proxy else 0,
                    1 if opt.ldl_device_updates else 0, opt.ldlq_chains, opt.group_lanes)
        return cin, cout, outs, co, keep

    @staticmethod
    def _finish(cout, outs, tm):
        for k, o in enumerate(outs):
            o.wscale, o.proxy = cout[k].wscale, cout[k].proxy
            o.proxy_rot_reg, o.seconds = cout[k].proxy_rot_reg, cout[k].seconds
        return outs, GroupTiming(**{k: getattr(tm, k) for k, _ in _TimingC._fields_})

    def quantize_group(self, lins: List[LinearIn], hp: HessPrep, opt: QuantOpts = None):
        """quantize_group(s, gemm, lins, hp, opt, tm, tag), src/quantizer.cpp:176-346.  Consumes hp.L."""
        opt = opt or QuantOpts()
        cin, cout, outs, co, keep = self._marshal(lins, hp.n, opt)
        tm = _TimingC()
        tm.rht, tm.ldl_cpu = hp.t_rot, hp.t_ldl
        _check(lib().qtip_quantize_group(self._h, len(lins), cin, hp.n, hp.seed, _ptr(hp.su), hp.creg, _ptr(hp.HRr),
                                         _ptr(hp.L), C.byref(co), cout, C.byref(tm)))
        hp.L = None
        return self._finish(cout, outs, tm)

    def quantize_group_h(self, lins: List[LinearIn], n, H, seed, opt: QuantOpts = None):
        """quantize_group(s, gemm, lins, n, H, seed, opt, tm, tag), src/quantizer.cpp:167-174."""
        opt = opt or QuantOpts()
        cin, cout, outs, co, keep = self._marshal(lins, n, opt)
        tm = _TimingC()
        if not _is_device(H):
            H = np.ascontiguousarray(H, np.float32)
        _check(lib().qtip_quantize_group_h(self._h, len(lins), cin, n, _ptr(H), 1 if _is_device(H) else 0, seed,
                                           C.byref(co), cout, C.byref(tm)))
        return self._finish(cout, outs, tm)


    def hessian_accumulate_dev(self, dX_bf16, rows, n, dH):
        """dH (n x n fp32, device) += X^T X for dX_bf16 (rows x n bf16 bits, device); src/model.cpp:352-363."""
        _check(lib().qtip_hessian_accumulate_dev(self._h, _ptr(dX_bf16), rows, n, _ptr(dH)))

    def hessian_finish_dev(self, dH, n, scale=1.0):
        """Mirror the computed triangle and scale (src/model.cpp:260-264, src/pipeline.cpp:160-166)."""
        _check(lib().qtip_hessian_finish_dev(self._h, _ptr(dH), n, float(scale)))

    # ---- NVFP4 fallback quantizer (src/nvfp4_gpu.hpp)
    @staticmethod
    def _nvfp4_marshal(ws, n):
        mats = (_Nvfp4MatrixC * len(ws))()
        outs, keep = [], []
        for k, w in enumerate(ws):
            w = np.ascontiguousarray(w, np.float32)
            assert w.ndim == 2 and w.shape[1] == n
            t = Nvfp4Tensor(m=w.shape[0], n=n, packed=np.zeros((w.shape[0], n // 2), np.uint8),
                            scales=np.zeros((w.shape[0], n // 16), np.uint8))
            mats[k].m, mats[k].w, mats[k].packed, mats[k].scales = w.shape[0], _ptr(w), _ptr(t.packed), _ptr(t.scales)
            outs.append(t)
            keep.append(w)
        return mats, outs, keep

    def nvfp4_quantize_group(self, ws, n, H=None, scale_search=True, calibrate=True, sigma_reg=1e-2,
                             factor_on_host=False):
        """nvfp4_quantize_group, src/nvfp4_gpu.hip:174-241 -> (tensors, calibrated).  factor_on_host: the calibration's
        Cholesky factorization on the host alone (default: its trailing updates on the GPU, same bits)."""
        mats, outs, keep = self._nvfp4_marshal(ws, n)
        o = _Nvfp4OptsC(1 if scale_search else 0, 1 if calibrate else 0, sigma_reg, 1 if factor_on_host else 0)
        used = C.c_int()
        Hc = None if H is None else np.ascontiguousarray(H, np.float32)
        _check(lib().qtip_nvfp4_quantize_group(self._h, len(ws), C.addressof(mats), n, _ptr(Hc), C.byref(o), C.byref(used)))
        for k, t in enumerate(outs):
            t.global_scale = mats[k].global_
        return outs, bool(used.value)

    def nvfp4_quantize_prepared(self, ws, n, L=None, dw=None, scale_search=True):
        """The device block loop on a prepared factor (L unit-lower n x n or None, dw [n] or None)."""
        mats, outs, keep = self._nvfp4_marshal(ws, n)
        Lc = None if L is None else np.ascontiguousarray(L, np.float32)
        dc = None if dw is None else np.ascontiguousarray(dw, np.float32)
        _check(lib().qtip_nvfp4_quantize_prepared(self._h, len(ws), C.addressof(mats), n, _ptr(Lc), _ptr(dc),
                                                  1 if scale_search else 0))
        for k, t in enumerate(outs):
            t.global_scale = mats[k].global_
        return outs

    def reserve_groups(self, n):
        _check(lib().qtip_reserve_groups(self._h, n))

    def run_groups(self, groups, opt: QuantOpts = None):
        """Several groups with the host LDL of group g+1 overlapping the GPU work of group g (run_qtip_groups,
        src/pipeline.cpp:229-312).  groups: list of (lins, n, H, seed).  Returns a list of (outs, timing, ldl_wait)."""
        opt = opt or QuantOpts()
        G = (_GroupC * len(groups))()
        held, keep = [], []
        co = None
        for g, (lins, n, H, seed) in enumerate(groups):
            cin, cout, outs, co, kp = self._marshal(lins, n, opt)
            if not _is_device(H):
                H = np.ascontiguousarray(H, np.float32)
            keep.append((kp, H, cin))
            held.append((cout, outs))
            G[g].nlin, G[g].lins, G[g].outs = len(lins), C.addressof(cin), C.addressof(cout)
            G[g].n, G[g].H, G[g].h_on_device, G[g].seed = n, _ptr(H), 1 if _is_device(H) else 0, seed
        tms = (_TimingC * len(groups))()
        waits = (C.c_double * len(groups))()
        if groups:
            _check(lib().qtip_run_groups(self._h, len(groups), C.addressof(G), C.byref(co), C.addressof(tms),
                                         C.addressof(waits)))
        res = []
        for g, (cout, outs) in enumerate(held):
            o, tm = self._finish(cout, outs, tms[g])
            res.append((o, tm, waits[g]))
        return res

    def group_lanes(self, shapes, opt: QuantOpts = None):
        """How many groups run_groups would run side by side for groups of these shapes: a list of (ms, n) with ms
        the out-features of the group's linears."""
        opt = opt or QuantOpts()
        G = (_GroupC * len(shapes))()
        keep = []
        for g, (ms, n) in enumerate(shapes):
            cin = (_LinearInC * len(ms))()
            for k, m in enumerate(ms):
                cin[k].m = m
            keep.append(cin)
            G[g].nlin, G[g].lins, G[g].n = len(ms), C.addressof(cin), n
        co = _OptsC(opt.sigma_reg, opt.scale_override, opt.ldl_threads, opt.feedback, 1 if opt.skip_proxy else 0,
                    1 if opt.ldl_device_updates else 0, opt.ldlq_chains, opt.group_lanes)
        lanes = C.c_int()
        _check(lib().qtip_group_lanes(self._h, len(shapes), C.addressof(G), C.byref(co), C.byref(lanes)))
        return lanes.value

    def nvfp4_prepare_device_updates(self, H, sigma_reg=1e-2, threads=16):
        """nvfp4_prepare (calibrated) with the factorization's trailing updates on the GPU -> (L, dw), same bits."""
        H = np.ascontiguousarray(H, np.float32)
        n = H.shape[0]
        L = np.zeros((n, n), np.float32)
        dw = np.zeros(n, np.float32)
        _check(lib().qtip_nvfp4_prepare_device_updates(self._h, _ptr(H), n, sigma_reg, threads, _ptr(L), _ptr(dw)))
        return L, dw

    def tlut_f16(self):
        out = np.zeros((512, 2), np.uint16)
        _check(lib().qtip_get_tlut_f16(self._h, _ptr(out)))
        return out


@dataclass
class Nvfp4Tensor:  # src/nvfp4.hpp:35-41
    m: int = 0
    n: int = 0
    packed: Optional[np.ndarray] = None   # [m][n/2], low nibble = first of two values
    scales: Optional[np.ndarray] = None   # [m][n/16] E4M3 block scales
    global_scale: float = 1.0


def nvfp4_quantize(w):
    """nvfp4_quantize, src/nvfp4.cpp:12-55 (host)."""
    w = np.ascontiguousarray(w, np.float32)
    m, n = w.shape
    t = Nvfp4Tensor(m=m, n=n, packed=np.zeros((m, n // 2), np.uint8), scales=np.zeros((m, max(n // 16, 0)), np.uint8))
    g = C.c_float()
    _check(lib().qtip_nvfp4_quantize(_ptr(w), m, n, _ptr(t.packed), _ptr(t.scales), C.byref(g)))
    t.global_scale = g.value
    return t


def nvfp4_dequantize(t: Nvfp4Tensor):
    """nvfp4_dequantize, src/nvfp4.cpp:57-70 (host)."""
    out = np.zeros((t.m, t.n), np.float32)
    _check(lib().qtip_nvfp4_dequantize(_ptr(np.ascontiguousarray(t.packed)), _ptr(np.ascontiguousarray(t.scales)),
                                       t.global_scale, t.m, t.n, _ptr(out)))
    return out


def nvfp4_proxy_error(w, what, H=None):
    """nvfp4_proxy_error, src/nvfp4.cpp:72-87 (host, fp64)."""
    w = np.ascontiguousarray(w, np.float32)
    what = np.ascontiguousarray(what, np.float32)
    Hc = None if H is None else np.ascontiguousarray(H, np.float32)
    out = C.c_double()
    _check(lib().qtip_nvfp4_proxy_error(_ptr(w), _ptr(what), w.shape[0], w.shape[1], _ptr(Hc), C.byref(out)))
    return out.value


def nvfp4_prepare(H, sigma_reg=1e-2, calibrate=True, threads=16):
    """Host preparation of the calibrated quantizer (src/nvfp4_gpu.hip:181-207) -> (L or None, dw)."""
    H = np.ascontiguousarray(H, np.float32)
    n = H.shape[0]
    L = np.zeros((n, n), np.float32) if calibrate else None
    dw = np.zeros(n, np.float32)
    _check(lib().qtip_nvfp4_prepare(_ptr(H), n, sigma_reg, 1 if calibrate else 0, threads, _ptr(L), _ptr(dw)))
    return L, dw


def f32_to_fp8e4m3(x):
    return int(lib().qtip_f32_to_fp8e4m3(float(x)))


class LayerFileWriter:
    """safetensors container of a quantized layer (SafeTensorsWriter, src/safetensors.cpp:93-137; tensor set of
    write_layer_file, src/pipeline.cpp:315-352).  Host only."""

    def __init__(self):
        self._h = C.c_void_p()
        _check(lib().qtip_st_create(C.byref(self._h)))

    def close(self):
        if self._h:
            lib().qtip_st_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def add(self, name, dtype, shape, data):
        data = np.ascontiguousarray(data)
        sh = (C.c_int64 * max(1, len(shape)))(*shape)
        _check(lib().qtip_st_add(self._h, name.encode(), dtype.encode(), C.addressof(sh), len(shape), _ptr(data),
                                 data.nbytes))

    def add_qtip_linear(self, prefix, out: "LinearOut", tlut_f16=None):
        co = _LinearOutC()
        tr = np.ascontiguousarray(out.trellis, np.uint16)
        su = np.ascontiguousarray(out.su_bf16, np.uint16)
        sv = np.ascontiguousarray(out.sv, np.float32)
        co.trellis, co.su_bf16, co.sv, co.wscale = _ptr(tr), _ptr(su), _ptr(sv), out.wscale
        tl = None if tlut_f16 is None else np.ascontiguousarray(tlut_f16, np.uint16)
        _check(lib().qtip_st_add_qtip_linear(self._h, prefix.encode(), C.addressof(co), out.m, out.n, _ptr(tl)))

    def add_nvfp4_linear(self, prefix, t: "Nvfp4Tensor"):
        """weight_packed / weight_scale / weight_global_scale of an NVFP4 linear (src/pipeline.cpp:342-346)."""
        self.add(prefix + "weight_packed", "U8", [t.m, t.n // 2], t.packed)
        self.add(prefix + "weight_scale", "F8_E4M3", [t.m, t.n // 16], t.scales)
        self.add(prefix + "weight_global_scale", "F32", [], np.array([t.global_scale], np.float32))

    def write(self, path, metadata=None):
        n = C.c_uint64()
        if metadata is None:
            _check(lib().qtip_st_write(self._h, path.encode(), None, 0, C.byref(n)))
        else:
            flat = []
            for k, v in metadata.items():
                flat += [k.encode(), v.encode()]
            arr = (C.c_char_p * max(1, len(flat)))(*flat)
            _check(lib().qtip_st_write(self._h, path.encode(), C.addressof(arr), len(metadata), C.byref(n)))
        return n.value


# ---------------------------------------------------------------- host packers
def device_alloc_calls():
    """Device allocations (hipMalloc) the library has made in this process so far."""
    return int(lib().qtip_selftest_device_alloc_calls())


def pack_trellis(states):
    states = np.ascontiguousarray(states, np.uint16).reshape(-1, 128)
    out = np.zeros((states.shape[0], 32), np.uint16)
    lib().qtip_pack_trellis(_ptr(states), states.shape[0], _ptr(out))
    return out


def unpack_trellis(packed):
    packed = np.ascontiguousarray(packed, np.uint16).reshape(-1, 32)
    out = np.zeros((packed.shape[0], 128), np.uint16)
    lib().qtip_unpack_trellis(_ptr(packed), packed.shape[0], _ptr(out))
    return out


def swizzle_for_kernel(packed, m, n):
    packed = np.ascontiguousarray(packed, np.uint16).reshape(-1)
    out = np.zeros_like(packed)
    _check(lib().qtip_swizzle_for_kernel(_ptr(packed), m, n, _ptr(out)))
    return out


def unswizzle_for_kernel(tr, m, n):
    tr = np.ascontiguousarray(tr, np.uint16).reshape(-1)
    out = np.zeros_like(tr)
    _check(lib().qtip_unswizzle_for_kernel(_ptr(tr), m, n, _ptr(out)))
    return out


def had_K(n):
    return lib().qtip_had_K(n)


def sign_vector(seed, count):
    out = np.zeros(count, np.float32)
    lib().qtip_sign_vector(seed, count, _ptr(out))
    return out
