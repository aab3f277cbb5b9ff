"""TEST INFRASTRUCTURE ONLY: ctypes front-end of the CPU oracle.

``oracle.lib`` wraps ``libmiq_oracle.so`` (the C restatement in ``miq_oracle.c``); ``oracle.ref`` wraps
``_ref/libaimet_ref.so`` (the reference's own DlQuantization CPU sources compiled in place behind
``ref_driver.cpp``) and is ``None`` where that library has not been built.  Only tests, the smoke check and the
bench's CPU-baseline leg may import this package; the product package never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_ORACLE_SO = os.path.join(_HERE, "libmiq_oracle.so")
_REF_SO = os.path.join(_HERE, "_ref", "libaimet_ref.so")

PDF_SIZE = 512
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_f64p = np.ctypeslib.ndpointer(np.float64, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(np.uint16, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(np.uint8, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_i64p = np.ctypeslib.ndpointer(np.int64, flags="C_CONTIGUOUS")
_i64 = C.c_int64


def build(with_ref=True):
    """Compile the restatement, and the compiled reference where the reference tree is present."""
    subprocess.run(["make", "-C", _HERE, "-s", "all"], check=True)
    if with_ref and os.path.isdir("/root/reference/ModelOptimizations/DlQuantization/src"):
        subprocess.run(["make", "-C", _HERE, "-s", "ref"], check=True)


class Encoding(C.Structure):
    _fields_ = [("min", C.c_double), ("max", C.c_double), ("delta", C.c_double), ("offset", C.c_double),
                ("bw", C.c_int)]

    def astuple(self):
        return (self.min, self.max, self.delta, self.offset, self.bw)


class _PdfStruct(C.Structure):
    _fields_ = [("xLeft", C.c_double * PDF_SIZE), ("pdf", C.c_double * PDF_SIZE), ("iterations", C.c_int),
                ("initialized", C.c_int), ("stats_updated", C.c_int)]


class _ProfileStruct(C.Structure):
    _fields_ = [("min", C.c_double), ("max", C.c_double), ("histogram", C.c_double * PDF_SIZE),
                ("iterations", C.c_int), ("initialized", C.c_int), ("stats_updated", C.c_int)]


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


class _Oracle:
    def __init__(self, path):
        L = self.L = C.CDLL(path)
        L.orc_fill_encoding_info.argtypes = [C.c_int, C.c_double, C.c_double, C.POINTER(Encoding)]
        L.orc_qdq_per_tensor_f32.argtypes = [_f32p, _i64, _f32p, C.c_double, C.c_double, C.c_int]
        L.orc_quantize_per_tensor_f32.argtypes = [_f32p, _i64, _f32p, C.c_double, C.c_double, C.c_int, C.c_int]
        L.orc_qdq_per_tensor_bf16.argtypes = [_u16p, _i64, _u16p, C.c_double, C.c_double, C.c_int]
        L.orc_per_channel_params_f32.argtypes = [_f64p, _f64p, _i64, C.c_int, _f32p, _f32p, _f32p, _f32p]
        L.orc_qdq_per_channel_f32.argtypes = [_f32p, _i64, _i64, _i64, _f32p, _f32p, _f32p, _f32p, _f32p]
        L.orc_quantize_per_channel_f32.argtypes = L.orc_qdq_per_channel_f32.argtypes
        L.orc_stochastic_f32.argtypes = [_f32p, _i64, _i64, _i64, _f32p, _f32p, _f32p, _f32p, _f32p, _f64p, C.c_int,
                                         C.c_float]
        L.orc_stochastic_uniforms.argtypes = [C.c_uint64, C.c_uint64, _i64, _i64, _f64p]
        L.orc_qdq_per_channel_bf16.argtypes = [_u16p, _i64, _i64, _i64, _u16p, _f32p, _f32p, _f32p, _f32p]
        L.orc_qdq_broadcast_f32.argtypes = [_f32p, _f32p, _i64, _i64, _i64p, _i64p, _f32p, _f32p, _f32p, _f32p]
        L.orc_ste_bwd_per_tensor_f32.argtypes = [_f32p, _f32p, _f32p, _i64, C.c_float, C.c_float]
        L.orc_ste_bwd_per_channel_f32.argtypes = [_f32p, _f32p, _f32p, _i64, _i64, _i64, _f32p, _f32p]
        L.orc_minmax_f32.argtypes = [_f32p, _i64, C.POINTER(C.c_float), C.POINTER(C.c_float)]
        L.orc_get_computed_encodings.argtypes = [C.c_int, C.c_double, C.c_double, C.c_int, C.c_int, C.c_int,
                                                 C.POINTER(Encoding)]
        L.orc_tf_compute_encoding.argtypes = [C.c_double, C.c_double, C.c_int, C.c_int, C.c_int, C.c_int,
                                              C.POINTER(Encoding)]
        L.orc_pdf_reset.argtypes = [C.POINTER(_PdfStruct)]
        L.orc_pdf_update_f32.argtypes = [C.POINTER(_PdfStruct), _f32p, _i64, C.c_void_p]
        L.orc_histogram_f32.argtypes = [_f32p, _i64, _u32p, C.c_float, C.c_float]
        L.orc_tfe_find_range.argtypes = [C.POINTER(_PdfStruct), C.POINTER(C.c_float), C.POINTER(C.c_float)]
        L.orc_tfe_candidates.argtypes = [C.POINTER(_PdfStruct), C.c_int, C.c_int, C.c_int, C.c_int, _f32p, _i32p,
                                         C.c_int]
        L.orc_tfe_candidates.restype = C.c_int
        L.orc_tfe_cost.argtypes = [C.POINTER(_PdfStruct), C.c_int, C.c_float, C.c_int]
        L.orc_tfe_cost.restype = C.c_double
        L.orc_tfe_compute_encoding.argtypes = [C.POINTER(_PdfStruct), C.c_int, C.c_int, C.c_int, C.c_int,
                                               C.POINTER(Encoding), C.c_void_p, C.POINTER(C.c_int)]
        L.orc_mse_minimize.argtypes = [C.POINTER(_PdfStruct), C.c_int, C.c_int, C.c_int, C.c_int,
                                       C.POINTER(C.c_float), C.POINTER(C.c_float), C.c_void_p, C.c_void_p, C.c_void_p,
                                       C.POINTER(C.c_int)]
        L.orc_mse_compute_encoding.argtypes = [C.POINTER(_PdfStruct), C.c_int, C.c_int, C.c_int, C.c_int,
                                               C.POINTER(Encoding)]
        L.orc_mse_cost.restype = C.c_float
        L.orc_mse_cost.argtypes = [C.c_int, _f32p, _f32p, C.c_int, C.c_float, C.c_float, C.c_int, C.c_int, C.c_int]
        L.orc_profile_reset.argtypes = [C.POINTER(_ProfileStruct)]
        L.orc_profile_update_f32.argtypes = [C.POINTER(_ProfileStruct), _f32p, _i64]
        L.orc_entropy_optimize_kl.argtypes = [C.POINTER(_ProfileStruct), C.c_int, C.c_int, C.c_int, C.c_int,
                                              C.POINTER(C.c_float), C.POINTER(C.c_float), C.c_void_p,
                                              C.POINTER(C.c_int)]
        L.orc_entropy_compute_encoding.argtypes = [C.POINTER(_ProfileStruct), C.c_int, C.c_int, C.c_int, C.c_int,
                                                   C.POINTER(Encoding)]
        L.orc_v2_qdq_f32.argtypes = [_f32p, _i64, _i64, _i64, C.c_void_p, C.c_void_p, C.c_void_p, _f32p, _f32p,
                                     C.c_int, C.c_int]
        L.orc_v2_qdq_bf16.argtypes = [_u16p, _i64, _i64, _i64, _u16p, C.c_void_p, _f32p, _f32p, C.c_int, C.c_int]
        L.orc_v2_qdq_bwd_f32.argtypes = [_f32p, _f32p, _i64, _i64, _i64, _f32p, _f32p, _f32p, C.c_int, C.c_int]
        L.orc_v2_qdq_bwd_params_f32.argtypes = [_f32p, _f32p, _i64, _i64, _i64, _f32p, _f32p, _f32p, C.c_int, C.c_int,
                                                _f64p, _f64p]
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]
        L.orc_bf16_to_f32.restype = C.c_float
        L.orc_f32_to_bf16.argtypes = [C.c_float]
        L.orc_f32_to_bf16.restype = C.c_uint16

    # -- encodings ---------------------------------------------------------------------------------------------
    def fill_encoding_info(self, bw, mn, mx):
        e = Encoding()
        self.L.orc_fill_encoding_info(bw, mn, mx, C.byref(e))
        return e

    def get_computed_encodings(self, bw, mn, mx, sym, strict, unsigned_sym):
        e = Encoding()
        self.L.orc_get_computed_encodings(bw, mn, mx, int(sym), int(strict), int(unsigned_sym), C.byref(e))
        return e

    def tf_compute_encoding(self, acc_min, acc_max, bw, sym=False, strict=False, unsigned_sym=False):
        e = Encoding()
        self.L.orc_tf_compute_encoding(acc_min, acc_max, bw, int(sym), int(strict), int(unsigned_sym), C.byref(e))
        return e

    # -- per-tensor --------------------------------------------------------------------------------------------
    def qdq_per_tensor(self, x, mn, mx, bw):
        x = _f32(x)
        out = np.empty_like(x)
        self.L.orc_qdq_per_tensor_f32(x.reshape(-1), x.size, out.reshape(-1), mn, mx, bw)
        return out

    def quantize_per_tensor(self, x, mn, mx, bw, shift_to_signed):
        x = _f32(x)
        out = np.empty_like(x)
        self.L.orc_quantize_per_tensor_f32(x.reshape(-1), x.size, out.reshape(-1), mn, mx, bw, int(shift_to_signed))
        return out

    def qdq_per_tensor_bf16(self, x_bits, mn, mx, bw):
        x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
        out = np.empty_like(x_bits)
        self.L.orc_qdq_per_tensor_bf16(x_bits.reshape(-1), x_bits.size, out.reshape(-1), mn, mx, bw)
        return out

    # -- stochastic rounding -----------------------------------------------------------------------------------
    def stochastic_uniforms(self, seed, call, n, first=0):
        """The product's documented generator: u(i) for i in [first, first + n)."""
        u = np.empty(n, np.float64)
        self.L.orc_stochastic_uniforms(seed, call, first, n, u)
        return u

    def stochastic(self, x, num_channel, n_per_channel, params, u, dequant=True, shift=0.0):
        """floor(t + u) quantize(-dequantize) with explicit uniform numbers; params = (min, max, delta, offset) float32
        vectors of length num_channel."""
        x = _f32(x)
        out = np.empty_like(x)
        mn, mx, d, o = (_f32(p).reshape(-1) for p in params)
        u = np.ascontiguousarray(u, dtype=np.float64).reshape(-1)
        assert u.size == x.size and mn.size == num_channel
        self.L.orc_stochastic_f32(x.reshape(-1), num_channel, x.size, n_per_channel, out.reshape(-1), mn, mx, d, o, u,
                                  int(dequant), float(shift))
        return out

    def stochastic_per_tensor(self, x, mn, mx, bw, u, dequant=True, shift_to_signed=False):
        e = self.fill_encoding_info(bw, mn, mx)
        params = tuple(np.array([v], np.float32) for v in (e.min, e.max, e.delta, e.offset))
        shift = float(2 ** (bw - 1)) if (shift_to_signed and not dequant) else 0.0
        return self.stochastic(x, 1, max(np.asarray(x).size, 1), params, u, dequant, shift)

    # -- per-channel -------------------------------------------------------------------------------------------
    def per_channel_params(self, enc_min, enc_max, bw):
        enc_min = np.ascontiguousarray(enc_min, dtype=np.float64)
        enc_max = np.ascontiguousarray(enc_max, dtype=np.float64)
        c = enc_min.size
        outs = [np.empty(c, np.float32) for _ in range(4)]
        self.L.orc_per_channel_params_f32(enc_min, enc_max, c, bw, *outs)
        return tuple(outs)

    def qdq_per_channel(self, x, num_channel, n_per_channel, params, quantize_only=False):
        x = _f32(x)
        out = np.empty_like(x)
        fn = self.L.orc_quantize_per_channel_f32 if quantize_only else self.L.orc_qdq_per_channel_f32
        fn(x.reshape(-1), num_channel, x.size, n_per_channel, out.reshape(-1), *[_f32(p) for p in params])
        return out

    def qdq_per_channel_bf16(self, x_bits, num_channel, n_per_channel, params):
        x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
        out = np.empty_like(x_bits)
        self.L.orc_qdq_per_channel_bf16(x_bits.reshape(-1), num_channel, x_bits.size, n_per_channel,
                                        out.reshape(-1), *[_f32(p) for p in params])
        return out

    def qdq_broadcast(self, x, input_strides, encoding_strides, params):
        x = _f32(x)
        out = np.empty_like(x)
        ist = np.ascontiguousarray(input_strides, dtype=np.int64)
        est = np.ascontiguousarray(encoding_strides, dtype=np.int64)
        self.L.orc_qdq_broadcast_f32(x.reshape(-1), out.reshape(-1), x.size, ist.size, ist, est,
                                     *[_f32(p) for p in params])
        return out

    # -- STE backward ------------------------------------------------------------------------------------------
    def ste_bwd_per_tensor(self, x, g, mn, mx):
        x, g = _f32(x), _f32(g)
        out = np.empty_like(x)
        self.L.orc_ste_bwd_per_tensor_f32(x.reshape(-1), g.reshape(-1), out.reshape(-1), x.size, mn, mx)
        return out

    def ste_bwd_per_channel(self, x, g, num_channel, n_per_channel, mn, mx):
        x, g = _f32(x), _f32(g)
        out = np.empty_like(x)
        self.L.orc_ste_bwd_per_channel_f32(x.reshape(-1), g.reshape(-1), out.reshape(-1), num_channel, x.size,
                                           n_per_channel, _f32(mn), _f32(mx))
        return out

    # -- statistics --------------------------------------------------------------------------------------------
    def minmax(self, x):
        x = _f32(x)
        mn, mx = C.c_float(), C.c_float()
        self.L.orc_minmax_f32(x.reshape(-1), x.size, C.byref(mn), C.byref(mx))
        return np.float32(mn.value), np.float32(mx.value)

    def histogram(self, x, bucket, pdf_offset):
        x = _f32(x)
        hist = np.zeros(PDF_SIZE, np.uint32)
        self.L.orc_histogram_f32(x.reshape(-1), x.size, hist, bucket, pdf_offset)
        return hist

    def new_pdf(self):
        return OraclePdf(self)

    def new_profile(self):
        return OracleProfile(self)

    # -- v2 ----------------------------------------------------------------------------------------------------
    def v2_qdq(self, x, num_channel, n_per_channel, scale, offset, qmin, qmax):
        """returns (dequantized, codes, mask)"""
        x = _f32(x)
        out, codes = np.empty_like(x), np.empty_like(x)
        mask = np.empty(x.shape, np.uint8)
        self.L.orc_v2_qdq_f32(x.reshape(-1), num_channel, x.size, n_per_channel, out.ctypes.data, codes.ctypes.data,
                              mask.ctypes.data, _f32(scale), _f32(offset), qmin, qmax)
        return out, codes, mask

    def v2_qdq_bf16(self, x_bits, num_channel, n_per_channel, scale, offset, qmin, qmax):
        x_bits = np.ascontiguousarray(x_bits, dtype=np.uint16)
        out = np.empty_like(x_bits)
        mask = np.empty(x_bits.shape, np.uint8)
        self.L.orc_v2_qdq_bf16(x_bits.reshape(-1), num_channel, x_bits.size, n_per_channel, out.reshape(-1),
                               mask.ctypes.data, _f32(scale), _f32(offset), qmin, qmax)
        return out, mask

    def v2_qdq_bwd(self, x, g, num_channel, n_per_channel, scale, offset, qmin, qmax):
        x, g = _f32(x), _f32(g)
        out = np.empty_like(x)
        self.L.orc_v2_qdq_bwd_f32(x.reshape(-1), g.reshape(-1), num_channel, x.size, n_per_channel,
                                  out.reshape(-1), _f32(scale), _f32(offset), qmin, qmax)
        return out

    def v2_qdq_bwd_params(self, x, g, num_channel, n_per_channel, scale, offset, qmin, qmax):
        """(grad_in float32, scale_grad float64[C], offset_grad float64[C])."""
        x, g = _f32(x), _f32(g)
        gin = np.empty_like(x)
        sg, og = np.zeros(num_channel, np.float64), np.zeros(num_channel, np.float64)
        self.L.orc_v2_qdq_bwd_params_f32(x.reshape(-1), g.reshape(-1), num_channel, x.size, n_per_channel,
                                         gin.reshape(-1), _f32(scale), _f32(offset), qmin, qmax, sg, og)
        return gin, sg, og

    # -- bf16 helpers ------------------------------------------------------------------------------------------
    def f32_to_bf16_bits(self, x):
        x = _f32(x)
        u = x.view(np.uint32).astype(np.uint64)
        nan = (u & 0x7fffffff) > 0x7f800000
        r = ((u + 0x7fff + ((u >> 16) & 1)) >> 16).astype(np.uint16)
        r[nan] = 0x7fc0
        return r

    @staticmethod
    def bf16_bits_to_f32(b):
        return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


class OraclePdf:
    """Stateful TF-Enhanced analyzer of the restatement (TfEnhancedEncodingAnalyzer<float>)."""

    def __init__(self, o):
        self.o = o
        self.s = _PdfStruct()
        o.L.orc_pdf_reset(C.byref(self.s))

    def update(self, x):
        x = _f32(x)
        hist = np.zeros(PDF_SIZE, np.uint32)
        self.o.L.orc_pdf_update_f32(C.byref(self.s), x.reshape(-1), x.size, hist.ctypes.data)
        return hist

    @property
    def initialized(self):
        return bool(self.s.initialized)

    @property
    def iterations(self):
        return self.s.iterations

    def x_left(self):
        return np.array(self.s.xLeft[:], np.float64)

    def pdf(self):
        return np.array(self.s.pdf[:], np.float64)

    def find_range(self):
        a, b = C.c_float(), C.c_float()
        self.o.L.orc_tfe_find_range(C.byref(self.s), C.byref(a), C.byref(b))
        return np.float32(a.value), np.float32(b.value)

    def candidates(self, bw, sym=False, strict=False, unsigned_sym=False):
        d = np.empty(512, np.float32)
        off = np.empty(512, np.int32)
        n = self.o.L.orc_tfe_candidates(C.byref(self.s), bw, int(sym), int(strict), int(unsigned_sym), d, off, 512)
        return d[:n].copy(), off[:n].copy()

    def cost(self, bw, delta, offset):
        return self.o.L.orc_tfe_cost(C.byref(self.s), bw, float(np.float32(delta)), int(offset))

    def compute_encoding(self, bw, sym=False, strict=False, unsigned_sym=False):
        """returns (Encoding, costs[ncand], best_index)"""
        e = Encoding()
        costs = np.full(512, np.nan, np.float64)
        best = C.c_int(-1)
        self.o.L.orc_tfe_compute_encoding(C.byref(self.s), bw, int(sym), int(strict), int(unsigned_sym), C.byref(e),
                                          costs.ctypes.data, C.byref(best))
        return e, costs, best.value

    def percentile_range(self, percentile):
        a, b = C.c_float(), C.c_float()
        self.o.L.orc_percentile_range(C.byref(self.s), C.c_float(percentile), C.byref(a), C.byref(b))
        return np.float32(a.value), np.float32(b.value)

    def compute_percentile_encoding(self, bw, percentile, sym=False, strict=False, unsigned_sym=False):
        """PercentileEncodingAnalyzer<float>::computeEncoding on the same PDF."""
        e = Encoding()
        self.o.L.orc_percentile_compute_encoding(C.byref(self.s), C.c_float(percentile), bw, int(sym), int(strict),
                                                 int(unsigned_sym), C.byref(e))
        return e

    def mse_minimize(self, bw, sym=False, strict=False, unsigned_sym=False):
        """MseEncodingAnalyzer<float>::_minimizeMSE on the same PDF: (best min, best max, min candidates, max
        candidates, bucket centres)."""
        a, b = C.c_float(), C.c_float()
        mins, maxs, centers = (np.empty(1100, np.float32) for _ in range(3))
        counts = (C.c_int * 3)()
        self.o.L.orc_mse_minimize(C.byref(self.s), bw, int(sym), int(strict), int(unsigned_sym), C.byref(a),
                                  C.byref(b), mins.ctypes.data, maxs.ctypes.data, centers.ctypes.data, counts)
        return (np.float32(a.value), np.float32(b.value), mins[:counts[0]].copy(), maxs[:counts[1]].copy(),
                centers[:counts[2]].copy())

    def compute_mse_encoding(self, bw, sym=False, strict=False, unsigned_sym=False):
        """MseEncodingAnalyzer<float>::computeEncoding on the same PDF."""
        e = Encoding()
        self.o.L.orc_mse_compute_encoding(C.byref(self.s), bw, int(sym), int(strict), int(unsigned_sym), C.byref(e))
        return e


class OracleProfile:
    """The rescaling 512-bin histogram of the entropy analyzer (TensorProfilingParams) and its searches."""

    def __init__(self, o):
        self.o = o
        self.s = _ProfileStruct()
        o.L.orc_profile_reset(C.byref(self.s))

    def update(self, x):
        x = _f32(x)
        self.o.L.orc_profile_update_f32(C.byref(self.s), x.reshape(-1), x.size)

    @property
    def initialized(self):
        return bool(self.s.initialized)

    @property
    def iterations(self):
        return self.s.iterations

    def range(self):
        return self.s.min, self.s.max

    def histogram(self):
        return np.array(self.s.histogram[:], np.float64)

    def optimize_kl(self, bw, sym=False, strict=False, unsigned_sym=False):
        """_optimizeKL: (min, max, divergence of every window tried)."""
        a, b = C.c_float(), C.c_float()
        div = np.empty(PDF_SIZE, np.float64)
        n = C.c_int(0)
        self.o.L.orc_entropy_optimize_kl(C.byref(self.s), bw, int(sym), int(strict), int(unsigned_sym), C.byref(a),
                                         C.byref(b), div.ctypes.data, C.byref(n))
        return np.float32(a.value), np.float32(b.value), div[:n.value].copy()

    def compute_encoding(self, bw, sym=False, strict=False, unsigned_sym=False):
        e = Encoding()
        self.o.L.orc_entropy_compute_encoding(C.byref(self.s), bw, int(sym), int(strict), int(unsigned_sym),
                                              C.byref(e))
        return e


class _Ref:
    """The reference's own CPU classes, compiled in place (present only where oracle/_ref was built)."""

    def __init__(self, path):
        L = self.L = C.CDLL(path)
        L.ref_fill_encoding_info.argtypes = [C.c_int, C.c_double, C.c_double, _f64p]
        L.ref_qdq_per_tensor.argtypes = [_f32p, _i64, _f32p, C.c_double, C.c_double, C.c_int]
        L.ref_quantize_per_tensor.argtypes = [_f32p, _i64, _f32p, C.c_double, C.c_double, C.c_int, C.c_int]
        L.ref_qdq_per_channel.argtypes = [_f32p, _i64, _i64, _i64, _f32p, _f32p, _f32p, _f32p, _f32p]
        L.ref_qdq_broadcast.argtypes = [_f32p, _f32p, _i64, _i64, _i64p, _i64p, _f32p, _f32p, _f32p, _f32p]
        L.ref_qdq_per_tensor_stochastic.argtypes = [_f32p, _i64, _f32p, C.c_double, C.c_double, C.c_int, C.c_uint]
        L.ref_quantize_per_tensor_stochastic.argtypes = [_f32p, _i64, _f32p, C.c_double, C.c_double, C.c_int, C.c_int,
                                                         C.c_uint]
        L.ref_qdq_per_channel_stochastic.argtypes = [_f32p, _i64, _i64, _i64, _f32p, _f32p, _f32p, _f32p, _f32p,
                                                     C.c_uint]
        L.ref_libc_uniforms.argtypes = [C.c_uint, _i64, _f64p]
        L.ref_get_computed_encodings.argtypes = [C.c_int, C.c_double, C.c_double, C.c_int, C.c_int, C.c_int, _f64p]
        for name in ("ref_tf_create", "ref_tfe_create"):
            getattr(L, name).restype = C.c_void_p
        for name in ("ref_tf_destroy", "ref_tfe_destroy"):
            getattr(L, name).argtypes = [C.c_void_p]
        L.ref_tf_update.argtypes = [C.c_void_p, _f32p, _i64]
        L.ref_tfe_update.argtypes = [C.c_void_p, _f32p, _i64]
        L.ref_tf_compute.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, _f64p]
        L.ref_tfe_compute.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, _f64p]
        L.ref_tfe_get_pdf.argtypes = [C.c_void_p, _f64p, _f64p, C.POINTER(C.c_int)]
        L.ref_tfe_get_pdf.restype = C.c_int
        L.ref_tfe_candidates.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _f32p, _i32p, _f64p]
        L.ref_tfe_candidates.restype = C.c_int
        L.ref_tfe_range.argtypes = [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float)]

    @staticmethod
    def _enc(out5):
        return (out5[0], out5[1], out5[2], out5[3], int(out5[4]))

    def fill_encoding_info(self, bw, mn, mx):
        o = np.empty(5)
        self.L.ref_fill_encoding_info(bw, mn, mx, o)
        return self._enc(o)

    def get_computed_encodings(self, bw, mn, mx, sym, strict, unsigned_sym):
        o = np.empty(5)
        self.L.ref_get_computed_encodings(bw, mn, mx, int(sym), int(strict), int(unsigned_sym), o)
        return self._enc(o)

    def qdq_per_tensor(self, x, mn, mx, bw):
        x = _f32(x)
        out = np.empty_like(x)
        self.L.ref_qdq_per_tensor(x.reshape(-1), x.size, out.reshape(-1), mn, mx, bw)
        return out

    def quantize_per_tensor(self, x, mn, mx, bw, shift_to_signed):
        x = _f32(x)
        out = np.empty_like(x)
        self.L.ref_quantize_per_tensor(x.reshape(-1), x.size, out.reshape(-1), mn, mx, bw, int(shift_to_signed))
        return out

    # ROUND_STOCHASTIC: srand(seed), then the reference's CPU loop; libc_uniforms replays the same rand() sequence
    def libc_uniforms(self, seed, n):
        u = np.empty(n, np.float64)
        self.L.ref_libc_uniforms(seed, n, u)
        return u

    def qdq_per_tensor_stochastic(self, x, mn, mx, bw, seed):
        x = _f32(x)
        out = np.empty_like(x)
        self.L.ref_qdq_per_tensor_stochastic(x.reshape(-1), x.size, out.reshape(-1), mn, mx, bw, seed)
        return out

    def quantize_per_tensor_stochastic(self, x, mn, mx, bw, shift_to_signed, seed):
        x = _f32(x)
        out = np.empty_like(x)
        self.L.ref_quantize_per_tensor_stochastic(x.reshape(-1), x.size, out.reshape(-1), mn, mx, bw,
                                                  int(shift_to_signed), seed)
        return out

    def qdq_per_channel_stochastic(self, x, num_channel, n_per_channel, params, seed):
        x = _f32(x)
        out = np.empty_like(x)
        mn, mx, d, o = (_f32(p).copy() for p in params)
        self.L.ref_qdq_per_channel_stochastic(x.reshape(-1), num_channel, x.size, n_per_channel, out.reshape(-1), mn,
                                              mx, d, o, seed)
        return out

    def qdq_per_channel(self, x, num_channel, n_per_channel, params):
        x = _f32(x)
        out = np.empty_like(x)
        self.L.ref_qdq_per_channel(x.reshape(-1), num_channel, x.size, n_per_channel, out.reshape(-1),
                                   *[_f32(p).copy() for p in params])
        return out

    def qdq_broadcast(self, x, input_strides, encoding_strides, params):
        x = _f32(x)
        out = np.empty_like(x)
        ist = np.ascontiguousarray(input_strides, dtype=np.int64)
        est = np.ascontiguousarray(encoding_strides, dtype=np.int64)
        self.L.ref_qdq_broadcast(x.reshape(-1), out.reshape(-1), x.size, ist.size, ist, est,
                                 *[_f32(p) for p in params])
        return out

    def new_tf(self):
        return _RefAnalyzer(self, enhanced=False)

    def new_tfe(self):
        return _RefAnalyzer(self, enhanced=True)

    def new_percentile(self, percentile):
        return _RefPercentile(self, percentile)

    def new_mse(self):
        return _RefMse(self)

    def new_entropy(self):
        return _RefEntropy(self)


class _RefAnalyzer:
    def __init__(self, ref, enhanced):
        self.r = ref
        self.enh = enhanced
        self.h = C.c_void_p(ref.L.ref_tfe_create() if enhanced else ref.L.ref_tf_create())

    def __del__(self):
        if getattr(self, "h", None):
            (self.r.L.ref_tfe_destroy if self.enh else self.r.L.ref_tf_destroy)(self.h)
            self.h = None

    def update(self, x):
        x = _f32(x)
        (self.r.L.ref_tfe_update if self.enh else self.r.L.ref_tf_update)(self.h, x.reshape(-1), x.size)

    def compute_encoding(self, bw, sym=False, strict=False, unsigned_sym=False):
        o = np.empty(5)
        fn = self.r.L.ref_tfe_compute if self.enh else self.r.L.ref_tf_compute
        fn(self.h, bw, int(sym), int(strict), int(unsigned_sym), o)
        return _Ref._enc(o)

    def pdf(self):
        xl, p = np.zeros(PDF_SIZE), np.zeros(PDF_SIZE)
        it = C.c_int(0)
        n = self.r.L.ref_tfe_get_pdf(self.h, xl, p, C.byref(it))
        return n, xl, p, it.value

    def find_range(self):
        a, b = C.c_float(), C.c_float()
        self.r.L.ref_tfe_range(self.h, C.byref(a), C.byref(b))
        return np.float32(a.value), np.float32(b.value)

    def candidates(self, bw, sym=False, strict=False, unsigned_sym=False):
        d = np.empty(512, np.float32)
        off = np.empty(512, np.int32)
        costs = np.empty(512, np.float64)
        n = self.r.L.ref_tfe_candidates(self.h, bw, int(sym), int(strict), int(unsigned_sym), 512, d, off, costs)
        return d[:n].copy(), off[:n].copy(), costs[:n].copy()


class _RefPercentile:
    """The reference's PercentileEncodingAnalyzer<float>, compiled in place."""

    def __init__(self, ref, percentile):
        L = self.L = ref.L
        L.ref_pct_create.restype = C.c_void_p
        L.ref_pct_create.argtypes = [C.c_float]
        L.ref_pct_destroy.argtypes = [C.c_void_p]
        L.ref_pct_update.argtypes = [C.c_void_p, _f32p, _i64]
        L.ref_pct_compute.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, _f64p]
        self.h = C.c_void_p(L.ref_pct_create(percentile))

    def __del__(self):
        if getattr(self, "h", None):
            self.L.ref_pct_destroy(self.h)
            self.h = None

    def update(self, x):
        x = _f32(x)
        self.L.ref_pct_update(self.h, x.reshape(-1), x.size)

    def compute_encoding(self, bw, sym=False, strict=False, unsigned_sym=False):
        o = np.empty(5)
        self.L.ref_pct_compute(self.h, bw, int(sym), int(strict), int(unsigned_sym), o)
        return _Ref._enc(o)


class _RefMse:
    """The reference's MseEncodingAnalyzer<float>, compiled in place."""

    def __init__(self, ref):
        L = self.L = ref.L
        L.ref_mse_create.restype = C.c_void_p
        L.ref_mse_create.argtypes = []
        L.ref_mse_destroy.argtypes = [C.c_void_p]
        L.ref_mse_update.argtypes = [C.c_void_p, _f32p, _i64]
        L.ref_mse_compute.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, _f64p]
        L.ref_mse_minimize.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float),
                                       C.POINTER(C.c_float)]
        L.ref_mse_cost.restype = C.c_float
        L.ref_mse_cost.argtypes = [C.c_void_p, C.c_int, _f32p, _f32p, C.c_int, C.c_float, C.c_float, C.c_int, C.c_int,
                                   C.c_int]
        self.h = C.c_void_p(L.ref_mse_create())

    def __del__(self):
        if getattr(self, "h", None):
            self.L.ref_mse_destroy(self.h)
            self.h = None

    def update(self, x):
        x = _f32(x)
        self.L.ref_mse_update(self.h, x.reshape(-1), x.size)

    def compute_encoding(self, bw, sym=False, strict=False, unsigned_sym=False):
        o = np.empty(5)
        self.L.ref_mse_compute(self.h, bw, int(sym), int(strict), int(unsigned_sym), o)
        return _Ref._enc(o)

    def minimize(self, bw, sym=False, strict=False, unsigned_sym=False):
        a, b = C.c_float(), C.c_float()
        self.L.ref_mse_minimize(self.h, bw, int(sym), int(strict), int(unsigned_sym), C.byref(a), C.byref(b))
        return np.float32(a.value), np.float32(b.value)

    def cost(self, bw, centers, pdf_at_center, cand_min, cand_max, sym=False, strict=False, unsigned_sym=False):
        centers, pdf_at_center = _f32(centers), _f32(pdf_at_center)
        return np.float32(self.L.ref_mse_cost(self.h, bw, centers, pdf_at_center, centers.size, cand_min, cand_max,
                                              int(sym), int(strict), int(unsigned_sym)))


class _RefEntropy:
    """The reference's EntropyEncodingAnalyzer<float>, compiled in place."""

    def __init__(self, ref):
        L = self.L = ref.L
        L.ref_entropy_create.restype = C.c_void_p
        L.ref_entropy_create.argtypes = []
        L.ref_entropy_destroy.argtypes = [C.c_void_p]
        L.ref_entropy_update.argtypes = [C.c_void_p, _f32p, _i64]
        L.ref_entropy_compute.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, _f64p]
        L.ref_entropy_get_histogram.argtypes = [C.c_void_p, _f64p, _f64p, C.POINTER(C.c_int)]
        L.ref_entropy_optimize.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_float),
                                           C.POINTER(C.c_float)]
        self.h = C.c_void_p(L.ref_entropy_create())

    def __del__(self):
        if getattr(self, "h", None):
            self.L.ref_entropy_destroy(self.h)
            self.h = None

    def update(self, x):
        x = _f32(x)
        self.L.ref_entropy_update(self.h, x.reshape(-1), x.size)

    def compute_encoding(self, bw, sym=False, strict=False, unsigned_sym=False):
        o = np.empty(5)
        self.L.ref_entropy_compute(self.h, bw, int(sym), int(strict), int(unsigned_sym), o)
        return _Ref._enc(o)

    def histogram(self):
        """(number of bins, histogram, (min, max), iterations)"""
        hist, mm, it = np.zeros(PDF_SIZE), np.zeros(2), C.c_int(0)
        n = self.L.ref_entropy_get_histogram(self.h, hist, mm, C.byref(it))
        return n, hist, (mm[0], mm[1]), it.value

    def optimize(self, bw, sym=False, strict=False, unsigned_sym=False):
        a, b = C.c_float(), C.c_float()
        self.L.ref_entropy_optimize(self.h, bw, int(sym), int(strict), int(unsigned_sym), C.byref(a), C.byref(b))
        return np.float32(a.value), np.float32(b.value)


def _load():
    if not os.path.exists(_ORACLE_SO):
        build(with_ref=True)
    return _Oracle(_ORACLE_SO)


lib = _load()
ref = _Ref(_REF_SO) if os.path.exists(_REF_SO) else None
