"""ctypes wrapper of the CPU oracle (oracle/lz_oracle.c).

TEST INFRASTRUCTURE: imported only by tests/, by __graft_entry__.smoke() and
by bench.py's cpu_baseline leg, always as the checker or the reported CPU
baseline, never by the product library.
"""
import ctypes
import glob
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
# LZ_ORACLE_LIB: another build of lz_oracle.c to load instead (the test that compares an
# -ffast-math build, the reference's own compiler setting, with this IEEE one)
LIB_PATH = os.environ.get("LZ_ORACLE_LIB") or os.path.join(HERE, "liblzoracle.so")
_fp = ctypes.POINTER(ctypes.c_float)
_lib = None


def build():
    subprocess.run(["make", "-C", HERE, "-B", "liblzoracle.so"], check=True, capture_output=True)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        L.lzo_benchmark.restype = ctypes.c_double
        L.lzo_blas_name.restype = ctypes.c_char_p
        L.lzo_use_blas.argtypes = [ctypes.c_char_p]
        _lib = L
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(_fp) if a is not None else None


def use_openblas():
    """Bind scipy's bundled OpenBLAS for the 36 GEMMs (single-threaded per call, as
    the reference sets it, src/Network.cpp:499).  Returns the provider name."""
    pats = ["/usr/local/lib/python3*/dist-packages/scipy.libs/libscipy_openblas*.so",
            "/usr/lib/python3*/site-packages/scipy.libs/libscipy_openblas*.so"]
    try:
        import scipy
        pats.insert(0, os.path.join(os.path.dirname(os.path.dirname(scipy.__file__)),
                                    "scipy.libs", "libscipy_openblas*.so"))
    except Exception:
        pass
    for pat in pats:
        for path in sorted(glob.glob(pat)):
            if "64_" in os.path.basename(path):
                continue  # ILP64 build: different integer width
            if lib().lzo_use_blas(path.encode()):
                return blas_name()
    return blas_name()


def use_builtin():
    lib().lzo_use_builtin()


def blas_name():
    return lib().lzo_blas_name().decode()


def winograd_transform_f(f, outputs, channels):
    f = _f32(f).reshape(outputs, channels, 3, 3)
    U = np.empty((36, channels, outputs), np.float32)
    lib().lzo_winograd_transform_f(_p(f), outputs, channels, _p(U))
    return U


def process_bn_var(v):
    w = _f32(v).copy()
    lib().lzo_process_bn_var(_p(w), w.size)
    return w


def transform_in(x, C):
    x = _f32(x).reshape(C, 361)
    V = np.empty((36, C, 25), np.float32)
    lib().lzo_transform_in(_p(x), _p(V), C)
    return V


def sgemm(U, V, C, K):
    U, V = _f32(U), _f32(V)
    M = np.empty((36, K, 25), np.float32)
    lib().lzo_sgemm(_p(U), _p(V), _p(M), C, K)
    return M


def transform_out(M, K):
    M = _f32(M)
    Y = np.zeros((K, 361), np.float32)
    lib().lzo_transform_out(_p(M), _p(Y), K)
    return Y


def batchnorm(data, means, scales, eltwise=None):
    d = _f32(data).copy()
    ch = d.reshape(-1, 361).shape[0]
    lib().lzo_batchnorm(ch, _p(d), _p(_f32(means)), _p(_f32(scales)),
                        _p(_f32(eltwise)) if eltwise is not None else None)
    return d


def convolve1(x, w, outputs, C):
    out = np.empty((outputs, 361), np.float32)
    lib().lzo_convolve1(outputs, C, _p(_f32(x)), _p(_f32(w)), None, _p(out))
    return out


class OraclePipe:
    """CPU pipe with the ForwardPipe call order: initialize, push_weights, forward."""

    def __init__(self):
        self.filters = 0
        self.w = None

    def initialize(self, channels):
        self.filters = int(channels)

    def push_weights(self, filter_size, channels, outputs, weights):
        nl = len(weights.m_conv_weights)
        self.U = [_f32(u) for u in weights.m_conv_weights]
        self.mean = [_f32(m) for m in weights.m_batchnorm_means]
        self.scale = [_f32(s) for s in weights.m_batchnorm_stddevs]
        self.pol_w = _f32(weights.m_conv_pol_w)
        self.val_w = _f32(weights.m_conv_val_w)
        self.nl = nl
        arr = lambda xs: (_fp * nl)(*[_p(x) for x in xs])
        self._U, self._mean, self._scale = arr(self.U), arr(self.mean), arr(self.scale)

    def forward(self, x, trace=False):
        x = _f32(x).reshape(18 * 361)
        pol = np.empty(722, np.float32)
        val = np.empty(361, np.float32)
        tr = np.empty((self.nl, self.filters, 361), np.float32) if trace else None
        lib().lzo_forward_flat(self.filters, self.nl, self._U, self._mean, self._scale,
                               _p(self.pol_w), _p(self.val_w), _p(x), _p(pol), _p(val), _p(tr))
        return (pol, val, tr) if trace else (pol, val)

    def forward_many(self, xs, threads=1):
        """Independent single-position forwards on `threads` threads (the shape of
        Network::benchmark, reference src/Network.cpp:128-149).
        Returns (pol [n][722], val [n][361], seconds)."""
        xs = _f32(xs).reshape(-1, 18 * 361)
        n = xs.shape[0]
        pol = np.empty((n, 722), np.float32)
        val = np.empty((n, 361), np.float32)
        secs = lib().lzo_benchmark(self.filters, self.nl, self._U, self._mean, self._scale,
                                   _p(self.pol_w), _p(self.val_w), _p(xs), n, n, int(threads),
                                   _p(pol), _p(val))
        return pol, val, secs


def heads(h, pol, val, temperature=1.0):
    """reference src/Network.cpp:833-851.  Returns dict(policy[362], logits[362],
    value (tanh), winrate, value_pre)."""
    policy = np.empty(362, np.float32)
    logits = np.empty(362, np.float32)
    vt, wr, vp = ctypes.c_float(), ctypes.c_float(), ctypes.c_float()
    a = [_f32(getattr(h, n)) for n in
         ["bn_pol_mean", "bn_pol_scale", "ip_pol_w", "ip_pol_b", "bn_val_mean", "bn_val_scale",
          "ip1_val_w", "ip1_val_b", "ip2_val_w", "ip2_val_b"]]
    lib().lzo_heads_flat(*[_p(x) for x in a], _p(_f32(pol)), _p(_f32(val)),
                         ctypes.c_float(temperature), _p(policy), _p(logits),
                         ctypes.byref(vt), ctypes.byref(wr), ctypes.byref(vp))
    return dict(policy=policy, logits=logits, value=vt.value, winrate=wr.value,
                value_pre=vp.value)
