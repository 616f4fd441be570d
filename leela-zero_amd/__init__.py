"""Python face of liblzhip: the MI355X network-forward backend for Leela Zero.

The classes mirror the reference's C++ interface for this path
(reference src/ForwardPipe.h:38-71): a pipe is `initialize`d with the filter
count, receives `push_weights`, and then answers `forward` calls.  All compute
happens in the HIP library; there is no CPU fallback -- if the library is not
built or no gfx950 device is present the calls raise.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "liblzhip.so")

FP32 = 0
FP16 = 1
OK, EINVAL, EDEVICE, EHALT, ENOMEM = 0, -1, -2, -3, -4

BOARD = 19
NPTS = 361
INPUT_CHANNELS = 18
INPUT_SIZE = 18 * 361
POL_SIZE = 2 * 361
VAL_SIZE = 361
MOVES = 362
VALUE_LAYER = 256
WINOGRAD_ALPHA = 6

K_PACK, K_IN, K_GEMM, K_OUT, K_HEAD, K_OUTIN, K_COUNT = 0, 1, 2, 3, 4, 5, 6
KERNEL_CLASSES = ["pack_input", "in_transform", "gemm", "out_transform", "head_conv",
                  "out_in_transform"]

# Every symbol include/lzhip.h declares.
EXPORTS = [
    "lzhip_create", "lzhip_create_from_file", "lzhip_destroy", "lzhip_push_weights", "lzhip_forward",
    "lzhip_forward_batch", "lzhip_forward_batch_device", "lzhip_lanes",
    "lzhip_forward_batch_device_lane", "lzhip_forward_batch_device_noalloc", "lzhip_sync", "lzhip_stream",
    "lzhip_drain", "lzhip_resume", "lzhip_get_stats", "lzhip_reset_stats",
    "lzhip_process_batch_stats", "lzhip_push_heads",
    "lzhip_evaluate_batch", "lzhip_timed_evaluations", "lzhip_forward_eval", "lzhip_winograd_transform_f", "lzhip_process_bn_var",
    "lzhip_ceil_multiple",
    "lzhip_debug_layer", "lzhip_get_act_scales", "lzhip_profile_forward", "lzhip_last_error",
    "lzhip_version",
]
# Every symbol include/lzhip_search.h declares.
SEARCH_EXPORTS = [
    "lzhip_symmetry_index", "lzhip_gather_features", "lzhip_get_output",
    "lzhip_get_output_average", "lzhip_netbench", "lzhip_set_value_head_not_stm",
    "lzhip_search_default_config", "lzhip_selfplay", "lzhip_board_replay",
]

BLACK, WHITE, EMPTY, PASS = 0, 1, 2, 361


def process_batch_stats():
    """The process-wide counters the engine prints after a search (reference
    src/UCTSearch.cpp:855-860): batches of one position, batches of more, positions
    evaluated, batch slots offered."""
    out = (ctypes.c_uint64 * 4)()
    _check(lib().lzhip_process_batch_stats(out))
    return dict(single_evals=int(out[0]), batch_evals=int(out[1]), positions=int(out[2]),
                slots=int(out[3]))


class NetworkHaltException(Exception):
    """forward() was woken by drain() (reference src/Network.h:66-67)."""


class LzhipError(RuntimeError):
    pass


class Stats(ctypes.Structure):
    _fields_ = [("requests", ctypes.c_uint64), ("batches", ctypes.c_uint64),
                ("batch_slots", ctypes.c_uint64), ("halted", ctypes.c_uint64),
                ("max_batch_seen", ctypes.c_uint32), ("max_batch", ctypes.c_uint32)]


_lib = None
_fp = ctypes.POINTER(ctypes.c_float)
_fpp = ctypes.POINTER(_fp)
_u8p = ctypes.POINTER(ctypes.c_uint8)
_ip = ctypes.POINTER(ctypes.c_int)


class CHeadWeights(ctypes.Structure):
    """lzhip_head_weights of include/lzhip_search.h."""
    _fields_ = [(n, _fp) for n in ["bn_pol_mean", "bn_pol_scale", "ip_pol_w", "ip_pol_b",
                                   "bn_val_mean", "bn_val_scale", "ip1_val_w", "ip1_val_b",
                                   "ip2_val_w", "ip2_val_b"]]


class SearchConfig(ctypes.Structure):
    """lzhip_search_config; SearchConfig.default() holds the engine's defaults."""
    _fields_ = [("threads", ctypes.c_int), ("visits", ctypes.c_int), ("moves", ctypes.c_int),
                ("cache_size", ctypes.c_int), ("reuse_tree", ctypes.c_int),
                ("random_moves", ctypes.c_int), ("virtual_loss", ctypes.c_int),
                ("device_heads", ctypes.c_int),
                ("puct", ctypes.c_float), ("logpuct", ctypes.c_float),
                ("logconst", ctypes.c_float), ("fpu_reduction", ctypes.c_float),
                ("fpu_root_reduction", ctypes.c_float),
                ("softmax_temp", ctypes.c_float), ("komi", ctypes.c_float),
                ("seed", ctypes.c_uint64)]

    @classmethod
    def default(cls, **kw):
        cfg = cls()
        _check(lib().lzhip_search_default_config(ctypes.byref(cfg)))
        for k, v in kw.items():
            if k not in dict(cls._fields_):
                raise ValueError("unknown search option %r" % k)
            setattr(cfg, k, v)
        return cfg


class SearchResult(ctypes.Structure):
    _fields_ = [("playouts", ctypes.c_uint64), ("wasted", ctypes.c_uint64),
                ("halted", ctypes.c_uint64), ("evals", ctypes.c_uint64),
                ("cache_lookups", ctypes.c_uint64), ("cache_hits", ctypes.c_uint64),
                ("nodes", ctypes.c_uint64), ("seconds", ctypes.c_double),
                ("visits_per_s", ctypes.c_double), ("moves_played", ctypes.c_int),
                ("passes_at_end", ctypes.c_int), ("final_score", ctypes.c_float),
                ("sched", Stats)]


def lib():
    """The loaded shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LzhipError("%s is missing: run __graft_entry__.build() (hipcc) first; "
                             "there is no fallback implementation" % LIB_PATH)
        # A process that also uses torch-ROCm must hold ONE HIP runtime: torch ships its
        # own copy, and whichever copy is loaded second finds no devices.  Loading
        # torch first makes this library bind to torch's copy (same SONAME).
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = ctypes.CDLL(LIB_PATH)
        L.lzhip_last_error.restype = ctypes.c_char_p
        L.lzhip_version.restype = ctypes.c_char_p
        L.lzhip_stream.restype = ctypes.c_void_p
        L.lzhip_stream.argtypes = [ctypes.c_void_p]
        L.lzhip_create.argtypes = [ctypes.c_int] * 4 + [ctypes.POINTER(ctypes.c_void_p)]
        L.lzhip_create_from_file.argtypes = [ctypes.c_char_p, ctypes.c_int, ctypes.c_int,
                                             ctypes.c_int, ctypes.POINTER(ctypes.c_void_p),
                                             ctypes.POINTER(ctypes.c_int),
                                             ctypes.POINTER(ctypes.c_int)]
        L.lzhip_destroy.argtypes = [ctypes.c_void_p]
        L.lzhip_push_weights.argtypes = [ctypes.c_void_p, ctypes.c_int, _fpp, _fpp, _fpp, _fp, _fp]
        L.lzhip_forward.argtypes = [ctypes.c_void_p, _fp, _fp, _fp]
        L.lzhip_forward_batch.argtypes = [ctypes.c_void_p, ctypes.c_int, _fp, _fp, _fp]
        L.lzhip_forward_batch_device.argtypes = [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 3
        L.lzhip_forward_batch_device_noalloc.argtypes = ([ctypes.c_void_p, ctypes.c_int]
                                                        + [ctypes.c_void_p] * 3)
        L.lzhip_lanes.argtypes = [ctypes.c_void_p]
        L.lzhip_forward_batch_device_lane.argtypes = ([ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
                                                      + [ctypes.c_void_p] * 3)
        L.lzhip_sync.argtypes = [ctypes.c_void_p]
        L.lzhip_drain.argtypes = [ctypes.c_void_p]
        L.lzhip_resume.argtypes = [ctypes.c_void_p]
        L.lzhip_get_stats.argtypes = [ctypes.c_void_p, ctypes.POINTER(Stats)]
        L.lzhip_reset_stats.argtypes = [ctypes.c_void_p]
        L.lzhip_process_batch_stats.argtypes = [ctypes.POINTER(ctypes.c_uint64)]
        L.lzhip_push_heads.argtypes = [ctypes.c_void_p] + [_fp] * 10
        L.lzhip_evaluate_batch.argtypes = [ctypes.c_void_p, ctypes.c_int, _fp, ctypes.c_float] + [_fp] * 5
        L.lzhip_forward_eval.argtypes = [ctypes.c_void_p, _fp, ctypes.c_float, _fp, _fp]
        L.lzhip_timed_evaluations.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, _fp,
                                              ctypes.c_float, _fp, _fp, _fp]
        L.lzhip_winograd_transform_f.argtypes = [_fp, ctypes.c_int, ctypes.c_int, _fp]
        L.lzhip_process_bn_var.argtypes = [_fp, ctypes.c_int]
        L.lzhip_ceil_multiple.argtypes = [ctypes.c_size_t, ctypes.c_size_t]
        L.lzhip_ceil_multiple.restype = ctypes.c_size_t
        L.lzhip_debug_layer.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int] + [_fp] * 5
        L.lzhip_get_act_scales.argtypes = [ctypes.c_void_p, _fp, ctypes.c_int]
        L.lzhip_profile_forward.argtypes = [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 3 + \
            [_fp, ctypes.POINTER(ctypes.c_int)]
        L.lzhip_symmetry_index.argtypes = [ctypes.c_int, ctypes.c_int]
        L.lzhip_gather_features.argtypes = [_u8p, ctypes.c_int, ctypes.c_int, ctypes.c_int, _fp]
        L.lzhip_get_output.argtypes = [ctypes.c_void_p, ctypes.POINTER(CHeadWeights), _u8p,
                                       ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_float,
                                       _fp, _fp]
        L.lzhip_get_output_average.argtypes = [ctypes.c_void_p, ctypes.POINTER(CHeadWeights), _u8p,
                                               ctypes.c_int, ctypes.c_int, ctypes.c_float, _fp, _fp]
        L.lzhip_set_value_head_not_stm.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.lzhip_netbench.argtypes = [ctypes.c_void_p, ctypes.POINTER(CHeadWeights), _u8p,
                                     ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                     ctypes.c_uint64, ctypes.POINTER(ctypes.c_int),
                                     ctypes.POINTER(ctypes.c_double)]
        L.lzhip_search_default_config.argtypes = [ctypes.POINTER(SearchConfig)]
        L.lzhip_selfplay.argtypes = [ctypes.c_void_p, ctypes.POINTER(CHeadWeights),
                                     ctypes.POINTER(SearchConfig), ctypes.POINTER(SearchResult),
                                     _ip, ctypes.c_int]
        L.lzhip_board_replay.argtypes = [_ip, ctypes.c_int, ctypes.c_float, _u8p, _u8p, _ip, _ip,
                                         _fp]
        _lib = L
    return _lib


def _check(rc):
    if rc == OK:
        return
    msg = lib().lzhip_last_error().decode("utf-8", "replace")
    if rc == EHALT:
        raise NetworkHaltException(msg)
    if rc == EINVAL:
        raise ValueError(msg)
    raise LzhipError("lzhip error %d: %s" % (rc, msg))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a):
    return a.ctypes.data_as(_fp) if a is not None else None


def winograd_transform_f(f, outputs, channels):
    """reference src/Network.cpp:159-223: f[o][c][3][3] -> U[36][c][o]."""
    f = _f32(f).reshape(outputs, channels, 3, 3)
    U = np.empty((36, channels, outputs), dtype=np.float32)
    _check(lib().lzhip_winograd_transform_f(_ptr(f), outputs, channels, _ptr(U)))
    return U


def ceil_multiple(a, b):
    """reference src/Utils.cpp:208-215: a rounded up to a multiple of b."""
    return int(lib().lzhip_ceil_multiple(a, b))


def process_bn_var(var):
    """reference src/Network.cpp:151-157: var -> 1/sqrt(var + 1e-5)."""
    w = _f32(var).copy()
    _check(lib().lzhip_process_bn_var(_ptr(w), w.size))
    return w


def symmetry_index(symmetry, idx):
    """Board index read by NN index `idx` under `symmetry` (reference
    src/Network.cpp:518-531, :968-993)."""
    r = lib().lzhip_symmetry_index(int(symmetry), int(idx))
    if r < 0:
        raise ValueError("symmetry in 0..7 and idx in 0..360 expected")
    return r


def _boards(boards):
    b = np.ascontiguousarray(boards, dtype=np.uint8).reshape(-1, NPTS)
    return b, b.ctypes.data_as(_u8p)


def gather_features(boards, to_move, symmetry=0):
    """Network::gather_features (reference src/Network.cpp:935-966): boards
    [n<=8][361] newest first with BLACK/WHITE/EMPTY -> planes [18][361]."""
    b, bp = _boards(boards)
    out = np.empty((INPUT_CHANNELS, NPTS), dtype=np.float32)
    _check(lib().lzhip_gather_features(bp, b.shape[0], int(to_move), int(symmetry), _ptr(out)))
    return out


def board_replay(moves, komi=7.5):
    """Replays a move list from the empty board with the driver's Go rules and
    returns dict(stones[361], legal[362], ko_point, superko, score)."""
    mv = np.ascontiguousarray(moves, dtype=np.int32).reshape(-1)
    stones = np.empty(NPTS, dtype=np.uint8)
    legal = np.empty(MOVES, dtype=np.uint8)
    ko, sk, score = ctypes.c_int(), ctypes.c_int(), ctypes.c_float()
    _check(lib().lzhip_board_replay(mv.ctypes.data_as(_ip), mv.size, float(komi),
                                    stones.ctypes.data_as(_u8p), legal.ctypes.data_as(_u8p),
                                    ctypes.byref(ko), ctypes.byref(sk), ctypes.byref(score)))
    return {"stones": stones, "legal": legal.astype(bool), "ko_point": ko.value,
            "superko": bool(sk.value), "score": score.value}


def _c_heads(heads):
    """(pointer argument, keep-alive objects) for a HeadWeights-like object; None
    stands for the parameters given to push_heads."""
    if heads is None:
        return None, None
    arrs, c = [], CHeadWeights()
    for name, size in zip(HeadWeights.FIELDS, HeadWeights.SIZES):
        a = _f32(getattr(heads, name)).reshape(-1)
        if a.size != size:
            raise ValueError("%s must have %d values" % (name, size))
        arrs.append(a)
        setattr(c, name, _ptr(a))
    return ctypes.byref(c), (c, arrs)


class ForwardPipeWeights:
    """reference src/ForwardPipe.h:40-54 with numpy arrays."""

    def __init__(self):
        self.m_conv_weights = []       # U[l]: [36][C_in][F]
        self.m_conv_biases = []        # zero after folding
        self.m_batchnorm_means = []    # [F], bias folded in
        self.m_batchnorm_stddevs = []  # [F], 1/sqrt(var+eps)
        self.m_conv_pol_w = None       # [2][F]
        self.m_conv_pol_b = None
        self.m_conv_val_w = None       # [F]
        self.m_conv_val_b = None


class HeadWeights:
    """Head parameters as Network holds them (reference src/Network.h:166-183),
    after process_bn_var and bias folding (src/Network.cpp:351-352,568-576)."""
    FIELDS = ["bn_pol_mean", "bn_pol_scale", "ip_pol_w", "ip_pol_b", "bn_val_mean",
              "bn_val_scale", "ip1_val_w", "ip1_val_b", "ip2_val_w", "ip2_val_b"]
    SIZES = [2, 2, 362 * 722, 362, 1, 1, 256 * 361, 256, 256, 1]


class HIPScheduler:
    """ForwardPipe on one MI355X (the place of OpenCLScheduler<net_t>,
    reference src/OpenCLScheduler.h:51-118).  `precision` plays the role of the
    net_t template argument, `max_batch` of cfg_batch_size."""

    def __init__(self, precision=FP32, max_batch=1, device=0):
        self.precision = int(precision)
        self.max_batch = int(max_batch)
        self.device = int(device)
        self._h = None
        self.n_layers = 0
        self.filters = 0
        self._keep = None

    @classmethod
    def from_file(cls, path, precision=FP16, max_batch=1, device=0):
        """Network::initialize from a weights file (reference src/Network.cpp:225-405,
        :540-576): plain or gzip text, format 1 or 2; tower and head parameters are
        pushed, so `heads=None` works in the callers above forward()."""
        self = cls(precision, max_batch, device)
        h = ctypes.c_void_p()
        f, b = ctypes.c_int(), ctypes.c_int()
        _check(lib().lzhip_create_from_file(os.fsencode(path), self.precision, self.max_batch,
                                            self.device, ctypes.byref(h), ctypes.byref(f),
                                            ctypes.byref(b)))
        self._h = h
        self.filters = f.value
        self.n_layers = 1 + 2 * b.value
        return self

    # -- ForwardPipe interface -------------------------------------------
    def initialize(self, channels):
        if self._h is not None:
            raise ValueError("initialize called twice")
        h = ctypes.c_void_p()
        _check(lib().lzhip_create(int(channels), self.precision, self.max_batch, self.device,
                                  ctypes.byref(h)))
        self._h = h
        self.filters = int(channels)

    def needs_autodetect(self):
        return False

    def push_weights(self, filter_size, channels, outputs, weights):
        self._need()
        if filter_size != WINOGRAD_ALPHA or channels != INPUT_CHANNELS or outputs != self.filters:
            raise ValueError("push_weights(6, 18, filters, weights) expected")
        nl = len(weights.m_conv_weights)
        U, mean, scale = [], [], []
        for l in range(nl):
            cin = channels if l == 0 else outputs
            u = _f32(weights.m_conv_weights[l])
            if u.size != 36 * cin * outputs:
                raise ValueError("layer %d: wrong filter size" % l)
            m, s = _f32(weights.m_batchnorm_means[l]), _f32(weights.m_batchnorm_stddevs[l])
            if m.size != outputs or s.size != outputs:
                raise ValueError("layer %d: wrong batch-norm size" % l)
            U.append(u); mean.append(m); scale.append(s)
        pw, vw = _f32(weights.m_conv_pol_w), _f32(weights.m_conv_val_w)
        if pw.size != 2 * outputs or vw.size != outputs:
            raise ValueError("head convolutions have the wrong size")
        arr = lambda xs: (_fp * nl)(*[_ptr(x) for x in xs])
        _check(lib().lzhip_push_weights(self._h, nl, arr(U), arr(mean), arr(scale), _ptr(pw), _ptr(vw)))
        self.n_layers = nl

    def forward(self, input):
        """One position through the batching queue: in[6498] -> (pol[722], val[361])."""
        self._need()
        x = _f32(input).reshape(-1)
        if x.size != INPUT_SIZE:
            raise ValueError("input must have 18*361 values")
        pol = np.empty(POL_SIZE, dtype=np.float32)
        val = np.empty(VAL_SIZE, dtype=np.float32)
        _check(lib().lzhip_forward(self._h, _ptr(x), _ptr(pol), _ptr(val)))
        return pol, val

    def drain(self):
        self._need()
        _check(lib().lzhip_drain(self._h))

    def resume(self):
        self._need()
        _check(lib().lzhip_resume(self._h))

    # -- the executor under the queue ---------------------------------------
    def forward_batch(self, inputs):
        """n <= max_batch positions, host arrays: [n][18][361] -> ([n][722], [n][361])."""
        self._need()
        x = _f32(inputs).reshape(-1, INPUT_SIZE)
        n = x.shape[0]
        pol = np.empty((n, POL_SIZE), dtype=np.float32)
        val = np.empty((n, VAL_SIZE), dtype=np.float32)
        _check(lib().lzhip_forward_batch(self._h, n, _ptr(x), _ptr(pol), _ptr(val)))
        return pol, val

    def lanes(self):
        """Number of lanes (streams with their own working buffers) of the handle."""
        self._need()
        return lib().lzhip_lanes(self._h)

    def forward_batch_device(self, n, d_in, d_pol, d_val, lane=0):
        """Asynchronous forward on device pointers (ints) on one lane; see sync().
        Forwards on different lanes run side by side and need buffers of their own."""
        self._need()
        _check(lib().lzhip_forward_batch_device_lane(self._h, int(lane), int(n), d_in, d_pol,
                                                     d_val))

    def forward_batch_device_noalloc(self, n, d_in, d_pol, d_val):
        """forward_batch_device on lane 0 with the working buffers in the library's static
        device array: no allocation on the way.  n <= 8, up to 256 filters."""
        self._need()
        _check(lib().lzhip_forward_batch_device_noalloc(self._h, int(n), d_in, d_pol, d_val))

    def sync(self):
        self._need()
        _check(lib().lzhip_sync(self._h))

    def stream(self):
        self._need()
        return lib().lzhip_stream(self._h)

    def profile_forward(self, n, d_in, d_pol, d_val):
        """Per-kernel-class device time (ms) and launch counts of one forward."""
        self._need()
        ms = np.zeros(K_COUNT, dtype=np.float32)
        cnt = (ctypes.c_int * K_COUNT)()
        _check(lib().lzhip_profile_forward(self._h, int(n), d_in, d_pol, d_val, _ptr(ms), cnt))
        return ms, np.array(list(cnt), dtype=np.int64)

    def stats(self):
        self._need()
        s = Stats()
        _check(lib().lzhip_get_stats(self._h, ctypes.byref(s)))
        return {k: int(getattr(s, k)) for k, _ in Stats._fields_}

    def reset_stats(self):
        self._need()
        _check(lib().lzhip_reset_stats(self._h))

    def act_scales(self):
        self._need()
        out = np.empty(self.n_layers + 1, dtype=np.float32)
        _check(lib().lzhip_get_act_scales(self._h, _ptr(out), out.size))
        return out

    # -- heads on the device --------------------------------------------------
    def push_heads(self, heads):
        self._need()
        arrs = []
        for name, size in zip(HeadWeights.FIELDS, HeadWeights.SIZES):
            a = _f32(getattr(heads, name)).reshape(-1)
            if a.size != size:
                raise ValueError("%s must have %d values" % (name, size))
            arrs.append(a)
        _check(lib().lzhip_push_heads(self._h, *[_ptr(a) for a in arrs]))

    def forward_eval(self, input, temperature=1.0):
        """One position through the batching queue with the heads computed on the
        device: returns (policy[362] in NN index order, value = tanh output)."""
        self._need()
        x = _f32(input).reshape(-1)
        if x.size != INPUT_SIZE:
            raise ValueError("input must have 18*361 values")
        policy = np.empty(MOVES, dtype=np.float32)
        value = ctypes.c_float()
        _check(lib().lzhip_forward_eval(self._h, _ptr(x), float(temperature), _ptr(policy),
                                        ctypes.byref(value)))
        return policy, value.value

    def evaluate_batch(self, inputs, temperature=1.0, want_raw=False):
        """Tower + heads: returns policy [n][362], value [n] (tanh), logits [n][362]
        (and the raw pol/val planes when want_raw)."""
        self._need()
        x = _f32(inputs).reshape(-1, INPUT_SIZE)
        n = x.shape[0]
        policy = np.empty((n, MOVES), dtype=np.float32)
        value = np.empty(n, dtype=np.float32)
        logits = np.empty((n, MOVES), dtype=np.float32)
        pol = np.empty((n, POL_SIZE), dtype=np.float32) if want_raw else None
        val = np.empty((n, VAL_SIZE), dtype=np.float32) if want_raw else None
        _check(lib().lzhip_evaluate_batch(self._h, n, _ptr(x), float(temperature), _ptr(policy),
                                          _ptr(value), _ptr(logits), _ptr(pol), _ptr(val)))
        if want_raw:
            return policy, value, logits, pol, val
        return policy, value, logits

    def timed_evaluations(self, inputs, reps, temperature=1.0):
        """`reps` evaluations (H2D + tower + device heads + D2H) of the same batch on one
        lane between two stream events: returns (milliseconds, policy, value)."""
        self._need()
        x = _f32(inputs).reshape(-1, INPUT_SIZE)
        n = x.shape[0]
        policy = np.empty((n, MOVES), dtype=np.float32)
        value = np.empty(n, dtype=np.float32)
        ms = np.zeros(1, dtype=np.float32)
        _check(lib().lzhip_timed_evaluations(self._h, n, int(reps), _ptr(x), float(temperature),
                                             _ptr(policy), _ptr(value), _ptr(ms)))
        return float(ms[0]), policy, value

    # -- callers above forward() ------------------------------------------------
    def get_output(self, heads, boards, to_move, symmetry=0, temperature=1.0):
        """Network::get_output_internal for one position (reference
        src/Network.cpp:811-864): returns (policy[362] in board order, winrate)."""
        self._need()
        c, keep = _c_heads(heads)
        b, bp = _boards(boards)
        policy = np.empty(MOVES, dtype=np.float32)
        win = ctypes.c_float()
        _check(lib().lzhip_get_output(self._h, c, bp, b.shape[0], int(to_move),
                                      int(symmetry), float(temperature), _ptr(policy),
                                      ctypes.byref(win)))
        del keep
        return policy, win.value

    def set_value_head_not_stm(self, on):
        """Network::m_value_head_not_stm (weights-file format 2, reference
        src/Network.cpp:395-400, :797-802): the value head speaks for black; get_output,
        get_output_average and the search turn it round when white is to move."""
        self._need()
        _check(lib().lzhip_set_value_head_not_stm(self._h, 1 if on else 0))

    def netbench(self, heads, boards, to_move, threads, iterations, seed=1):
        """Network::benchmark (reference src/Network.cpp:128-149, GTP `netbench`): `threads`
        threads evaluate the position under random symmetries, cache off, until
        `iterations` evaluations have been started.  Returns (evaluations, seconds)."""
        self._need()
        c, keep = _c_heads(heads)
        b, bp = _boards(boards)
        done = ctypes.c_int()
        secs = ctypes.c_double()
        _check(lib().lzhip_netbench(self._h, c, bp, b.shape[0], int(to_move), int(threads),
                                    int(iterations), int(seed), ctypes.byref(done),
                                    ctypes.byref(secs)))
        del keep
        return done.value, secs.value

    def get_output_average(self, heads, boards, to_move, temperature=1.0):
        """Network::get_output with Ensemble::AVERAGE (reference
        src/Network.cpp:762-775): mean over the 8 symmetries, evaluated as one
        device batch.  Returns (policy[362], winrate)."""
        self._need()
        c, keep = _c_heads(heads)
        b, bp = _boards(boards)
        policy = np.empty(MOVES, dtype=np.float32)
        win = ctypes.c_float()
        _check(lib().lzhip_get_output_average(self._h, c, bp, b.shape[0],
                                              int(to_move), float(temperature), _ptr(policy),
                                              ctypes.byref(win)))
        del keep
        return policy, win.value

    def selfplay(self, heads, cfg):
        """Multi-threaded tree search self-play against this backend; returns
        (SearchResult, moves)."""
        self._need()
        c, keep = _c_heads(heads)
        res = SearchResult()
        moves = (ctypes.c_int * max(int(cfg.moves), 1))()
        _check(lib().lzhip_selfplay(self._h, c, ctypes.byref(cfg), ctypes.byref(res),
                                    moves, len(moves)))
        del keep
        return res, list(moves)[:res.moves_played]

    # -- introspection ----------------------------------------------------------
    def debug_layer(self, layer, act_in, res=None):
        """One conv layer, every stage in the reference's layouts:
        act_in [n][C_in][361] -> V [n][36][C_in][25], M [n][36][F][25], Y [n][F][361]."""
        self._need()
        cin = INPUT_CHANNELS if layer == 0 else self.filters
        a = _f32(act_in).reshape(-1, cin, NPTS)
        n = a.shape[0]
        r = None if res is None else _f32(res).reshape(n, self.filters, NPTS)
        V = np.empty((n, 36, cin, 25), dtype=np.float32)
        M = np.empty((n, 36, self.filters, 25), dtype=np.float32)
        Y = np.empty((n, self.filters, NPTS), dtype=np.float32)
        _check(lib().lzhip_debug_layer(self._h, int(layer), n, _ptr(a), _ptr(r), _ptr(V), _ptr(M), _ptr(Y)))
        return V, M, Y

    def close(self):
        if self._h is not None:
            lib().lzhip_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _need(self):
        if self._h is None:
            raise ValueError("initialize() has not been called")


def version():
    return lib().lzhip_version().decode()
