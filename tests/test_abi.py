"""CPU-side checks of the C-ABI library: it loads without a GPU, exports every
symbol the header declares, and its host-only entry points agree with the oracle."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(pkg):
    header = open(os.path.join(ROOT, "include", "lzhip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = sorted(set(re.findall(r"\b(lzhip_[a-z0-9_]+)\s*\(", header)))
    assert len(declared) >= 20
    L = ctypes.CDLL(pkg.LIB_PATH)
    for name in declared:
        assert hasattr(L, name), name
    assert sorted(pkg.EXPORTS) == declared


def test_library_exports_every_search_symbol(pkg):
    header = open(os.path.join(ROOT, "include", "lzhip_search.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = sorted(set(re.findall(r"\b(lzhip_[a-z0-9_]+)\s*\(", header)))
    assert len(declared) == 9
    L = ctypes.CDLL(pkg.LIB_PATH)
    for name in declared:
        assert hasattr(L, name), name
    assert sorted(pkg.SEARCH_EXPORTS) == declared
    # struct sizes the ctypes mirror assumes
    assert ctypes.sizeof(pkg.SearchConfig) == 72
    assert ctypes.sizeof(pkg.CHeadWeights) == 80
    cfg = pkg.SearchConfig.default()
    assert (cfg.threads, cfg.visits, cfg.moves, cfg.virtual_loss) == (16, 1600, 20, 3)
    assert abs(cfg.puct - 0.5) < 1e-7 and abs(cfg.komi - 7.5) < 1e-7
    assert cfg.fpu_reduction == 0.25 and cfg.fpu_root_reduction == 0.25 and cfg.seed == 1
    assert L.lzhip_selfplay(None, None, None, None, None, 0) == pkg.EINVAL
    assert L.lzhip_get_output(None, None, None, 1, 0, 0, ctypes.c_float(1.0), None, None) == pkg.EINVAL


def test_version_and_error_string(pkg):
    assert "gfx950" in pkg.version()
    assert isinstance(pkg.lib().lzhip_last_error(), bytes)


def test_null_arguments_are_rejected(pkg):
    L = pkg.lib()
    assert L.lzhip_create(64, 0, 1, 0, None) == pkg.EINVAL
    assert L.lzhip_forward(None, None, None, None) == pkg.EINVAL
    assert L.lzhip_drain(None) == pkg.EINVAL
    assert L.lzhip_destroy(None) == pkg.OK
    assert L.lzhip_winograd_transform_f(None, 1, 1, None) == pkg.EINVAL


def test_transform_f_matches_oracle(pkg, orc):
    rng = np.random.default_rng(0)
    for K, C in ((8, 18), (5, 3), (16, 16)):
        f = rng.standard_normal((K, C, 3, 3)).astype(np.float32)
        got = pkg.winograd_transform_f(f, K, C)
        want = orc.winograd_transform_f(f, K, C)
        assert got.shape == want.shape == (36, C, K)
        assert np.abs(got - want).max() <= 1e-6


def test_bn_var_matches_oracle(pkg, orc):
    v = np.random.default_rng(1).uniform(0.01, 4, 33).astype(np.float32)
    assert np.abs(pkg.process_bn_var(v) - orc.process_bn_var(v)).max() <= 1e-7


def test_ceil_multiple_known_answers(pkg):
    """The padding helper against the reference's own known answers
    (UtilsTest.CeilMultiple, src/tests/utils_unittest.cpp:47-68)."""
    cases = [(0, 1, 0), (0, 3, 0), (6, 1, 6), (23, 1, 23), (2, 2, 2), (4, 2, 4), (6, 2, 6),
             (0, 3, 0), (3, 3, 3), (9, 3, 9), (3, 5, 5), (6, 5, 10), (9, 5, 10), (23, 5, 25),
             (99, 100, 100)]
    for a, b, want in cases:
        assert pkg.ceil_multiple(a, b) == want, (a, b)
    # the paddings the pipe applies with it: filters to 64 channels, tile rows to 256
    assert pkg.ceil_multiple(18, 64) == 64 and pkg.ceil_multiple(192, 64) == 192
    assert pkg.ceil_multiple(64 * 25, 256) == 1792


def test_python_pipe_validates_call_order(pkg, netgen):
    pipe = pkg.HIPScheduler(pkg.FP32, 2)
    with pytest.raises(ValueError):
        pipe.forward(np.zeros(pkg.INPUT_SIZE, np.float32))
    with pytest.raises(ValueError):
        pipe.drain()


def test_weights_file_round_trip(netgen, tmp_path):
    net = netgen.make_network(1, 8, seed=5)
    for name in ("w.txt", "w.txt.gz"):
        p = tmp_path / name
        netgen.save_weights(net, p)
        back = netgen.load_weights(p)
        assert (back.blocks, back.filters) == (1, 8)
        for a, b in zip(net.lines(), back.lines()):
            assert np.array_equal(np.asarray(a, np.float32).ravel(), np.asarray(b).ravel())
    bad = tmp_path / "bad.txt"
    bad.write_text("3\n")
    with pytest.raises(ValueError):
        netgen.load_weights(bad)
    lines = open(tmp_path / "w.txt").read().split("\n")
    (tmp_path / "short.txt").write_text("\n".join(lines[:-3]) + "\n")
    with pytest.raises(ValueError):
        netgen.load_weights(tmp_path / "short.txt")


GOLDEN_NET = os.path.join(ROOT, "tests", "golden", "0k.txt.gz")


def test_reference_weights_fixture_loads(netgen, orc, tmp_path):
    """tests/golden/0k.txt.gz is the weights file the reference's own unit tests load
    (src/tests/0k.txt, gzip-compressed; the reference reads gzip too): format version 1,
    one residual block of 8 filters."""
    net = netgen.load_weights(GOLDEN_NET)
    assert (net.blocks, net.filters, net.value_head_not_stm) == (1, 8, False)
    sizes = [np.asarray(v).size for v in net.lines()]
    assert sizes == [1296, 8, 8, 8, 576, 8, 8, 8, 576, 8, 8, 8,
                     16, 2, 2, 2, 261364, 362, 8, 1, 1, 1, 92416, 256, 256, 1]
    # the file survives a write/read cycle of this package's writer
    out = tmp_path / "again.txt"
    netgen.save_weights(net, out)
    back = netgen.load_weights(out)
    for a, b in zip(net.lines(), back.lines()):
        assert np.array_equal(np.asarray(a, np.float32).ravel(), np.asarray(b, np.float32).ravel())
    # and the CPU oracle evaluates it to a proper distribution
    w, h = netgen.prepare(net, orc.winograd_transform_f, orc.process_bn_var)
    ref = orc.OraclePipe()
    ref.initialize(net.filters)
    ref.push_weights(6, 18, net.filters, w)
    pol, val = ref.forward(netgen.synthetic_inputs(1, seed=9)[0])
    hd = orc.heads(h, pol, val)
    assert abs(float(hd["policy"].sum()) - 1.0) < 1e-5 and 0.0 < hd["winrate"] < 1.0
    assert hd["policy"].max() < 0.9      # a real network: not a saturated one-hot


def test_create_from_file_refuses_what_the_engine_refuses(pkg, netgen, tmp_path):
    """lzhip_create_from_file reads the file before it touches a device, so the refusals of
    the engine's reader (reference src/Network.cpp:225-405) can be checked here: missing file,
    wrong version, a line count that is not 19 + 8 blocks, a token that is no number, a policy
    layer of another board size.  A good file gets as far as the device (which this host
    lacks, or which then serves it)."""
    import gzip
    import torch
    good = os.path.join(ROOT, "tests", "golden", "0k.txt.gz")
    lines = gzip.open(good, "rt").read().splitlines()
    assert len(lines) == 1 + 4 + 14 + 8 * 1

    def attempt(path):
        return pkg.HIPScheduler.from_file(str(path), pkg.FP32, 2)

    def write(name, ls):
        path = tmp_path / name
        path.write_text("\n".join(ls) + "\n")
        return path

    with pytest.raises(ValueError, match="Could not open weights file"):
        attempt(tmp_path / "missing.txt")
    with pytest.raises(ValueError, match="wrong version"):
        attempt(write("v3.txt", ["3"] + lines[1:]))
    with pytest.raises(ValueError, match="wrong version"):
        attempt(write("empty.txt", [""]))
    with pytest.raises(ValueError, match="Inconsistent number of weights"):
        attempt(write("short.txt", lines[:-1]))
    bad = list(lines)
    bad[7] = bad[7].replace(" ", " x ", 1)
    with pytest.raises(ValueError, match="Error on line 8"):
        attempt(write("token.txt", bad))
    other = list(lines)
    other[1 + 4 + 8 + 4] = " ".join(other[1 + 4 + 8 + 4].split()[:-362])   # one move fewer
    with pytest.raises(ValueError, match="not for 19x19 boards"):
        attempt(write("board.txt", other))
    narrow = list(lines)
    narrow[3] = " ".join(narrow[3].split()[:-1])                          # a mean goes missing
    with pytest.raises(ValueError, match="Inconsistent number of weights"):
        attempt(write("narrow.txt", narrow))
    # plain text and gzip are both read; without a device the good file ends at the device
    plain = write("plain.txt", lines)
    for path in (good, plain):
        if torch.cuda.is_available():
            pipe = attempt(path)
            assert (pipe.filters, pipe.n_layers) == (8, 3)
            pipe.close()
        else:
            with pytest.raises(pkg.LzhipError):
                attempt(path)

