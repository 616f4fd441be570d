"""Parity of the HIP path (through the C ABI) with the CPU oracle on identical
seeded networks and inputs.  Tolerances:
  fp32: policy probabilities and value within 1e-4 max abs; raw planes rel-L2 <= 1e-5
  fp16: policy within 2e-2, value within 2e-2; raw planes rel-L2 <= 2e-2
Deep random-init networks saturate softmax/tanh, so the raw 1x1 planes and the
logits are compared relatively as well.
"""
import threading

import numpy as np
import pytest

from helpers import max_abs, rel_l2

pytestmark = pytest.mark.gpu


def make_pipes(pkg, netgen, orc, blocks, filters, seed, precision, max_batch):
    net = netgen.make_network(blocks, filters, seed)
    w, h = netgen.prepare(net)
    w_ref, h_ref = netgen.prepare(net, orc.winograd_transform_f, orc.process_bn_var)
    ref = orc.OraclePipe()
    ref.initialize(filters)
    ref.push_weights(6, 18, filters, w_ref)
    pipe = pkg.HIPScheduler(precision, max_batch)
    pipe.initialize(filters)
    pipe.push_weights(6, 18, filters, w)
    pipe.push_heads(h)
    return net, pipe, ref, h_ref


@pytest.mark.parametrize("precision", [0, 1])
@pytest.mark.parametrize("filters,n", [(8, 3), (64, 3), (192, 3), (192, 30), (128, 3), (128, 40),
                                       (256, 3), (256, 16), (256, 20), (256, 40)])
def test_single_layer_stages(pkg, netgen, orc, precision, filters, n):
    """V, M and Y of one convolution layer against the oracle's stages, for the input
    layer (18 planes) and a residual-tower layer with a skip connection.  The M stage is
    the check the reference's tuner makes of every GEMM it times, against a plain sgemm
    (reference src/Tuner.cpp:262-301); 128 and 256 filters put the streaming GEMMs of both
    storage types under it, at 3 boards (one 32-row block per work-group) and at 40 (several
    blocks per work-group, a last block of 8 rows).  The fp16 GEMM and output transform run
    in the layout a forward of that many boards keeps its tiles in: slabs of 16 channels at
    3 and 16 boards, of 32 at 20 (256 filters), 30 (192) and 40 (128), rows at 40 boards of
    256 filters."""
    print("case: single_layer precision=%d filters=%d n=%d" % (precision, filters, n), flush=True)
    net, pipe, ref, _ = make_pipes(pkg, netgen, orc, 1, filters, 40 + filters, precision,
                                   max(4, n))
    rng = np.random.default_rng(filters)
    tol = 1e-5 if precision == 0 else 4e-3
    # layer 0 on real input planes
    x = netgen.synthetic_inputs(n, seed=3)
    V, M, Y = pipe.debug_layer(0, x)
    for i in range(n):
        Vr = orc.transform_in(x[i], 18)
        Mr = orc.sgemm(ref.U[0], Vr, 18, filters)
        Yr = orc.batchnorm(orc.transform_out(Mr, filters), ref.mean[0], ref.scale[0])
        assert rel_l2(V[i], Vr) <= tol, ("V layer0", i)
        assert rel_l2(M[i], Mr) <= tol, ("M layer0", i)
        assert rel_l2(Y[i], Yr) <= tol, ("Y layer0", i)
    # layer 2 (second conv of the block) with a residual input
    a = np.abs(rng.standard_normal((n, filters, 361))).astype(np.float32)
    r = np.abs(rng.standard_normal((n, filters, 361))).astype(np.float32)
    if precision == 1:  # make the inputs exactly representable in half precision
        a = a.astype(np.float16).astype(np.float32)
        r = r.astype(np.float16).astype(np.float32)
    V, M, Y = pipe.debug_layer(2, a, r)
    for i in range(n):
        Vr = orc.transform_in(a[i], filters)
        Mr = orc.sgemm(ref.U[2], Vr, filters, filters)
        Yr = orc.batchnorm(orc.transform_out(Mr, filters), ref.mean[2], ref.scale[2], r[i])
        assert rel_l2(V[i], Vr) <= tol, ("V layer2", i)
        assert rel_l2(M[i], Mr) <= tol, ("M layer2", i)
        assert rel_l2(Y[i], Yr) <= 2 * tol, ("Y layer2", i)
    pipe.close()


def check_outputs(pkg, orc, pipe, ref, h_ref, x, precision, idx=None, all_raw=False):
    """Raw planes, logits, policy and value of the HIP pipe against the oracle.

    The reference's answer is itself only defined up to its BLAS back-end's summation
    order (OpenBLAS / Eigen / MKL builds exist).  On random-init networks the logits
    reach 1e3..1e8, so a last-ulp change of the planes can move a non-saturated
    probability by more than 1e-4.  Each position is therefore also evaluated with the
    oracle's second sgemm provider; where the two oracle runs disagree by more than a
    fifth of the tolerance, the position is reported as ill-conditioned (with the gap
    between its two largest logits) and compared at 10x their disagreement instead.  At
    most one position of a case may take that route.  Raw planes and logits are always
    compared at the strict relative tolerance, for every position checked; with all_raw
    the raw planes of every position of the batch are (the oracle runs them on all host
    threads), whatever idx selects for the head outputs.  Every position checked must also
    pass the engine's own run-time self-check (Network::compare_net_outputs, reference
    src/Network.cpp:666-691): the L2 norm over the 362 policy entries and the winrate
    (1 + value) / 2 at most 0.2, with no relaxation for ill-conditioned positions."""
    raw_tol = 1e-5 if precision == 0 else 2e-2
    p_tol = 1e-4 if precision == 0 else 2e-2
    policy, value, logits, pol, val = pipe.evaluate_batch(x, want_raw=True)
    worst = dict(pol=0.0, val=0.0, logits=0.0, policy=0.0, value=0.0, ill_conditioned=0,
                 engine_selfcheck=0.0)
    if all_raw:
        import os
        rp_all, rv_all, _ = ref.forward_many(x, threads=min(16, os.cpu_count() or 1))
        for i in range(x.shape[0]):
            e_pol, e_val = rel_l2(pol[i], rp_all[i]), rel_l2(val[i], rv_all[i])
            assert e_pol <= raw_tol and e_val <= raw_tol, ("raw planes", i, e_pol, e_val)
            worst["pol"] = max(worst["pol"], e_pol)
            worst["val"] = max(worst["val"], e_val)
    have_blas = orc.use_openblas() != "builtin"
    orc.use_builtin()
    for i in (range(x.shape[0]) if idx is None else idx):
        rp, rv = ref.forward(x[i])
        hd = orc.heads(h_ref, rp, rv)
        tol_i = p_tol
        if have_blas:
            orc.use_openblas()
            rp2, rv2 = ref.forward(x[i])
            orc.use_builtin()
            hd2 = orc.heads(h_ref, rp2, rv2)
            noise = max(max_abs(hd["policy"], hd2["policy"]), abs(hd["value"] - hd2["value"]))
            if noise > p_tol / 5:
                worst["ill_conditioned"] += 1
                tol_i = max(p_tol, 10 * noise)
                top = np.sort(hd["logits"])[-2:]
                print("ill-conditioned position %d: top-2 logit gap %.4g, oracle back ends "
                      "differ by %.3g, compared at %.3g" % (i, float(top[1] - top[0]), noise,
                                                            tol_i), flush=True)
        worst["pol"] = max(worst["pol"], rel_l2(pol[i], rp))
        worst["val"] = max(worst["val"], rel_l2(val[i], rv))
        e_l = rel_l2(logits[i], hd["logits"])
        worst["logits"] = max(worst["logits"], e_l)
        assert e_l <= raw_tol, ("logits", i, e_l)
        e_p = max_abs(policy[i], hd["policy"])
        e_v = abs(float(value[i]) - hd["value"])
        worst["policy"] = max(worst["policy"], e_p)
        worst["value"] = max(worst["value"], e_v)
        assert e_p <= tol_i and e_v <= tol_i, (i, e_p, e_v, tol_i)
        d = np.asarray(policy[i], np.float64) - np.asarray(hd["policy"], np.float64)
        e_engine = float(np.sqrt(np.sum(d * d) + (0.5 * (float(value[i]) - hd["value"])) ** 2))
        worst["engine_selfcheck"] = max(worst["engine_selfcheck"], e_engine)
        assert e_engine <= 0.2, ("engine self-check bar", i, e_engine)
        assert abs(float(policy[i].sum()) - 1.0) < 1e-4
    print("parity", worst, flush=True)
    assert worst["pol"] <= raw_tol and worst["val"] <= raw_tol, worst
    assert worst["ill_conditioned"] <= 1, worst
    return worst


@pytest.mark.parametrize("blocks,filters,batch,precision", [
    (1, 8, 3, 0),       # the shape of the reference's test network (1 block x 8 filters)
    (6, 128, 1, 0),     # the smallest benchmark configuration: 6x128 fp32 batch 1
    (15, 192, 8, 0),    # 15x192 fp32 batch 8
    (1, 8, 3, 1),
    (6, 128, 4, 1),     # the same small net in fp16: the non-saturated fp16 check
    (2, 96, 5, 1),
])
def test_forward_parity(pkg, netgen, orc, blocks, filters, batch, precision):
    print("case: forward %dx%d b%d precision=%d" % (blocks, filters, batch, precision), flush=True)
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, blocks, filters, 1000 + blocks, precision,
                                       batch)
    x = netgen.synthetic_inputs(batch, seed=blocks * 7 + filters)
    check_outputs(pkg, orc, pipe, ref, h_ref, x, precision)
    pipe.close()


@pytest.mark.parametrize("precision", [0, 1])
@pytest.mark.parametrize("batch", [72, 64, 52, 41, 36, 35, 33, 32, 24, 21, 18, 17, 16, 10, 9, 8, 2, 1])
def test_forward_parity_wide_batches(pkg, netgen, orc, precision, batch):
    """256 filters at batch sizes on both sides of every change of kernel shape (GEMM, fp16:
    the streaming kernel with 1, 2, 4, 8 and 16 blocks of 32 tile rows per work-group, which
    change at 9, 18, 36 and 72 boards; fp32:
    256x256 tiles from 41 boards, 128x128 from 21, 128x64 with padded rows below; fused
    transform: 64 channels per work-group from 21 boards, 32 from 17, 16 below), in both
    precisions, including batches whose tile count is not a multiple of any tile height."""
    print("case: wide 3x256 b%d precision=%d" % (batch, precision), flush=True)
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 3, 256, 3000, precision, batch)
    x = netgen.synthetic_inputs(batch, seed=batch)
    check_outputs(pkg, orc, pipe, ref, h_ref, x, precision,
                  idx=sorted({0, min(1, batch - 1), batch // 2, batch - 1}))
    pipe.close()


@pytest.mark.parametrize("blocks,filters,batch", [(20, 256, 32), (40, 256, 64), (15, 192, 16),
                                                  (10, 128, 24)])
def test_forward_parity_deep_fp16(pkg, netgen, orc, blocks, filters, batch):
    """Deep fp16 towers: the two large fp16 benchmark configurations (20x256 batch 32, 40x256
    batch 64) at full size, and 15x192 and 10x128 (the streaming GEMM with 6 and 4 wavefronts
    under per-layer activation scales): raw planes of every position of the batch against the oracle, head outputs of
    three of them."""
    print("case: deep fp16 %dx%d b%d" % (blocks, filters, batch), flush=True)
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, blocks, filters, 2000 + blocks,
                                       pkg.FP16, batch)
    x = netgen.synthetic_inputs(batch, seed=blocks)
    s = pipe.act_scales()
    print("act scales: first %s last %s" % (s[:3], s[-3:]), flush=True)
    assert np.all(s >= 1.0) and np.all(np.log2(s) == np.round(np.log2(s)))
    check_outputs(pkg, orc, pipe, ref, h_ref, x, pkg.FP16, idx=[0, batch // 2, batch - 1],
                  all_raw=True)
    pipe.close()


def test_forward_parity_deep_fp16_with_plain_half_storage(pkg, netgen, orc):
    """40x256 at batch 64 with batch-norm statistics that keep the activations O(1) through
    all 40 blocks, as a trained network's do: the activation scales then come out as 1 for
    every layer, i.e. plain half-precision storage as in the reference's half pipeline, the
    heads are not saturated, and policy and value of all 64 positions are held to the fp16
    tolerance where it bites (no position may take the ill-conditioned route here)."""
    from helpers import normalise_network
    print("case: deep fp16, normalised 40x256 b64", flush=True)
    blocks, filters, batch = 40, 256, 64
    net = normalise_network(netgen.make_network(blocks, filters, 2100),
                            netgen.synthetic_inputs(4, seed=2101))
    w, h = netgen.prepare(net)
    w_ref, h_ref = netgen.prepare(net, orc.winograd_transform_f, orc.process_bn_var)
    ref = orc.OraclePipe()
    ref.initialize(filters)
    ref.push_weights(6, 18, filters, w_ref)
    pipe = pkg.HIPScheduler(pkg.FP16, batch)
    pipe.initialize(filters)
    pipe.push_weights(6, 18, filters, w)
    pipe.push_heads(h)
    s = pipe.act_scales()
    print("act scales: min %g max %g" % (s.min(), s.max()), flush=True)
    assert np.all(s == 1.0), s
    x = netgen.synthetic_inputs(batch, seed=2102)
    worst = check_outputs(pkg, orc, pipe, ref, h_ref, x, pkg.FP16, all_raw=True)
    assert worst["ill_conditioned"] == 0, worst
    # not a saturated case: the mean policy maximum is far from one-hot, values spread
    policy, value, _ = pipe.evaluate_batch(x)
    print("policy max: mean %.3f; |value|: mean %.3f max %.3f"
          % (policy.max(axis=1).mean(), np.abs(value).mean(), np.abs(value).max()), flush=True)
    assert policy.max(axis=1).mean() < 0.9 and np.abs(value).mean() < 0.95
    pipe.close()


def test_failed_push_weights_leaves_the_handle_unchanged(pkg, netgen, orc):
    """push_weights is all or nothing.  An fp16 push whose calibration cannot settle (a
    layer with an infinite batch-norm scale: its activations are infinite at any scale) fails
    after the filters of every layer went up; the handle must then refuse forwards exactly as
    before any push, and accept a second push with good weights, whose results are right."""
    print("case: failed push_weights", flush=True)
    net = netgen.make_network(2, 64, 71)
    w, h = netgen.prepare(net)
    bad = pkg.ForwardPipeWeights()
    bad.__dict__.update(w.__dict__)
    bad.m_batchnorm_stddevs = [v.copy() for v in w.m_batchnorm_stddevs]
    bad.m_batchnorm_stddevs[3][:] = np.inf
    x = netgen.synthetic_inputs(3, seed=72)
    pipe = pkg.HIPScheduler(pkg.FP16, 4)
    pipe.initialize(64)
    with pytest.raises(pkg.LzhipError):
        pipe.push_weights(6, 18, 64, bad)
    with pytest.raises(ValueError, match="push_weights has not been called"):
        pipe.forward_batch(x)
    import torch
    d = torch.zeros(3, 18, 361, device="cuda")
    o1, o2 = torch.zeros(3, 722, device="cuda"), torch.zeros(3, 361, device="cuda")
    with pytest.raises(ValueError, match="push_weights has not been called"):
        pipe.forward_batch_device_noalloc(3, d.data_ptr(), o1.data_ptr(), o2.data_ptr())
    pipe.push_weights(6, 18, 64, w)            # accepted: the failed push left nothing behind
    pol, val = pipe.forward_batch(x)
    w_ref, _ = netgen.prepare(net, orc.winograd_transform_f, orc.process_bn_var)
    ref = orc.OraclePipe()
    ref.initialize(64)
    ref.push_weights(6, 18, 64, w_ref)
    for i in range(3):
        rp, rv = ref.forward(x[i])
        assert rel_l2(pol[i], rp) <= 2e-2 and rel_l2(val[i], rv) <= 2e-2
    pipe.close()


def test_golden_fixtures_on_device(pkg, netgen):
    import os
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "tower_golden.npz"))
    for tag in ("b1f8", "b2f16"):
        blocks, filters, seed = [int(v) for v in g[tag + "_cfg"]]
        net = netgen.make_network(blocks, filters, seed)
        w, h = netgen.prepare(net)
        for precision, raw_tol, p_tol in ((pkg.FP32, 1e-5, 1e-4), (pkg.FP16, 2e-2, 2e-2)):
            pipe = pkg.HIPScheduler(precision, 4)
            pipe.initialize(filters)
            pipe.push_weights(6, 18, filters, w)
            pipe.push_heads(h)
            policy, value, logits, pol, val = pipe.evaluate_batch(g[tag + "_x"], want_raw=True)
            assert rel_l2(pol, g[tag + "_pol"]) <= raw_tol
            assert rel_l2(val, g[tag + "_val"]) <= raw_tol
            assert max_abs(policy, g[tag + "_policy"]) <= p_tol
            assert max_abs(value, g[tag + "_value"]) <= p_tol
            pipe.close()


@pytest.mark.parametrize("precision", [0, 1])
def test_reference_weights_file_on_device(pkg, netgen, orc, precision):
    """The weights file of the reference's own unit tests (1 block x 8 filters, loaded
    through the text-format reader) against the oracle: 8 filters exercise the padding of
    the channel dimension to 64 with real weights."""
    import os
    print("case: reference weights file precision=%d" % precision, flush=True)
    net = netgen.load_weights(os.path.join(os.path.dirname(__file__), "golden", "0k.txt.gz"))
    w, h = netgen.prepare(net)
    w_ref, h_ref = netgen.prepare(net, orc.winograd_transform_f, orc.process_bn_var)
    ref = orc.OraclePipe()
    ref.initialize(net.filters)
    ref.push_weights(6, 18, net.filters, w_ref)
    pipe = pkg.HIPScheduler(precision, 8)
    pipe.initialize(net.filters)
    pipe.push_weights(6, 18, net.filters, w)
    pipe.push_heads(h)
    check_outputs(pkg, orc, pipe, ref, h_ref, netgen.synthetic_inputs(8, seed=31), precision)
    pipe.close()


def test_handle_created_from_a_weights_file(pkg, netgen, orc, tmp_path):
    """lzhip_create_from_file (reading, Winograd transform, bias folding, push of tower and
    heads in one call) gives bit for bit what the Python reader plus push_weights/push_heads
    give, for the reference's own test file (gzip) and for a seeded 2-block net written as
    format 2 in plain text; the heads it pushed serve `heads=None`, and format 2 turns the
    value round for white."""
    import os
    print("case: create from file", flush=True)
    x = netgen.synthetic_inputs(5, seed=41)
    ref_file = os.path.join(os.path.dirname(__file__), "golden", "0k.txt.gz")
    net2 = netgen.make_network(2, 24, 43)
    net2.value_head_not_stm = True
    v2_file = str(tmp_path / "v2.txt")
    netgen.save_weights(net2, v2_file)
    for path in (ref_file, v2_file):
        net = netgen.load_weights(path)
        w, h = netgen.prepare(net)
        a = pkg.HIPScheduler(pkg.FP32, 8)
        a.initialize(net.filters)
        a.push_weights(6, 18, net.filters, w)
        a.push_heads(h)
        b = pkg.HIPScheduler.from_file(path, pkg.FP32, 8)
        assert (b.filters, b.n_layers) == (net.filters, net.n_layers)
        pa, pb = a.forward_batch(x), b.forward_batch(x)
        assert np.array_equal(pa[0], pb[0]) and np.array_equal(pa[1], pb[1])
        ea, eb = a.evaluate_batch(x), b.evaluate_batch(x)
        assert np.array_equal(ea[0], eb[0]) and np.array_equal(ea[1], eb[1])
        # callers above forward(): the heads pushed from the file, and the format-2 flag
        boards = np.full((1, 361), pkg.EMPTY, np.uint8)
        boards[0, 72] = pkg.BLACK
        pol_a, win_a = a.get_output(h, boards, pkg.WHITE, 2)
        pol_b, win_b = b.get_output(None, boards, pkg.WHITE, 2)
        assert np.array_equal(pol_a, pol_b)
        want = 1.0 - win_a if net.value_head_not_stm else win_a
        assert abs(win_b - want) < 1e-7
        a.close()
        b.close()


@pytest.mark.parametrize("precision", [0, 1])
@pytest.mark.parametrize("filters,maxb", [(64, 8), (128, 40), (192, 16), (192, 40), (256, 40)])
def test_batch_composition_does_not_change_results(pkg, netgen, orc, precision, filters, maxb):
    """A position evaluated alone, in a partial batch and in a full batch gives
    bit-identical planes: rows of the GEMM are independent, and a network's layers run one
    kernel family at every batch (whatever the tile shapes, blocks per work-group or channel
    groups the batch selects, a value is summed in the same order).  fp32 at 192 filters takes
    the streaming GEMM in handles of up to 16 positions and the tiled one in larger ones."""
    print("case: batch composition %d filters precision=%d" % (filters, precision), flush=True)
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 2, filters, 77, precision, maxb)
    x = netgen.synthetic_inputs(maxb, seed=5)
    pol_all, val_all = pipe.forward_batch(x)
    for lo, hi in ((2, 5), (4, 5), (0, min(17, maxb)), (1, min(34, maxb)), (0, 1)):
        pol, val = pipe.forward_batch(x[lo:hi])
        assert np.array_equal(pol_all[lo:hi], pol) and np.array_equal(val_all[lo:hi], val), (lo, hi)
    # a larger batch after a smaller one (stale rows in the padded tile range)
    pol_b, val_b = pipe.forward_batch(x)
    assert np.array_equal(pol_all, pol_b) and np.array_equal(val_all, val_b)
    with pytest.raises(ValueError):
        pipe.forward_batch(np.zeros((maxb + 1, 18, 361), np.float32))
    pipe.close()


def test_scheduler_concurrent_requests(pkg, netgen, orc):
    """Many threads call forward() at once: each gets its own position's result,
    identical to the batch executor's, and the batches fill."""
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 2, 64, 78, pkg.FP32, 8)
    x = netgen.synthetic_inputs(24, seed=6)
    pol_ref = np.concatenate([pipe.forward_batch(x[i:i + 8])[0] for i in range(0, 24, 8)])
    out = [None] * 24
    pipe.reset_stats()

    def work(i):
        for rep in range(3):
            out[i] = pipe.forward(x[i])

    th = [threading.Thread(target=work, args=(i,)) for i in range(24)]
    [t.start() for t in th]
    [t.join() for t in th]
    for i in range(24):
        assert np.array_equal(out[i][0], pol_ref[i])
    st = pipe.stats()
    assert st["requests"] == 72 and st["halted"] == 0
    assert st["max_batch_seen"] <= 8 and st["batches"] < 72
    pipe.close()


def test_drain_and_resume(pkg, netgen, orc):
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 1, 8, 79, pkg.FP32, 4)
    x = netgen.synthetic_inputs(1, seed=7)[0]
    pipe.forward(x)
    pipe.drain()
    with pytest.raises(pkg.NetworkHaltException):
        pipe.forward(x)
    pipe.resume()
    pol, val = pipe.forward(x)
    rp, rv = ref.forward(x)
    assert rel_l2(pol, rp) < 1e-5
    assert pipe.stats()["halted"] == 1
    pipe.close()


def test_device_resident_forward_and_profile(pkg, netgen, orc):
    """The device-pointer entry point (what the bench times) gives the same planes as
    the host entry point, and the per-kernel timing hook reports every launch."""
    import torch
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 2, 64, 80, pkg.FP16, 4)
    x = netgen.synthetic_inputs(4, seed=8)
    pol_h, val_h = pipe.forward_batch(x)
    d_in = torch.from_numpy(x).cuda()
    d_pol = torch.zeros(4, 722, device="cuda")
    d_val = torch.zeros(4, 361, device="cuda")
    torch.cuda.synchronize()
    pipe.forward_batch_device(4, d_in.data_ptr(), d_pol.data_ptr(), d_val.data_ptr())
    pipe.sync()
    assert np.array_equal(d_pol.cpu().numpy(), pol_h) and np.array_equal(d_val.cpu().numpy(), val_h)
    ms, cnt = pipe.profile_forward(4, d_in.data_ptr(), d_pol.data_ptr(), d_val.data_ptr())
    # 2 blocks = 5 conv layers: 5 GEMMs, 4 fused out->in transforms, 1 plain of each
    assert list(cnt) == [1, 1, 5, 1, 1, 4]
    assert np.all(ms > 0) and np.all(ms < 50)
    assert np.array_equal(d_pol.cpu().numpy(), pol_h)
    pipe.close()


def test_lanes_run_side_by_side_with_equal_results(pkg, netgen, orc):
    """Forwards of different batches enqueued on the handle's two lanes, many in a row with no
    synchronisation between them, give bit for bit what each batch gives alone on lane 0;
    host-buffer calls from four threads (more than there are lanes) likewise.  A lane that does not
    exist is refused."""
    import threading
    import torch
    print("case: lanes", flush=True)
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 3, 128, 81, pkg.FP16, 16)
    assert pipe.lanes() == 3      # up to batch 48; two above
    xa = netgen.synthetic_inputs(16, seed=21)
    xb = netgen.synthetic_inputs(11, seed=22)
    want_a = pipe.forward_batch(xa)
    want_b = pipe.forward_batch(xb)
    d_a, d_b = torch.from_numpy(xa).cuda(), torch.from_numpy(xb).cuda()
    pol = [torch.zeros(16, 722, device="cuda") for _ in range(2)]
    val = [torch.zeros(16, 361, device="cuda") for _ in range(2)]
    torch.cuda.synchronize()
    for rep in range(6):
        pipe.forward_batch_device(16, d_a.data_ptr(), pol[0].data_ptr(), val[0].data_ptr(), lane=0)
        pipe.forward_batch_device(11, d_b.data_ptr(), pol[1].data_ptr(), val[1].data_ptr(), lane=1)
    pipe.sync()
    assert np.array_equal(pol[0].cpu().numpy(), want_a[0])
    assert np.array_equal(val[0].cpu().numpy(), want_a[1])
    assert np.array_equal(pol[1].cpu().numpy()[:11], want_b[0])
    assert np.array_equal(val[1].cpu().numpy()[:11], want_b[1])
    # the roles swapped: lane 1 takes the batch lane 0 had
    pipe.forward_batch_device(16, d_a.data_ptr(), pol[1].data_ptr(), val[1].data_ptr(), lane=1)
    pipe.forward_batch_device(11, d_b.data_ptr(), pol[0].data_ptr(), val[0].data_ptr(), lane=0)
    pipe.sync()
    assert np.array_equal(pol[1].cpu().numpy(), want_a[0])
    assert np.array_equal(pol[0].cpu().numpy()[:11], want_b[0])
    # the third lane, alone and beside the others
    for rep in range(3):
        pipe.forward_batch_device(11, d_b.data_ptr(), pol[0].data_ptr(), val[0].data_ptr(), lane=0)
        pipe.forward_batch_device(16, d_a.data_ptr(), pol[1].data_ptr(), val[1].data_ptr(), lane=2)
    pipe.sync()
    assert np.array_equal(pol[1].cpu().numpy(), want_a[0])
    assert np.array_equal(val[1].cpu().numpy(), want_a[1])
    assert np.array_equal(pol[0].cpu().numpy()[:11], want_b[0])
    for lane in (3, -1):
        with pytest.raises(ValueError):
            pipe.forward_batch_device(4, d_a.data_ptr(), pol[0].data_ptr(), val[0].data_ptr(),
                                      lane=lane)

    bad = []
    def caller(x, want):
        for _ in range(8):
            got = pipe.forward_batch(x)
            if not (np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])):
                bad.append(1)
    th = [threading.Thread(target=caller, args=(xa, want_a)),
          threading.Thread(target=caller, args=(xb, want_b)),
          threading.Thread(target=caller, args=(xa[:5], (want_a[0][:5], want_a[1][:5]))),
          threading.Thread(target=caller, args=(xb[:2], (want_b[0][:2], want_b[1][:2])))]
    for t in th:
        t.start()
    for t in th:
        t.join()
    assert not bad
    # against the oracle as well, so that "equal" is not "equally wrong"
    for i in (0, 10):
        rp, rv = ref.forward(xb[i])
        assert rel_l2(want_b[0][i], rp) <= 2e-2 and rel_l2(want_b[1][i], rv) <= 2e-2
    pipe.close()
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 1, 64, 82, pkg.FP16, 52)
    assert pipe.lanes() == 2
    pipe.close()


def test_graph_replays_match_stream_launches(pkg, netgen, orc):
    """The forward is replayed from a captured HIP graph.  Replays of several graphs
    (different batch sizes and buffers), with other work and synchronisations in between,
    must reproduce the first results bit for bit, and match a pipe that launches every
    kernel on the stream (the default; graphs are enabled with LZHIP_GRAPH=1)."""
    import os
    import torch
    _, plain, _, _ = make_pipes(pkg, netgen, orc, 3, 64, 81, pkg.FP16, 8)
    os.environ["LZHIP_GRAPH"] = "1"
    try:
        net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 3, 64, 81, pkg.FP16, 8)
    finally:
        del os.environ["LZHIP_GRAPH"]
    x = netgen.synthetic_inputs(8, seed=9)
    want8 = plain.forward_batch(x)
    want3 = plain.forward_batch(x[:3])
    d_in = torch.from_numpy(x).cuda()
    d_pol = torch.zeros(8, 722, device="cuda")
    d_val = torch.zeros(8, 361, device="cuda")
    for rep in range(4):
        got8 = pipe.forward_batch(x)                      # graph (8, internal buffers)
        assert np.array_equal(got8[0], want8[0]) and np.array_equal(got8[1], want8[1]), rep
        got3 = pipe.forward_batch(x[:3])                  # graph (3, internal buffers)
        assert np.array_equal(got3[0], want3[0]) and np.array_equal(got3[1], want3[1]), rep
        d_pol.zero_()
        torch.cuda.synchronize()
        pipe.forward_batch_device(8, d_in.data_ptr(), d_pol.data_ptr(), d_val.data_ptr())
        pipe.sync()                                       # graph (8, caller buffers)
        assert np.array_equal(d_pol.cpu().numpy(), want8[0]), rep
        assert np.array_equal(d_val.cpu().numpy(), want8[1]), rep
        policy, value, _ = pipe.evaluate_batch(x[:5])     # eager head kernel after a graph
        assert policy.shape == (5, 362)
    pipe.close()
    plain.close()


@pytest.mark.parametrize("filters,maxb,batches", [
    (256, 32, (1, 5, 8, 9, 16, 17, 20, 21, 23, 32)),
    (192, 42, (1, 7, 10, 15, 21, 22, 37, 42)),
    (128, 64, (1, 8, 9, 18, 32, 33, 36, 44, 45, 64)),
])
def test_fused_launches_match_separate_launches(pkg, netgen, orc, filters, maxb, batches):
    """An fp16 tower of 128, 192 or 256 filters sends the transform of a layer and the GEMM of
    the next as one launch where that is faster and the forward has the device to itself, up
    to the batch where the transform changes to its 64-channel shape, and up to that batch it
    keeps its tile arrays slab by slab instead of row by row.  Handles that always fuse
    (LZHIP_FUSE=2), that never fuse (0) and that decide per forward (the default), each with
    the slab layout and (LZHIP_SLAB=0) without,
    must give the same bits, at batches that take each of the shapes (1, 2, 4 or 8 blocks of 32
    rows per GEMM work-group, 16- or 32-channel transform groups), on one lane and with all
    lanes busy; and the result agrees with the oracle."""
    import os
    import torch
    print("case: fused launches, %d filters" % filters, flush=True)
    pipes = {}
    for slab in ("0", None):
        for mode in ("2", "0", None):
            for key, v in (("LZHIP_FUSE", mode), ("LZHIP_SLAB", slab)):
                if v is None:
                    os.environ.pop(key, None)
                else:
                    os.environ[key] = v
            try:
                net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 4, filters, 3100, pkg.FP16, maxb)
            finally:
                os.environ.pop("LZHIP_FUSE", None)
                os.environ.pop("LZHIP_SLAB", None)
            pipes[(mode, slab)] = pipe
    x = netgen.synthetic_inputs(maxb, seed=3101)
    base = pipes[("0", "0")]                      # separate launches, row layout
    for n in batches:
        want = base.forward_batch(x[:n])
        for key, pipe in pipes.items():
            if pipe is base:
                continue
            got = pipe.forward_batch(x[:n])
            assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]), (n, key)
    rp, rv = ref.forward(x[7])
    nb = batches[4]
    want = base.forward_batch(x[:nb])
    assert rel_l2(want[0][7], rp) <= 2e-2 and rel_l2(want[1][7], rv) <= 2e-2
    # every lane at once, many forwards in a row without synchronisation, always fused
    d_in = torch.from_numpy(x).cuda()
    for key in (("2", None), ("2", "0"), ("0", None)):
        pipe = pipes[key]
        outs = [(torch.zeros(nb, 722, device="cuda"), torch.zeros(nb, 361, device="cuda"))
                for _ in range(pipe.lanes())]
        torch.cuda.synchronize()
        for rep in range(8):
            for k, (pol, val) in enumerate(outs):
                pipe.forward_batch_device(nb, d_in.data_ptr(), pol.data_ptr(), val.data_ptr(), lane=k)
        pipe.sync()
        for pol, val in outs:
            assert np.array_equal(pol.cpu().numpy(), want[0]), key
            assert np.array_equal(val.cpu().numpy(), want[1]), key
    for pipe in pipes.values():
        pipe.close()


def test_random_batches_on_all_lanes_match_the_plain_forward(pkg, netgen, orc):
    """A seeded sequence of 400 forwards of random batches (1 to 32 boards, 256 filters) dealt to
    random lanes with no synchronisation between them -- so that consecutive forwards of a lane
    change between the slab widths and the row layout, between fused and separate launches,
    and between having the device alone and sharing it -- gives, forward by forward, the bits
    of a handle that never fuses and keeps its tiles row by row."""
    import os
    import torch
    print("case: random batches on all lanes", flush=True)
    maxb = 32
    os.environ["LZHIP_FUSE"] = "0"
    os.environ["LZHIP_SLAB"] = "0"
    try:
        net, plain, ref, h_ref = make_pipes(pkg, netgen, orc, 3, 256, 3300, pkg.FP16, maxb)
    finally:
        os.environ.pop("LZHIP_FUSE", None)
        os.environ.pop("LZHIP_SLAB", None)
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 3, 256, 3300, pkg.FP16, maxb)
    x = netgen.synthetic_inputs(maxb, seed=3301)
    want = {}
    rng = np.random.default_rng(3302)
    plan = [(int(rng.integers(1, maxb + 1)), int(rng.integers(0, pipe.lanes()))) for _ in range(400)]
    for n, _ in plan:
        if n not in want:
            want[n] = plain.forward_batch(x[:n])
    d_in = torch.from_numpy(x).cuda()
    outs = [(torch.zeros(maxb, 722, device="cuda"), torch.zeros(maxb, 361, device="cuda"))
            for _ in plan]
    torch.cuda.synchronize()
    for i, (n, lane) in enumerate(plan):
        pipe.forward_batch_device(n, d_in.data_ptr(), outs[i][0].data_ptr(), outs[i][1].data_ptr(),
                                  lane=lane)
        if i % 97 == 96:
            pipe.sync()           # now and then a forward finds the device empty
    pipe.sync()
    for i, (n, lane) in enumerate(plan):
        assert np.array_equal(outs[i][0].cpu().numpy()[:n], want[n][0]), (i, n, lane)
        assert np.array_equal(outs[i][1].cpu().numpy()[:n], want[n][1]), (i, n, lane)
    pipe.close()
    plain.close()


def test_error_behaviour_on_device(pkg, netgen):
    """Calls out of order and arguments out of range are refused with an error code and a
    message, never executed: forward before push_weights, push_weights twice, an even layer
    count, wrong tensor sizes, empty and oversized batches, bad precision/batch/filter
    arguments at creation, device heads before push_heads.  The pipe keeps working
    afterwards."""
    print("case: error behaviour", flush=True)
    net = netgen.make_network(1, 64, 5)
    w, h = netgen.prepare(net)
    x = netgen.synthetic_inputs(3, seed=2)
    pipe = pkg.HIPScheduler(pkg.FP32, 2)
    pipe.initialize(64)
    with pytest.raises(ValueError):
        pipe.forward_batch(x[:1])                      # no weights yet
    with pytest.raises(ValueError):
        pipe.push_weights(6, 18, 32, w)                # filter count differs from initialize
    bad = pkg.ForwardPipeWeights()
    bad.__dict__.update(w.__dict__)
    bad.m_conv_weights = w.m_conv_weights[:2]          # two layers: not 1 + 2*blocks
    bad.m_batchnorm_means = w.m_batchnorm_means[:2]
    bad.m_batchnorm_stddevs = w.m_batchnorm_stddevs[:2]
    with pytest.raises(ValueError):
        pipe.push_weights(6, 18, 64, bad)
    pipe.push_weights(6, 18, 64, w)
    with pytest.raises(ValueError):
        pipe.push_weights(6, 18, 64, w)                # twice
    with pytest.raises(ValueError):
        pipe.forward_batch(x)                          # 3 > max_batch 2
    with pytest.raises(ValueError):
        pipe.forward_batch(np.zeros((0, 18, 361), np.float32))
    with pytest.raises(ValueError):
        pipe.forward(np.zeros(100, np.float32))
    with pytest.raises(ValueError):
        pipe.evaluate_batch(x[:1])                     # device heads not pushed
    pol, val = pipe.forward_batch(x[:2])
    assert np.isfinite(pol).all() and np.isfinite(val).all()
    assert b"" == pkg.lib().lzhip_last_error()[:0]
    pipe.close()
    for args in ((pkg.FP32, 0), (pkg.FP32, 5000), (7, 4)):
        p = pkg.HIPScheduler(*args)
        with pytest.raises((ValueError, pkg.LzhipError)):
            p.initialize(64)
    p = pkg.HIPScheduler(pkg.FP32, 2)
    with pytest.raises((ValueError, pkg.LzhipError)):
        p.initialize(0)
    for prec, filters in ((pkg.FP32, 576), (pkg.FP16, 576), (pkg.FP16, 1100)):
        p = pkg.HIPScheduler(prec, 2)
        with pytest.raises(ValueError):
            p.initialize(filters)                      # no GEMM pipeline for this width
    p = pkg.HIPScheduler(pkg.FP32, 2, device=99)
    with pytest.raises(pkg.LzhipError):
        p.initialize(64)


@pytest.mark.parametrize("precision", [1, 0])
@pytest.mark.parametrize("filters,batch", [(128, 1), (128, 9), (128, 30), (128, 52), (128, 72),
                                           (192, 2), (192, 16), (192, 17), (192, 40), (192, 64)])
def test_streaming_gemm_at_narrower_widths(pkg, netgen, orc, filters, batch, precision):
    """Nets of 128 and 192 filters run the streaming GEMM with 4 and 6 wavefronts per
    work-group (256 filters: 8); in fp32 only the 128-filter ones do, 192 filters stay on the
    tiled kernels there.  The batches take every number of blocks per work-group (1, 2, 4, 8,
    16), with tile counts that are not multiples of the 32-row block."""
    print("case: streaming width %d b%d precision=%d" % (filters, batch, precision), flush=True)
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 1, filters, 5100 + filters, precision,
                                       batch)
    x = netgen.synthetic_inputs(batch, seed=filters + batch)
    check_outputs(pkg, orc, pipe, ref, h_ref, x, precision,
                  idx=sorted({0, batch // 2, batch - 1}))
    pipe.close()


@pytest.mark.parametrize("filters,batch", [(640, 4), (768, 3), (896, 2), (1024, 12), (1024, 8),
                                           (384, 28), (448, 30), (320, 52)])
def test_fp16_widths_on_the_tiled_gemm(pkg, netgen, orc, filters, batch):
    """fp16 widths served by the tiled GEMM kernels (above 256 filters; 64-filter nets are in
    the small-network cases): the widest ones -- 10, 12, 14 and 16 k-slices, at 1024 filters
    the one-pass 256x256 tile (from 11 boards) and the 128x64 tile below it -- and widths
    at batches that take the 128x128 persistent and the 128x64 tiles."""
    print("case: fp16 width %d b%d" % (filters, batch), flush=True)
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 1, filters, 5000 + filters, pkg.FP16,
                                       batch)
    x = netgen.synthetic_inputs(batch, seed=filters + batch)
    check_outputs(pkg, orc, pipe, ref, h_ref, x, pkg.FP16, idx=[0, batch - 1])
    pipe.close()


@pytest.mark.parametrize("precision", [0, 1])
@pytest.mark.parametrize("filters,batch", [(384, 6), (512, 44), (320, 3)])
def test_other_widths(pkg, netgen, orc, precision, filters, batch):
    """Widths other than the benchmark's: 6, 8 and 5 k-slices in fp16 (12, 16, 10 in fp32),
    with the large-tile GEMM at 512 filters."""
    print("case: width %d b%d precision=%d" % (filters, batch, precision), flush=True)
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 1, filters, 4000 + filters, precision,
                                       batch)
    x = netgen.synthetic_inputs(batch, seed=filters)
    check_outputs(pkg, orc, pipe, ref, h_ref, x, precision, idx=[0, batch - 1])
    pipe.close()


def test_bit_packed_and_float_requests_agree(pkg, netgen, orc):
    """Queued requests whose planes hold only 0 and 1 travel one bit per value; any other
    value sends the request down the float path.  Both must give bit-for-bit what the
    batch executor gives for the same planes handed over as floats."""
    print("case: bit-packed requests", flush=True)
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 2, 64, 91, pkg.FP32, 4)
    x = netgen.synthetic_inputs(4, seed=12)
    x[1, 3, 17] = 0.25          # not a 0/1 plane
    x[2, 16, :] = 1.0
    x[3, 17, 360] = 1.0         # the very last value: the partial last word
    pol, val = pipe.forward_batch(x)
    for i in range(4):
        p1, v1 = pipe.forward(x[i])
        assert np.array_equal(p1, pol[i]) and np.array_equal(v1, val[i]), i
    policy, value, _ = pipe.evaluate_batch(x)
    for i in (0, 1, 3):
        pe, ve = pipe.forward_eval(x[i])
        assert np.abs(pe - policy[i]).max() <= 1e-6 and abs(ve - value[i]) <= 1e-6, i
    pipe.close()


def test_fp16_range_beyond_the_calibration_positions(pkg, netgen, orc):
    """Stored activations are scaled at push_weights from 8 synthetic positions (target
    maximum 16) and clamped at 2040 on storage, by the fused and the unfused output
    transform alike.  Planes 64 times larger than anything the calibration saw still sit
    inside that range and agree with the oracle; planes 4096 times larger run into the clamp
    and must come out finite, with a policy that sums to one; and a single layer whose
    outputs exceed the clamp stores exactly min(y, 2040)."""
    print("case: fp16 range", flush=True)
    net, pipe, ref, h_ref = make_pipes(pkg, netgen, orc, 3, 128, 6100, pkg.FP16, 4)
    x = netgen.synthetic_inputs(4, seed=61)
    big = (64.0 * x).astype(np.float32)
    policy, value, logits, pol, val = pipe.evaluate_batch(big, want_raw=True)
    for i in range(4):
        rp, rv = ref.forward(big[i])
        assert rel_l2(pol[i], rp) <= 2e-2 and rel_l2(val[i], rv) <= 2e-2, i
    huge = (4096.0 * x).astype(np.float32)
    policy, value, logits, pol, val = pipe.evaluate_batch(huge, want_raw=True)
    assert np.isfinite(pol).all() and np.isfinite(val).all() and np.isfinite(logits).all()
    assert np.isfinite(policy).all() and np.isfinite(value).all()
    assert np.allclose(policy.sum(axis=1), 1.0, atol=1e-3)
    # one layer through the unfused kernel, inputs chosen so that many outputs pass 2040
    rng = np.random.default_rng(62)
    # (inputs stay inside the stored range themselves, so that V = B^T d B stays in half range)
    a = np.minimum(np.abs(rng.standard_normal((2, 128, 361))) * 600.0, 2000.0)
    a = a.astype(np.float16).astype(np.float32)
    V, M, Y = pipe.debug_layer(1, a)
    clipped = 0
    for i in range(2):
        Vr = orc.transform_in(a[i], 128)
        Mr = orc.sgemm(ref.U[1], Vr, 128, 128)
        Yr = orc.batchnorm(orc.transform_out(Mr, 128), ref.mean[1], ref.scale[1])
        want = np.minimum(Yr, 2040.0)
        clipped += int((Yr > 2040.0).sum())
        assert Y[i].max() <= 2040.0
        assert rel_l2(Y[i], want) <= 4e-3
    assert clipped > 100, clipped
    pipe.close()
