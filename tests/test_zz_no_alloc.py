"""The entry point that allocates nothing (lzhip_forward_batch_device_noalloc): same
planes, bit for bit, as lzhip_forward_batch_device, on two calls in a row, the second
with a smaller batch, in both storage types; sizes beyond its static working memory
are refused with a message."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _pipe(pkg, netgen, blocks, filters, seed, precision, max_batch):
    net = netgen.make_network(blocks, filters, seed=seed)
    w, _ = netgen.prepare(net)
    pipe = pkg.HIPScheduler(precision, max_batch=max_batch, device=0)
    pipe.initialize(filters)
    pipe.push_weights(6, 18, filters, w)
    return pipe


@pytest.mark.parametrize("precision_name", ["FP32", "FP16"])
@pytest.mark.parametrize("filters,max_batch", [(192, 8), (256, 8), (128, 64), (256, 64)])
def test_no_alloc_forward_matches_the_allocating_one(pkg, netgen, precision_name, filters,
                                                     max_batch):
    """256 filters at max_batch 8 fill the static array exactly; a handle made for 64
    positions has lane buffers with more tile rows per position than the static array
    (the serving case: a large handle, small no-alloc calls)."""
    import torch
    precision = getattr(pkg, precision_name)
    print("case: no-alloc forward", precision_name, filters, max_batch, flush=True)
    pipe = _pipe(pkg, netgen, 3, filters, 91, precision, max_batch)
    x = netgen.synthetic_inputs(8, seed=92)
    d_in = torch.from_numpy(x).cuda()
    for n in (8, 3):    # the second call is smaller: the array still holds the first one's tiles
        want_pol = torch.zeros(n, 722, device="cuda")
        want_val = torch.zeros(n, 361, device="cuda")
        got_pol = torch.full((n, 722), -7.0, device="cuda")
        got_val = torch.full((n, 361), -7.0, device="cuda")
        torch.cuda.synchronize()
        pipe.forward_batch_device(n, d_in.data_ptr(), want_pol.data_ptr(), want_val.data_ptr())
        pipe.sync()
        pipe.forward_batch_device_noalloc(n, d_in.data_ptr(), got_pol.data_ptr(),
                                          got_val.data_ptr())
        pipe.sync()
        assert np.isfinite(want_pol.cpu().numpy()).all()
        assert np.array_equal(got_pol.cpu().numpy(), want_pol.cpu().numpy())
        assert np.array_equal(got_val.cpu().numpy(), want_val.cpu().numpy())
    pipe.close()


def test_no_alloc_forwards_of_two_handles_share_the_array_in_turn(pkg, netgen):
    """Two handles of different width and storage type on one GPU, their no-alloc forwards
    enqueued alternately on their own streams with no host synchronisation in between: the
    library orders them on the device, and each gives what its allocating forward gives."""
    import torch
    print("case: no-alloc, two handles", flush=True)
    a = _pipe(pkg, netgen, 3, 256, 95, pkg.FP16, 8)
    b = _pipe(pkg, netgen, 2, 64, 96, pkg.FP32, 8)
    xa = torch.from_numpy(netgen.synthetic_inputs(8, seed=97)).cuda()
    xb = torch.from_numpy(netgen.synthetic_inputs(5, seed=98)).cuda()
    want = []
    for pipe, x, n in ((a, xa, 8), (b, xb, 5)):
        pol = torch.zeros(n, 722, device="cuda")
        val = torch.zeros(n, 361, device="cuda")
        torch.cuda.synchronize()
        pipe.forward_batch_device(n, x.data_ptr(), pol.data_ptr(), val.data_ptr())
        pipe.sync()
        want.append((pol.cpu().numpy(), val.cpu().numpy()))
    outs = [[(torch.full((8, 722), -7.0, device="cuda"), torch.full((8, 361), -7.0, device="cuda"))
             for _ in range(6)] for _ in range(2)]
    torch.cuda.synchronize()
    for rep in range(6):
        a.forward_batch_device_noalloc(8, xa.data_ptr(), outs[0][rep][0].data_ptr(),
                                       outs[0][rep][1].data_ptr())
        b.forward_batch_device_noalloc(5, xb.data_ptr(), outs[1][rep][0].data_ptr(),
                                       outs[1][rep][1].data_ptr())
    a.sync()
    b.sync()
    for rep in range(6):
        assert np.array_equal(outs[0][rep][0].cpu().numpy(), want[0][0]), rep
        assert np.array_equal(outs[0][rep][1].cpu().numpy(), want[0][1]), rep
        assert np.array_equal(outs[1][rep][0].cpu().numpy()[:5], want[1][0]), rep
        assert np.array_equal(outs[1][rep][1].cpu().numpy()[:5], want[1][1]), rep
    a.close()
    b.close()


def test_no_alloc_forward_refuses_what_does_not_fit(pkg, netgen):
    import torch
    print("case: no-alloc refusals", flush=True)
    pipe = _pipe(pkg, netgen, 1, 64, 93, pkg.FP16, 16)
    d_in = torch.zeros(16, 18, 361, device="cuda")
    d_pol = torch.zeros(16, 722, device="cuda")
    d_val = torch.zeros(16, 361, device="cuda")
    with pytest.raises(ValueError, match="1..8 positions"):
        pipe.forward_batch_device_noalloc(9, d_in.data_ptr(), d_pol.data_ptr(), d_val.data_ptr())
    with pytest.raises(ValueError):
        pipe.forward_batch_device_noalloc(0, d_in.data_ptr(), d_pol.data_ptr(), d_val.data_ptr())
    pipe.close()
    wide = _pipe(pkg, netgen, 1, 320, 94, pkg.FP16, 4)
    with pytest.raises(ValueError, match="256 filters"):
        wide.forward_batch_device_noalloc(2, d_in.data_ptr(), d_pol.data_ptr(), d_val.data_ptr())
    wide.close()
