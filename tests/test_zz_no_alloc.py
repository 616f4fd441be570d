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
def test_no_alloc_forward_matches_the_allocating_one(pkg, netgen, precision_name):
    import torch
    precision = getattr(pkg, precision_name)
    print("case: no-alloc forward", precision_name, flush=True)
    pipe = _pipe(pkg, netgen, 3, 192, 91, precision, 8)
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
