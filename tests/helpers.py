"""Shared helpers of the parity tests: an independent float64 model of the
network (direct convolutions through torch's conv2d, no Winograd) and the
error metrics the tests report."""
import numpy as np


def conv3x3_f64(x, w):
    """x [n][C][19][19] float64, w [K][C][3][3]: zero-padded correlation."""
    import torch
    import torch.nn.functional as F
    return F.conv2d(torch.from_numpy(np.asarray(x, np.float64)),
                    torch.from_numpy(np.asarray(w, np.float64)), padding=1).numpy()


def tower_f64(net, x, eps=1e-5):
    """Float64 forward of a RawNetwork on x [n][18][361] with direct convolutions.
    Returns dict(pol [n][722], val [n][361], acts=[per-layer activations])."""
    n = x.shape[0]
    a = np.asarray(x, np.float64).reshape(n, 18, 19, 19)

    def bn(y, l):
        m = (np.asarray(net.bn_mean[l], np.float64) - np.asarray(net.conv_b[l], np.float64))
        s = 1.0 / np.sqrt(np.asarray(net.bn_var[l], np.float64) + eps)
        return s[None, :, None, None] * (y - m[None, :, None, None])

    acts = []
    a = np.maximum(0.0, bn(conv3x3_f64(a, net.conv_w[0]), 0))
    acts.append(a)
    for l in range(1, net.n_layers, 2):
        t = np.maximum(0.0, bn(conv3x3_f64(a, net.conv_w[l]), l))
        acts.append(t)
        a = np.maximum(0.0, bn(conv3x3_f64(t, net.conv_w[l + 1]), l + 1) + a)
        acts.append(a)
    flat = a.reshape(n, net.filters, 361)
    pol = np.einsum("oc,ncp->nop", np.asarray(net.pol_conv_w, np.float64).reshape(2, -1), flat)
    val = np.einsum("oc,ncp->nop", np.asarray(net.val_conv_w, np.float64).reshape(1, -1), flat)
    return dict(pol=pol.reshape(n, 722), val=val.reshape(n, 361), acts=acts)


def heads_f64(net, pol, val, temperature=1.0, eps=1e-5):
    """Float64 head arithmetic on raw planes pol[722], val[361]."""
    p = np.asarray(pol, np.float64).reshape(2, 361)
    m = np.asarray(net.pol_bn_mean, np.float64) - np.asarray(net.pol_conv_b, np.float64)
    s = 1.0 / np.sqrt(np.asarray(net.pol_bn_var, np.float64) + eps)
    p = np.maximum(0.0, s[:, None] * (p - m[:, None])).reshape(722)
    logits = np.asarray(net.pol_fc_w, np.float64).reshape(362, 722) @ p + np.asarray(net.pol_fc_b, np.float64)
    e = np.exp((logits - logits.max()) / temperature)
    policy = e / e.sum()
    v = np.asarray(val, np.float64).reshape(361)
    m = np.asarray(net.val_bn_mean, np.float64) - np.asarray(net.val_conv_b, np.float64)
    s = 1.0 / np.sqrt(np.asarray(net.val_bn_var, np.float64) + eps)
    v = np.maximum(0.0, s[0] * (v - m[0]))
    h1 = np.maximum(0.0, np.asarray(net.val_fc1_w, np.float64).reshape(256, 361) @ v
                    + np.asarray(net.val_fc1_b, np.float64))
    o = float(np.asarray(net.val_fc2_w, np.float64).reshape(256) @ h1 + np.asarray(net.val_fc2_b, np.float64)[0])
    return dict(policy=policy, logits=logits, value=np.tanh(o), winrate=(1 + np.tanh(o)) / 2, value_pre=o)


def normalise_network(net, x, branch_rms=0.15):
    """Gives a RawNetwork the batch-norm statistics a trained network has: every layer's
    mean and variance are set from what its convolution puts out on the positions x
    [n][18][361] (float32 direct convolutions), so that the normalised output has zero mean
    and unit RMS -- and RMS `branch_rms` on the second convolution of each block, which
    keeps the residual stream O(1) however deep the tower is.  The two head planes are
    normalised the same way.  Returns net (modified in place)."""
    import torch
    import torch.nn.functional as F
    n = x.shape[0]
    a = torch.from_numpy(np.asarray(x, np.float32).reshape(n, 18, 19, 19))

    def conv_bn(inp, l, rms):
        y = F.conv2d(inp, torch.from_numpy(net.conv_w[l]), padding=1)
        mean = y.mean(dim=(0, 2, 3))
        var = y.var(dim=(0, 2, 3), unbiased=False) / (rms * rms)
        net.bn_mean[l] = mean.numpy().astype(np.float32)
        net.bn_var[l] = np.maximum(var.numpy(), 1e-6).astype(np.float32)
        net.conv_b[l] = np.zeros(net.filters, np.float32)
        s = 1.0 / torch.sqrt(torch.from_numpy(net.bn_var[l]) + 1e-5)
        return s[None, :, None, None] * (y - torch.from_numpy(net.bn_mean[l])[None, :, None, None])

    a = torch.relu(conv_bn(a, 0, 1.0))
    for l in range(1, net.n_layers, 2):
        t = torch.relu(conv_bn(a, l, 1.0))
        a = torch.relu(conv_bn(t, l + 1, branch_rms) + a)
    flat = a.reshape(n, net.filters, 361)
    pol = torch.einsum("oc,ncp->nop", torch.from_numpy(net.pol_conv_w.reshape(2, -1)), flat)
    val = torch.einsum("oc,ncp->nop", torch.from_numpy(net.val_conv_w.reshape(1, -1)), flat)
    net.pol_bn_mean = pol.mean(dim=(0, 2)).numpy().astype(np.float32)
    net.pol_bn_var = pol.var(dim=(0, 2), unbiased=False).numpy().astype(np.float32)
    net.val_bn_mean = val.mean(dim=(0, 2)).numpy().astype(np.float32)
    net.val_bn_var = val.var(dim=(0, 2), unbiased=False).numpy().astype(np.float32)
    return net


def rel_l2(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    d = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / d) if d > 0 else float(np.linalg.norm(a - b))


def max_abs(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max())
