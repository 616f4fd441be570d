"""Seeded synthetic networks and positions, and the weight preparation that
Network::initialize performs before a pipe sees the weights.

Network definition (the benchmark configurations): 3x3 conv 18->F + BN + ReLU,
`blocks` residual blocks, policy head 1x1 conv F->2 + BN + ReLU + FC 722->362,
value head 1x1 conv F->1 + BN + ReLU + FC 361->256 + ReLU + FC 256->1 + tanh.
Weights are He-normal N(0, 2/fan_in), conv and FC biases zero, BN means
N(0, 0.1^2), BN variances U(0.5, 1.5).
"""
import gzip
import io

import numpy as np

from . import (INPUT_CHANNELS, NPTS, MOVES, VALUE_LAYER, ForwardPipeWeights, HeadWeights,
               process_bn_var, winograd_transform_f)


class RawNetwork:
    """A network as a Leela Zero weights file describes it (reference
    README.md:205-262; src/Network.cpp:268-348): spatial 3x3 filters
    [F][C][3][3], conv biases, BN means and variances, head parameters."""

    def __init__(self, blocks, filters):
        self.blocks = blocks
        self.filters = filters
        self.conv_w, self.conv_b, self.bn_mean, self.bn_var = [], [], [], []
        self.pol_conv_w = self.pol_conv_b = self.pol_bn_mean = self.pol_bn_var = None
        self.pol_fc_w = self.pol_fc_b = None
        self.val_conv_w = self.val_conv_b = self.val_bn_mean = self.val_bn_var = None
        self.val_fc1_w = self.val_fc1_b = self.val_fc2_w = self.val_fc2_b = None
        self.value_head_not_stm = False  # format version 2

    @property
    def n_layers(self):
        return 1 + 2 * self.blocks

    def lines(self):
        """The parameter vectors in file order (src/Network.cpp:281-348)."""
        out = []
        for l in range(self.n_layers):
            out += [self.conv_w[l], self.conv_b[l], self.bn_mean[l], self.bn_var[l]]
        out += [self.pol_conv_w, self.pol_conv_b, self.pol_bn_mean, self.pol_bn_var,
                self.pol_fc_w, self.pol_fc_b,
                self.val_conv_w, self.val_conv_b, self.val_bn_mean, self.val_bn_var,
                self.val_fc1_w, self.val_fc1_b, self.val_fc2_w, self.val_fc2_b]
        return out


def make_network(blocks, filters, seed):
    rng = np.random.default_rng(seed)
    F = filters
    net = RawNetwork(blocks, F)

    def he(shape, fan_in):
        return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)

    for l in range(net.n_layers):
        cin = INPUT_CHANNELS if l == 0 else F
        net.conv_w.append(he((F, cin, 3, 3), 9 * cin))
        net.conv_b.append(np.zeros(F, np.float32))
        net.bn_mean.append((rng.standard_normal(F) * 0.1).astype(np.float32))
        net.bn_var.append(rng.uniform(0.5, 1.5, F).astype(np.float32))
    net.pol_conv_w = he((2, F), F)
    net.pol_conv_b = np.zeros(2, np.float32)
    net.pol_bn_mean = (rng.standard_normal(2) * 0.1).astype(np.float32)
    net.pol_bn_var = rng.uniform(0.5, 1.5, 2).astype(np.float32)
    net.pol_fc_w = he((MOVES, 2 * NPTS), 2 * NPTS)
    net.pol_fc_b = np.zeros(MOVES, np.float32)
    net.val_conv_w = he((1, F), F)
    net.val_conv_b = np.zeros(1, np.float32)
    net.val_bn_mean = (rng.standard_normal(1) * 0.1).astype(np.float32)
    net.val_bn_var = rng.uniform(0.5, 1.5, 1).astype(np.float32)
    net.val_fc1_w = he((VALUE_LAYER, NPTS), NPTS)
    net.val_fc1_b = np.zeros(VALUE_LAYER, np.float32)
    net.val_fc2_w = he((1, VALUE_LAYER), VALUE_LAYER)
    net.val_fc2_b = np.zeros(1, np.float32)
    return net


def synthetic_inputs(n, seed):
    """n positions [n][18][361]: 8 own-stone and 8 opponent-stone history planes,
    each point own with p=0.2, else opponent with p=0.2 (never both); plane 16
    all ones (side to move), plane 17 all zeros."""
    rng = np.random.default_rng(seed)
    u = rng.random((n, 8, NPTS))
    x = np.zeros((n, INPUT_CHANNELS, NPTS), np.float32)
    x[:, 0:8] = (u < 0.2)
    x[:, 8:16] = (u >= 0.2) & (u < 0.4)
    x[:, 16] = 1.0
    return x


def prepare(net, transform_f=winograd_transform_f, bn_var=process_bn_var):
    """What Network::initialize does between loading the file and init_net
    (reference src/Network.cpp:540-576, :351-352): Winograd-transform the 3x3
    filters, turn variances into 1/sqrt(var+eps), fold conv biases into the BN
    means.  Returns (ForwardPipeWeights, HeadWeights)."""
    F = net.filters
    w = ForwardPipeWeights()
    for l in range(net.n_layers):
        cin = INPUT_CHANNELS if l == 0 else F
        w.m_conv_weights.append(transform_f(net.conv_w[l], F, cin))
        w.m_batchnorm_means.append((net.bn_mean[l] - net.conv_b[l]).astype(np.float32))
        w.m_conv_biases.append(np.zeros(F, np.float32))
        w.m_batchnorm_stddevs.append(bn_var(net.bn_var[l]))
    w.m_conv_pol_w = np.asarray(net.pol_conv_w, np.float32).reshape(2, F)
    w.m_conv_pol_b = np.zeros(2, np.float32)
    w.m_conv_val_w = np.asarray(net.val_conv_w, np.float32).reshape(F)
    w.m_conv_val_b = np.zeros(1, np.float32)
    h = HeadWeights()
    h.bn_pol_mean = (net.pol_bn_mean - net.pol_conv_b).astype(np.float32)
    h.bn_pol_scale = bn_var(net.pol_bn_var)
    h.ip_pol_w = np.asarray(net.pol_fc_w, np.float32).reshape(MOVES, 2 * NPTS)
    h.ip_pol_b = np.asarray(net.pol_fc_b, np.float32)
    h.bn_val_mean = (net.val_bn_mean - net.val_conv_b).astype(np.float32)
    h.bn_val_scale = bn_var(net.val_bn_var)
    h.ip1_val_w = np.asarray(net.val_fc1_w, np.float32).reshape(VALUE_LAYER, NPTS)
    h.ip1_val_b = np.asarray(net.val_fc1_b, np.float32)
    h.ip2_val_w = np.asarray(net.val_fc2_w, np.float32).reshape(VALUE_LAYER)
    h.ip2_val_b = np.asarray(net.val_fc2_b, np.float32)
    return w, h


# ---------------------------------------------------------------------------
# Leela Zero text weight files (reference src/Network.cpp:225-405).

def save_weights(net, path):
    """Write format version 1 (or 2) text, gzip-compressed if path ends in .gz."""
    buf = io.StringIO()
    buf.write("2\n" if net.value_head_not_stm else "1\n")
    for v in net.lines():
        buf.write(" ".join(repr(float(x)) for x in np.asarray(v, np.float32).reshape(-1)))
        buf.write("\n")
    data = buf.getvalue().encode("ascii")
    if str(path).endswith(".gz"):
        with gzip.open(path, "wb") as f:
            f.write(data)
    else:
        with open(path, "wb") as f:
            f.write(data)


def load_weights(path):
    """Parse a v1/v2 weights file, plain or gzip (the reference reads both
    through gzopen, src/Network.cpp:357-405).  Block count = (lines-1-4-14)/8,
    filter count = number of values on the conv-bias line (:243-259).
    Raises ValueError where the reference reports failure and exits."""
    with open(path, "rb") as f:
        raw = f.read()
    if raw[:2] == b"\x1f\x8b":
        raw = gzip.decompress(raw)
    text = raw.decode("ascii", "strict").split("\n")
    if text and text[-1] == "":
        text.pop()
    if not text:
        raise ValueError("empty weights file")
    try:
        version = int(text[0].split()[0])
    except (ValueError, IndexError):
        raise ValueError("Weights file is the wrong version.")
    if version not in (1, 2):
        raise ValueError("Weights file is the wrong version.")
    nlines = len(text)
    residual = nlines - (1 + 4 + 14)
    if residual < 0 or residual % 8 != 0:
        raise ValueError("Inconsistent number of weights in the file.")
    blocks = residual // 8
    vecs = []
    for i, line in enumerate(text[1:]):
        try:
            vecs.append(np.array(line.split(), dtype=np.float32))
        except ValueError:
            raise ValueError("Failed to parse weight file. Error on line %d." % (i + 2))
    filters = vecs[1].size
    net = RawNetwork(blocks, filters)
    net.value_head_not_stm = version == 2
    k = 0
    for l in range(net.n_layers):
        cin = INPUT_CHANNELS if l == 0 else filters
        if vecs[k].size != filters * cin * 9:
            raise ValueError("layer %d: expected %d filter values, found %d"
                             % (l, filters * cin * 9, vecs[k].size))
        net.conv_w.append(vecs[k].reshape(filters, cin, 3, 3))
        net.conv_b.append(vecs[k + 1]); net.bn_mean.append(vecs[k + 2]); net.bn_var.append(vecs[k + 3])
        k += 4
    (net.pol_conv_w, net.pol_conv_b, net.pol_bn_mean, net.pol_bn_var, net.pol_fc_w,
     net.pol_fc_b, net.val_conv_w, net.val_conv_b, net.val_bn_mean, net.val_bn_var,
     net.val_fc1_w, net.val_fc1_b, net.val_fc2_w, net.val_fc2_b) = vecs[k:k + 14]
    if net.pol_fc_w.size != 2 * NPTS * MOVES:
        raise ValueError("The weights file is not for 19x19 boards.")
    net.pol_conv_w = net.pol_conv_w.reshape(2, filters)
    net.val_conv_w = net.val_conv_w.reshape(1, filters)
    net.pol_fc_w = net.pol_fc_w.reshape(MOVES, 2 * NPTS)
    net.val_fc1_w = net.val_fc1_w.reshape(VALUE_LAYER, NPTS)
    net.val_fc2_w = net.val_fc2_w.reshape(1, VALUE_LAYER)
    return net
