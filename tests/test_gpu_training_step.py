"""Two SGD steps of a small convolutional network (conv - batch norm - ReLU - max pool - strided conv - ReLU - global average
pool - linear - softmax cross entropy) with the backward pass written out by hand from the backward kernels, run on the
device and by the CPU oracle: losses and every updated parameter must agree to the float32 tolerance.  This is the kernel
sequence the reference's training examples issue through autograd (chainerx_cc/examples/mnist/train_mnist.cc:48-75,
examples/imagenet_py/train_imagenet.py); autograd itself is outside the backend."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close

pytestmark = pytest.mark.gpu


class OracleOps:
    """Adapts the oracle's functions to the call shapes used below."""
    array = staticmethod(lambda a: np.array(a))
    get = staticmethod(lambda a: np.asarray(a))
    conv, relu, max_pool, average_pool, linear, log_softmax = O.conv, O.relu, O.max_pool, O.average_pool, O.linear, O.log_softmax
    exp, add, subtract, multiply, sum = O.exp, O.add, O.subtract, O.multiply, O.sum
    max_pool_grad, average_pool_grad, conv_transpose = O.max_pool_grad, O.average_pool_grad, O.conv_transpose

    @staticmethod
    def conv_grad_weight(w, x, gy, stride, pad):
        return O.conv_grad_weight(w.shape, x, gy, stride, pad)

    @staticmethod
    def batch_norm(x, gamma, beta, rm, rv):
        out, nrm, nrv, state = O.batch_norm(x, gamma, beta, rm, rv, 2e-5, 0.9)
        rm[...] = nrm
        rv[...] = nrv
        return out, state

    batch_norm_grad = staticmethod(O.batch_norm_grad)

    @staticmethod
    def relu_grad(x, g):
        return O.if_less_else(x, 0, 0, g)

    @staticmethod
    def dot(a, b):
        return O.dot(np.ascontiguousarray(a), np.ascontiguousarray(b))

    @staticmethod
    def onehot(t, n, dtype):
        return (t[:, None] == np.arange(n)[None, :]).astype(dtype)

    @staticmethod
    def scale(a, s):
        return O.multiply(a, np.asarray(s, a.dtype))

    @staticmethod
    def broadcast(a, shape):
        return np.broadcast_to(a, shape)


class DeviceOps:
    def __init__(self, chx):
        self.c = chx
        for name in ('conv', 'relu', 'max_pool', 'average_pool', 'linear', 'log_softmax', 'exp', 'add', 'subtract', 'multiply', 'sum',
                     'max_pool_grad', 'average_pool_grad', 'conv_transpose', 'dot', 'batch_norm_grad'):
            setattr(self, name, getattr(chx, name))
        self.array = chx.array
        self.get = lambda a: a.get()

    def conv_grad_weight(self, w, x, gy, stride, pad):
        return self.c.conv_grad_weight(w.dtype, w.shape, x, gy, stride, pad)

    def batch_norm(self, x, gamma, beta, rm, rv):
        return self.c.batch_norm(x, gamma, beta, rm, rv, 2e-5, 0.9)

    def relu_grad(self, x, g):
        return self.c.if_less_else(x, 0, 0, g)

    def onehot(self, t, n, dtype):
        return self.c.equal(t[:, None], self.c.arange(n, dtype=t.dtype)).astype(dtype)

    def scale(self, a, s):
        return self.c.multiply(a, s)

    def broadcast(self, a, shape):
        return a.broadcast_to(shape)


def train_steps(F, p, x, t, steps=2, lr=0.05):
    """Forward, hand-written backward and an SGD update; returns the losses."""
    losses = []
    n = x.shape[0]
    for _ in range(steps):
        # forward
        c1 = F.conv(x, p['w1'], None, 1, 1)
        b1, bn_state = F.batch_norm(c1, p['gamma'], p['beta'], p['rm'], p['rv'])
        r1 = F.relu(b1)
        m1 = F.max_pool(r1, 2, 2, 0)
        c2 = F.conv(m1, p['w2'], p['b2'], 2, 1)
        r2 = F.relu(c2)
        a2 = F.average_pool(r2, r2.shape[2], 1, 0, 'zero')
        h = a2.reshape((n, -1))
        logits = F.linear(h, p['w3'], p['b3'])
        logp = F.log_softmax(logits, 1)
        onehot = F.onehot(t, logits.shape[1], logp.dtype)
        losses.append(float(F.get(F.scale(F.sum(F.multiply(logp, onehot)), -1.0 / n))))
        # backward
        dlogits = F.scale(F.subtract(F.exp(logp), onehot), 1.0 / n)
        gw3 = F.dot(dlogits.T, h)
        gb3 = F.sum(dlogits, 0)
        gh = F.dot(dlogits, p['w3'])
        ga2 = gh.reshape(a2.shape)
        gr2 = F.average_pool_grad(r2, ga2, r2.shape[2], 1, 0, 'zero')
        gc2 = F.relu_grad(c2, gr2)
        gw2 = F.conv_grad_weight(p['w2'], m1, gc2, 2, 1)
        gb2 = F.sum(gc2, (0, 2, 3))
        gm1 = F.conv_transpose(gc2, p['w2'], None, 2, 1, m1.shape[2:])
        gr1 = F.max_pool_grad(r1, gm1, 2, 2, 0)
        gb1 = F.relu_grad(b1, gr1)
        gc1, ggamma, gbeta = F.batch_norm_grad(c1, p['gamma'], gb1, bn_state)
        gw1 = F.conv_grad_weight(p['w1'], x, gc1, 1, 1)
        # SGD
        for name, g in (('w1', gw1), ('gamma', ggamma), ('beta', gbeta), ('w2', gw2), ('b2', gb2), ('w3', gw3), ('b3', gb3)):
            p[name] = F.subtract(p[name], F.scale(g, lr))
    return losses


def test_two_sgd_steps_match_the_oracle():
    import chainer_amd as chx
    rng = np.random.default_rng(60)
    n = 8
    x = rng.standard_normal((n, 3, 12, 12)).astype('float32')
    t = rng.integers(0, 10, n).astype('int32')
    p0 = {
        'w1': (rng.standard_normal((8, 3, 3, 3)) * 0.3).astype('float32'),
        'gamma': rng.uniform(0.5, 1.5, 8).astype('float32'), 'beta': (rng.standard_normal(8) * 0.1).astype('float32'),
        'rm': np.zeros(8, 'float32'), 'rv': np.ones(8, 'float32'),
        'w2': (rng.standard_normal((16, 8, 3, 3)) * 0.2).astype('float32'), 'b2': np.zeros(16, 'float32'),
        'w3': (rng.standard_normal((10, 16)) * 0.3).astype('float32'), 'b3': np.zeros(10, 'float32'),
    }
    po = {k: v.copy() for k, v in p0.items()}
    pd = {k: chx.array(v) for k, v in p0.items()}
    lo = train_steps(OracleOps, po, x, t)
    ld = train_steps(DeviceOps(chx), pd, chx.array(x), chx.array(t))
    assert lo[1] < lo[0], 'the oracle step must reduce the loss: %r' % (lo,)
    assert np.allclose(ld, lo, rtol=1e-5, atol=1e-6), (ld, lo)
    for k in po:
        assert_close(pd[k].get(), po[k], 2e-5, 'parameter %s after two steps' % k)


def test_resnet_training_step_matches_the_oracle():
    """One SGD step of a bottleneck ResNet (one block per stage, 64x64 images) through configs.resnet50_train_step: conv / batch
    norm (batch statistics) / ReLU / pooling / linear forward, every backward kernel, the update.  Device against oracle."""
    import copy
    import chainer_amd as chx
    from chainer_amd import configs as cfg
    p0 = cfg.resnet50_params(seed=7, dtype=np.float32, n_out=10, blocks=(1, 1, 1, 1))
    rng = np.random.default_rng(70)
    x = rng.standard_normal((8, 3, 64, 64)).astype('float32')
    t = rng.integers(0, 10, 8).astype('int32')
    po = copy.deepcopy(p0)
    pd = cfg.tree_map(chx.array, copy.deepcopy(p0))
    loss_o = float(np.asarray(cfg.resnet50_train_step(OracleOps, po, x, t, 0.05)))
    loss_d = float(cfg.resnet50_train_step(cfg.DeviceTrainOps(chx), pd, chx.array(x), chx.array(t), 0.05).get())
    assert abs(loss_d - loss_o) <= 1e-4 * abs(loss_o), (loss_d, loss_o)

    def compare(a, b, path):
        if isinstance(a, dict):
            for k in a:
                compare(a[k], b[k], path + '/' + str(k))
        elif isinstance(a, list):
            for i, (u, v) in enumerate(zip(a, b)):
                compare(u, v, path + '/' + str(i))
        else:
            assert_close(a.get(), np.asarray(b), 2e-3, 'parameter %s after one step' % path)
    compare(pd, po, '')
    changed = np.abs(np.asarray(po['conv1']) - p0['conv1']).max()
    assert changed > 0, 'the step must have updated the first filters'
