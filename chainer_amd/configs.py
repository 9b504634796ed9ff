"""The five benchmark/parity workloads, written once against a routine namespace ``F``.

``F`` is either ``chainer_amd`` (device arrays, HIP kernels) or any module exposing the same
routine names on numpy arrays; the parity tests pass the CPU oracle there.  The graphs follow the
reference's example models and the Chainer functions' ``forward_chainerx`` decompositions:

* mlp:       examples/mnist/train_mnist.py, chainerx_cc/examples/mnist/train_mnist.cc:48-75
* sweep:     elementwise / reduction kernels one by one
* cifar:     3x3 conv stack with fixed batch norm (examples/cifar)
* resnet50:  chainerx_cc/examples/imagenet_py/resnet50.py:103-127,202-225 (stride on the first 1x1)
* lstm_lm:   examples/ptb/train_ptb.py:28-50 with L.LSTM = Linear(x) + Linear(h) -> F.lstm

Parameters and inputs are drawn from ``numpy.random.Generator(PCG64(seed))`` on the host.
"""
import numpy as np


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def _he_normal(rng, shape, dtype):
    fan_in = int(np.prod(shape[1:]))
    return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32).astype(dtype)


def _bn_params(rng, c, dtype):
    return {
        'gamma': rng.uniform(0.5, 1.5, c).astype(np.float32).astype(dtype),
        'beta': (rng.standard_normal(c) * 0.1).astype(np.float32).astype(dtype),
        'mean': (rng.standard_normal(c) * 0.1).astype(np.float32).astype(dtype),
        'var': rng.uniform(0.5, 1.5, c).astype(np.float32).astype(dtype),
    }


def tree_map(fn, tree):
    if isinstance(tree, dict):
        return {k: tree_map(fn, v) for k, v in tree.items()}
    if isinstance(tree, (list, tuple)):
        return [tree_map(fn, v) for v in tree]
    return fn(tree)


BN_EPS = 2e-5


def _bn(F, x, p):
    # chainer.functions.fixed_batch_normalization on a 4-D input with 1-D parameters: axis (0, 2, 3)
    # (chainer/functions/normalization/batch_normalization.py:832-840), eps 2e-5.
    return F.fixed_batch_norm(x, p['gamma'], p['beta'], p['mean'], p['var'], BN_EPS, (0, 2, 3))


# ---------------------------------------------------------------------------------------------
# C1: MNIST-shaped MLP + softmax cross entropy (fp32, batch 100)
# ---------------------------------------------------------------------------------------------
def mlp_params(seed=1, dtype=np.float32, n_in=784, n_units=1000, n_out=10):
    rng = _rng(seed)

    def lecun(shape):  # N(0, 1/fan_in), Chainer's default initializer
        return (rng.standard_normal(shape) / np.sqrt(shape[1])).astype(dtype)

    return {
        'w1': lecun((n_units, n_in)), 'b1': np.zeros(n_units, dtype),
        'w2': lecun((n_units, n_units)), 'b2': np.zeros(n_units, dtype),
        'w3': lecun((n_out, n_units)), 'b3': np.zeros(n_out, dtype),
    }


def mlp_input(seed=1, batch=100, dtype=np.float32, n_in=784, n_out=10):
    rng = _rng(seed + 1000)
    x = rng.random((batch, n_in)).astype(dtype)
    t = rng.integers(0, n_out, batch).astype(np.int32)
    return x, t


def mlp_forward(F, p, x, t):
    h = F.relu(F.linear(x, p['w1'], p['b1']))
    h = F.relu(F.linear(h, p['w2'], p['b2']))
    y = F.linear(h, p['w3'], p['b3'])
    return y, F.softmax_cross_entropy(y, t)


# ---------------------------------------------------------------------------------------------
# C3: CIFAR-shaped conv net inference (fp32 NCHW, batch 256)
# ---------------------------------------------------------------------------------------------
CIFAR_CHANNELS = (64, 64, 128, 128, 256, 256)


def cifar_params(seed=3, dtype=np.float32, n_out=10):
    rng = _rng(seed)
    p = {'convs': [], 'bns': []}
    c_in = 3
    for c_out in CIFAR_CHANNELS:
        p['convs'].append(_he_normal(rng, (c_out, c_in, 3, 3), dtype))
        p['bns'].append(_bn_params(rng, c_out, dtype))
        c_in = c_out
    p['fc_w'] = _he_normal(rng, (n_out, c_in), dtype)
    p['fc_b'] = np.zeros(n_out, dtype)
    return p


def cifar_input(seed=3, batch=256, dtype=np.float32):
    return _rng(seed + 1000).standard_normal((batch, 3, 32, 32)).astype(dtype)


def cifar_forward(F, p, x):
    h = x
    for i, (w, bn) in enumerate(zip(p['convs'], p['bns'])):
        h = F.relu(_bn(F, F.conv(h, w, None, 1, 1), bn))
        if i % 2 == 1:
            h = F.max_pool(h, 2, 2, 0)
    h = F.average_pool(h, h.shape[2], 1, 0, 'zero')  # global average pooling
    return F.linear(h, p['fc_w'], p['fc_b'])


# ---------------------------------------------------------------------------------------------
# C4: ResNet-50 inference (fp16 NCHW, batch 128)
# ---------------------------------------------------------------------------------------------
RESNET50_BLOCKS = (3, 4, 6, 3)


RESNET50_RESIDUAL_GAMMA_SCALE = 0.25


def resnet50_params(seed=4, dtype=np.float16, n_out=1000, residual_gamma_scale=RESNET50_RESIDUAL_GAMMA_SCALE, blocks=None):
    """He-normal filters and batch-norm statistics drawn as for the CIFAR net.  One deviation: gamma of the last
    batch norm of every residual branch is scaled by `residual_gamma_scale`.  With statistics that are drawn at random
    instead of measured, nothing normalises the residual stream: its magnitude grows ~1.4x per block and passes the
    float16 maximum in stage 4 (on the CPU oracle as well); the scale keeps every activation below ~100."""
    rng = _rng(seed)
    p = {'conv1': _he_normal(rng, (64, 3, 7, 7), dtype), 'bn1': _bn_params(rng, 64, dtype), 'stages': []}
    c_in = 64
    for si, n_blocks in enumerate(blocks or RESNET50_BLOCKS):
        mid = 64 * 2 ** si
        c_out = 4 * mid
        stage = []
        for bi in range(n_blocks):
            blk = {
                'conv1': _he_normal(rng, (mid, c_in, 1, 1), dtype), 'bn1': _bn_params(rng, mid, dtype),
                'conv2': _he_normal(rng, (mid, mid, 3, 3), dtype), 'bn2': _bn_params(rng, mid, dtype),
                'conv3': _he_normal(rng, (c_out, mid, 1, 1), dtype), 'bn3': _bn_params(rng, c_out, dtype),
            }
            g3 = blk['bn3']['gamma'].astype(np.float32) * np.float32(residual_gamma_scale)
            blk['bn3']['gamma'] = g3.astype(dtype)
            if bi == 0:
                blk['conv4'] = _he_normal(rng, (c_out, c_in, 1, 1), dtype)
                blk['bn4'] = _bn_params(rng, c_out, dtype)
            stage.append(blk)
            c_in = c_out
        p['stages'].append(stage)
    p['fc_w'] = _he_normal(rng, (n_out, c_in), dtype)
    p['fc_b'] = np.zeros(n_out, dtype)
    return p


def resnet50_params_mixed(**kwargs):
    """resnet50_params with the batch normalisation parameters and running statistics in float32: how a float16 network is trained
    (Chainer's mixed16 keeps them in float32, chainer/links/normalization/batch_normalization.py:213-268).  BatchNorm then computes
    in float32 (ResultType(x, gamma, beta), CX/routines/normalization.cc:176-180); an all-float16 call sums its statistics into
    float16 arrays, which overflow beyond a few thousand elements per channel."""
    p = resnet50_params(**kwargs)

    def widen(tree):
        for k, v in (tree.items() if isinstance(tree, dict) else enumerate(tree)):
            if isinstance(v, dict) and 'gamma' in v:
                tree[k] = {name: a.astype(np.float32) for name, a in v.items()}
            elif isinstance(v, (dict, list)):
                widen(v)
    widen(p)
    return p


def resnet50_input(seed=4, batch=128, dtype=np.float16, size=224):
    return _rng(seed + 1000).standard_normal((batch, 3, size, size)).astype(np.float32).astype(dtype)


def _bottleneck(F, blk, x, stride):
    h = F.relu(_bn(F, F.conv(x, blk['conv1'], None, stride, 0), blk['bn1']))
    h = F.relu(_bn(F, F.conv(h, blk['conv2'], None, 1, 1), blk['bn2']))
    h = _bn(F, F.conv(h, blk['conv3'], None, 1, 0), blk['bn3'])
    if 'conv4' in blk:
        sc = _bn(F, F.conv(x, blk['conv4'], None, stride, 0), blk['bn4'])
    else:
        sc = x
    return F.relu(F.add(h, sc))


def resnet50_forward(F, p, x):
    h = F.relu(_bn(F, F.conv(x, p['conv1'], None, 2, 3), p['bn1']))
    h = F.max_pool(h, 3, 2, 1, False)  # 112 -> 56
    for si, stage in enumerate(p['stages']):
        for bi, blk in enumerate(stage):
            h = _bottleneck(F, blk, h, 2 if (bi == 0 and si > 0) else 1)
    h = F.average_pool(h, h.shape[2], 1, 0, 'zero')
    return F.linear(h, p['fc_w'], p['fc_b'])


def _conv_bn_act(F, x, w, stride, pad, bn, residual=None, relu=True):
    """conv -> fixed batch norm -> (+ residual) -> ReLU through the fused entry point when `F` has one, else composed."""
    if hasattr(F, 'conv_bn_act'):
        return F.conv_bn_act(x, w, None, stride, pad, False, (bn['gamma'], bn['beta'], bn['mean'], bn['var']), BN_EPS, residual, relu)
    h = _bn(F, F.conv(x, w, None, stride, pad), bn)
    if residual is not None:
        h = F.add(h, residual)
    return F.relu(h) if relu else h


def resnet50_forward_fused(F, p, x):
    """The same network with every conv -> batch norm (-> add) -> ReLU group issued as one fused call."""
    h = _conv_bn_act(F, x, p['conv1'], 2, 3, p['bn1'])
    h = F.max_pool(h, 3, 2, 1, False)
    for si, stage in enumerate(p['stages']):
        for bi, blk in enumerate(stage):
            stride = 2 if (bi == 0 and si > 0) else 1
            sc = _conv_bn_act(F, h, blk['conv4'], stride, 0, blk['bn4'], relu=False) if 'conv4' in blk else h
            t = _conv_bn_act(F, h, blk['conv1'], stride, 0, blk['bn1'])
            t = _conv_bn_act(F, t, blk['conv2'], 1, 1, blk['bn2'])
            h = _conv_bn_act(F, t, blk['conv3'], 1, 0, blk['bn3'], residual=sc, relu=True)
    h = F.average_pool(h, h.shape[2], 1, 0, 'zero')
    return F.linear(h, p['fc_w'], p['fc_b'])


# ---------------------------------------------------------------------------------------------
# ResNet-50 training step: forward in training mode, the backward pass written out from the backward kernels, SGD.
# This is the kernel sequence the reference's ImageNet example issues through autograd
# (chainerx_cc/examples/imagenet_py/train_imagenet.py with resnet50.py); autograd itself is outside the backend.
# `F` supplies the kernels: DeviceTrainOps below for the device, an adapter over the CPU oracle in the tests.
# ---------------------------------------------------------------------------------------------
class DeviceTrainOps:
    """The call shapes resnet50_train_step uses, over the chainer_amd routines."""

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
        return self.c.batch_norm(x, gamma, beta, rm, rv, BN_EPS, 0.9)

    def relu_grad(self, x, g):
        """Gradient of Relu(x) = Maximum(0, x) as the reference's backward issues it: IfLessElse(x, 0, 0, g) on the input of the
        activation (chainerx/routines/misc.cc:34-58, 210-216), one kernel."""
        return self.c.if_less_else(x, 0, 0, g)

    def onehot(self, t, n, dtype):
        return self.c.equal(t[:, None], self.c.arange(n, dtype=t.dtype)).astype(dtype)

    def scale(self, a, s):
        return self.c.multiply(a, s)


def _unit_forward(F, x, w, bn, stride, pad, relu):
    """conv -> batch norm (batch statistics, running statistics updated in place) -> optional ReLU; returns (y, saved)."""
    c = F.conv(x, w, None, stride, pad)
    b, state = F.batch_norm(c, bn['gamma'], bn['beta'], bn['mean'], bn['var'])
    y = F.relu(b) if relu else b
    return y, (x, w, bn, stride, pad, c, state, b if relu else None)


def _unit_backward(F, saved, gy, grads, need_gx=True):
    x, w, bn, stride, pad, c, state, pre = saved
    g = F.relu_grad(pre, gy) if pre is not None else gy
    gc, ggamma, gbeta = F.batch_norm_grad(c, bn['gamma'], g, state)
    grads.append((bn, 'gamma', ggamma))
    grads.append((bn, 'beta', gbeta))
    grads.append((w, None, F.conv_grad_weight(w, x, gc, stride, pad)))
    return F.conv_transpose(gc, w, None, stride, pad, x.shape[2:]) if need_gx else None


def resnet50_train_step(F, p, x, t, lr=0.01):
    """One SGD step on softmax cross entropy (mean over the batch); updates `p` in place and returns the loss array."""
    n = x.shape[0]
    # ---- forward ----
    h0, s_stem = _unit_forward(F, x, p['conv1'], p['bn1'], 2, 3, True)
    h = F.max_pool(h0, 3, 2, 1, False)
    tape = []
    for si, stage in enumerate(p['stages']):
        for bi, blk in enumerate(stage):
            stride = 2 if (bi == 0 and si > 0) else 1
            a, s1 = _unit_forward(F, h, blk['conv1'], blk['bn1'], stride, 0, True)
            b, s2 = _unit_forward(F, a, blk['conv2'], blk['bn2'], 1, 1, True)
            c, s3 = _unit_forward(F, b, blk['conv3'], blk['bn3'], 1, 0, False)
            if 'conv4' in blk:
                sc, s4 = _unit_forward(F, h, blk['conv4'], blk['bn4'], stride, 0, False)
            else:
                sc, s4 = h, None
            pre = F.add(c, sc)
            h = F.relu(pre)
            tape.append((s1, s2, s3, s4, pre))
    pooled = F.average_pool(h, h.shape[2], 1, 0, 'zero')
    feat = pooled.reshape((n, -1))
    logits = F.linear(feat, p['fc_w'], p['fc_b'])
    logp = F.log_softmax(logits, 1)
    onehot = F.onehot(t, logits.shape[1], logp.dtype)
    loss = F.scale(F.sum(F.multiply(logp, onehot)), -1.0 / n)
    # ---- backward ----
    grads = []  # (container, key or None for the array itself, gradient)
    dlogits = F.scale(F.subtract(F.exp(logp), onehot), 1.0 / n)
    g_fc_w = F.dot(dlogits.T, feat)
    g_fc_b = F.sum(dlogits, 0)
    gh = F.average_pool_grad(h, F.dot(dlogits, p['fc_w']).reshape(pooled.shape), h.shape[2], 1, 0, 'zero')
    for (s1, s2, s3, s4, pre) in reversed(tape):
        g = F.relu_grad(pre, gh)
        gb = _unit_backward(F, s3, g, grads)
        ga = _unit_backward(F, s2, gb, grads)
        gx = _unit_backward(F, s1, ga, grads)
        gh = F.add(gx, _unit_backward(F, s4, g, grads) if s4 is not None else g)
    g0 = F.max_pool_grad(h0, gh, 3, 2, 1)
    _unit_backward(F, s_stem, g0, grads, need_gx=False)
    # ---- SGD ----
    updates = {}
    for container, key, g in grads:
        if key is None:
            updates[id(container)] = F.subtract(container, F.scale(g, lr))
        else:
            container[key] = F.subtract(container[key], F.scale(g.reshape(container[key].shape), lr))

    _replace_leaves(p, updates)  # filters are values of dicts: replace them where they live
    p['fc_w'] = F.subtract(p['fc_w'], F.scale(g_fc_w, lr))
    p['fc_b'] = F.subtract(p['fc_b'], F.scale(g_fc_b, lr))
    return loss


def _replace_leaves(tree, updates):
    """tree[k] = updates[id(tree[k])] for every leaf that has an update.  A module-level function on purpose: a recursive closure
    inside the step would form a reference cycle that keeps a whole generation of device arrays alive until the garbage
    collector happens to run."""
    for k, v in (tree.items() if isinstance(tree, dict) else enumerate(tree)):
        if isinstance(v, (dict, list)):
            _replace_leaves(v, updates)
        elif id(v) in updates:
            tree[k] = updates[id(v)]


def resnet50_flops(batch=128, size=224):
    """Multiply-add count x2 of every conv and the final linear layer."""
    total = 0

    def conv(c_in, c_out, k, hw_out):
        return 2 * c_in * c_out * k * k * hw_out * hw_out

    hw = size // 2
    total += conv(3, 64, 7, hw)
    hw = hw // 2
    c_in = 64
    for si, n_blocks in enumerate(RESNET50_BLOCKS):
        mid = 64 * 2 ** si
        c_out = 4 * mid
        for bi in range(n_blocks):
            if bi == 0 and si > 0:
                hw //= 2
            total += conv(c_in, mid, 1, hw) + conv(mid, mid, 3, hw) + conv(mid, c_out, 1, hw)
            if bi == 0:
                total += conv(c_in, c_out, 1, hw)
            c_in = c_out
    total += 2 * c_in * 1000
    return total * batch


# ---------------------------------------------------------------------------------------------
# C5: 2-layer LSTM language model inference (fp32, batch 128, seq 35)
# ---------------------------------------------------------------------------------------------
def lstm_lm_params(seed=5, dtype=np.float32, vocab=10000, units=650):
    rng = _rng(seed)

    def u(shape):
        return rng.uniform(-0.05, 0.05, shape).astype(dtype)

    p = {'embed': u((vocab, units)), 'layers': [], 'out_w': u((vocab, units)), 'out_b': u((vocab,))}
    for _ in range(2):
        p['layers'].append({'up_w': u((4 * units, units)), 'up_b': u((4 * units,)), 'lat_w': u((4 * units, units))})
    return p


def lstm_lm_input(seed=5, batch=128, seq=35, vocab=10000):
    return _rng(seed + 1000).integers(0, vocab, (batch, seq)).astype(np.int32)


def lstm_lm_forward(F, p, ids, zeros, take_mode=None, fused=False):
    """Runs the sequence; returns log-probabilities of the last step and the final (h, c) of both layers.
    ``zeros(shape, dtype)`` makes the initial state on the same backend as ``F``.  ``fused`` takes the opt-in one-kernel
    Lstm cell and LogSoftmax (``F.lstm_fused``, ``F.log_softmax_fused``) instead of the routine chains."""
    lstm = F.lstm_fused if fused else F.lstm
    log_softmax = F.log_softmax_fused if fused else F.log_softmax
    batch, seq = ids.shape
    units = p['embed'].shape[1]
    dtype = p['embed'].dtype
    hs = [zeros((batch, units), dtype) for _ in range(2)]
    cs = [zeros((batch, units), dtype) for _ in range(2)]
    y = None
    for t in range(seq):
        x = F.take(p['embed'], ids[:, t], 0, take_mode)
        for li, layer in enumerate(p['layers']):
            gates = F.add(F.linear(x, layer['up_w'], layer['up_b']), F.linear(hs[li], layer['lat_w']))
            hs[li], cs[li] = lstm(cs[li], gates)
            x = hs[li]
        y = F.linear(x, p['out_w'], p['out_b'])
    return log_softmax(y, 1), hs, cs
