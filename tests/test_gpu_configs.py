"""The five workloads end to end through the C ABI, against the CPU oracle on sizes the oracle finishes in seconds,
and through size-independent properties at the full benchmark size."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close, assert_exact

pytestmark = pytest.mark.gpu


def to_dev(chx, cfg, p):
    return cfg.tree_map(chx.array, p)


def test_mlp_full_size():
    """Config 1 at its real size: fp32 batch 100, 784-1000-1000-10, softmax cross entropy."""
    import chainer_amd as chx
    from chainer_amd import configs as cfg
    p = cfg.mlp_params()
    x, t = cfg.mlp_input()
    y1, l1 = cfg.mlp_forward(chx, to_dev(chx, cfg, p), chx.array(x), chx.array(t))
    y2, l2 = cfg.mlp_forward(O, p, x, t)
    assert_close(y1.get(), y2, 1e-5, 'logits', elementwise=True)
    assert_close(l1.get(), l2, 1e-5, 'loss', elementwise=True)
    assert_exact(chx.argmax(y1, 1).get(), O.argmax(y2, 1), 'predictions')


def test_cifar_convnet():
    """Config 3 (fp32) on a batch of 4 against the oracle."""
    import chainer_amd as chx
    from chainer_amd import configs as cfg
    p = cfg.cifar_params()
    x = cfg.cifar_input(batch=4)
    assert_close(cfg.cifar_forward(chx, to_dev(chx, cfg, p), chx.array(x)).get(), cfg.cifar_forward(O, p, x), 1e-5, 'cifar logits', elementwise=True)


def test_resnet50_fp16_against_oracle_and_batch_invariance():
    """Config 4: batch 2 at 224x224 against the oracle (2e-2), then the full batch of 128: every image's logits must not
    depend on the batch it is computed in (same kernels, same per-output accumulation order)."""
    import chainer_amd as chx
    from chainer_amd import configs as cfg
    p = cfg.resnet50_params()
    pd = to_dev(chx, cfg, p)
    x = cfg.resnet50_input(batch=128)
    ref = cfg.resnet50_forward(O, p, x[:2])
    y2 = cfg.resnet50_forward(chx, pd, chx.array(x[:2])).get()
    assert np.isfinite(ref.astype(np.float32)).all()
    assert_close(y2, ref, 2e-2, 'batch 2 vs oracle', elementwise=True)
    assert np.array_equal(y2.argmax(1), ref.argmax(1))
    y128 = cfg.resnet50_forward(chx, pd, chx.array(x)).get()
    assert y128.shape == (128, 1000) and np.isfinite(y128.astype(np.float32)).all()
    assert_close(y128[:2], y2, 1e-3, 'batch 128 vs batch 2')
    y_tail = cfg.resnet50_forward(chx, pd, chx.array(x[120:])).get()
    assert_close(y128[120:], y_tail, 1e-3, 'last images of the batch')


def test_lstm_language_model():
    """Config 5 on a reduced vocabulary against the oracle, and the real-size gather/projection shapes bit-exact / 1e-5."""
    import chainer_amd as chx
    from chainer_amd import configs as cfg
    p = cfg.lstm_lm_params(vocab=1000, units=64)
    ids = cfg.lstm_lm_input(batch=8, seq=5, vocab=1000)
    o1, h1, c1 = cfg.lstm_lm_forward(chx, to_dev(chx, cfg, p), chx.array(ids), chx.zeros)
    o2, h2, c2 = cfg.lstm_lm_forward(O, p, ids, np.zeros)
    assert_close(o1.get(), o2, 1e-5, 'log-probabilities', elementwise=True)
    assert_close(h1[1].get(), h2[1], 1e-5, 'h')
    assert_close(c1[0].get(), c2[0], 1e-5, 'c')
    # full-size model, two time steps (the oracle's 650x10000 projection takes about a second per step)
    p = cfg.lstm_lm_params()
    ids = cfg.lstm_lm_input(seq=2)
    o1, h1, _ = cfg.lstm_lm_forward(chx, to_dev(chx, cfg, p), chx.array(ids), chx.zeros)
    o2, h2, _ = cfg.lstm_lm_forward(O, p, ids, np.zeros)
    assert_close(o1.get(), o2, 1e-5, 'full-size log-probabilities', elementwise=True)
    assert_exact(chx.argmax(o1, 1).get(), O.argmax(o2, 1), 'full-size predictions')
