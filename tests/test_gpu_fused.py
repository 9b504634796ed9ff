"""The opt-in fused entry point hipcx_conv_bn_act against the composition of the reference's separate kernels
(conv -> fixed_batch_norm -> add -> relu) evaluated by the CPU oracle."""
import numpy as np
import pytest

from oracle import native as O
from helpers import assert_close, channels_last

pytestmark = pytest.mark.gpu


def ref_block(x, w, b, stride, pad, bn, residual, relu):
    y = O.conv(x, w, b, stride, pad)
    if bn is not None:
        y = O.fixed_batch_norm(y, *bn, 2e-5, (0, 2, 3))
    if residual is not None:
        y = O.add(y, residual)
    return O.relu(y) if relu else y


CASES = [  # N, C, H, W, K, R, stride, pad
    (2, 64, 8, 8, 64, 1, 1, 0), (3, 32, 14, 14, 128, 1, 2, 0), (2, 16, 12, 12, 32, 3, 1, 1), (4, 64, 7, 7, 256, 1, 1, 0),
    (2, 128, 7, 7, 128, 3, 1, 1), (1, 3, 20, 20, 16, 7, 2, 3), (2, 24, 6, 6, 40, 3, 2, 1), (2, 3, 32, 32, 64, 7, 2, 3),
]


@pytest.mark.parametrize('dt,tol', [('float16', 2e-2), ('float32', 1e-5)])
def test_conv_bn_act_matches_composition(dt, tol):
    import chainer_amd as chx
    rng = np.random.default_rng(0)
    for (N, C, H, W, K, R, st, pd) in CASES:
        x = rng.standard_normal((N, C, H, W)).astype(dt)
        w = (rng.standard_normal((K, C, R, R)) / np.sqrt(C * R * R)).astype(dt)
        b = rng.standard_normal(K).astype(dt)
        bn = [rng.uniform(0.5, 1.5, K).astype(dt), (rng.standard_normal(K) * 0.1).astype(dt), (rng.standard_normal(K) * 0.1).astype(dt),
              rng.uniform(0.5, 1.5, K).astype(dt)]
        oh = (H + 2 * pd - R) // st + 1
        res = rng.standard_normal((N, K, oh, oh)).astype(dt)
        for use_bn, use_res, relu, bias in [(True, True, True, False), (True, False, True, False), (True, False, False, True),
                                            (False, True, True, True), (False, False, False, False)]:
            ref = ref_block(x, w, b if bias else None, st, pd, bn if use_bn else None, res if use_res else None, relu)
            for lay, X in (('nchw', chx.array(x)), ('nhwc', channels_last(chx, x))):
                y = chx.conv_bn_act(X, chx.array(w), chx.array(b) if bias else None, st, pd, False,
                                    [chx.array(a) for a in bn] if use_bn else None, 2e-5, chx.array(res) if use_res else None, relu)
                assert_close(y.get(), ref, tol, '%s %s bn=%s res=%s relu=%s %s' % (dt, lay, use_bn, use_res, relu, (N, C, H, W, K, R, st, pd)))


def test_relu_lets_nan_through_and_params_may_be_keepdims():
    import chainer_amd as chx
    rng = np.random.default_rng(1)
    x = rng.standard_normal((1, 32, 4, 4)).astype('float16')
    x[0, 0, 1, 1] = np.nan
    w = (rng.standard_normal((32, 32, 1, 1)) / 6).astype('float16')
    bn = [np.ones(32, 'float16'), np.zeros(32, 'float16'), np.zeros(32, 'float16'), np.ones(32, 'float16')]
    y = chx.conv_bn_act(chx.array(x), chx.array(w), None, 1, 0, False, [chx.array(a.reshape(1, 32, 1, 1)) for a in bn], 2e-5, None, True).get()
    ref = ref_block(x, w, None, 1, 0, bn, None, True)
    assert np.isnan(y[0, :, 1, 1]).all() and np.array_equal(np.isnan(y), np.isnan(ref))
    with pytest.raises(chx.DimensionError):
        chx.conv_bn_act(chx.array(x), chx.array(w), None, 1, 0, False, [chx.array(a[:5]) for a in bn], 2e-5, None, True)


def test_resnet50_fused_forward():
    """The fused network against the oracle's unfused one (batch 2), and against the unfused hip path at batch 16."""
    import chainer_amd as chx
    from chainer_amd import configs as cfg
    p = cfg.resnet50_params()
    pd = cfg.tree_map(chx.array, p)
    x = cfg.resnet50_input(batch=16)
    ref = cfg.resnet50_forward(O, p, x[:2])
    y = cfg.resnet50_forward_fused(chx, pd, chx.array(x[:2])).get()
    assert_close(y, ref, 2e-2, 'fused vs oracle')
    assert np.array_equal(y.argmax(1), ref.argmax(1))
    y16 = cfg.resnet50_forward_fused(chx, pd, chx.array(x)).get()
    u16 = cfg.resnet50_forward(chx, pd, chx.array(x)).get()
    assert_close(y16, u16, 2e-2, 'fused vs unfused hip')
