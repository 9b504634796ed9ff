#!/usr/bin/env python3
"""Per-operation and per-workload measurements of the hip kernels against the MI355X rooflines.

    python -m chainer_amd.bench_ops [--section sweep,mlp,cifar,resnet_layers,lstm,backward,train,linalg]
    python bench.py --ops [sections]        (the same, plus a CPU baseline column)

Every figure is device time between two events recorded on the launch stream around `iters` back-to-back calls
(after warm-up), divided by `iters`; the sweep section also replays ten calls captured into one HIP graph and keeps the
smaller figure, because the host needs longer to issue a call than the shortest kernels run.  Bandwidth figures divide the *algorithmic* bytes of the operation (each operand
once, no temporaries) by that time; the fraction is taken against the published peaks (8 TB/s HBM, 2.5 PFLOP/s dense
fp16 MFMA, 157.3 TFLOP/s fp32 MFMA).  Chains of kernels (log_softmax = 7 launches, softmax_cross_entropy, the LSTM
cell) are timed as the chain and priced against the bytes a single fused pass would move.

`run(sections, cpu=namespace)` additionally times each operation on a CPU implementation of the same routine names that
the caller passes in (bench.py passes its single-threaded restatement of the ChainerX native backend; bounded sample
sizes) for the "next to the native backend" column.  This module itself only knows the hip kernels.  Output: one JSON
object per line.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

HBM_PEAK = 8000.0  # GB/s
MFMA_PEAK = {'float16': 2500.0, 'float32': 157.3}  # TFLOP/s
FAMILY_REPS = 4  # calls per operation in the `families` section (after one warm-up call)


def device_time(fn, iters=20, warmup=5, rounds=3):
    """Seconds per call: HIP events around `iters` back-to-back calls, best of `rounds` (a round that happens to grow the
    allocator's pool or to load a code object is not the kernel's time)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    best = None
    for _ in range(rounds):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        e1.synchronize()
        t = e0.elapsed_time(e1) / iters * 1e-3
        best = t if best is None else min(best, t)
    return best


def graph_time(fn, iters=20):
    """Seconds per replay of `fn` captured into a HIP graph (launch overhead of its kernels removed)."""
    import torch
    from chainer_amd.graph import capture
    g = capture(fn)
    g.replay()
    torch.cuda.synchronize()
    seconds = device_time(g.replay, iters, 3)
    g.release()
    return seconds


def kernel_time(fn, reps=10):
    """Seconds per call of `fn` with the host out of the picture: `reps` back-to-back calls captured into one HIP graph and
    replayed (a call through ctypes costs the host 10-20 us, which would otherwise bound every kernel shorter than that)."""
    def burst():
        return [fn() for _ in range(reps)]
    return graph_time(burst) / reps


def op_time(fn):
    """The smaller of the eager and the graph-burst figure: the kernel's time, whichever way the host gets out of the way."""
    return min(device_time(fn), kernel_time(fn))


def cpu_time(fn, min_s=0.2):
    fn()
    t0 = time.perf_counter()
    n = 0
    while True:
        fn()
        n += 1
        dt = time.perf_counter() - t0
        if dt > min_s:
            return dt / n


def emit(**kw):
    print(json.dumps(kw), flush=True)


def bw_row(section, name, shape, seconds, nbytes, launches=1, cpu_s=None, note=None):
    row = dict(section=section, op=name, shape=list(shape), us=round(seconds * 1e6, 2), launches=launches,
               algorithmic_MB=round(nbytes / 1e6, 2), GBps=round(nbytes / seconds / 1e9, 1),
               hbm_frac=round(nbytes / seconds / 1e9 / HBM_PEAK, 4))
    if cpu_s is not None:
        row['cpu_native_1core_us'] = round(cpu_s * 1e6, 1)
    if note:
        row['note'] = note
    emit(**row)


def section_sweep(chx, oracle, with_cpu):
    """Config 2: elementwise / reduction sweep, float32 [4096,4096] and [64,1048576]."""
    rng = np.random.default_rng(2)
    for shape in ((4096, 4096), (64, 1048576)):
        x = rng.standard_normal(shape).astype(np.float32)
        b = rng.standard_normal(shape[1]).astype(np.float32)
        X, B = chx.array(x), chx.array(b)
        n, s = x.size, 4
        rows = shape[0]
        small = x[:max(1, rows // 64)] if with_cpu else None  # CPU sample: 1/64 of the rows, scaled back up
        scale = rows / max(1, rows // 64)
        ops = [
            ('x+b', lambda: chx.add(X, B), 2 * n * s + b.nbytes, 1, (lambda: oracle.add(small, b)) if with_cpu else None),
            ('x*b', lambda: chx.multiply(X, B), 2 * n * s + b.nbytes, 1, (lambda: oracle.multiply(small, b)) if with_cpu else None),
            ('exp', lambda: chx.exp(X), 2 * n * s, 1, (lambda: oracle.exp(small)) if with_cpu else None),
            ('tanh', lambda: chx.tanh(X), 2 * n * s, 1, (lambda: oracle.tanh(small)) if with_cpu else None),
            ('sum axis1', lambda: chx.sum(X, 1), n * s + rows * s, 1, (lambda: oracle.sum(small, 1)) if with_cpu else None),
            ('max axis1', lambda: chx.amax(X, 1), n * s + rows * s, 1, (lambda: oracle.amax(small, 1)) if with_cpu else None),
            ('argmax axis1', lambda: chx.argmax(X, 1), n * s + rows * 8, 1, (lambda: oracle.argmax(small, 1)) if with_cpu else None),
            ('log_softmax axis1', lambda: chx.log_softmax(X, 1), (2 if shape[1] * s <= 65536 else 3) * n * s, 7,
             (lambda: oracle.log_softmax(small, 1)) if with_cpu else None),
            ('log_softmax axis1, fused opt-in entry', lambda: chx.log_softmax_fused(X, 1), (2 if shape[1] * s <= 65536 else 3) * n * s,
             1 if shape[1] * s <= 65536 else 2, None),
        ]
        for name, fn, nbytes, launches, cfn in ops:
            t = op_time(fn)
            cpu = cpu_time(cfn) * scale if cfn is not None else None
            note = None
            if 'fused' in name:
                note = 'hipcx_log_softmax: one read + one write for rows up to 64 KiB, two reads + one write beyond; not the drop-in kernel boundary'
            elif launches > 1:
                note = ('7 kernel launches as the ChainerX routine decomposes it (moves 8*N*4 bytes: ceiling %.0f%% of the '
                        'fused-ideal figure used here)' % (100.0 * nbytes / (8 * n * s)))
            bw_row('sweep', name, shape, t, nbytes, launches, cpu, note)


def section_mlp(chx, oracle, with_cpu):
    """Config 1: MNIST-shaped MLP forward + softmax cross entropy, float32 batch 100 (launch-latency bound)."""
    from chainer_amd import configs as cfg
    p = cfg.mlp_params()
    x, t = cfg.mlp_input()
    pd = cfg.tree_map(chx.array, p)
    X, T = chx.array(x), chx.array(t)
    fn = lambda: cfg.mlp_forward(chx, pd, X, T)
    eager = device_time(fn)
    graph = graph_time(fn)
    flops = 2 * 100 * (784 * 1000 + 1000 * 1000 + 1000 * 10)
    row = dict(section='mlp', op='forward+loss', batch=100, eager_us=round(eager * 1e6, 1), graph_replay_us=round(graph * 1e6, 1),
               kernel_launches=3 + 3 + 2 + 15, GFLOP=round(flops / 1e9, 4), TFLOPs_graph=round(flops / graph / 1e12, 2))
    if with_cpu:
        row['cpu_native_1core_us'] = round(cpu_time(lambda: cfg.mlp_forward(oracle, p, x, t)) * 1e6, 1)
    emit(**row)


def section_cifar(chx, oracle, with_cpu):
    """Config 3: CIFAR-shaped convnet inference, float32 batch 256."""
    from chainer_amd import configs as cfg
    p = cfg.cifar_params()
    x = cfg.cifar_input()
    pd = cfg.tree_map(chx.array, p)
    X = chx.array(x)
    fn = lambda: cfg.cifar_forward(chx, pd, X)
    eager = device_time(fn, 10, 3)
    graph = graph_time(fn, 10)
    flops = 78.22e9
    row = dict(section='cifar', op='forward', batch=256, dtype='float32', eager_ms=round(eager * 1e3, 3),
               graph_replay_ms=round(graph * 1e3, 3), img_per_s=round(256 / graph, 1), TFLOPs=round(flops / graph / 1e12, 2),
               fp32_mfma_frac=round(flops / graph / 1e12 / MFMA_PEAK['float32'], 4))
    if with_cpu:
        xs = x[:2]
        row['cpu_native_1core_img_per_s'] = round(2 / cpu_time(lambda: cfg.cifar_forward(oracle, p, xs), 1.0), 3)
    emit(**row)


RESNET_LAYERS = [  # N, C, H, W, K, R, S, stride, pad, occurrences in ResNet-50
    (128, 3, 224, 224, 64, 7, 7, 2, 3, 1),
    (128, 64, 56, 56, 64, 1, 1, 1, 0, 1), (128, 64, 56, 56, 64, 3, 3, 1, 1, 3), (128, 64, 56, 56, 256, 1, 1, 1, 0, 4),
    (128, 256, 56, 56, 64, 1, 1, 1, 0, 2), (128, 256, 56, 56, 128, 1, 1, 2, 0, 1), (128, 256, 56, 56, 512, 1, 1, 2, 0, 1),
    (128, 128, 28, 28, 128, 3, 3, 1, 1, 4), (128, 128, 28, 28, 512, 1, 1, 1, 0, 4), (128, 512, 28, 28, 128, 1, 1, 1, 0, 3),
    (128, 512, 28, 28, 256, 1, 1, 2, 0, 1), (128, 512, 28, 28, 1024, 1, 1, 2, 0, 1), (128, 256, 14, 14, 256, 3, 3, 1, 1, 6),
    (128, 256, 14, 14, 1024, 1, 1, 1, 0, 6), (128, 1024, 14, 14, 256, 1, 1, 1, 0, 5), (128, 1024, 14, 14, 512, 1, 1, 2, 0, 1),
    (128, 1024, 14, 14, 2048, 1, 1, 2, 0, 1), (128, 512, 7, 7, 512, 3, 3, 1, 1, 3), (128, 512, 7, 7, 2048, 1, 1, 1, 0, 3),
    (128, 2048, 7, 7, 512, 1, 1, 1, 0, 2),
]


def section_resnet_layers(chx, oracle, with_cpu):
    """Config 4 layer by layer: every distinct convolution (float16 NCHW in and out), and the bandwidth-bound kernels at
    the largest activation shape."""
    rng = np.random.default_rng(4)
    total = 0.0
    for (N, C, H, W, K, R, S, st, pd, cnt) in RESNET_LAYERS:
        x = rng.standard_normal((N, C, H, W)).astype(np.float16)
        w = (rng.standard_normal((K, C, R, S)) / np.sqrt(C * R * S)).astype(np.float16)
        X, Wd = chx.array(x), chx.array(w)
        OH = (H + 2 * pd - R) // st + 1
        flops = 2.0 * N * OH * OH * K * C * R * S
        nbytes = 2.0 * (x.size + w.size + N * K * OH * OH)
        t = op_time(lambda: chx.conv(X, Wd, None, st, pd))
        total += t * cnt
        emit(section='resnet_layers', op='conv', shape=[N, C, H, W], filters=[K, C, R, S], stride=st, pad=pd, count=cnt,
             us=round(t * 1e6, 1), TFLOPs=round(flops / t / 1e12, 1), mfma_frac=round(flops / t / 1e12 / MFMA_PEAK['float16'], 4),
             GBps=round(nbytes / t / 1e9, 1), hbm_frac=round(nbytes / t / 1e9 / HBM_PEAK, 4),
             bound='hbm' if nbytes / 8e12 > flops / 2.5e15 else 'mfma')
    emit(section='resnet_layers', op='all convolutions of one forward pass', ms=round(total * 1e3, 3), TFLOPs=round(987.6e9 / total / 1e12, 1))
    shape = (128, 256, 56, 56)
    x = rng.standard_normal(shape).astype(np.float16)
    X, Y = chx.array(x), chx.array(x)
    prm = [chx.array(rng.uniform(0.5, 1.5, shape[1]).astype(np.float16)) for _ in range(4)]
    n = x.size * 2
    bw_row('resnet_layers', 'fixed_batch_norm', shape, op_time(lambda: chx.fixed_batch_norm(X, *prm, 2e-5, (0, 2, 3))), 2 * n)
    bw_row('resnet_layers', 'relu', shape, op_time(lambda: chx.relu(X)), 2 * n)
    bw_row('resnet_layers', 'add (residual)', shape, op_time(lambda: chx.add(X, Y)), 3 * n)
    xp = chx.array(rng.standard_normal((128, 64, 112, 112)).astype(np.float16))
    bw_row('resnet_layers', 'max_pool 3x3/2 pad 1', (128, 64, 112, 112), op_time(lambda: chx.max_pool(xp, 3, 2, 1)), xp.nbytes * 1.25)
    xa = chx.array(rng.standard_normal((128, 2048, 7, 7)).astype(np.float16))
    bw_row('resnet_layers', 'average_pool 7x7 (global)', (128, 2048, 7, 7), op_time(lambda: chx.average_pool(xa, 7, 1, 0, 'zero')),
           xa.nbytes + 128 * 2048 * 2)


def section_lstm(chx, oracle, with_cpu):
    """Config 5: 2-layer LSTM language model inference, float32, batch 128, 35 steps, vocabulary 10000."""
    from chainer_amd import configs as cfg
    p = cfg.lstm_lm_params()
    ids = cfg.lstm_lm_input()
    pd = cfg.tree_map(chx.array, p)
    I = chx.array(ids)
    fn = lambda: cfg.lstm_lm_forward(chx, pd, I, chx.zeros)
    eager = device_time(fn, 3, 1)
    graph = graph_time(fn, 5)
    flops = 60.57e9 + 58.24e9
    row = dict(section='lstm', op='35-step forward', batch=128, eager_ms=round(eager * 1e3, 2), graph_replay_ms=round(graph * 1e3, 2),
               TFLOPs_graph=round(flops / graph / 1e12, 2), tokens_per_s_graph=round(128 * 35 / graph, 0), kernel_launches=35 * 86 + 7,
               note='eager time is host launch overhead (~3000 kernel calls); take runs in the default bounds mode (mode=None, what the '
                    'reference caller passes): an out-of-range id is recorded on the device and raised by the next get / synchronize')
    emit(**row)
    fused = graph_time(lambda: cfg.lstm_lm_forward(chx, pd, I, chx.zeros, None, True), 5)
    emit(section='lstm', op='35-step forward, fused opt-in Lstm cell and LogSoftmax', batch=128, graph_replay_ms=round(fused * 1e3, 2),
         TFLOPs_graph=round(flops / fused / 1e12, 2), tokens_per_s_graph=round(128 * 35 / fused, 0), kernel_launches=35 * 14 + 1,
         note='hipcx_lstm_cell and hipcx_log_softmax replace the ~25-kernel cell and the 7-kernel LogSoftmax chains; not the drop-in kernel boundary')
    # NStepLstm at the same size: 2 layers x 35 steps, batch 128, 650 units (float32)
    rng = np.random.default_rng(5)
    u = 650
    ws = [[chx.array(rng.uniform(-0.05, 0.05, (u, u)).astype(np.float32)) for _ in range(8)] for _ in range(2)]
    bs = [[chx.array(rng.uniform(-0.05, 0.05, (u,)).astype(np.float32)) for _ in range(8)] for _ in range(2)]
    xs = [chx.array(rng.standard_normal((128, u)).astype(np.float32)) for _ in range(35)]
    hx = chx.zeros((2, 128, u), 'float32')
    cx = chx.zeros((2, 128, u), 'float32')
    nflops = 2 * 35 * 2 * 2.0 * 128 * u * 4 * u
    composed = graph_time(lambda: chx.n_step_lstm(2, hx, cx, ws, bs, xs), 5)
    hoisted = graph_time(lambda: chx.n_step_lstm(2, hx, cx, ws, bs, xs, fused=True), 5)
    emit(section='lstm', op='n_step_lstm 2 layers x 35 steps, as the reference composes it', batch=128, units=u,
         graph_replay_ms=round(composed * 1e3, 2), TFLOPs_graph=round(nflops / composed / 1e12, 2),
         note='the composition restacks the eight gate matrices at every time step')
    emit(section='lstm', op='n_step_lstm 2 layers x 35 steps, opt-in: weights stacked once, one input Dot per layer, fused cell', batch=128,
         units=u, graph_replay_ms=round(hoisted * 1e3, 2), TFLOPs_graph=round(nflops / hoisted / 1e12, 2))
    entry = graph_time(lambda: chx.n_step_lstm(2, hx, cx, ws, bs, xs, kernel=True), 5)
    emit(section='lstm', op='n_step_lstm 2 layers x 35 steps, hipcx_n_step_lstm (the RnnKernel entry)', batch=128, units=u,
         graph_replay_ms=round(entry * 1e3, 2), TFLOPs_graph=round(nflops / entry / 1e12, 2), fp32_mfma_frac=round(nflops / entry / 157.3e12, 4),
         kernel_launches=36 + 12,
         note='weights packed once per call, one launch per wavefront stage (36), gates stay in the MFMA accumulators; the reference '
              'hands RnnKernel to its cuda backend only (routines/n_step_rnn.cc:210), so this entry is opt-in for a hip plugin')
    W = pd['embed']
    t = op_time(lambda: chx.take(W, I, 0))
    bw_row('lstm', 'take [10000,650] rows by [128,35] ids', (128, 35, 650), t, 2 * 128 * 35 * 650 * 4 + ids.nbytes)
    if with_cpu:
        ids2 = ids[:, :1]
        emit(section='lstm', op='cpu native 1 core, one time step', ms=round(cpu_time(lambda: cfg.lstm_lm_forward(oracle, p, ids2, np.zeros), 1.0) * 1e3, 1))


def section_backward(chx, oracle, with_cpu):
    """Backward / training kernels at ResNet-50 layer shapes (float16, batch 32).  The convolution gradients are compositions of
    the forward kernels (Im2Col / Col2Im copies plus one matrix product) -- functional, not tuned; batch normalisation, its
    gradient and the pooling gradients have kernels of their own.  Timed as bursts of ten calls in one HIP-graph replay (issued
    eagerly from Python the short ones would be host-bound, and a graph of a single kernel measures the replay's own latency)."""
    rng = np.random.default_rng(6)
    n, c, k, hw = 32, 256, 256, 14
    x = chx.array(rng.standard_normal((n, c, hw, hw)).astype(np.float16))
    w = chx.array((rng.standard_normal((k, c, 3, 3)) / np.sqrt(9 * c)).astype(np.float16))
    gy = chx.array(rng.standard_normal((n, k, hw, hw)).astype(np.float16))
    flops = 2.0 * n * hw * hw * k * c * 9
    for name, fn in (('conv_grad_weight 3x3', lambda: chx.conv_grad_weight('float16', w.shape, x, gy, 1, 1)),
                     ('conv_transpose 3x3', lambda: chx.conv_transpose(gy, w, None, 1, 1, (hw, hw))),
                     ('conv 3x3 (forward, for scale)', lambda: chx.conv(x, w, None, 1, 1))):
        t = op_time(fn)
        emit(section='backward', op=name, shape=[n, c, hw, hw, k], us=round(t * 1e6, 1), TFLOPs=round(flops / t / 1e12, 2),
             fp16_mfma_frac=round(flops / t / 1e12 / MFMA_PEAK['float16'], 4))
    shape = (32, 256, 56, 56)
    xb = chx.array(rng.standard_normal(shape).astype(np.float16))
    gb = chx.array(rng.standard_normal(shape).astype(np.float16))
    # float16 activations with float32 parameters and statistics (the mixed-precision call: the reference then computes in float32;
    # with float16 parameters its float16 sums over 100352 elements per channel overflow to inf, and so do this library's)
    prm = [chx.array(rng.uniform(0.5, 1.5, 256).astype(np.float32)) for _ in range(2)]
    rm, rv = chx.array(np.zeros(256, np.float32)), chx.array(np.ones(256, np.float32))
    nbytes = xb.nbytes
    out_state = []
    out_state[:] = [chx.batch_norm(xb, prm[0], prm[1], rm, rv)]
    t = op_time(lambda: chx.batch_norm(xb, prm[0], prm[1], rm, rv))
    bw_row('backward', 'batch_norm (training forward)', shape, t, 4 * nbytes, 5,
           note='algorithmic bytes: three reads (sum, centred sum of squares, normalise) and one write')
    state = out_state[0][1]
    t = op_time(lambda: chx.batch_norm_grad(xb, prm[0], gb, state))
    bw_row('backward', 'batch_norm_grad', shape, t, 5 * nbytes, 3,
           note='algorithmic bytes: x and gout read twice, gx written')
    xp = chx.array(rng.standard_normal((32, 64, 112, 112)).astype(np.float16))
    gp = chx.array(rng.standard_normal((32, 64, 56, 56)).astype(np.float16))
    t = op_time(lambda: chx.max_pool_grad(xp, gp, 3, 2, 1))
    bw_row('backward', 'max_pool_grad 3x3/2 pad 1', (32, 64, 112, 112), t, 2 * xp.nbytes + gp.nbytes, 2,
           note='window ArgMax kernel + gather kernel; bits of the Im2Col / ArgMax / Col2Im composition')
    xa = chx.array(rng.standard_normal((128, 2048, 7, 7)).astype(np.float16))
    ga = chx.array(rng.standard_normal((128, 2048, 1, 1)).astype(np.float16))
    t = op_time(lambda: chx.average_pool_grad(xa, ga, 7, 1, 0, 'zero'))
    bw_row('backward', 'average_pool_grad 7x7 (global)', (128, 2048, 7, 7), t, xa.nbytes + ga.nbytes)


def section_train(chx, oracle, with_cpu):
    """ResNet-50 training step (forward with batch statistics, hand-written backward, SGD) with float16 filters and activations and
    float32 batch normalisation parameters -- the kernel sequence of the reference's ImageNet example without its autograd bookkeeping.  Not the headline metric: it shows the backward set end to end."""
    import copy
    from chainer_amd import configs as cfg
    F = cfg.DeviceTrainOps(chx)
    p0 = cfg.resnet50_params_mixed()
    for batch in (32, 128):
        x = chx.array(cfg.resnet50_input(batch=batch))
        t = chx.array(np.random.default_rng(8).integers(0, 1000, batch).astype(np.int32))
        pd = cfg.tree_map(chx.array, copy.deepcopy(p0))
        step = lambda: cfg.resnet50_train_step(F, pd, x, t, 0.0)  # lr 0: the timed steps do not walk the weights into overflow
        eager = device_time(step, 2, 1, 1)
        graph = graph_time(step, 3)
        flops = 3.0 * cfg.resnet50_flops(batch)
        emit(section='train', op='ResNet-50 training step, float16 (batch norm parameters float32)', batch=batch, eager_ms=round(eager * 1e3, 2),
             graph_replay_ms=round(graph * 1e3, 2), img_per_s_graph=round(batch / graph, 1), TFLOPs_graph=round(flops / graph / 1e12, 1),
             note='3x the forward flops (forward, data gradient, weight gradient); eager time includes ~1500 Python-issued kernel calls')
        del pd


def section_linalg(chx, oracle, with_cpu):
    """Dense decompositions (float32): blocked LU / Cholesky, QR by columns and Jacobi rounds, all spread over many workgroups above
    about 64 to 100 rows.  The CPU column is LAPACK through numpy, which is what the native backend calls."""
    rng = np.random.default_rng(8)
    for n in (64, 256, 1024):
        a = (rng.standard_normal((n, n)) + np.sqrt(n) * np.eye(n)).astype(np.float32)
        sym = ((a + a.T) / 2).astype(np.float32)
        spd = (a @ a.T).astype(np.float32)
        b = rng.standard_normal((n, 8)).astype(np.float32)
        A, S, P, B = chx.array(a), chx.array(sym), chx.array(spd), chx.array(b)
        cases = (('solve (8 right-hand sides)', lambda: chx.solve(A, B), lambda: oracle.solve(a, b), 2 / 3 * n ** 3),
                 ('inv', lambda: chx.inv(A), lambda: oracle.inv(a), 2.0 * n ** 3),
                 ('cholesky', lambda: chx.cholesky(P), lambda: oracle.cholesky(spd), n ** 3 / 3),
                 ('qr reduced', lambda: chx.qr(A), lambda: oracle.qr(a), 8 / 3 * n ** 3),
                 ('eigh', lambda: chx.eigh(S), lambda: oracle.eigh(sym), None),
                 ('svd full', lambda: chx.svd(A), lambda: oracle.svd(a), None))
        for name, fn, cpu_fn, flops in cases:
            t = device_time(fn, 3 if n <= 256 else 1, 1)
            row = dict(section='linalg', op=name, shape=[n, n], dtype='float32', us=round(t * 1e6, 1))
            if flops is not None:
                row['GFLOPs'] = round(flops / t / 1e9, 2)
            if with_cpu:
                row['cpu_us'] = round(cpu_time(cpu_fn) * 1e6, 1)
            emit(**row)


def section_dot(chx, oracle, with_cpu):
    """Dot: the matrix products of the five workloads (as the Linear link hands them over: x row-major, W^T a view of the
    [out, in] weights) and a calibration product with both operands stored along the reduction axis."""
    rng = np.random.default_rng(5)
    cases = [
        ('MLP layer 1 (config 1)', 'float32', 100, 784, 1000),
        ('LSTM gates (config 5)', 'float32', 128, 650, 2600),
        ('LSTM output layer, 35 steps (config 5)', 'float32', 4480, 650, 10000),
        ('ResNet-50 classifier (config 4)', 'float16', 128, 2048, 1000),
        ('calibration', 'float16', 4096, 4096, 4096),
        ('calibration', 'float16', 8192, 8192, 8192),
    ]
    for name, dt, m, k, n in cases:
        a = rng.standard_normal((m, k)).astype(dt)
        wt = (rng.standard_normal((n, k)) / np.sqrt(k)).astype(dt)
        A, B = chx.array(a), chx.array(wt).T
        t = op_time(lambda: chx.dot(A, B))
        flops = 2.0 * m * n * k
        nbytes = (m * k + n * k + m * n) * a.dtype.itemsize
        peak = MFMA_PEAK[dt]
        row = dict(section='dot', op='dot %s [%d,%d] . [%d,%d]^T (%s)' % (dt, m, k, n, k, name), us=round(t * 1e6, 2), TFLOPs=round(flops / t / 1e12, 2),
                   mfma_frac=round(flops / t / 1e12 / peak, 4), GBps=round(nbytes / t / 1e9, 1), hbm_frac=round(nbytes / t / 1e9 / HBM_PEAK, 4),
                   bound='mfma' if flops / (peak * 1e12) >= nbytes / (HBM_PEAK * 1e9) else 'hbm')
        if with_cpu and m * n * k <= 4e8:
            row['cpu_native_1core_us'] = round(cpu_time(lambda: oracle.dot(a, np.ascontiguousarray(wt.T))) * 1e6, 1)
        emit(**row)


def section_families(chx, oracle, with_cpu):
    """One operation per hot-path kernel family, each called FAMILY_REPS times in a row (eagerly, nothing else in between), with
    its algorithmic bytes and flops: the run a counter profile (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE /
    SQ_VALU_MFMA_BUSY_CYCLES) is taken of, so that counters per dispatch can be set against what the operation has to move or
    compute.  `kernel` is a pattern the dispatched kernel's name matches; operations follow each other in the order printed."""
    rng = np.random.default_rng(8)
    reps = FAMILY_REPS
    f16, f32 = np.float16, np.float32
    act = chx.array(rng.standard_normal((128, 256, 56, 56)).astype(f16))
    act2 = chx.array(rng.standard_normal((128, 256, 56, 56)).astype(f16))
    n_act = 128 * 256 * 56 * 56
    bn = [chx.array(v.astype(f16)) for v in (rng.uniform(0.5, 1.5, 256), rng.normal(0, 0.1, 256), rng.normal(0, 0.1, 256), rng.uniform(0.5, 1.5, 256))]
    pool_in = chx.array(rng.standard_normal((128, 64, 112, 112)).astype(f16))
    x32 = chx.array(rng.standard_normal((4096, 4096)).astype(f32))
    table = chx.array(rng.standard_normal((10000, 650)).astype(f32))
    ids = chx.array(rng.integers(0, 10000, (128, 35)).astype(np.int32))
    a1, w1 = chx.array(rng.random((100, 784)).astype(f32)), chx.array((rng.standard_normal((1000, 784)) / 28).astype(f32))
    a5, w5 = chx.array(rng.standard_normal((128, 650)).astype(f32)), chx.array(rng.uniform(-0.05, 0.05, (2600, 650)).astype(f32))
    a5o, w5o = chx.array(rng.standard_normal((4480, 650)).astype(f32)), chx.array(rng.uniform(-0.05, 0.05, (10000, 650)).astype(f32))
    a4, w4 = chx.array(rng.standard_normal((128, 2048)).astype(f16)), chx.array((rng.standard_normal((1000, 2048)) / 45).astype(f16))
    ag, wg = chx.array(rng.standard_normal((4096, 4096)).astype(f16)), chx.array((rng.standard_normal((4096, 4096)) / 64).astype(f16))
    cx, cw = chx.array(rng.standard_normal((256, 64, 32, 32)).astype(f32)), chx.array((rng.standard_normal((64, 64, 3, 3)) / 24).astype(f32))
    px = chx.array(rng.standard_normal((128, 512, 28, 28)).astype(f16))
    pw = chx.array((rng.standard_normal((128, 512, 1, 1)) / 23).astype(f16))
    u = 650
    ws = [[chx.array(rng.uniform(-0.05, 0.05, (u, u)).astype(f32)) for _ in range(8)] for _ in range(2)]
    bs = [[chx.array(rng.uniform(-0.05, 0.05, (u,)).astype(f32)) for _ in range(8)] for _ in range(2)]
    xs = [chx.array(rng.standard_normal((128, u)).astype(f32)) for _ in range(35)]
    hx, cxs = chx.array(np.zeros((2, 128, u), f32)), chx.array(np.zeros((2, 128, u), f32))
    ops = [
        # name, kernel pattern, call, algorithmic bytes per dispatch, flops per dispatch, dispatches of that kernel per call
        ('residual add float16 [128,256,56,56]', r'EwKernel.*(Add|BinaryAA)', lambda: chx.add(act, act2), 3 * n_act * 2, 0, 1),
        ('relu float16 [128,256,56,56]', r'EwKernel.*(IfLess|Select|Relu)', lambda: chx.relu(act), 2 * n_act * 2, 0, 1),
        ('exp float32 [4096,4096]', r'EwKernel.*UnaryOp', lambda: chx.exp(x32), 2 * 4096 * 4096 * 4, 0, 1),
        ('fixed_batch_norm float16 [128,256,56,56]', r'BnChannelsFirstKernel', lambda: chx.fixed_batch_norm(act, *bn, axis=(0, 2, 3)), 2 * n_act * 2, 0, 1),
        ('max_pool 3x3/2 pad 1 float16 [128,64,112,112]', r'MaxPoolRowsS2Kernel', lambda: chx.max_pool(pool_in, 3, 2, 1, False),
         (128 * 64 * 112 * 112 + 128 * 64 * 56 * 56) * 2, 0, 1),
        ('take float32 [10000,650] by [128,35]', r'TakeRowsKernel', lambda: chx.take(table, ids, 0), 2 * 128 * 35 * 650 * 4 + 128 * 35 * 4, 0, 1),
        ('dot float32 [100,784].[784,1000] (config 1)', r'SmallDot', lambda: chx.dot(a1, w1.T), (100 * 784 + 784 * 1000 + 100 * 1000) * 4, 2.0 * 100 * 784 * 1000, 1),
        ('dot float32 [128,650].[650,2600] (config 5 gates)', r'SmallDot', lambda: chx.dot(a5, w5.T), (128 * 650 + 650 * 2600 + 128 * 2600) * 4, 2.0 * 128 * 650 * 2600, 1),
        ('dot float32 [4480,650].[650,10000] (config 5 output layer)', r'IGemmFastKernel<float', lambda: chx.dot(a5o, w5o.T),
         (4480 * 650 + 650 * 10000 + 4480 * 10000) * 4, 2.0 * 4480 * 650 * 10000, 1),
        ('dot float16 [128,2048].[2048,1000] (config 4 classifier)', r'SmallDot', lambda: chx.dot(a4, w4.T), (128 * 2048 + 2048 * 1000 + 128 * 1000) * 2, 2.0 * 128 * 2048 * 1000, 1),
        ('dot float16 [4096,4096].[4096,4096] (calibration)', r'GemmPpKernel', lambda: chx.dot(ag, wg.T), 3 * 4096 * 4096 * 2, 2.0 * 4096 ** 3, 1),
        ('conv float32 3x3 [256,64,32,32] -> 64 (config 3)', r'IGemmFastKernel<float', lambda: chx.conv(cx, cw, None, 1, 1),
         (2 * 256 * 64 * 32 * 32 + 64 * 64 * 9) * 4, 2.0 * 256 * 32 * 32 * 64 * 64 * 9, 1),
        ('conv float16 1x1 [128,512,28,28] -> 128', r'PwConvKernel', lambda: chx.conv(px, pw), (128 * 512 * 784 + 128 * 512 + 128 * 128 * 784) * 2, 2.0 * 128 * 784 * 128 * 512, 1),
        ('n_step_lstm float32 2 layers x 35 steps, batch 128, 650 units (RnnKernel entry)', r'LstmStepKernel',
         lambda: chx.n_step_lstm(2, hx, cxs, ws, bs, xs, kernel=True), 0, 2.0 * 128 * 4 * u * 2 * u * 2 * 35 / 36, 36),
    ]
    for name, pattern, fn, nbytes, flops, per_call in ops:
        fn()
        chx.synchronize()
        for _ in range(reps):
            fn()
        chx.synchronize()
        emit(section='families', op=name, kernel=pattern, calls=reps + 1, dispatches_per_call=per_call, algorithmic_bytes=int(nbytes), flops=float(flops))


def section_copy(chx, oracle, with_cpu):
    """A plain copy of known size (128 MiB read + 128 MiB written): the calibration point for HBM traffic counters."""
    x = chx.array(np.zeros(64 * 1024 * 1024, np.float16))
    t = op_time(lambda: chx.copy(x))
    bw_row('copy', 'copy float16 [67108864]', (64 * 1024 * 1024,), t, 2 * x.nbytes)


SECTIONS = {'copy': section_copy, 'sweep': section_sweep, 'dot': section_dot, 'families': section_families, 'mlp': section_mlp, 'cifar': section_cifar, 'resnet_layers': section_resnet_layers, 'lstm': section_lstm, 'backward': section_backward, 'train': section_train, 'linalg': section_linalg}


def run(sections, cpu=None):
    import chainer_amd as chx
    if not chx.device_available():
        sys.exit('bench_ops: no HIP device visible')
    for name in sections:
        SECTIONS[name](chx, cpu, cpu is not None)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--section', default=','.join(k for k in SECTIONS if k not in ('copy', 'families')))
    args = ap.parse_args()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    if root not in sys.path:
        sys.path.insert(0, root)
    run(args.section.split(','))


if __name__ == '__main__':
    main()
