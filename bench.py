#!/usr/bin/env python3
"""Headline benchmark: ResNet-50 float16 inference at batch 128 through the hip backend's kernels.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 128]

A step is one forward pass of the network of chainer_amd/configs.py (53 convolutions, fixed batch
norm, ReLU, residual adds, pooling, linear) over one synthetic batch that is already resident in
device memory.  Every operation is one C-ABI kernel call, decomposed as the ChainerX routines do.
One JSON line is printed; besides the contract keys it carries

  roofline      the implicit-GEMM convolution kernel (the dominant one): algorithmic flops of its
                launches in one step / their summed duration, measured with HIP events recorded on
                the launch stream around each launch (hipcx_profile_start/stop) in extra steps run
                after the timed region, against the dense fp16 MFMA peak.  `by_bound` splits the
                same launches by what bounds each one on paper (flops / 2.5 PFLOP/s against bytes /
                8 TB/s): the MFMA-bound launches against the MFMA peak, the HBM-bound ones against
                the HBM peak, and `max_bound_frac` = sum of each launch's larger bound time / sum
                of the measured durations.  `stream_copy` is a plain device copy timed in the same
                run: the HBM rate this box actually reaches.
  cpu_baseline  the CPU oracle (a single-threaded restatement of the ChainerX native backend) on a
                small batch of the same network, timed on this host.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16 matrix peak
HBM_PEAK_GBS = 8000.0          # MI355X HBM3E peak
# HBM bytes per launch of the dominant kernels (fetch + write, averaged over the 53 convolutions and the linear layer of one
# step), from two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) scaled by what the same counters read for a 128 MiB copy
# kernel (x1.999, x1.000): profiles/resnet50_conv_hbm_traffic.txt.  The algorithmic figure is 99.2 MB per launch.
CONV_HBM_TRAFFIC_BYTES_PER_LAUNCH = 111.4e6


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--batch', type=int, default=128)
    ap.add_argument('--eager', action='store_true', help='time eager launches instead of a HIP graph replay')
    ap.add_argument('--ops', nargs='?', const='copy,sweep,dot,mlp,cifar,resnet_layers,lstm,backward,train,linalg', default=None,
                    help='instead of the headline step, print per-operation roofline lines (chainer_amd.bench_ops) with a CPU baseline column')
    ap.add_argument('--cpu-batch', type=int, default=8, help='images for the CPU baseline (0 = skip)')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py: this build runs on one GPU only (inference shards trivially along the batch axis; '
                 'no multi-GPU path is built). Run with --gpus 1.')

    if args.ops is not None:
        from chainer_amd import bench_ops
        from oracle import native as oracle  # CPU baseline column only
        bench_ops.run(args.ops.split(','), cpu=oracle)
        return

    import torch
    import chainer_amd as chx
    from chainer_amd import _lib, configs as cfg

    if not torch.cuda.is_available():
        sys.exit('bench.py: no HIP device visible')

    params_host = cfg.resnet50_params()
    params = cfg.tree_map(chx.array, params_host)
    x = chx.array(cfg.resnet50_input(batch=args.batch))

    def step():
        return cfg.resnet50_forward(chx, params, x)

    # Warm-up runs eagerly (first-call kernel attribute set-up happens here); the step is then captured once into a HIP
    # graph on a side stream and the timed region replays it, so that the ~250 kernel launches of a step cost one host
    # call.  Every allocation inside the capture comes from the capture's private pool and stays valid across replays.
    for _ in range(max(args.warmup, 1)):
        y = step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        y = step()
    torch.cuda.synchronize()
    eager_ms = (time.perf_counter() - t0) / 3 * 1e3
    graph = None
    if not args.eager:
        from chainer_amd.graph import capture
        graph = capture(step)
        y = graph.result
        graph.replay()
        torch.cuda.synchronize()
        eager_out = step().get()
        if not np.array_equal(y.get().view(np.uint16), eager_out.view(np.uint16)):
            sys.exit('bench.py: graph replay differs from eager execution')

    def run():
        if graph is not None:
            graph.replay()
        else:
            step()

    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    img_s = args.batch * args.steps / elapsed
    if graph is None:
        y = step()
    finite = bool(np.isfinite(y.get().astype(np.float32)).all())

    # ---- roofline of the dominant kernel: event-bracketed implicit-GEMM launches, extra steps ----
    lib = _lib.load()
    prof_steps = max(1, min(args.steps, 5))
    _lib.check(lib.hipcx_profile_start())
    for _ in range(prof_steps):
        step()
    n = ctypes.c_int64()
    ms = ctypes.c_double()
    flops = ctypes.c_double()
    nbytes = ctypes.c_double()
    _lib.check(lib.hipcx_profile_stop(ctypes.byref(n), ctypes.byref(ms), ctypes.byref(flops), ctypes.byref(nbytes)))
    rec_n = ctypes.c_int64()
    rec_ms = (ctypes.c_double * n.value)()
    rec_flops = (ctypes.c_double * n.value)()
    rec_bytes = (ctypes.c_double * n.value)()
    _lib.check(lib.hipcx_profile_records(n.value, rec_ms, rec_flops, rec_bytes, ctypes.byref(rec_n)))
    groups = {'mfma': [0, 0.0, 0.0, 0.0], 'hbm': [0, 0.0, 0.0, 0.0]}  # launches, ms, flops, bytes
    bound_ms = 0.0
    for i in range(min(n.value, rec_n.value)):
        t_mfma = rec_flops[i] / (MFMA_F16_PEAK_TFLOPS * 1e12) * 1e3
        t_hbm = rec_bytes[i] / (HBM_PEAK_GBS * 1e9) * 1e3
        g = groups['mfma' if t_mfma >= t_hbm else 'hbm']
        g[0] += 1
        g[1] += rec_ms[i]
        g[2] += rec_flops[i]
        g[3] += rec_bytes[i]
        bound_ms += max(t_mfma, t_hbm)
    gm, gh = groups['mfma'], groups['hbm']
    by_bound = {
        'mfma_bound': {'launches_per_step': gm[0] // prof_steps, 'kernel_ms_per_step': round(gm[1] / prof_steps, 3),
                       'achieved_tflops': round(gm[2] / (gm[1] * 1e-3) / 1e12, 1) if gm[1] > 0 else 0.0,
                       'frac_of_mfma_peak': round(gm[2] / (gm[1] * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS, 4) if gm[1] > 0 else None},
        'hbm_bound': {'launches_per_step': gh[0] // prof_steps, 'kernel_ms_per_step': round(gh[1] / prof_steps, 3),
                      'achieved_gbs': round(gh[3] / (gh[1] * 1e-3) / 1e9, 1) if gh[1] > 0 else 0.0,
                      'frac_of_hbm_peak': round(gh[3] / (gh[1] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4) if gh[1] > 0 else None},
        'max_bound_ms_per_step': round(bound_ms / prof_steps, 3),
        'max_bound_frac': round(bound_ms / ms.value, 4) if ms.value > 0 else None,
    }

    # ---- a plain device copy (1 GiB read + 1 GiB written), ten back-to-back launches between two events (a launch lasts ~0.4 ms,
    # far longer than the host needs to issue it): what this box's HBM delivers ----
    big = chx.array(np.zeros(512 * 1024 * 1024, np.float16))
    from chainer_amd.bench_ops import device_time
    copy_s = device_time(lambda: chx.copy(big), iters=10, warmup=2, rounds=2)
    stream_copy = {'bytes': 2 * big.nbytes, 'us': round(copy_s * 1e6, 1), 'gbs': round(2 * big.nbytes / copy_s / 1e9, 1),
                   'frac_of_hbm_peak': round(2 * big.nbytes / copy_s / 1e9 / HBM_PEAK_GBS, 4)}
    del big

    launches_per_step = n.value // prof_steps
    avg_launch_ms = ms.value / max(n.value, 1)
    achieved_tflops = flops.value / (ms.value * 1e-3) / 1e12 if ms.value > 0 else 0.0
    roofline = {
        'kernel': 'NchwConvKernel / PwConvKernel / StemConv7x7s2Kernel / SmallDotKernel (every convolution and the linear layer of a pass, MFMA implicit GEMM)',
        'bound': 'mfma',
        'achieved': round(achieved_tflops, 2),
        'peak': MFMA_F16_PEAK_TFLOPS,
        'unit': 'TFLOP/s',
        'frac': round(achieved_tflops / MFMA_F16_PEAK_TFLOPS, 4),
        'traffic': CONV_HBM_TRAFFIC_BYTES_PER_LAUNCH if args.batch == 128 else None,
        'launches_per_step': launches_per_step,
        'avg_launch_us': round(avg_launch_ms * 1e3, 2),
        'kernel_ms_per_step': round(ms.value / prof_steps, 3),
        'algorithmic_gflop_per_step': round(flops.value / prof_steps / 1e9, 2),
        'algorithmic_gb_per_step': round(nbytes.value / prof_steps / 1e9, 3),
        'achieved_gbs': round(nbytes.value / (ms.value * 1e-3) / 1e9, 1) if ms.value > 0 else 0.0,
        'by_bound': by_bound,
        'stream_copy': stream_copy,
    }

    # ---- opt-in fused path (reported beside the headline, never as `value`): conv+bn(+add)+relu groups as one call ----
    fused = None
    if not args.eager:
        def fstep():
            return cfg.resnet50_forward_fused(chx, params, x)
        fgraph = capture(fstep)
        yf = fgraph.result
        for _ in range(max(args.warmup, 1)):
            fgraph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fgraph.replay()
        torch.cuda.synchronize()
        fel = time.perf_counter() - t0
        a = yf.get().astype(np.float64)
        b = y.get().astype(np.float64)
        fused = {
            'what': 'same network through hipcx_conv_bn_act: batch norm, residual add and ReLU run in the convolution epilogue '
                    '(53 fused calls + 2 pooling + linear/add instead of ~190 kernel calls); not the drop-in kernel boundary',
            'value': round(args.batch * args.steps / fel, 1), 'unit': 'img/s', 'ms_per_step': round(fel / args.steps * 1e3, 3),
            'max_rel_diff_vs_unfused': float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30)),
        }

    # ---- CPU baseline: the oracle on a bounded sample of the same workload ----
    cpu = None
    if args.cpu_batch > 0:
        from oracle import native as oracle
        xs = cfg.resnet50_input(batch=args.cpu_batch)
        t0 = time.perf_counter()
        ref = cfg.resnet50_forward(oracle, params_host, xs)
        cpu_s = time.perf_counter() - t0
        got = cfg.resnet50_forward(chx, params, chx.array(xs)).get().astype(np.float64)
        refd = ref.astype(np.float64)
        rel = float(np.abs(got - refd).max() / max(np.abs(refd).max(), 1e-30))
        cpu = {
            'value': round(args.cpu_batch / cpu_s, 3),
            'unit': 'img/s',
            'cores': 1,
            'kind': 'port',
            'sample': '%d images, one forward pass of the same ResNet-50 (fp16 storage, fp32 accumulation), %.1f s'
                      % (args.cpu_batch, cpu_s),
            'max_rel_err_vs_gpu': rel,
        }

    out = {
        'metric': 'ResNet-50 fp16 inference img/s @bs%d on 1 MI355X' % args.batch,
        'value': round(img_s, 1),
        'unit': 'img/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': round(ms_per_step, 3),
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'f16',
        'data': 'synthetic',
        'config': {
            'workload': 'ResNet-50 inference, fp16 NCHW [%d,3,224,224], bottlenecks [3,4,6,3], fixed batch norm, '
                        'one kernel call per ChainerX routine kernel (unfused)' % args.batch,
            'batch': args.batch,
            'residual_gamma_scale': cfg.RESNET50_RESIDUAL_GAMMA_SCALE,
            'outputs_finite': finite,
            'launch': 'eager' if graph is None else 'hip graph replay (bit-identical to eager, checked)',
            'eager_ms_per_step': round(eager_ms, 3),
        },
        'roofline': roofline,
        'fused_opt_in': fused,
        'cpu_baseline': cpu,
    }
    print(json.dumps(out))


if __name__ == '__main__':
    main()
