#!/usr/bin/env python3
"""ROIAlign forward+backward throughput on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2] [--impl auto]

One step = one forward pass plus one backward pass (gradient overwritten) of the
operator over one batch of synthetic, seeded input that is already resident in
HBM, issued through the launcher library's C ABI on one HIP stream.  Prints ONE
JSON line: whole-job ROIs/s, the roofline figures of the dominant pass measured
with HIP events around each pass, and the CPU baseline (the reference's own
kernels compiled for the host where that build is present, else the CPU
restatement), timed on this machine's cores on a bounded sample.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth



def kernel_source_digest():
    """Digest of the ROIAlign kernel sources: a traffic summary names the digest of the
    sources it was measured on, and is only quoted while they are unchanged."""
    import glob
    import hashlib
    h = hashlib.sha256()
    files = sorted(glob.glob(os.path.join(ROOT, 'mobulaop_amd', 'csrc', 'roialign_*.h')) +
                   [os.path.join(ROOT, 'mobulaop_amd', 'opzoo', 'ROIAlign', 'ROIAlign.hip')])
    for f in files:
        h.update(open(f, 'rb').read())
    return h.hexdigest()[:16]


def conv_source_digest():
    """Digest of the Conv2D kernel sources, named by profiles/conv2d_cfg5_mfma.txt the same way."""
    import glob
    import hashlib
    h = hashlib.sha256()
    files = sorted(glob.glob(os.path.join(ROOT, 'mobulaop_amd', 'csrc', 'conv_*.h')) +
                   [os.path.join(ROOT, 'mobulaop_amd', 'opzoo', 'Convolution', 'Convolution.hip')])
    for f in files:
        h.update(open(f, 'rb').read())
    return h.hexdigest()[:16]


def measured_traffic(path, kernel):
    """HBM bytes per launch of `kernel` from a summary under profiles/ (two rocprofv3 --pmc
    runs of this script, FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter
    reads for a copy of known size): the `total MB` column of the NCHW table.  None when
    the file is absent, was measured on other kernel sources, or does not list the kernel."""
    try:
        text = open(path).read()
    except OSError:
        return None
    if 'kernel sources: ' + kernel_source_digest() not in text:
        return None
    for line in text.split('-- channels-last')[0].splitlines():
        parts = line.split()
        if len(parts) >= 6 and parts[0].startswith(kernel):
            try:
                return float(parts[-1]) * 1e6
            except ValueError:
                return None
    return None



def cpu_baseline(w, budget_s=25.0, gpu_result=None):
    """Reference kernels on the host cores: forward+backward ROIs/s on a
    bounded sample (the first ROIs of the same workload, full channel count).
    `gpu_result(n)` returns what the library computes for the same n ROIs; the
    largest differences between the two go into the report."""
    import numpy as np
    from oracle import roialign as oracle
    kind = 'reference' if oracle.ref_available('omp') else 'port'
    impl = 'ref_omp' if kind == 'reference' else 'oracle'
    x = w['data'].astype(np.float32)
    pooled, scale, S = w['pooled_size'], w['spatial_scale'], w['sampling_ratio']
    R = w['rois'].shape[0]
    n = min(R, 64)
    best = None
    spent = 0.0
    while True:
        rois = w['rois'][:n]
        dy = w['dy'][:n] if w['dy'] is not None else None
        t0 = time.perf_counter()
        y_cpu = oracle.forward(x, rois, pooled, scale, S, impl=impl)
        dx_cpu = oracle.backward(dy, rois, x.shape, scale, S, impl=impl) if dy is not None else None
        dt = time.perf_counter() - t0
        spent += dt
        best = (n, dt)
        # grow the sample until one pass costs a few seconds or covers everything
        if n >= R or dt > budget_s / 4 or spent > budget_s:
            break
        n = min(R, n * 4)
    n, dt = best
    # the CPU gets its best of a few more passes over the final sample (warm caches, settled threads)
    passes = 1
    while passes < 8 and spent + dt < min(budget_s, 12.0):
        t0 = time.perf_counter()
        oracle.forward(x, rois, pooled, scale, S, impl=impl)
        if dy is not None:
            oracle.backward(dy, rois, x.shape, scale, S, impl=impl)
        again = time.perf_counter() - t0
        spent += again
        dt = min(dt, again)
        passes += 1
    out = {'value': n / dt, 'unit': 'ROIs/s', 'cores': oracle.num_threads(), 'kind': kind,
           'sample': 'first {} of {} ROIs of {} ({}), best of {} passes, {:.2f} s each'.format(
               n, R, w['name'], 'fwd+bwd' if w['dy'] is not None else 'fwd only', passes, dt)}
    if gpu_result is not None:
        # the same sample through the library: max |gpu - cpu| / max |cpu| per pass
        def rel(a, b):
            a, b = a.astype(np.float32), b.astype(np.float32)
            return float(np.abs(a - b).max() / max(float(np.abs(b).max()), 1e-30))
        y_gpu, dx_gpu = gpu_result(n)
        if w['data'].dtype.itemsize == 2:   # 16-bit storage: the checker's result is rounded the same way
            y_cpu = y_cpu.astype(w['data'].dtype)
        out['gpu_vs_cpu'] = {'forward_max_rel': rel(y_gpu, y_cpu)}
        if dx_cpu is not None:
            out['gpu_vs_cpu']['backward_max_rel'] = rel(dx_gpu, dx_cpu)
    return out


MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X published dense fp32 matrix rate
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X published dense bf16 matrix rate


def short_roialign_run(name, steps=20, warmup=3, nhwc=False):
    """One of the other BASELINE configurations (nhwc: on channels-last tensors through the
    channels-last entry points), a few steps through the C ABI: ms per
    step, fraction of the HBM peak on the algorithmic bytes, and the largest difference
    from the CPU oracle on the first ROIs (relative to the largest expected value)."""
    import numpy as np
    import torch
    from mobulaop_amd import abi, workloads
    from oracle import roialign as oracle
    w = workloads.make_workload(name)
    pooled, scale, S = w['pooled_size'], w['spatial_scale'], w['sampling_ratio']
    x, rois = abi.to_dev(w['data']), abi.to_dev(w['rois'])
    has_bwd = w['dy'] is not None
    dy = abi.to_dev(w['dy']) if has_bwd else None
    if nhwc:   # [N,H,W,C] and [R,PH,PW,C]
        x = x.permute(0, 2, 3, 1).contiguous()
        dy = dy.permute(0, 2, 3, 1).contiguous() if has_bwd else None
    dx = torch.empty_like(x) if has_bwd else None
    run_forward = abi.forward_nhwc if nhwc else abi.forward
    run_backward = abi.backward_nhwc if nhwc else abi.backward
    stream = torch.cuda.current_stream().cuda_stream
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
    fwd_ms = bwd_ms = 0.0
    for k in range(warmup + steps):   # the passes, one step at a time
        ev[0].record()
        run_forward(x, rois, pooled, scale, S, stream=stream)
        ev[1].record()
        if has_bwd:
            run_backward(dy, rois, x.shape, scale, S, dx=dx, assign=True, stream=stream)
        ev[2].record()
        torch.cuda.synchronize()
        if k >= warmup:
            fwd_ms += ev[0].elapsed_time(ev[1]) / steps
            bwd_ms += ev[1].elapsed_time(ev[2]) / steps
    # the step as the bench line's own workload is timed: `steps` of them back to back
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run_forward(x, rois, pooled, scale, S, stream=stream)
        if has_bwd:
            run_backward(dy, rois, x.shape, scale, S, dx=dx, assign=True, stream=stream)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    b_fwd, b_bwd = workloads.algorithmic_bytes(w)
    nbytes = b_fwd + (b_bwd if has_bwd else 0)
    n = min(32, rois.shape[0])
    part = rois[:n].contiguous()

    def rel(a, b):
        a, b = a.astype(np.float32), b.astype(np.float32)
        return float(np.abs(a - b).max() / max(float(np.abs(b).max()), 1e-30))
    want = oracle.forward(w['data'].astype(np.float32), w['rois'][:n], pooled, scale, S)
    if w['data'].dtype.itemsize == 2:
        want = want.astype(w['data'].dtype)
    got_y = run_forward(x, part, pooled, scale, S)
    parity = {'forward': rel((got_y.permute(0, 3, 1, 2) if nhwc else got_y).cpu().numpy(), want)}
    if has_bwd:
        got = run_backward(dy[:n].contiguous(), part, x.shape, scale, S, assign=True)
        got = (got.permute(0, 3, 1, 2) if nhwc else got).cpu().numpy()
        parity['backward'] = rel(got, oracle.backward(w['dy'][:n], w['rois'][:n], w['data'].shape, scale, S,
                                                     impl='ordered'))
    out = {'step': ('forward + backward(assign)' if has_bwd else 'forward') +
                   (', channels-last tensors' if nhwc else ''), 'ms_per_step': ms,
           'forward_ms': fwd_ms, 'frac': nbytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
           'rois_per_s': rois.shape[0] / (ms * 1e-3), 'parity_max_rel': parity,
           'parity_sample': 'first {} ROIs against the CPU oracle'.format(n)}
    if has_bwd:
        out['backward_ms'] = bwd_ms
    return out


def short_conv_run(mode='fp32', steps=20, warmup=5):
    """cfg5 with fp32 products, with operands rounded to bf16, or with every operand split
    into two bf16 (three products): ms per step (forward + data gradient + weight gradient),
    fraction of the matrix peak of that type, parity against torch's conv2d on the CPU (outputs
    and data gradient of the first two images, the weight gradient of the whole batch)."""
    import torch
    import torch.nn.functional as F
    from mobulaop_amd import native
    N, C, H, W, D, K = 32, 256, 56, 56, 256, 3
    g = torch.Generator().manual_seed(1005)
    xh = torch.randn(N, C, H, W, generator=g)
    wh = torch.randn(D, C, K, K, generator=g) * (2.0 / (C * K * K)) ** 0.5
    dyh = torch.randn(N, D, H, W, generator=g)
    x, w, dy = xh.cuda(), wh.cuda(), dyh.cuda()
    y, dx, dw = torch.empty_like(dy), torch.empty_like(x), torch.empty_like(w)
    lib = native.library()
    stream = torch.cuda.current_stream().cuda_stream
    geo = [ctypes.c_int(v) for v in (N, C, H, W, D, K, K, 1, 1, 1, 1, 1, 1)]
    native.set_option('conv_compute', {'fp32': 0, 'bf16': 1, 'bf16x3': 2}[mode])

    def ptr(t):
        return ctypes.c_void_p(t.data_ptr())

    def call(fn, *a):
        native.begin_call(stream, [])
        fn(ctypes.c_int(0), *a)
        native.end_call(fn.__name__)

    def step():
        call(lib.conv2d_forward_c6a7aa85, ctypes.c_int(y.numel()), ptr(x), ptr(w), ptr(w), ctypes.c_int(0), *geo, ptr(y))
        call(lib.conv2d_backward_data_ecf81c91, ctypes.c_int(dx.numel()), ptr(dy), ptr(w), ctypes.c_int(0), *geo, ptr(dx))
        call(lib.conv2d_backward_weight_ecf81c91, ctypes.c_int(dw.numel()), ptr(dy), ptr(x), ctypes.c_int(0), *geo,
             ptr(dw))
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    flops = 3 * 2.0 * N * D * H * W * C * K * K
    xr = xh[:2].clone().requires_grad_(True)
    yr = F.conv2d(xr, wh, padding=1)
    yr.backward(dyh[:2])
    wr = wh.clone().requires_grad_(True)
    F.conv2d(xh, wr, padding=1).backward(dyh)

    def rel(a, b):
        return float((a.cpu().double() - b.double()).abs().max() / b.double().abs().max())
    native.set_option('conv_compute', 0)
    peak = MFMA_FP32_PEAK_TFLOPS if mode == 'fp32' else MFMA_BF16_PEAK_TFLOPS
    parity = {'forward': rel(y[:2], yr.detach()), 'data_gradient': rel(dx[:2], xr.grad),
              'weight_gradient': rel(dw, wr.grad)}
    return {'step': 'forward + data gradient + weight gradient, %s products' % mode, 'ms_per_step': ms,
            'frac': flops / (ms * 1e-3) / 1e12 / peak, 'bound': 'mfma ' + ('fp32' if mode == 'fp32' else 'bf16'),
            'tflops': flops / (ms * 1e-3) / 1e12,
            'parity_max_rel': parity,
            # BASELINE.json asks for 1e-3 relative against the reference
            'within_1e-3': max(parity.values()) <= 1e-3,
            'parity_sample': 'first 2 images (outputs, data gradient) and the whole batch (weight gradient) '
                             'against torch conv2d on the CPU'}


def bench_conv(args):
    """cfg5: opzoo Conv2D, N=32, 256 -> 256 channels, 56x56, 3x3, stride 1, pad 1; fp32 tensors.
    One step = forward + data gradient + weight gradient through the C ABI.
    --conv-compute picks how the products are formed: fp32 matrix cores, operands rounded
    to bf16, or two bf16 per operand (three products, fp32-like results)."""
    import torch
    from mobulaop_amd import native
    assert torch.cuda.is_available(), 'bench.py needs a GPU'
    N, C, H, W, D, K = 32, 256, 56, 56, 256, 3
    g = torch.Generator().manual_seed(1005)
    x = torch.randn(N, C, H, W, generator=g).cuda()
    w = (torch.randn(D, C, K, K, generator=g) * (2.0 / (C * K * K)) ** 0.5).cuda()
    dy = torch.randn(N, D, H, W, generator=g).cuda()
    y, dx, dw = torch.empty_like(dy), torch.empty_like(x), torch.empty_like(w)
    lib = native.library()
    lib.mobula_hip_last_kernel_ms.restype = ctypes.c_double
    lib.mobula_hip_last_kernel_ms.argtypes = [ctypes.POINTER(ctypes.c_char_p)]
    stream = torch.cuda.current_stream().cuda_stream
    geo = [ctypes.c_int(v) for v in (N, C, H, W, D, K, K, 1, 1, 1, 1, 1, 1)]
    mode = {'fp32': 0, 'bf16': 1, 'bf16x3': 2}[args.conv_compute]
    native.set_option('conv_compute', mode)
    # dense peak of the matrix-core instruction the products run on; the split mode is
    # priced on the products that count (one per multiply-add of the convolution)
    peak = MFMA_FP32_PEAK_TFLOPS if mode == 0 else MFMA_BF16_PEAK_TFLOPS

    def ptr(t):
        return ctypes.c_void_p(t.data_ptr())

    def call(fn, *a):
        native.begin_call(stream, [])
        fn(ctypes.c_int(0), *a)
        native.end_call(fn.__name__)

    calls = [
        lambda: call(lib.conv2d_forward_c6a7aa85, ctypes.c_int(y.numel()), ptr(x), ptr(w), ptr(w),
                     ctypes.c_int(0), *geo, ptr(y)),
        lambda: call(lib.conv2d_backward_data_ecf81c91, ctypes.c_int(dx.numel()), ptr(dy), ptr(w),
                     ctypes.c_int(0), *geo, ptr(dx)),
        lambda: call(lib.conv2d_backward_weight_ecf81c91, ctypes.c_int(dw.numel()), ptr(dy), ptr(x),
                     ctypes.c_int(0), *geo, ptr(dw)),
    ]

    def step():
        for c in calls:
            c()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    native.set_option('kernel_timing', 1)
    kernel_ms = {}
    for _ in range(args.steps):
        for c in calls:
            c()
            name = ctypes.c_char_p()
            ms = lib.mobula_hip_last_kernel_ms(ctypes.byref(name))
            if ms >= 0 and name.value:
                kernel_ms.setdefault(name.value.decode(), []).append(ms)
    native.set_option('kernel_timing', 0)
    kernel_ms = {k: sum(v) / len(v) for k, v in kernel_ms.items()}
    flops_each = 2.0 * N * D * H * W * C * K * K          # per product; three products per step
    dom = max(kernel_ms, key=kernel_ms.get)
    achieved = flops_each / (kernel_ms[dom] * 1e-3) / 1e12
    out = {
        'metric': 'conv2d_fwd_bwd_tflops', 'value': 3 * flops_each / (ms_per_step * 1e-3) / 1e12,
        'unit': 'TFLOP/s', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': ms_per_step, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': {0: 'f32', 1: 'bf16', 2: 'bf16x3'}[mode], 'data': 'synthetic',
        'config': {'workload': 'cfg5: conv2d x 32x256x56x56, 256 filters 3x3 stride 1 pad 1',
                   'step': 'forward + data gradient + weight gradient', 'compute': args.conv_compute},
        'roofline': {'bound': 'mfma', 'kernel': dom, 'achieved': achieved, 'peak': peak,
                     'unit': 'TFLOP/s', 'frac': achieved / peak, 'traffic': None,
                     'algorithmic_flops': flops_each, 'avg_ms': kernel_ms[dom]},
        'kernels_ms': kernel_ms,
    }
    if not args.no_cpu_baseline:
        # the C restatement of the reference algorithm (im2col + product per image), one thread,
        # on the first image of the same tensors
        from oracle import conv as oracle
        xs, ws, dys = x[:1].cpu().numpy(), w.cpu().numpy(), dy[:1].cpu().numpy()
        t0 = time.perf_counter()
        oracle.conv2d_forward(xs, ws, None, (1, 1), (1, 1), (1, 1))
        oracle.conv2d_backward(dys, xs, ws, (1, 1), (1, 1), (1, 1), with_bias=False)
        dt = time.perf_counter() - t0
        out['cpu_baseline'] = {'value': 3 * flops_each / N / dt / 1e12, 'unit': 'TFLOP/s', 'cores': 1,
                               'kind': 'port', 'sample': 'first image of 32, one pass, {:.2f} s'.format(dt)}
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=30)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--workload', default='cfg2', choices=['cfg1', 'cfg2', 'cfg3', 'cfg4', 'cfg5'])
    ap.add_argument('--impl', default='auto', choices=['auto', 'tiled', 'naive'])
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--sampling-ratio', type=int, default=None,
                    help='replace the sampling ratio of the workload (0: adaptive grid); the configuration '
                         'string of the report says so')
    ap.add_argument('--layout', default='nchw', choices=['nchw', 'nhwc'],
                    help='nhwc: channels-last tensors through the channels-last entry points (an extension; '
                         'the reference interface, and the default here, is nchw)')
    ap.add_argument('--conv-compute', default='fp32', choices=['fp32', 'bf16', 'bf16x3'],
                    help='cfg5 only: how the convolution forms its products')
    ap.add_argument('--traffic-file', default=os.path.join(ROOT, 'profiles', 'roialign_cfg2_hbm_traffic.txt'),
                    help='counter summary that roofline.traffic is read from (cfg2, NCHW)')
    ap.add_argument('--option', action='append', default=[], metavar='NAME=VALUE',
                    help='set a library option (mobula_hip_set_option) before the run, for experiments')
    ap.add_argument('--no-other-configs', action='store_true',
                    help='leave out the short runs of the other BASELINE configurations (the "configs" object)')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py: this build measures one GPU only (the path would shard by image, each GPU '
                 'taking the ROIs of its images, with no exchange between them); run with --gpus 1')

    if args.workload == 'cfg5':
        return bench_conv(args)

    import torch
    from mobulaop_amd import workloads
    from mobulaop_amd import abi
    assert torch.cuda.is_available(), 'bench.py needs a GPU'
    for item in args.option:
        from mobulaop_amd import native
        name, _, value = item.partition('=')
        native.set_option(name, int(value))

    w = workloads.make_workload(args.workload)
    if args.sampling_ratio is not None:
        w['sampling_ratio'] = args.sampling_ratio
        w['name'] += ' with sampling_ratio replaced'
    pooled, scale, S = w['pooled_size'], w['spatial_scale'], w['sampling_ratio']
    nhwc = args.layout == 'nhwc'
    x = abi.to_dev(w['data'].transpose(0, 2, 3, 1) if nhwc else w['data'])
    rois = abi.to_dev(w['rois'])
    has_bwd = w['dy'] is not None
    dy = abi.to_dev(w['dy'].transpose(0, 2, 3, 1) if nhwc else w['dy']) if has_bwd else None
    R = rois.shape[0]
    abi.set_impl(args.impl)
    stream = torch.cuda.current_stream().cuda_stream  # launches and events share this stream

    dx = torch.empty_like(x) if has_bwd else None
    run_forward = abi.forward_nhwc if nhwc else abi.forward
    run_backward = abi.backward_nhwc if nhwc else abi.backward

    def step(events=None):
        if events is not None:
            events[0].record()
        y = run_forward(x, rois, pooled, scale, S, stream=stream)
        if events is not None:
            events[1].record()
        if has_bwd:
            run_backward(dy, rois, x.shape, scale, S, dx=dx, assign=True, stream=stream)
        if events is not None:
            events[2].record()
        return y

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # the throughput loop: K steps back to back, nothing else in the stream
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    # per-pass times: the same steps again with an event before, between and after the passes
    # (the event records cost the stream a few microseconds each, hence a loop of their own)
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(args.steps)]
    for k in range(args.steps):
        step(evs[k])
    torch.cuda.synchronize()

    # Per-kernel time of the dominant kernel of each pass: the library brackets it
    # with HIP events on the launch stream (option "kernel_timing"); measured in
    # a loop of its own after the throughput loop, same inputs, same stream.
    from mobulaop_amd import native
    lib = native.library()
    lib.mobula_hip_last_kernel_ms.restype = ctypes.c_double
    lib.mobula_hip_last_kernel_ms.argtypes = [ctypes.POINTER(ctypes.c_char_p)]
    native.set_option('kernel_timing', 1)
    kernel_ms = {}

    def note_kernel():
        name = ctypes.c_char_p()
        ms = lib.mobula_hip_last_kernel_ms(ctypes.byref(name))
        if ms >= 0 and name.value:
            kernel_ms.setdefault(name.value.decode(), []).append(ms)

    for _ in range(args.steps):
        run_forward(x, rois, pooled, scale, S, stream=stream)
        note_kernel()
        if has_bwd:
            run_backward(dy, rois, x.shape, scale, S, dx=dx, assign=True, stream=stream)
            note_kernel()
    native.set_option('kernel_timing', 0)
    kernel_ms = {k: sum(v) / len(v) for k, v in kernel_ms.items()}

    # End to end through the operator: mobula.op.ROIAlign on torch tensors with autograd
    # (allocation of y and dx, Python binding, the same kernels), wall clock per step.
    op_ms = None
    if has_bwd and w['data'].dtype.itemsize == 4:
        import mobulaop_amd as mobula
        mobula.op.load('ROIAlign')
        x_op = (x.permute(0, 3, 1, 2) if nhwc else x).detach().requires_grad_(True)
        dy_op = dy.permute(0, 3, 1, 2) if nhwc else dy
        kw = dict(pooled_size=pooled, spatial_scale=scale, sampling_ratio=S)

        def op_step():
            y_op = mobula.op.ROIAlign(x_op, rois, **kw)
            y_op.backward(dy_op)
            x_op.grad = None

        for _ in range(args.warmup):
            op_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            op_step()
        torch.cuda.synchronize()
        op_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # The same step recorded once in a HIP graph and replayed: what a caller gets who captures
    # the calls (all kernels run on every replay; the links between the two streams of a
    # call become edges of the graph).  Not for the adaptive backward, which reads a count
    # back from the device inside the call.
    graph_ms = None
    if not has_bwd or S > 0:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            inner = torch.cuda.current_stream().cuda_stream
            y_graph = run_forward(x, rois, pooled, scale, S, stream=inner)
            if has_bwd:
                run_backward(dy, rois, x.shape, scale, S, dx=dx, assign=True, stream=inner)
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        y_eager = step()
        torch.cuda.synchronize()
        assert torch.equal(y_graph, y_eager), 'graph replay and direct calls differ'
        del graph, y_graph, y_eager
        native.unpin_workspace()   # recording pinned the thread's workspace

    # Backward twice from the same inputs: the largest difference between the two
    # results (the reference's atomics give a different summation order each run).
    repeat_diff = None
    if has_bwd:
        dx_again = torch.empty_like(dx)
        run_backward(dy, rois, x.shape, scale, S, dx=dx, assign=True, stream=stream)
        run_backward(dy, rois, x.shape, scale, S, dx=dx_again, assign=True, stream=stream)
        torch.cuda.synchronize()
        repeat_diff = float((dx.float() - dx_again.float()).abs().max())
        del dx_again

    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in evs) / args.steps
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in evs) / args.steps if has_bwd else 0.0
    ms_per_step = wall * 1e3 / args.steps
    b_fwd, b_bwd = workloads.algorithmic_bytes(w)

    def gbs(nbytes, ms):
        return nbytes / (ms * 1e-3) / 1e9 if ms > 0 else 0.0

    # The dominant kernel: the longest of the bracketed ones.  Its algorithmic
    # bytes are those of its pass (each tensor of the pass once): the helper
    # kernels around it exist only to feed it.
    pass_of = {'forward_blocked_kernel': ('forward', b_fwd), 'forward_merged_kernel': ('forward', b_fwd),
               'backward_blocked_kernel': ('backward', b_bwd)}
    if kernel_ms:
        dom_kernel = max(kernel_ms, key=kernel_ms.get)
        dom_ms = kernel_ms[dom_kernel]
        dom_bytes = pass_of.get(dom_kernel, ('forward', b_fwd))[1]
    else:  # the straightforward kernels carry no bracket: fall back to the slower pass
        dom_kernel = ('backward' if bwd_ms > fwd_ms else 'forward') + ' pass'
        dom_bytes, dom_ms = (b_bwd, bwd_ms) if bwd_ms > fwd_ms else (b_fwd, fwd_ms)
    passes = {'forward': {'ms': fwd_ms, 'GB/s': gbs(b_fwd, fwd_ms), 'frac': gbs(b_fwd, fwd_ms) / HBM_PEAK_GBS,
                          'rois_per_s': R / (fwd_ms * 1e-3)}}
    total_bytes = b_fwd
    if has_bwd:
        passes['backward'] = {'ms': bwd_ms, 'GB/s': gbs(b_bwd, bwd_ms),
                              'frac': gbs(b_bwd, bwd_ms) / HBM_PEAK_GBS}
        total_bytes += b_bwd
    gpu_ms = fwd_ms + bwd_ms
    passes['fwd_bwd' if has_bwd else 'fwd'] = {
        'ms': gpu_ms, 'GB/s': gbs(total_bytes, gpu_ms), 'frac': gbs(total_bytes, gpu_ms) / HBM_PEAK_GBS}

    out = {
        'metric': 'roialign_fwd_bwd_rois_per_sec' if has_bwd else 'roialign_fwd_rois_per_sec',
        'value': R / (ms_per_step * 1e-3), 'unit': 'ROIs/s', 'n_gpus': 1, 'steps': args.steps,
        'warmup': args.warmup, 'ms_per_step': ms_per_step, 'higher_is_better': True,
        'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'f16 storage, f32 accumulate' if w['data'].dtype.itemsize == 2 else 'f32',
        'data': 'synthetic',
        'config': {'workload': '{}: data {} rois {} pooled {} scale {} sampling_ratio {}'.format(
            w['name'], 'x'.join(map(str, w['data'].shape)), R, 'x'.join(map(str, pooled)), scale, S),
            'impl': args.impl, 'layout': args.layout,
            'step': 'forward + backward(assign)' if has_bwd else 'forward'},
        'roofline': {'bound': 'hbm', 'kernel': dom_kernel, 'achieved': gbs(dom_bytes, dom_ms),
                     'peak': HBM_PEAK_GBS, 'unit': 'GB/s', 'frac': gbs(dom_bytes, dom_ms) / HBM_PEAK_GBS,
                     'traffic': None if nhwc or w['name'] != 'cfg2' else measured_traffic(args.traffic_file, dom_kernel),
                     'algorithmic_bytes': dom_bytes, 'avg_ms': dom_ms,
                     # the whole step (every helper kernel and gap included) on the algorithmic bytes of both passes
                     'step_frac': total_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS},
        'kernels_ms': kernel_ms,
        'passes': passes,
        # share of the map inside some ROI's box: the e*|x| term of the algorithmic bytes counts all of it
        'touched_fraction': workloads.touched_fraction(w),
        # what a kernel with no reuse of corner values would move per forward pass
        'gather_bytes': workloads.gather_bytes(w),
    }
    if repeat_diff is not None:
        out['backward_run_to_run_max_abs'] = repeat_diff
    if op_ms is not None:
        out['passes']['operator_fwd_bwd'] = {'ms': op_ms, 'rois_per_s': R / (op_ms * 1e-3)}
    if graph_ms is not None:
        out['passes']['graph_replay'] = {'ms': graph_ms, 'rois_per_s': R / (graph_ms * 1e-3)}
    if not args.no_cpu_baseline:
        def gpu_result(n):
            # NCHW results for the first n ROIs, whatever layout the timed loop used
            x_nchw = x.permute(0, 3, 1, 2).contiguous() if nhwc else x
            part = rois[:n].contiguous()
            y_n = abi.forward(x_nchw, part, pooled, scale, S)
            dx_n = None
            if has_bwd:
                dy_nchw = (dy.permute(0, 3, 1, 2) if nhwc else dy)[:n].contiguous()
                dx_n = abi.backward(dy_nchw, part, x_nchw.shape, scale, S, assign=True).cpu().numpy()
            return y_n.cpu().numpy(), dx_n
        out['cpu_baseline'] = cpu_baseline(w, gpu_result=gpu_result)
    if args.workload == 'cfg2' and not args.no_other_configs and not nhwc and args.sampling_ratio is None:
        # the other configurations of BASELINE.json, a few steps each (parity cases, shown
        # for orientation; `value` above is cfg2 alone)
        del x, dy, dx
        torch.cuda.empty_cache()
        out['configs'] = {'cfg2': {'step': 'forward + backward(assign)', 'ms_per_step': ms_per_step,
                                   'frac': total_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS}}
        for name in ('cfg1', 'cfg3', 'cfg4'):
            out['configs'][name] = short_roialign_run(name)
            torch.cuda.empty_cache()
        # cfg2 again on channels-last tensors: the entry points that need no layout pass
        out['configs']['cfg2_nhwc'] = short_roialign_run('cfg2', nhwc=True)
        torch.cuda.empty_cache()
        out['configs']['cfg5'] = short_conv_run('fp32')
        out['configs']['cfg5_bf16'] = short_conv_run('bf16')
        out['configs']['cfg5_bf16x3'] = short_conv_run('bf16x3')
    print(json.dumps(out))


if __name__ == '__main__':
    main()
