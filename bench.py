#!/usr/bin/env python3
"""Benchmark of the fused SAPA-B forward (qk -> softmax -> av, one launch) on
one MI355X; the default workload is the largest FPN level (B=16, C=256, d=64,
K=5, 100x168 -> 200x336, fp32).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--settle-ms MS] [--dtype fp32|bf16]
                    [--workload fpn_large|fpn_mid|fpn_small|segformer_16|segformer_32|segformer_64|
                                stress|deform_p25|deform_p9|deform_p5]
                    [--pass forward|train] [--no-cpu-baseline] [--calibration-copy]

A step is one fused forward over the whole synthetic batch, inputs already
resident in HBM.  Prints ONE JSON line: output Gpix/s, the HBM roofline of
the kernel (algorithmic bytes / measured launch time against 8 TB/s) and the
CPU baseline (the unfold-based PyTorch math of the reference's own forward
check, restated in oracle/torch_oracle.py, timed on this host's cores over a
bounded sample of the same workload).
"""
import argparse
import ctypes
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# published dense peaks of the arithmetic a workload could be bound by instead:
# fp32 on the vector or the matrix pipe, 16-bit inputs on the matrix pipe
FP32_PEAK_TFLOPS = 157.3
BF16_MFMA_PEAK_TFLOPS = 2500.0

# name -> (B, C, d, H, W, K, s); FPN levels of an 800x1333 input, stride 8/16/32
WORKLOADS = {
    'fpn_large': (16, 256, 64, 100, 168, 5, 2),
    'fpn_mid': (16, 256, 64, 50, 84, 5, 2),
    'fpn_small': (16, 256, 64, 25, 42, 5, 2),
    'stress': (4, 512, 64, 64, 64, 7, 4),
    # SegFormer-style decoder chain 16^2 -> 32^2 -> 64^2 -> 128^2 (B=8, C=256, d=32): one
    # workload per stage; query / key come from 1x1 projections ~N(0, .02) of
    # random features (sapa_base.py:21-22,42-46)
    'segformer_16': (8, 256, 32, 16, 16, 5, 2),
    'segformer_32': (8, 256, 32, 32, 32, 5, 2),
    'segformer_64': (8, 256, 32, 64, 64, 5, 2),
}
# SAPA-D (fused deform_qk -> softmax -> deform_av), BASELINE config 4:
# name -> (B, C, d, G, H, W, P, s); offsets ~N(0, 0.75) clipped to +-4 cells
DEFORM_WORKLOADS = {
    'deform_p25': (8, 256, 32, 4, 64, 64, 25, 2),
    'deform_p9': (8, 256, 32, 4, 64, 64, 9, 2),
    'deform_p5': (8, 256, 32, 4, 64, 64, 5, 2),
}

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE + WRITE_SIZE,
# scaled by what the same counters read for a plain copy of known size), per
# (workload, dtype, layout): bytes, the summary under profiles/ they come from
# and the kernel they were measured on.  A run whose dispatched kernel is not
# that kernel stops with an error instead of printing a stale figure.
MEASURED_TRAFFIC = {
    ('fpn_large', 'fp32', 'nchw'): (1831119034, 'profiles/sapa_b_fused_fpn_large_fp32.md', 'sapa_b_tiled_kernel'),
    ('fpn_large', 'bf16', 'nchw'): (944266161, 'profiles/sapa_b_fused_fpn_large_bf16.md', 'sapa_b_wmat16_kernel'),
    ('fpn_large', 'fp32', 'channels_last'): (1720501334, 'profiles/sapa_b_nhwc_fused_fpn_large_fp32.md',
                                             'sapa_b_nhwc_kernel'),
    ('fpn_large', 'bf16', 'channels_last'): (862391142, 'profiles/sapa_b_nhwc_fused_fpn_large_bf16.md',
                                             'sapa_b_nhwc_wm16_kernel'),
    ('fpn_small', 'fp32', 'nchw'): (137685860, 'profiles/sapa_b_fused_fpn_small_fp32.md', 'sapa_b_tiled_kernel'),
    ('segformer_16', 'fp32', 'nchw'): (11936679, 'profiles/sapa_b_mfma_fused_segformer_16_fp32.md',
                                       'sapa_b_mfma_kernel'),
    ('stress', 'bf16', 'nchw'): (371333608, 'profiles/sapa_b_mfma_fused_stress_bf16.md', 'sapa_b_mfma_kernel'),
    ('stress', 'fp32', 'channels_last'): (647422060, 'profiles/sapa_b_nhwc_mm_fused_stress_fp32.md',
                                          'sapa_b_nhwc_mm_kernel'),
    ('stress', 'bf16', 'channels_last'): (323264189, 'profiles/sapa_b_nhwc16_fused_stress_bf16.md',
                                          'sapa_b_nhwc16_kernel'),
    ('deform_p25', 'fp32', 'nchw'): (459730983, 'profiles/sapa_d_wmat_fused_deform_p25_fp32_nchw.md',
                                     'deform_fused_wmat_kernel'),
    ('deform_p25', 'bf16', 'nchw'): (228881067, 'profiles/sapa_d_wmat16_fused_deform_p25_bf16_nchw.md',
                                     'deform_fused_wmat16_kernel'),
    ('deform_p25', 'fp32', 'nchw_reference_order'): (828689742, 'profiles/sapa_d_lds_fused_deform_p25_fp32.md',
                                                     'deform_lds_kernel'),
    ('deform_p9', 'fp32', 'nchw'): (399849952, 'profiles/sapa_d_lds_fused_deform_p9_fp32.md', 'deform_lds_kernel'),
    ('deform_p25', 'fp32', 'channels_last'): (356737114, 'profiles/sapa_d_nhwc_fused_deform_p25_fp32.md',
                                              'deform_fused_wmat_kernel'),
    ('deform_p25', 'bf16', 'channels_last'): (178447650, 'profiles/sapa_d_wmat16_fused_deform_p25_bf16.md',
                                              'deform_fused_wmat16_kernel'),
}


def measured_traffic(workload, dtype, layout, kernel):
    """(bytes, {'file', 'kernel'}) for the run's configuration, (None, None) if
    it was never measured; exits if it was measured on another kernel than the
    one this run dispatched to."""
    hit = MEASURED_TRAFFIC.get((workload, dtype, layout))
    if hit is None:
        return None, None
    nbytes, source, measured_on = hit
    if measured_on != kernel:
        sys.exit(f'bench.py: the traffic figure for {workload}/{dtype}/{layout} in {source} was measured on '
                 f'{measured_on}, this run dispatched to {kernel}: re-measure it (rocprofv3 --pmc FETCH_SIZE / '
                 'WRITE_SIZE) and update MEASURED_TRAFFIC')
    return nbytes, {'file': source, 'kernel': measured_on}


def algorithmic_bytes(B, C, d, H, W, s, esize):
    """Read q, key, value once, write the output once."""
    return esize * (B * H * s * W * s * (d + C) + B * H * W * (d + C))


def algorithmic_flops(B, C, d, H, W, K, s):
    """Fused SAPA-B: K*K multiply-adds per query channel and per value channel
    of every output pixel, plus the softmax."""
    return B * H * s * W * s * (2 * d * K * K + 2 * C * K * K + 5 * K * K)


def deform_algorithmic_flops(B, C, d, G, H, W, P, s):
    """Fused SAPA-D: per pixel, group and point a bilinear sample (4 multiply-adds)
    and one more multiply-add for each of the group's d query and C/G value channels."""
    return B * H * s * W * s * G * P * 2 * 5 * (d + C // G)


def make_inputs(cfg, dtype, device, seed=0, heavy_tails=False, projected=False):
    B, C, d, H, W, K, s = cfg
    g = torch.Generator(device=device).manual_seed(seed)
    if projected:
        # q, key = 1x1 projections ~N(0, .02) (zero bias) of GroupNorm(32)-normalised
        # random features; the value is the un-normalised low-res feature
        y = torch.randn(B, C, H * s, W * s, generator=g, device=device)
        x = torch.randn(B, C, H, W, generator=g, device=device)
        wq = torch.randn(d, C, 1, 1, generator=g, device=device) * 0.02
        wk = torch.randn(d, C, 1, 1, generator=g, device=device) * 0.02
        gn = torch.nn.functional.group_norm
        q = torch.nn.functional.conv2d(gn(y, 32), wq)
        key = torch.nn.functional.conv2d(gn(x, 32), wk)
        return q.to(dtype).contiguous(), key.to(dtype).contiguous(), x.to(dtype).contiguous()
    q = torch.randn(B, d, H * s, W * s, generator=g, device=device)
    if heavy_tails:
        # a random 10 % of the query replaced by Student-t(3) draws (the stress
        # workload: logits with outliers for the softmax)
        z = torch.randn(4, *q.shape, generator=g, device=device)
        t3 = z[0] / (z[1:].pow(2).mean(0)).sqrt()
        q = torch.where(torch.rand(q.shape, generator=g, device=device) < 0.1, t3, q)
        del z, t3
    # keys L2-magnitude-varied via a per-channel scale ~U(0.5, 2)
    scale = torch.rand(d, generator=g, device=device) * 1.5 + 0.5
    key = torch.randn(B, d, H, W, generator=g, device=device) * scale.view(1, d, 1, 1)
    v = torch.randn(B, C, H, W, generator=g, device=device)
    return q.to(dtype).contiguous(), key.to(dtype).contiguous(), v.to(dtype).contiguous()


def deform_algorithmic_bytes(B, C, d, G, H, W, P, s, esize):
    """Read q, key, value, offset once, write the output once."""
    hi, lo = B * H * s * W * s, B * H * W
    return esize * (hi * (G * d + 2 * G * P + C) + lo * (G * d + C))


def make_deform_inputs(cfg, dtype, device, seed=0):
    B, C, d, G, H, W, P, s = cfg
    g = torch.Generator(device=device).manual_seed(seed)
    q = torch.randn(B, G * d, H * s, W * s, generator=g, device=device)
    key = torch.randn(B, G * d, H, W, generator=g, device=device)
    v = torch.randn(B, C, H, W, generator=g, device=device)
    off = (0.75 * torch.randn(B, 2 * G * P, H * s, W * s, generator=g, device=device)).clamp(-4, 4)
    return tuple(t.to(dtype).contiguous() for t in (q, key, v, off))


def measured_ceiling(lib, dev, stream, args, timed, write_bytes):
    """What the memory system gives a kernel that only moves bytes: workgroups
    that each read one contiguous run and write one contiguous run, in the
    9 : 16 read : write mix of a fused SAPA-B forward at up_factor 2 with
    C = 4 d (FPN shapes: q + key + value in, the result out), sized to this
    workload's output, timed with the step's own protocol; a copy, a fill and
    a read of the same size for context.  The best of the mix variants is the
    ceiling.  (SAPA-D and the SegFormer stages read relatively more; the
    9 : 16 figure is still the nearest of the built mixes.)"""
    from sapa_amd import _lib
    unit_w = 16 * 4096
    units = max(write_bytes // unit_w, 1)
    src = torch.empty(units * 16 * 4096 // 4, dtype=torch.int32, device=dev).fill_(12345)
    dst = torch.empty(units * 16 * 4096 // 4, dtype=torch.int32, device=dev)
    res = {}
    # name: reads, writes (x 4 KiB per unit), units, units per workgroup, streaming loads | 2 * streaming stores
    for name, r, w, n, reps, nt in (('mix_9_16_runs_36K_64K_streaming', 9, 16, units, 1, 3),
                                    ('mix_9_16_runs_36K_64K_streaming_loads', 9, 16, units, 1, 1),
                                    ('mix_9_16_runs_36K_64K_plain', 9, 16, units, 1, 0),
                                    ('mix_9_16_runs_72K_128K_streaming', 9, 16, units, 2, 3),
                                    # readers and writers in different workgroups (runs of 128K): units // 32 groups
                                    ('mix_9_16_readers_and_writers_apart', 9, 16, max(units // 32, 1), 2, 4 | 3),
                                    ('copy_runs_32K_streaming', 8, 8, units, 1, 3),
                                    ('fill_runs_256K_plain', 0, 16, units, 4, 0),
                                    ('read_runs_256K_streaming', 16, 0, units, 4, 1)):
        def step():
            _lib.check(lib.sapa_stream_mix(src.data_ptr(), dst.data_ptr(), n, r, w, reps, nt, stream.cuda_stream),
                       'sapa_stream_mix')
        ms, _ = timed(step)
        moved = n * reps * 25 * 65536 if nt & 4 else n * (r + w) * 4096
        res[name] = {'ms': ms, 'GB/s': moved / (ms * 1e-3) / 1e9}
    del src, dst
    best = max((k for k in res if k.startswith('mix')), key=lambda k: res[k]['GB/s'])
    # reads and writes share the memory bus: a stream of both takes about as long as its read
    # part at the read-only rate plus its write part at the write-only rate
    rd, wr = res['read_runs_256K_streaming']['GB/s'], res['fill_runs_256K_plain']['GB/s']
    additive_ms = (units * 9 * 4096 / rd + units * 16 * 4096 / wr) / 1e6
    return {'GB/s': res[best]['GB/s'], 'variant': best, 'kernel': 'stream_mix_kernel (sapa_stream_mix)',
            'bytes_moved': units * 25 * 4096,
            'read_plus_write_floor': {'ms': additive_ms, 'GB/s': units * 25 * 4096 / additive_ms / 1e6,
                                      'note': 'the mix\'s read bytes at the measured read-only rate plus its '
                                              'write bytes at the measured fill rate'},
            'variants': res}


def timed_median(fn, budget_s):
    """Median wall time of fn() over at least 3 runs within the budget."""
    fn()  # warm-up
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 20):
        t0 = time.perf_counter()
        out = fn()
        times.append(time.perf_counter() - t0)
        if time.perf_counter() - t_start > 3 * budget_s:
            break
    times.sort()
    return times[len(times) // 2], len(times), out


def cpu_baseline(fn, tensors, pix_per_image, median_budget_s=8.0, batch_budget_s=60.0):
    """CPU time of fn(image tensors...) on this host's cores: the median over
    repeated runs on image 0, then the whole batch once, image by image (the
    unfold formulation needs several GB per image, so the batch is chunked),
    summed -- or as many images as fit batch_budget_s, and the count says so.
    Returns the record for the JSON line and image 0's output."""
    imgs = [[t[i:i + 1].float().cpu() for t in tensors] for i in range(tensors[0].shape[0])]
    cores = torch.get_num_threads()
    med, runs, out = timed_median(lambda: fn(*imgs[0]), median_budget_s)
    total, done = 0.0, 0
    for im in imgs:
        t0 = time.perf_counter()
        fn(*im)
        total += time.perf_counter() - t0
        done += 1
        if total > batch_budget_s:
            break
    rec = {'value': pix_per_image * done / total / 1e9, 'unit': 'Gpix/s', 'cores': cores, 'kind': 'port',
           'sample': f'{done} of {len(imgs)} images of the batch, one at a time, fp32, {total:.1f} s in all '
                     f'(torch CPU, {cores} threads)',
           'image0_median': {'value': pix_per_image / med / 1e9, 'unit': 'Gpix/s', 'runs': runs}}
    return rec, out


def module_cases(args, dev, dtype, stream, only=None, warmup=None, steps=None):
    """SAPA.forward(y, x) = GroupNorm(32) on both features, 1x1 q / k projections,
    fused operator (sapa_base.py:26-40), timed as the reference composes it and with
    the projections of this build: {case: {'ms', 'max_abs_diff_vs_first_image0'}}."""
    import sapa_amd
    B, C, d, H, W, K, s = WORKLOADS[args.workload]
    g = torch.Generator(device=dev).manual_seed(0)
    y = torch.randn(B, C, H * s, W * s, generator=g, device=dev).to(dtype)
    x = torch.randn(B, C, H, W, generator=g, device=dev).to(dtype)
    m = sapa_amd.SAPA(C, embedding_dim=d, up_factor=s, up_kernel_size=K).to(dev).to(dtype)
    CL = torch.channels_last
    ycl, xcl = y.contiguous(memory_format=CL), x.contiguous(memory_format=CL)
    cases = [('GroupNorm -> Conv2d -> fused operator, contiguous features', {}, (y, x)),
             ('fold_norm, contiguous features', {'fold_norm': True}, (y, x)),
             ('channels_last=True, contiguous features', {'channels_last': True}, (y, x)),
             ('channels_last=True, channels_last features', {'channels_last': True}, (ycl, xcl)),
             ('GroupNorm -> Conv2d -> fused operator, channels_last features', {}, (ycl, xcl))]
    if only is not None:
        cases = [cases[i] for i in only]
    warmup = max(args.warmup // 10, 3) if warmup is None else warmup
    steps = max(args.steps // 10, 5) if steps is None else steps
    res, ref = {}, None
    with torch.no_grad():
        for name, kw, feats in cases:
            m.fold_norm, m.channels_last = kw.get('fold_norm', False), kw.get('channels_last', False)
            out = m(*feats)
            if ref is None:
                ref = out[:1].float()
            err = (out[:1].float() - ref).abs().max().item()
            for _ in range(warmup):
                m(*feats)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            n = steps
            e0.record(stream)
            for _ in range(n):
                m(*feats)
            e1.record(stream)
            torch.cuda.synchronize()
            res[name] = {'ms': e0.elapsed_time(e1) / n, 'max_abs_diff_vs_first_image0': err}
    return res


def module_pass(args, dev, dtype, stream):
    """The caller of the hot path (module_cases) as the main line."""
    if args.workload not in WORKLOADS:
        sys.exit('bench.py: --pass module covers the SAPA-B workloads')
    B, C, d, H, W, K, s = WORKLOADS[args.workload]
    res = module_cases(args, dev, dtype, stream,
                       only=[args.module_case] if args.module_case >= 0 else None)
    if args.calibration_copy:
        # a copy of known size in the same run: what the profiler's byte counters read for it
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    pix = B * H * s * W * s
    best = min(res, key=lambda k: res[k]['ms'] if 'contiguous features' in k or len(res) == 1 else 1e9)
    print(json.dumps({
        'metric': 'upsampled Gpix/s, SAPA module forward (GroupNorm + q/k projections + fused operator), 1 GPU',
        'value': pix / (res[best]['ms'] * 1e-3) / 1e9, 'unit': 'Gpix/s', 'n_gpus': 1,
        'steps': max(args.steps // 10, 5), 'warmup': max(args.warmup // 10, 3),
        'ms_per_step': res[best]['ms'], 'higher_is_better': True, 'scaling': 'weak',
        'vs_baseline': None, 'dtype': {'fp32': 'f32', 'bf16': 'bf16'}[args.dtype], 'data': 'synthetic',
        'config': {'workload': f'{args.workload}: SAPA module, features B={B} C={C} {H}x{W} / '
                               f'{H * s}x{W * s}, embedding_dim={d}, K={K}, s={s}, {args.dtype}; '
                               f'main line = "{best}"'},
        'cases': res}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=200)
    # the GPU's clocks take ~50 ms of work to settle: warm up for about that long
    ap.add_argument('--warmup', type=int, default=200)
    ap.add_argument('--recompute-attention', action='store_true',
                    help="--pass train, SAPA-B: the backward pass recomputes the attention weights "
                         'instead of taking the fp32 ones the forward pass keeps by default')
    ap.add_argument('--dtype', default='fp32', choices=['fp32', 'bf16'])
    ap.add_argument('--workload', default='fpn_large',
                    choices=sorted(WORKLOADS) + sorted(DEFORM_WORKLOADS))
    ap.add_argument('--pass', dest='direction', default='forward', choices=['forward', 'train', 'module'],
                    help="'train' times the fused forward plus its backward (all input "
                         'gradients) through the autograd API instead of the forward alone; '
                         "'module' times the whole SAPA module forward (GroupNorm, q / k "
                         'projections, fused operator) in its configurations')
    ap.add_argument('--layout', default='nchw', choices=['nchw', 'channels_last'],
                    help="memory order of the SAPA-B tensors: 'nchw' = contiguous, the "
                         "reference's contract (default); 'channels_last' = torch.channels_last, "
                         'served by the *_nhwc entry points.  With the default, the forward '
                         'SAPA-B line also carries the channels_last timing of the same '
                         "workload under 'channels_last'")
    ap.add_argument('--module-case', type=int, default=-1,
                    help="with --pass module: run only case N of the list (0 = the reference's "
                         'composition on contiguous features ... 3 = channels_last projections on '
                         'channels_last features), e.g. under a profiler; default: all')
    ap.add_argument('--settle-ms', type=float, default=40.0,
                    help='GPU time (ms) of untimed launches of the same step before the warm-up '
                         'steps, to let the power management settle after idle; 0 = none')
    ap.add_argument('--reference-order', action='store_true',
                    help='SAPA-D, contiguous tensors: time sapa_deform_fused_forward (sums in the '
                         "reference's order) as the main line instead of the matrix-form path that "
                         'sapa_amd.deform_sapa_fused takes by default where it is faster')
    ap.add_argument('--only-main', action='store_true',
                    help='skip the channels_last timing that a default (contiguous) SAPA-B / SAPA-D '
                         'forward line carries along (e.g. under a profiler)')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--no-after-idle', action='store_true',
                    help="skip the 'after_idle' timing (W warm-up + K timed steps straight after a pause, "
                         'no settle launches) that a forward line carries next to the settled main figure')
    ap.add_argument('--no-ceiling', action='store_true',
                    help="skip 'roofline.measured_ceiling' (a kernel that only streams this workload's "
                         'bytes in and out in long contiguous runs, sapa_stream_mix)')
    ap.add_argument('--calibration-copy', action='store_true',
                    help='after the timed region, run 5 device copies of 1 GiB (a kernel of '
                         'known traffic: 1 GiB read + 1 GiB written) for scaling profiler '
                         'byte counters')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py: this build measures one GPU only (the operators are '
                 'single-device: a batch shards over GPUs by image, with no communication). '
                 'Use --gpus 1.')
    if not torch.cuda.is_available():
        sys.exit('bench.py: no GPU visible')

    from sapa_amd import _lib
    lib = _lib.lib()  # raises if the HIP library is missing: no fallback

    dev = torch.device('cuda:0')
    torch.cuda.set_device(dev)
    dtype = {'fp32': torch.float32, 'bf16': torch.bfloat16}[args.dtype]
    stream = torch.cuda.current_stream(dev)
    if args.direction == 'module':
        return module_pass(args, dev, dtype, stream)
    deform = args.workload in DEFORM_WORKLOADS
    if deform:
        cfg = DEFORM_WORKLOADS[args.workload]
        B, C, d, G, H, W, P, s = cfg
        q, key, v, off = make_deform_inputs(cfg, dtype, dev)
    else:
        cfg = WORKLOADS[args.workload]
        B, C, d, H, W, K, s = cfg
        q, key, v = make_inputs(cfg, dtype, dev, heavy_tails=args.workload == 'stress',
                                projected=args.workload.startswith('segformer'))
    out = torch.empty(B, C, H * s, W * s, dtype=dtype, device=dev)
    code = _lib.dtype_code(out)
    if deform:
        nhwc_ok = s in (1, 2, 4) and P <= 32 and d % 4 == 0 and d <= 64 and (C // G) % 4 == 0
    else:
        nhwc_ok = ((K, s) in ((3, 2), (5, 2), (7, 2), (5, 4), (7, 4))
                   and d % 4 == 0 and C % 4 == 0)
    if args.layout == 'channels_last':
        if not nhwc_ok or args.direction == 'module':
            sys.exit('bench.py: --layout channels_last covers the workloads with '
                     '(K, s) in {(3,2), (5,2), (7,2), (5,4), (7,4)} (SAPA-B) / P <= 32 (SAPA-D), '
                     '--pass forward and --pass train')
        q, key, v, out = (t.contiguous(memory_format=torch.channels_last) for t in (q, key, v, out))
        if deform:
            off = off.contiguous(memory_format=torch.channels_last)

    if deform:
        def fused_step(entry, q, key, v, out, off):
            fn = getattr(lib, entry)

            def step():
                _lib.check(fn(q.data_ptr(), key.data_ptr(), v.data_ptr(), off.data_ptr(),
                              out.data_ptr(), B, G * d, C, H, W, P, s, G, code,
                              stream.cuda_stream), entry)
            return step
        # contiguous tensors through the matrix-form kernels (key and value copied to
        # channels-last order in a workspace): what sapa_amd.deform_sapa_fused does by
        # default where it is the faster path (16-bit tensors from 4 points, fp32 from 13)
        ws_bytes = lib.sapa_deform_fused_forward_workspace(B, G * d, C, H, W, P, s, G, code)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)

        def ws_step():
            _lib.check(lib.sapa_deform_fused_forward_ws(
                q.data_ptr(), key.data_ptr(), v.data_ptr(), off.data_ptr(), out.data_ptr(), ws.data_ptr(),
                B, G * d, C, H, W, P, s, G, 0, code, stream.cuda_stream), 'sapa_deform_fused_forward_ws')
        main_is_ws = args.layout == 'nchw' and ws_bytes > 0 and not args.reference_order
        step = ws_step if main_is_ws else fused_step(
            'sapa_deform_fused_forward_nhwc' if args.layout == 'channels_last' else 'sapa_deform_fused_forward',
            q, key, v, out, off)
    else:
        def fused_step(entry, q, key, v, out):
            fn = getattr(lib, entry)

            def step():
                _lib.check(fn(q.data_ptr(), key.data_ptr(), v.data_ptr(), out.data_ptr(), B, d, C,
                              H, W, K, s, code, stream.cuda_stream), entry)
            return step
        step = fused_step('sapa_fused_forward_nhwc' if args.layout == 'channels_last'
                          else 'sapa_fused_forward', q, key, v, out)

    train = args.direction == 'train'
    if train:
        import sapa_amd
        go = torch.randn(B, C, H * s, W * s, device=dev).to(dtype)
        if args.layout == 'channels_last':
            # the forward runs on the channels-last kernels; the backward pass has no
            # channels-last kernels: autograd copies its operands to contiguous order and
            # the gradients come back in that order (the step below includes those copies)
            go = go.contiguous(memory_format=torch.channels_last)
        leaves = [t.requires_grad_() for t in ((q, key, v, off) if deform else (q, key, v))]
        if deform:
            def step():
                y = sapa_amd.deform_sapa_fused(q, key, v, off, P, s, G)
                torch.autograd.grad(y, leaves, go)
        else:
            def step():
                y = sapa_amd.sapa_fused(q, key, v, K, s, save_attention=not args.recompute_attention)
                torch.autograd.grad(y, leaves, go)

    settle = {'ms': args.settle_ms, 'launches': 0}

    def timed(step):
        # Power management first: from idle this GPU runs its first 3-4 launches at
        # full clocks, drops by ~25 % for the next ~30 launches and recovers within
        # ~40 (a transient of the part, the same after any pause) -- a timed region
        # that starts a handful of launches after idle measures that dip, not the
        # kernel.  So the same launch is repeated, untimed, for --settle-ms of GPU
        # time before the W warm-up steps; the JSON line says how many that were.
        if args.settle_ms > 0:
            t0, n = time.perf_counter(), 0
            while (time.perf_counter() - t0) * 1e3 < args.settle_ms:
                for _ in range(10):
                    step()
                torch.cuda.synchronize()
                n += 10
            settle['launches'] = max(settle['launches'], n)
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        # HIP events on the stream the kernel is launched on
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(stream)
        for _ in range(args.steps):
            step()
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps, (time.perf_counter() - t0) * 1e3 / args.steps

    after_idle = None
    if args.direction == 'forward' and not args.no_after_idle:
        # the literal protocol first: W warm-up steps and K timed steps straight after a
        # pause (the GPU has idled through input generation's tail and this sleep), with
        # no settle launches.  It contains the power-management dip described in timed().
        step()      # first-call costs (module load, descriptor set-up) are not what either protocol times
        torch.cuda.synchronize()
        time.sleep(1.0)
        keep, args.settle_ms = args.settle_ms, 0.0
        ms_idle, _ = timed(step)
        args.settle_ms = keep
        after_idle = {'ms_per_step': ms_idle, 'protocol': f'1 s pause, {args.warmup} warm-up steps, '
                      f'{args.steps} timed steps, no settle launches'}
    ms, wall_ms = timed(step)
    main_kernel = _lib.last_kernel()
    ms_cl = None
    if args.layout == 'nchw' and nhwc_ok and args.direction == 'forward' and not args.only_main:
        # the same workload with every tensor in torch.channels_last order
        cl = [t.contiguous(memory_format=torch.channels_last)
              for t in ((q, key, v, out, off) if deform else (q, key, v, out))]
        ms_cl, _ = timed(fused_step('sapa_deform_fused_forward_nhwc' if deform
                                    else 'sapa_fused_forward_nhwc', *cl))
        cl_kernel = _lib.last_kernel()
        err_cl = (cl[3][:1].float() - out[:1].float()).abs().max().item()
        del cl

    half = None
    if (not deform and args.dtype == 'fp32' and args.layout == 'nchw' and args.direction == 'forward'
            and not args.only_main):
        # the same workload and layout with bf16 tensors (the inputs rounded to bf16)
        hq, hk, hv = (t.to(torch.bfloat16) for t in (q, key, v))
        hout = torch.empty_like(out, dtype=torch.bfloat16)

        def half_step():
            _lib.check(lib.sapa_fused_forward(hq.data_ptr(), hk.data_ptr(), hv.data_ptr(), hout.data_ptr(), B, d, C,
                                              H, W, K, s, 3, stream.cuda_stream), 'sapa_fused_forward')
        ms_h, _ = timed(half_step)
        hbytes = algorithmic_bytes(B, C, d, H, W, s, 2)
        half = {'dtype': 'bf16', 'ms_per_step': ms_h, 'value': B * H * s * W * s / (ms_h * 1e-3) / 1e9,
                'unit': 'Gpix/s', 'algorithmic_bytes': hbytes,
                'roofline_frac': hbytes / (ms_h * 1e-3) / 1e9 / HBM_PEAK_GBS,
                'kernel': _lib.last_kernel() + ' (fused mode)',
                'note': 'same workload, contiguous (NCHW) bf16 tensors (python bench.py --dtype bf16 makes this '
                        'the main line); parity bar 1e-2 max(|b|, rms(b)), held by the tests to half a bf16 '
                        'spacing of the double-precision result on the rounded inputs'}
        if nhwc_ok:
            # and with every tensor in torch.channels_last order
            hc = [t.contiguous(memory_format=torch.channels_last) for t in (hq, hk, hv, hout)]

            def half_cl_step():
                _lib.check(lib.sapa_fused_forward_nhwc(hc[0].data_ptr(), hc[1].data_ptr(), hc[2].data_ptr(),
                                                       hc[3].data_ptr(), B, d, C, H, W, K, s, 3, stream.cuda_stream),
                           'sapa_fused_forward_nhwc')
            ms_hc, _ = timed(half_cl_step)
            half['channels_last'] = {
                'ms_per_step': ms_hc, 'value': B * H * s * W * s / (ms_hc * 1e-3) / 1e9, 'unit': 'Gpix/s',
                'roofline_frac': hbytes / (ms_hc * 1e-3) / 1e9 / HBM_PEAK_GBS,
                'kernel': _lib.last_kernel() + ' (fused mode)',
                'max_abs_diff_vs_nchw_image0': (hc[3][:1].float() - hout[:1].float()).abs().max().item(),
                'note': 'python bench.py --dtype bf16 --layout channels_last makes this the main line'}
            del hc
        del hq, hk, hv, hout

    module = None
    if (not deform and args.dtype == 'fp32' and args.layout == 'nchw' and args.direction == 'forward'
            and not args.only_main):
        # the caller of the hot path: the whole SAPA module forward on this workload's features (the
        # reference's composition, and GroupNorm folded into this library's projection kernels)
        module = {'unit': 'ms per forward', 'note': 'python bench.py --pass module [--dtype bf16] makes this the main line',
                  'fp32': {k: round(v['ms'], 4) for k, v in module_cases(
                      args, dev, torch.float32, stream, only=[0, 1, 3], warmup=5, steps=10).items()},
                  'bf16': {k: round(v['ms'], 4) for k, v in module_cases(
                      args, dev, torch.bfloat16, stream, only=[0, 1, 3], warmup=5, steps=10).items()}}

    reference_order = None
    if deform and main_is_ws and args.direction == 'forward' and not args.only_main:
        # the same contiguous tensors through the kernel that keeps the reference's order of sums
        ws_out = out[:1].clone()
        ms_r, _ = timed(fused_step('sapa_deform_fused_forward', q, key, v, out, off))
        reference_order = {'ms_per_step': ms_r, 'kernel': _lib.last_kernel(),
                           'max_abs_diff_vs_main_image0': (out[:1].float() - ws_out.float()).abs().max().item(),
                           'note': 'sapa_deform_fused_forward (sapa_amd.deform_sapa_fused(..., matrix_form=False)); '
                                   'python bench.py --reference-order makes this the main line'}
        step()      # the main line's result back into `out` for the checks below

    ceiling = None
    if args.direction == 'forward' and not args.no_ceiling:
        ceiling = measured_ceiling(lib, dev, stream, args, timed,
                                   out.numel() * out.element_size())

    if args.calibration_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    pix = B * H * s * W * s
    esize = out.element_size()
    if deform:
        abytes = deform_algorithmic_bytes(B, C, d, G, H, W, P, s, esize)
        what = 'fused SAPA-D forward (deform_qk->softmax->deform_av)'
        wl = (f'{args.workload}: SAPA-D B={B} C={C} d={d} G={G} P={P} {H}x{W}->{H * s}x{W * s} '
              f's={s} {args.dtype}, NCHW, offsets ~N(0,0.75) clipped to +-4')
        wl = wl.replace('NCHW', 'channels_last') if args.layout == 'channels_last' else wl
    else:
        abytes = algorithmic_bytes(B, C, d, H, W, s, esize)
        what = 'fused SAPA-B forward (qk->softmax->av)'
        style = ('SegFormer-style stage, q / k from 1x1 projections ~N(0,.02) of GroupNorm-ed features'
                 if args.workload.startswith('segformer') else 'FPN-style')
        wl = (f'{args.workload}: SAPA-B {style} B={B} C={C} d={d} '
              f'{H}x{W}->{H * s}x{W * s} K={K} s={s} {args.dtype}, '
              + ('channels_last' if args.layout == 'channels_last' else 'NCHW')
              + (', 10% of q Student-t(3)' if args.workload == 'stress' else ''))
    # the kernel the library dispatched this workload to
    kern = main_kernel + ' (fused mode)'
    if train:
        # backward: read grad_out, q, key, value (offset); write every input gradient
        hi_px, lo_px = B * H * s * W * s, B * H * W
        qc = G * d if deform else d
        abytes += esize * (hi_px * (C + 2 * qc) + 2 * lo_px * (qc + C))
        if deform:
            abytes += esize * hi_px * 2 * (2 * G * P)
        what = what.replace('forward', 'forward + backward')
        kern = 'several (see profiles/)'
        if args.layout == 'channels_last':
            kern += '; forward on the channels-last kernels, backward through contiguous copies'
    traffic = traffic_source = None
    if not train:
        tlayout = 'nchw_reference_order' if deform and args.layout == 'nchw' and args.reference_order else args.layout
        traffic, traffic_source = measured_traffic(args.workload, args.dtype, tlayout, main_kernel)
    achieved = abytes / (ms * 1e-3) / 1e9
    flops = (deform_algorithmic_flops(B, C, d, G, H, W, P, s) if deform
             else algorithmic_flops(B, C, d, H, W, K, s)) * (3 if train else 1)
    # the arithmetic bound next to the HBM one: fp32 tensors multiply at the fp32 rate whichever
    # pipe takes them; 16-bit tensors can take the products to the 16-bit matrix instructions
    cpeak = FP32_PEAK_TFLOPS if args.dtype == 'fp32' else BF16_MFMA_PEAK_TFLOPS
    t_hbm, t_cmp = abytes / (HBM_PEAK_GBS * 1e9), flops / (cpeak * 1e12)
    compute_bound = {'bound': 'mfma', 'achieved': flops / (ms * 1e-3) / 1e12, 'peak': cpeak, 'unit': 'TFLOP/s',
                     'frac': flops / (ms * 1e-3) / 1e12 / cpeak, 'algorithmic_flops': flops,
                     'floor_us': t_cmp * 1e6,
                     'note': ('fp32 multiply-adds, vector or matrix pipe' if args.dtype == 'fp32'
                              else 'products on the 16-bit matrix instructions')}
    rec = {
        'metric': f'upsampled Gpix/s, {what}, 1 GPU',
        'value': pix / (ms * 1e-3) / 1e9,
        'unit': 'Gpix/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': ms,
        'wall_ms_per_step': wall_ms,
        'settle': settle,
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'f32' if args.dtype == 'fp32' else 'bf16',
        'data': 'synthetic',
        'config': {'workload': wl},
        'roofline': {
            'bound': 'hbm',
            'achieved': achieved,
            'peak': HBM_PEAK_GBS,
            'unit': 'GB/s',
            'frac': achieved / HBM_PEAK_GBS,
            'traffic': traffic,
            'traffic_source': traffic_source,
            'algorithmic_bytes': abytes,
            'kernel': kern,
            # a working set below the 256 MB Infinity Cache stays cache-resident
            # when the same buffers are iterated: the rate is then no HBM rate
            'cache_resident': abytes < 256e6,
            'floor_us': t_hbm * 1e6,
            # the bound whose floor is the higher one is the nearer one: 'bound' above says
            # which roofline the main figures are quoted on, 'nearer_bound' which of the two
            # the workload would hit first on this part
            'nearer_bound': 'hbm' if t_hbm >= t_cmp else 'mfma',
            'compute': compute_bound,
        },
    }
    if t_cmp > t_hbm:
        # quote the main roofline on the bound that is actually nearer; the HBM figures stay beside it
        hbm = {k: rec['roofline'][k] for k in ('achieved', 'peak', 'unit', 'frac', 'floor_us')}
        rec['roofline'].update({'bound': 'mfma', 'achieved': compute_bound['achieved'], 'peak': cpeak,
                                'unit': 'TFLOP/s', 'frac': compute_bound['frac'], 'floor_us': t_cmp * 1e6,
                                'hbm': hbm})
        del rec['roofline']['compute']
    if after_idle is not None:
        after_idle['frac'] = abytes / (after_idle['ms_per_step'] * 1e-3) / 1e9 / HBM_PEAK_GBS
        after_idle['value'] = pix / (after_idle['ms_per_step'] * 1e-3) / 1e9
        rec['after_idle'] = after_idle
    if ceiling is not None:
        ceiling['frac_of_peak'] = ceiling['GB/s'] / HBM_PEAK_GBS
        ceiling['kernel_vs_ceiling'] = achieved / ceiling['GB/s']
        if ms_cl is not None:
            ceiling['channels_last_kernel_vs_ceiling'] = abytes / (ms_cl * 1e-3) / 1e9 / ceiling['GB/s']
        rec['roofline']['measured_ceiling'] = ceiling
    if ms_cl is not None:
        rec['channels_last'] = {
            'ms_per_step': ms_cl, 'value': pix / (ms_cl * 1e-3) / 1e9, 'unit': 'Gpix/s',
            'roofline_frac': abytes / (ms_cl * 1e-3) / 1e9 / HBM_PEAK_GBS,
            'kernel': cl_kernel + ' (fused mode)',
            'max_abs_diff_vs_nchw_image0': err_cl,
            'parity_bar': ('16-bit tensors: 1e-2 max(|b|, rms(b)) against the double-precision result on the '
                           'rounded inputs' if args.dtype != 'fp32' else
                           'channel sums in tree order (SAPA-D: matrix form): not the reference order, so not '
                           'bit-identical to it; held by the tests to "no worse than the reference order '
                           'against the double-precision result", with the count outside 1e-6 + 1e-5 |b| of '
                           'the reference-order fp32 result printed and bounded there'),
            'note': 'same workload and algorithmic bytes, every tensor in torch.channels_last '
                    'order (python bench.py --layout channels_last makes this the main line)'}
    if half is not None:
        rec['bf16'] = half
    if module is not None:
        rec['module_forward'] = module
    if reference_order is not None:
        reference_order['value'] = pix / (reference_order['ms_per_step'] * 1e-3) / 1e9
        reference_order['roofline_frac'] = abytes / (reference_order['ms_per_step'] * 1e-3) / 1e9 / HBM_PEAK_GBS
        rec['reference_order'] = reference_order
    if deform and not train and main_is_ws:
        rec['config']['workspace_bytes'] = ws_bytes
        rec['config']['entry'] = 'sapa_deform_fused_forward_ws (key / value copied to channels-last order inside the timed call)'
    if not args.no_cpu_baseline and not train:
        from oracle import torch_oracle
        if deform:
            # grid_sample formulation of deformsapa/deformsapa/forward_check.py:6-40
            rec['cpu_baseline'], ref = cpu_baseline(
                lambda a, b, c, o: torch_oracle.deform_sapa_fused(a, b, c, o, P, s, G), (q, key, v, off),
                H * s * W * s)
        else:
            # unfold + einsum formulation of sapa/sapa/forward_check.py:9-24
            rec['cpu_baseline'], ref = cpu_baseline(
                lambda a, b, c: torch_oracle.sapa_fused(a, b, c, K, s), (q, key, v), H * s * W * s)
        # Sanity check only (the parity tests proper are tests/test_gpu_*): the timed GPU
        # output of image 0 against the CPU baseline's output.  That path sums in another
        # order (einsum / grid_sample), so this is fp32 against fp32 at the reference's own
        # check tolerance, allclose(atol=1e-5) (sapa/sapa/forward_check.py:37-39).
        got = out[:1].float().cpu()
        err = (got - ref).abs()
        if args.dtype != 'fp32':
            tol, bar = 1e-2 * torch.maximum(ref.abs(), ref.pow(2).mean().sqrt()), '1e-2 max(|b|, rms(b))'
        elif deform:
            # grid_sample normalises and de-normalises the coordinates in fp32,
            # which moves each sample by a few 1e-7 cells
            tol, bar = 1e-4 + 1e-4 * ref.abs(), '1e-4 + 1e-4 |b|'
        else:
            tol, bar = 1e-5 + 1e-5 * ref.abs(), '1e-5 + 1e-5 |b|'
        rec['sanity_vs_cpu_baseline_output'] = {'max_abs_err': err.max().item(), 'bar': bar,
                                                'outside_bar': int((err > tol).sum().item()),
                                                'elements': err.numel()}
        if args.dtype == 'fp32' and args.layout == 'nchw':
            # the stated bar, 1e-6 + 1e-5 |b|, against the reference kernels' own arithmetic
            # (the C restatement of their loops in fp32, one fused multiply-add per term in
            # kernel order): image 0 of the timed output
            from oracle import c_oracle
            cpu0 = [t[:1].float().cpu() for t in ((q, key, v, off) if deform else (q, key, v))]
            ref32 = (c_oracle.deform_sapa_fused(*cpu0, P, s, G, 'f32') if deform
                     else c_oracle.sapa_fused(*cpu0, K, s, 'f32'))
            e32 = (got - ref32).abs()
            outside = int((e32 > 1e-6 + 1e-5 * ref32.abs()).sum().item())
            same_order = main_kernel in ('sapa_b_tiled_kernel', 'deform_lds_kernel', 'sapa_b_mfma_kernel')
            rec['parity_image0'] = {
                'against': "oracle/c_oracle 'f32' (the reference kernels' arithmetic and order of sums)",
                'bar': '1e-6 + 1e-5 |b|', 'outside_bar': outside, 'elements': e32.numel(),
                'max_abs_err': e32.max().item(), 'bit_identical': bool(torch.equal(got, ref32)),
                'route': ('sums in the reference order: meets the stated bar literally' if same_order else
                          'sums in another order than the reference (matrix form): two fp32 orders of the '
                          'same sum differ by their rounding, so the tests hold this route to "no worse than '
                          'the reference order against the double-precision result" and bound this count')}
    print(json.dumps(rec))


if __name__ == '__main__':
    main()
