#!/usr/bin/env python3
"""Benchmark of the flash-attention hot path on one MI355X.

A step = one forward + one backward (split backend) at the headline
configuration: B=4, Hq=Hkv=32, Sq=Sk=4096, D=128, bf16, causal, q/k/v/dO ~ N(0,1)
from a seed, sm_scale = 1/sqrt(128), inputs resident in HBM.  FLOP conventions
are the reference's (modules/flash/tests/performance_forward.py:108-113):
forward 4*B*H*S^2*D*0.5 (causal), backward 2.5x forward.

Prints ONE JSON line.  `value` is the whole step's TFLOPS; the forward and both
backward variants are reported separately next to it, each also as a fraction of
the dense bf16 MFMA peak.  `roofline` describes the kernel that takes the largest
share of the step; `cpu_baseline` is PyTorch's math SDPA (the reference's own test
oracle) on the host CPU on a bounded sample of the same workload.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6      # MI355X dense bf16/fp16 MFMA: 256 CU x 2.4 GHz x 4096 FLOP/clk/CU

# HBM bytes per launch at the headline shape, from rocprofv3 FETCH_SIZE / WRITE_SIZE
# runs scaled by a 256 MiB elementwise probe (summaries and commands: profiles/*.txt).
# Counters cannot be read from inside this process, so the figures are recorded here.
HBM_BYTES_PER_LAUNCH = {'fwd_kernel': 6.9703e8, 'bwd_dkdv_kernel': 8.1939e8, 'bwd_dq_kernel': 7.7205e8}


def cpu_baseline(B, H, S, D, causal, seed):
    """PyTorch math SDPA on the host CPU, fwd + bwd by autograd, on H_s heads of one
    batch element (fp32, the precision the reference's oracle runs at)."""
    import torch
    from oracle import fa_ref
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    h_s = 8
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(1, h_s, S, D, generator=g).requires_grad_()
    k = torch.randn(1, h_s, S, D, generator=g).requires_grad_()
    v = torch.randn(1, h_s, S, D, generator=g).requires_grad_()
    do = torch.randn(1, h_s, S, D, generator=g)
    ct, wl, wr = (3, -2147483647, -2147483647) if causal else (0, 0, 0)
    sm = 1.0 / math.sqrt(D)
    t0 = time.perf_counter()
    fa_ref.sdpa_math_ref(q, k, v, None, sm, ct, wl, wr).backward(do)   # warm-up, also sizes the sample
    once = time.perf_counter() - t0
    reps = max(4, min(64, int(math.ceil(12.0 / max(once, 1e-3)))))     # about 12 s of CPU work
    t0 = time.perf_counter()
    for _ in range(reps):
        q.grad = k.grad = v.grad = None
        o = fa_ref.sdpa_math_ref(q, k, v, None, sm, ct, wl, wr)
        o.backward(do)
    dt = (time.perf_counter() - t0) / reps
    flops = 3.5 * 4.0 * 1 * h_s * S * S * D * (0.5 if causal else 1.0)
    return {
        'value': flops / dt / 1e12, 'unit': 'TFLOPS', 'cores': threads, 'kind': 'port',
        'sample': f'fwd+bwd of {h_s} heads of one batch element (fp32, S={S}, D={D}, causal={causal}), '
                  f'{reps} reps, {dt:.2f} s each; same FLOP formula as the GPU rows',
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--no-cpu', action='store_true', help='skip the host-CPU baseline leg')
    ap.add_argument('--traffic-probe', action='store_true',
                    help='also run one elementwise kernel of known HBM traffic (256 MiB read + 256 MiB '
                         'written) so that FETCH_SIZE / WRITE_SIZE counters can be scaled')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py: this build runs on one GPU only (attention shards by batch/head with no '
              'exchange); use --gpus 1', file=sys.stderr)
        sys.exit(2)

    import torch
    from aotriton_amd import flash
    from aotriton_amd.pyaotriton.v3.flash import attn_bwd_kernel, attn_bwd_params

    dev = torch.device('cuda', 0)
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(0)
    B, H, S, D = 4, 32, 4096, 128
    causal = True
    dtype = torch.bfloat16
    seed = 1234
    g = torch.Generator(device='cpu').manual_seed(seed)

    def rn():
        return torch.randn(B, H, S, D, generator=g, dtype=torch.float32).to(dtype).to(dev)

    q, k, v, do = rn(), rn(), rn(), rn()
    o = torch.empty_like(q)
    L = torch.empty(B * H, S, device=dev, dtype=torch.float32)
    delta = torch.empty_like(L)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    null = torch.empty([0], device=dev, dtype=torch.uint64)
    atomic = torch.zeros([1], device=dev, dtype=torch.int32)
    sm = 1.0 / math.sqrt(D)
    ok = flash.hipError_t.hipSuccess

    def fwd():
        atomic.zero_()
        assert flash.attn_fwd(q, k, v, None, sm, L, o, 0.0, null, null, 0, null, null, None, causal, atomic) == ok

    def bwd(backend):
        ext = flash.attn_options()
        ext.force_backend_index = backend
        assert flash.attn_bwd(q, k, v, None, sm, o, do, dq, dk, dv, None, None, L, delta, 0.0, null, null, 0,
                              causal, extargs=ext) == ok

    bparams = attn_bwd_params()
    flash._fill_bwd(bparams, q, k, v, None, sm, o, do, dq, dk, dv, None, None, L, delta, 0.0, null, null, 0, causal)

    def bwd_slot(slot):
        assert attn_bwd_kernel(bparams, attn_bwd_params.kVersion, flash._stream(), slot) == ok

    def timed(fn, n):
        """Average duration (ms) of fn over n launches, HIP events on the launch stream."""
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        e1.synchronize()
        return e0.elapsed_time(e1) / n

    if args.traffic_probe:
        x = torch.zeros(64 * 1024 * 1024, device=dev, dtype=torch.float32)
        y = torch.empty_like(x)
        torch.add(x, 1.0, out=y)          # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del x, y

    for _ in range(args.warmup):
        fwd()
        bwd(0)
    bwd(1)
    torch.cuda.synchronize()

    # the step: exactly K timed steps bracketed by synchronisation
    t0 = time.perf_counter()
    for _ in range(args.steps):
        fwd()
        bwd(0)
    torch.cuda.synchronize()
    step_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    n = max(args.steps, 5)
    t_fwd = timed(fwd, n)
    t_split = timed(lambda: bwd(0), n)
    t_fused = timed(lambda: bwd(1), n)
    t_pre = timed(lambda: bwd_slot(0), n)
    t_dkdv = timed(lambda: bwd_slot(1), n)
    t_dq = timed(lambda: bwd_slot(2), n)
    torch.cuda.synchronize()

    f_fwd = 4.0 * B * H * S * S * D * (0.5 if causal else 1.0)
    f_bwd = 2.5 * f_fwd
    tf = lambda fl, ms: fl / (ms * 1e-3) / 1e12
    value = tf(f_fwd + f_bwd, step_ms)

    # Dominant kernel of the step and the GEMM work it is required to do:
    # forward 2 GEMMs, dK/dV 4 GEMMs (S, dP, dV, dK), dQ 3 GEMMs (S, dP, dQ); one
    # causal GEMM = 2*B*H*S^2*D*0.5 FLOP.
    gemm = 2.0 * B * H * S * S * D * (0.5 if causal else 1.0)
    kernels = {'fwd_kernel': (t_fwd, 2 * gemm), 'bwd_dkdv_kernel': (t_dkdv, 4 * gemm),
               'bwd_dq_kernel': (t_dq, 3 * gemm)}
    dom = max(kernels, key=lambda kname: kernels[kname][0])
    dom_ms, dom_fl = kernels[dom]
    roofline = {'bound': 'mfma', 'kernel': dom, 'achieved': tf(dom_fl, dom_ms), 'peak': PEAK_BF16_TFLOPS,
                'unit': 'TFLOP/s', 'frac': tf(dom_fl, dom_ms) / PEAK_BF16_TFLOPS,
                'traffic': HBM_BYTES_PER_LAUNCH.get(dom), 'avg_ms': dom_ms, 'flop_per_launch': dom_fl}

    out = {
        'metric': 'attn fwd/bwd TFLOPS and % bf16 MFMA peak, B4 H32 S4096 D128 causal, 1 GPU',
        'value': value, 'unit': 'TFLOPS', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': step_ms, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'bf16', 'data': 'synthetic',
        'config': {'workload': 'attention fwd + bwd(split), B=4 Hq=Hkv=32 Sq=Sk=4096 D=128 bf16 causal, '
                               'q,k,v,dO~N(0,1) seed 1234, sm_scale=1/sqrt(128)'},
        'peak_tflops_used': PEAK_BF16_TFLOPS,
        'device': {'name': props.name, 'multiProcessorCount': props.multi_processor_count,
                   'clock_rate_khz': getattr(props, 'clock_rate', None)},
        'fwd': {'ms': t_fwd, 'tflops': tf(f_fwd, t_fwd), 'frac_peak': tf(f_fwd, t_fwd) / PEAK_BF16_TFLOPS},
        'bwd_split': {'ms': t_split, 'tflops': tf(f_bwd, t_split), 'frac_peak': tf(f_bwd, t_split) / PEAK_BF16_TFLOPS,
                      'kernels_ms': {'bwd_preprocess': t_pre, 'bwd_dkdv': t_dkdv, 'bwd_dq': t_dq}},
        'bwd_fused': {'ms': t_fused, 'tflops': tf(f_bwd, t_fused), 'frac_peak': tf(f_bwd, t_fused) / PEAK_BF16_TFLOPS},
        'roofline': roofline,
    }
    if not args.no_cpu:
        out['cpu_baseline'] = cpu_baseline(B, H, S, D, causal, seed)
    print(json.dumps(out))


if __name__ == '__main__':
    main()
