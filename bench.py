#!/usr/bin/env python3
"""Benchmark of the flash-attention hot path on one MI355X.

A step = one forward + one backward (split backend, as fa_attn_bwd runs it by default:
at this shape dS is kept in the library's HBM workspace between the dK/dV and the dQ
kernel) at the headline configuration: B=4, Hq=Hkv=32, Sq=Sk=4096, D=128, bf16, causal, q/k/v/dO ~ N(0,1)
from a seed, sm_scale = 1/sqrt(128), inputs resident in HBM.  FLOP conventions
are the reference's (modules/flash/tests/performance_forward.py:108-113):
forward 4*B*H*S^2*D*0.5 (causal), backward 2.5x forward.

Prints ONE JSON line.  `value` is the whole step's TFLOPS over K back-to-back steps.
The forward, both backward variants and the single kernels are timed one launch at a
time the way the reference times kernels (python/tune/gpu_utils.py:293-370): a buffer
larger than the last-level cache is zeroed before every launch, warm-up >= 25 ms,
>= 100 ms of timed launches, HIP events on the launch stream, median with the 20th and
80th percentile.  `roofline` describes the kernel that takes the largest share of the
step; `cpu_baseline` is PyTorch's math SDPA (the reference's own test oracle) on the host
CPU on a bounded sample of the same workload.  `c4` and `c5` time the benchmark's
configurations 4 (GQA, 16 packed sequences) and 5 (D=256, window + bias + dropout) at
full size; they are extra keys, `value` stays the headline.
"""
import argparse
import json
import math
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2516.6      # MI355X dense bf16/fp16 MFMA: 256 CU x 2.4 GHz x 4096 FLOP/clk/CU
FLUSH_BYTES = 512 << 20        # zeroed before each timed launch: above the 256 MB last-level cache


def hbm_bytes_from_profile(kernel):
    """HBM bytes per launch of `kernel` at the headline shape: the 'total ... B' figure of the
    committed rocprofv3 summary of that kernel (FETCH_SIZE / WRITE_SIZE runs, scaled by a
    256 MiB elementwise probe).  Counters cannot be read from inside this process."""
    names = {'fwd_kernel': 'attn_fwd', 'bwd_dkdv_kernel': 'bwd_dkdv', 'bwd_dq_kernel': 'bwd_dq',
             'bwd_dkdv_kernel (storing dS)': 'bwd_dkdv_storing_ds', 'bwd_dqs_kernel': 'bwd_dqs'}
    path = os.path.join(ROOT, 'profiles', f'{names.get(kernel, kernel)}_b4_h32_s4096_d128_bf16_causal.txt')
    try:
        m = re.search(r'total ([0-9.e+]+) B', open(path).read())
        return float(m.group(1)) if m else None
    except OSError:
        return None


def cpu_baseline(B, H, S, D, causal, seed):
    """PyTorch math SDPA on the host CPU, fwd + bwd by autograd, on H_s heads of one
    batch element (fp32, the precision the reference's oracle runs at)."""
    import torch
    from oracle import fa_ref
    threads = min(os.cpu_count() or 1, 16)        # a one-GPU box gives a job 16 cores
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
        'os_cpu_count': os.cpu_count(), 'torch_num_threads': torch.get_num_threads(),
        'sample': f'fwd+bwd of {h_s} heads of one batch element (fp32, S={S}, D={D}, causal={causal}), '
                  f'{reps} reps, {dt:.2f} s each; same FLOP formula as the GPU rows',
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--no-cpu', action='store_true', help='skip the host-CPU baseline leg')
    ap.add_argument('--no-extra', action='store_true', help='skip configurations 4 and 5')
    ap.add_argument('--plain', action='store_true',
                    help='headline kernels only, a few launches each, no cache flush (for profiler runs)')
    ap.add_argument('--traffic-probe', action='store_true',
                    help='also run one elementwise kernel of known HBM traffic (256 MiB read + 256 MiB '
                         'written) so that FETCH_SIZE / WRITE_SIZE counters can be scaled')
    ap.add_argument('--tile-entry', default=None, metavar='D,causal,dtype',
                    help='run the forward, dK/dV and dQ kernels of one tile-table entry a few times and print their '
                         'times (for profiler runs), e.g. 64,1,bf16: B = 4, H = 4096 / D, S = 4096; D up to 512, dtype bf16, fp16 or fp32')
    ap.add_argument('--only', default=None, choices=['c4', 'c5'],
                    help='run only the forward and the backward of configuration 4 (packed sequences) or 5 (D=256, window + '
                         'bias + dropout) a few times and print their times (for profiler runs)')
    ap.add_argument('--recompute', action='store_true',
                    help='with --only: workspace limit 0, i.e. the backward whose dQ kernel recomputes S and dP')
    ap.add_argument('--mfma-peak', action='store_true',
                    help='only measure what the matrix pipe sustains (register-only MFMA loop, constant '
                         'and random operands) and print that as one JSON line')
    args = ap.parse_args()
    if args.gpus != 1:
        print('bench.py: this build runs on one GPU only (attention shards by batch/head with no '
              'exchange); use --gpus 1', file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from aotriton_amd import flash
    from aotriton_amd._lib import lib
    from aotriton_amd.pyaotriton.v3.flash import attn_bwd_kernel, attn_bwd_params

    dev = torch.device('cuda', 0)
    torch.cuda.set_device(dev)
    props = torch.cuda.get_device_properties(0)
    stream_ptr = flash._stream().native() or None
    device = {'name': props.name, 'multiProcessorCount': lib.fa_get_multiprocessor_count(stream_ptr),
              'clock_rate_khz': lib.fa_get_clock_rate_khz(stream_ptr)}
    ok = flash.hipError_t.hipSuccess
    tf = lambda fl, ms: fl / (ms * 1e-3) / 1e12
    flush = torch.empty(FLUSH_BYTES, device=dev, dtype=torch.int8)

    def do_bench(fn, warmup_ms=25.0, rep_ms=100.0, max_reps=400):
        """Per-launch times of fn (ms): {'median','p20','p80','mean','reps'}."""
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(3):
            fn()
        e1.record()
        e1.synchronize()
        est = max(e0.elapsed_time(e1) / 3, 1e-3)
        for _ in range(max(1, int(warmup_ms / est))):
            fn()
        n = max(5, min(max_reps, int(math.ceil(rep_ms / est))))
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(n)]
        ends = [torch.cuda.Event(enable_timing=True) for _ in range(n)]
        for i in range(n):
            flush.zero_()
            starts[i].record()
            fn()
            ends[i].record()
        torch.cuda.synchronize()
        t = sorted(s.elapsed_time(e) for s, e in zip(starts, ends))
        q = lambda p: t[min(n - 1, int(p * n))]
        return {'median': q(0.5), 'p20': q(0.2), 'p80': q(0.8), 'mean': sum(t) / n, 'reps': n}

    def make_c4():
        """(forward, backward, forward FLOP, description) of configuration 4"""
        rng = np.random.default_rng(1234)
        lens = rng.integers(256, 8193, size=16)
        cu = np.zeros(17, dtype=np.int32)
        cu[1:] = np.cumsum(lens)
        T, Hq, Hk = int(cu[-1]), 32, 8
        gg = torch.Generator(device=dev).manual_seed(1234)
        mk = lambda h: torch.randn(1, T, h, 128, device=dev, dtype=torch.float32, generator=gg).to(torch.bfloat16).transpose(1, 2)
        q4, k4, v4, do4 = mk(Hq), mk(Hk), mk(Hk), mk(Hq)
        o4, dq4, dk4, dv4 = torch.empty_like(q4), torch.empty_like(q4), torch.empty_like(k4), torch.empty_like(v4)
        L4 = torch.empty(Hq, T, device=dev, dtype=torch.float32)
        d4 = torch.empty_like(L4)
        cuq = torch.from_numpy(cu).to(dev)
        mx = int(lens.max())
        sm4 = 1.0 / math.sqrt(128)

        def fwd4():
            assert flash.attn_fwd_compact_varlen(q4, k4, v4, None, cuq, cuq, mx, mx, sm4, L4, o4, 0.0, null, null, 0,
                                                 null, null, None, True, atomic) == ok

        def bwd4():
            assert flash.attn_bwd_compact_varlen(q4, k4, v4, cuq, cuq, mx, mx, None, sm4, o4, do4, dq4, dk4, dv4, None,
                                                 L4, d4, 0.0, null, null, 0, True) == ok

        fl4 = sum(4.0 * Hq * float(n) ** 2 * 128 * 0.5 for n in lens)
        return fwd4, bwd4, fl4, (f'GQA Hq=32 Hkv=8 D=128 bf16 causal, 16 packed sequences U[256,8192] (seed 1234), '
                                 f'{T} tokens, THD storage')

    def make_c5():
        """(forward, backward(with_db), forward FLOP, description) of configuration 5"""
        gg = torch.Generator(device=dev).manual_seed(1234)
        B5, H5, S5, D5 = 2, 16, 8192, 256
        rn5 = lambda *s, sc=1.0: (torch.randn(*s, device=dev, dtype=torch.float32, generator=gg) * sc).to(torch.float16)
        q5, k5, v5, do5 = (rn5(B5, H5, S5, D5) for _ in range(4))
        b5 = torch.empty(B5, H5, S5, S5, device=dev, dtype=torch.float16)
        for i in range(B5):
            for h in range(H5):
                b5[i, h] = rn5(S5, S5, sc=0.5)
        o5, dq5, dk5, dv5 = torch.empty_like(q5), torch.empty_like(q5), torch.empty_like(k5), torch.empty_like(v5)
        db5 = torch.empty_like(b5)
        L5 = torch.empty(B5 * H5, S5, device=dev, dtype=torch.float32)
        d5 = torch.empty_like(L5)
        u64 = lambda x: torch.tensor([x], device=dev, dtype=torch.uint64)
        seed5, off5, so5, oo5 = u64(0x1234), u64(0), u64(0), u64(0)
        sm5 = 1.0 / math.sqrt(D5)

        def fwd5():
            assert flash.attn_fwd(q5, k5, v5, b5, sm5, L5, o5, 0.1, seed5, off5, 0, so5, oo5, None, (1024, 0), atomic) == ok

        def bwd5(with_db):
            assert flash.attn_bwd(q5, k5, v5, b5, sm5, o5, do5, dq5, dk5, dv5, db5 if with_db else None, None, L5, d5,
                                  0.1, so5, oo5, 0, (1024, 0)) == ok

        fl5 = 4.0 * B5 * H5 * D5 * 7872000.0          # visible (query, key) pairs per head: sum_i (min(i, 1024) + 1)
        return fwd5, bwd5, fl5, ('B=2 H=16 S=8192 D=256 fp16, window (1024, 0), bias (B,H,S,S) ~ N(0,0.5), dropout 0.1 '
                                 'seed 0x1234 offset 0')

    if args.only:
        null = torch.empty([0], device=dev, dtype=torch.uint64)
        atomic = torch.zeros([1], device=dev, dtype=torch.int32)
        if args.recompute:
            lib.fa_set_bwd_workspace_limit(0)
        f, b, fl, work = make_c4() if args.only == 'c4' else make_c5()
        runs = {'fwd': f, 'bwd': b} if args.only == 'c4' else {'fwd': f, 'bwd_no_db': lambda: b(False)}
        res = {}
        for name, fn in runs.items():
            fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(3):
                fn()
            e1.record()
            e1.synchronize()
            res[name + '_ms'] = e0.elapsed_time(e1) / 3
        print(json.dumps({'only': args.only, 'workload': work, 'forward_flop': fl, **res}))
        return

    if args.tile_entry:
        d_s, c_s, t_s = args.tile_entry.split(',')
        D, causal = int(d_s), bool(int(c_s))
        dtype = {'bf16': torch.bfloat16, 'fp16': torch.float16, 'fp32': torch.float32}[t_s]
        B, S = 4, 4096
        H = 4096 // D
        g = torch.Generator(device=dev).manual_seed(1234)
        rn = lambda: torch.randn(B, H, S, D, device=dev, dtype=torch.float32, generator=g).to(dtype)
        q, k, v, do = rn(), rn(), rn(), rn()
        o, dq, dk, dv = (torch.empty_like(q) for _ in range(4))
        L = torch.empty(B * H, S, device=dev, dtype=torch.float32)
        delta = torch.empty_like(L)
        null = torch.empty([0], device=dev, dtype=torch.uint64)
        atomic = torch.zeros([1], device=dev, dtype=torch.int32)
        sm = 1.0 / math.sqrt(D)
        bp = attn_bwd_params()
        flash._fill_bwd(bp, q, k, v, None, sm, o, do, dq, dk, dv, None, None, L, delta, 0.0, null, null, 0, causal)
        fns = {'fwd': lambda: flash.attn_fwd(q, k, v, None, sm, L, o, 0.0, null, null, 0, null, null, None, causal, atomic),
               'bwd_preprocess': lambda: attn_bwd_kernel(bp, attn_bwd_params.kVersion, flash._stream(), 0),
               'bwd_dkdv': lambda: attn_bwd_kernel(bp, attn_bwd_params.kVersion, flash._stream(), 1),
               'bwd_dq': lambda: attn_bwd_kernel(bp, attn_bwd_params.kVersion, flash._stream(), 2)}
        res = {}
        for name, fn in fns.items():
            assert fn() == ok
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record()
            for _ in range(5):
                fn()
            e1.record()
            e1.synchronize()
            res[name + '_ms'] = e0.elapsed_time(e1) / 5
        gemm = 2.0 * B * H * S * S * D * (0.5 if causal else 1.0)
        print(json.dumps({'tile_entry': args.tile_entry, 'B': B, 'H': H, 'S': S, 'D': D, 'causal': causal,
                          'flop_per_gemm': gemm, **res}))
        return

    if args.mfma_peak:
        grid, iters = 512, 40000
        out = torch.empty(grid * 256, device=dev, dtype=torch.float32)
        clk = torch.zeros(2, device=dev, dtype=torch.int64)
        res = {}
        for name, rnd in (('constant_operands', 0), ('random_operands', 1)):
            run = lambda: lib.fa_probe_mfma_rate(rnd, grid, iters, out.data_ptr(), clk.data_ptr(), stream_ptr)
            assert run() == 0
            r = do_bench(run, warmup_ms=50.0, rep_ms=200.0, max_reps=8)
            c = clk.cpu().tolist()
            fl = grid * 4.0 * iters * 32 * 32768.0
            res[name] = {'ms': r['median'], 'tflops': tf(fl, r['median']),
                         'shader_clock_ghz': c[0] / (c[1] / 100e6) / 1e9 if c[1] else None}
        print(json.dumps({'metric': 'sustained v_mfma_f32_32x32x16_bf16 rate, register-only loop', 'unit': 'TFLOPS',
                          'device': device, 'peak_tflops_used': PEAK_BF16_TFLOPS, **res}))
        return

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

    def fwd():
        # (the persistent counter is accepted and not used: the work lists are static, nothing has to be zeroed)
        assert flash.attn_fwd(q, k, v, None, sm, L, o, 0.0, null, null, 0, null, null, None, causal, atomic) == ok

    def bwd(backend, workspace=True):
        lib.fa_set_bwd_workspace_limit(-1 if workspace else 0)      # 0: the dQ kernel recomputes S and dP
        ext = flash.attn_options()
        ext.force_backend_index = backend
        assert flash.attn_bwd(q, k, v, None, sm, o, do, dq, dk, dv, None, None, L, delta, 0.0, null, null, 0,
                              causal, extargs=ext) == ok
        lib.fa_set_bwd_workspace_limit(-1)

    bparams = attn_bwd_params()
    flash._fill_bwd(bparams, q, k, v, None, sm, o, do, dq, dk, dv, None, None, L, delta, 0.0, null, null, 0, causal)

    def bwd_slot(slot):
        assert attn_bwd_kernel(bparams, attn_bwd_params.kVersion, flash._stream(), slot) == ok

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
    if args.plain:
        for slot in (0, 1, 2, 3, 4, 5, 6):
            for _ in range(3):
                bwd_slot(slot)
        torch.cuda.synchronize()
        print(json.dumps({'plain': True, 'ms_per_step': step_ms, 'steps': args.steps}))
        return

    r_fwd = do_bench(fwd)
    r_split = do_bench(lambda: bwd(0))
    r_recomp = do_bench(lambda: bwd(0, workspace=False))
    r_fused = do_bench(lambda: bwd(1))
    r_pre = do_bench(lambda: bwd_slot(0))
    r_dkdv = do_bench(lambda: bwd_slot(1))
    r_dq = do_bench(lambda: bwd_slot(2))
    bwd(0)                                        # the workspace holds this shape's dS for slot 6
    r_prep = do_bench(lambda: bwd_slot(4))
    r_dkdv_s = do_bench(lambda: bwd_slot(5))
    r_dqs = do_bench(lambda: bwd_slot(6))
    torch.cuda.synchronize()

    f_fwd = 4.0 * B * H * S * S * D * (0.5 if causal else 1.0)
    f_bwd = 2.5 * f_fwd
    value = tf(f_fwd + f_bwd, step_ms)

    def row(fl, r, extra=None):
        d = {'ms': r['median'], 'ms_p20': r['p20'], 'ms_p80': r['p80'], 'reps': r['reps'],
             'tflops': tf(fl, r['median']), 'frac_peak': tf(fl, r['median']) / PEAK_BF16_TFLOPS}
        if extra:
            d.update(extra)
        return d

    # Dominant kernel of the step (the kernels the default step launches) and the GEMM work it is
    # required to do: forward 2 GEMMs, dK/dV 4 GEMMs (S, dP, dV, dK), dQ from stored dS 1 GEMM; one
    # causal GEMM = 2*B*H*S^2*D*0.5 FLOP.
    gemm = 2.0 * B * H * S * S * D * (0.5 if causal else 1.0)
    kernels = {'fwd_kernel': (r_fwd, 2 * gemm), 'bwd_dkdv_kernel (storing dS)': (r_dkdv_s, 4 * gemm),
               'bwd_dqs_kernel': (r_dqs, 1 * gemm)}
    dom = max(kernels, key=lambda kname: kernels[kname][0]['mean'])
    dom_r, dom_fl = kernels[dom]
    dom_ms = dom_r['mean']
    # the backward as a whole in the reference's convention (5 GEMMs of algorithmic work; 5 executed
    # when dS is kept, 7 when the dQ kernel recomputes)
    bwd_kernels_ms = r_prep['mean'] + r_dkdv_s['mean'] + r_dqs['mean']
    elem = 2 * B * H * S * D                                   # bytes of one bf16 activation tensor
    ds_bytes = 2.0 * B * H * S * S * (0.5 if causal else 1.0)  # one 16-bit dS value per visible (query, key) pair
    algorithmic_bytes = {'fwd_kernel': 4 * elem + 4 * B * H * S,            # Q, K, V in, O out, LSE out
                         # Q, K, V, dO in, dK, dV out, the two row statistics in, dS out
                         'bwd_dkdv_kernel (storing dS)': 6 * elem + 8 * B * H * S + ds_bytes,
                         'bwd_dqs_kernel': 2 * elem + ds_bytes}             # K in, dQ out, dS in
    roofline = {'bound': 'mfma', 'kernel': dom, 'achieved': tf(dom_fl, dom_ms), 'peak': PEAK_BF16_TFLOPS,
                'unit': 'TFLOP/s', 'frac': tf(dom_fl, dom_ms) / PEAK_BF16_TFLOPS,
                'traffic': hbm_bytes_from_profile(dom), 'algorithmic_bytes': algorithmic_bytes[dom],
                'avg_ms': dom_ms, 'median_ms': dom_r['median'], 'flop_per_launch': dom_fl,
                'frac_ref_convention': tf(f_bwd, bwd_kernels_ms) / PEAK_BF16_TFLOPS,
                'frac_ref_convention_note': 'whole split backward: 2.5 x forward FLOP (5 GEMMs) over the summed '
                                            'mean durations of its three kernels (delta and row statistics, '
                                            'dK/dV writing dS, dQ from dS); frac counts the GEMMs the dominant '
                                            'kernel executes'}

    out = {
        'metric': 'attn fwd/bwd TFLOPS and % bf16 MFMA peak, B4 H32 S4096 D128 causal, 1 GPU',
        'value': value, 'unit': 'TFLOPS', 'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup,
        'ms_per_step': step_ms, 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
        'dtype': 'bf16', 'data': 'synthetic',
        'config': {'workload': 'attention fwd + bwd(split), B=4 Hq=Hkv=32 Sq=Sk=4096 D=128 bf16 causal, '
                               'q,k,v,dO~N(0,1) seed 1234, sm_scale=1/sqrt(128)'},
        'peak_tflops_used': PEAK_BF16_TFLOPS,
        'device': device,
        'timing': 'per launch: 512 MiB zeroed before it, warm-up >= 25 ms, >= 100 ms of launches, HIP events, '
                  'median (p20, p80); value/ms_per_step: K back-to-back steps between synchronisations',
        'fwd': row(f_fwd, r_fwd),
        'bwd_split': row(f_bwd, r_split, {'kernels_ms': {'delta_and_row_statistics': r_prep['median'],
                                                         'bwd_dkdv_storing_ds': r_dkdv_s['median'],
                                                         'bwd_dq_from_ds': r_dqs['median']},
                                          'workspace_bytes': ds_bytes * 2 if causal else ds_bytes}),
        'bwd_split_recompute': row(f_bwd, r_recomp, {'kernels_ms': {'bwd_dq_with_delta': r_dq['median'],
                                                                    'bwd_dkdv': r_dkdv['median'],
                                                                    'bwd_preprocess_standalone_not_launched': r_pre['median']},
                                                     'note': 'workspace limit 0: the dQ kernel recomputes S and dP (7 GEMMs)'}),
        'bwd_fused': row(f_bwd, r_fused),
        'roofline': roofline,
    }

    if not args.no_extra:
        del q, k, v, do, o, dq, dk, dv
        torch.cuda.empty_cache()
        # --- configuration 4: GQA, 16 packed sequences U[256, 8192], causal, bf16, D=128 -------------
        fwd4, bwd4, fl4, work4 = make_c4()
        out['c4'] = {'workload': work4, 'fwd': row(fl4, do_bench(fwd4)), 'bwd_split': row(2.5 * fl4, do_bench(bwd4))}
        del fwd4, bwd4
        torch.cuda.empty_cache()
        # --- configuration 5: B2 H16 S8192 D256 fp16, window (1024, 0) + bias + dropout 0.1 ----------
        fwd5, bwd5, fl5, work5 = make_c5()

        def with_limit0(fn):
            lib.fa_set_bwd_workspace_limit(0)
            fn()
            lib.fa_set_bwd_workspace_limit(-1)

        out['c5'] = {'workload': work5,
                     'fwd': row(fl5, do_bench(fwd5, max_reps=100)),
                     'bwd_split_no_db': row(2.5 * fl5, do_bench(lambda: bwd5(False), max_reps=60)),
                     'bwd_split_no_db_recompute': row(2.5 * fl5, do_bench(lambda: with_limit0(lambda: bwd5(False)), max_reps=60),
                                                      {'note': 'workspace limit 0: the dQ kernel recomputes S and dP, with bias and dropout'}),
                     'bwd_split_with_db': row(2.5 * fl5, do_bench(lambda: bwd5(True), max_reps=60),
                                              {'note': 'dB is a dense (B,H,S,S) tensor: 4 GiB written, zeros outside the band'})}
        del fwd5, bwd5
        torch.cuda.empty_cache()
        # --- the two other kernel families: head dim 512 (bf16) and fp32 tensors, causal ---------------
        def family(Bx, Hx, Sx, Dx, dt, peak):
            gg = torch.Generator(device=dev).manual_seed(1234)
            rnx = lambda: torch.randn(Bx, Hx, Sx, Dx, device=dev, dtype=torch.float32, generator=gg).to(dt)
            qx, kx, vx, dox = rnx(), rnx(), rnx(), rnx()
            ox, dqx, dkx, dvx = (torch.empty_like(qx) for _ in range(4))
            Lx = torch.empty(Bx * Hx, Sx, device=dev, dtype=torch.float32)
            dx = torch.empty_like(Lx)
            smx = 1.0 / math.sqrt(Dx)

            def fwdx():
                assert flash.attn_fwd(qx, kx, vx, None, smx, Lx, ox, 0.0, null, null, 0, null, null, None, True, atomic) == ok

            def bwdx():
                assert flash.attn_bwd(qx, kx, vx, None, smx, ox, dox, dqx, dkx, dvx, None, None, Lx, dx, 0.0, null, null,
                                      0, True) == ok

            flx = 4.0 * Bx * Hx * Sx * Sx * Dx * 0.5
            rf, rb = do_bench(fwdx, max_reps=30), do_bench(bwdx, max_reps=12)
            return {'fwd': {'ms': rf['median'], 'tflops': tf(flx, rf['median']), 'frac_peak': tf(flx, rf['median']) / peak},
                    'bwd_split': {'ms': rb['median'], 'tflops': tf(2.5 * flx, rb['median']),
                                  'frac_peak': tf(2.5 * flx, rb['median']) / peak},
                    'peak_tflops_used': peak}

        out['d512'] = {'workload': 'B=4 H=16 S=4096 D=512 bf16 causal', **family(4, 16, 4096, 512, torch.bfloat16, PEAK_BF16_TFLOPS)}
        out['fp32'] = {'workload': 'B=4 H=32 S=4096 D=128 fp32 causal (fp32 MFMA peak)',
                       **family(4, 32, 4096, 128, torch.float32, 157.3)}
        # a head dim that is no multiple of 8 (one of the reference's test grid): packed copies in the
        # library's workspace, the 128-column MFMA kernels on those; next to the headline's figures
        d113 = family(4, 32, 4096, 113, torch.bfloat16, PEAK_BF16_TFLOPS)
        out['d113'] = {'workload': 'B=4 H=32 S=4096 D=113 bf16 causal (rows of 226 bytes: packed copies, FLOP counted at D=113)',
                       **d113, 'ms_over_d128': {'fwd': d113['fwd']['ms'] / r_fwd['median'],
                                                'bwd_split': d113['bwd_split']['ms'] / r_split['median']}}

    if not args.no_cpu:
        out['cpu_baseline'] = cpu_baseline(B, H, S, D, causal, seed)
    print(json.dumps(out))


if __name__ == '__main__':
    main()
