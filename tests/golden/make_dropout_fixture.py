"""Writes tests/golden/dropout_mask_reference.npz and tests/golden/philox_seed1234.json.

Runs in the build container only (it needs /root/reference and a Triton with the CPU
interpreter); only the files it writes travel anywhere else.

Part 1 runs the reference's own ``debug_simulate_encoded_softmax`` Triton kernel
(modules/flash/kernel/dropout_rng.py:86-126, which calls fast_dropout_mask,
dropout.py:41-71) under ``TRITON_INTERPRET=1`` on CPU tensors, with the grid of
modules/flash/csrc/attn_debug.cc:13-20 (cdiv(Sq, 64), H, B) and the fixed tile
BLOCK_M 64 / BLOCK_N 32 (modules/flash/aot/debug_simulate_encoded_softmax.py:21-25),
and stores the sign bits of its output.  The cases are small but exercise every term
of the Philox counter: several batch elements and heads, more than one 64-row tile,
key counts that are not multiples of 4 or of 32, two dropout rates, a seed above
2**32, and non-zero offset1 and offset2 together.

Part 2 is an independent probe of the Triton library itself (nothing from the
reference): ``tl.randint4x`` plus the join/join/reshape idiom, recorded for seed
0x1234 and a few counters, and the fp32 threshold expression.

Usage:  python tests/golden/make_dropout_fixture.py
"""
import json
import os
import sys

os.environ['TRITON_INTERPRET'] = '1'

import numpy as np  # noqa: E402
import torch  # noqa: E402
import triton  # noqa: E402
import triton.language as tl  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
REF_KERNELS = '/root/reference/modules/flash/kernel'

# (B, H, Sq, Sk, p, seed, offset1, offset2)
CASES = [
    (2, 3, 5, 10, 0.1, 0x1234, 0, 0),
    (2, 3, 70, 131, 0.5, 0x1_0000_0005, 0x1D4000, 0xB42),
    (1, 2, 65, 33, 0.1, 0xDEAD_BEEF_0000_0001, 3, (1 << 32) - 40),
    (3, 1, 7, 64, 0.25, 0x1BF52, 11, 0),
]


def scalar(value, np_dtype, tl_dtype):
    """A kernel scalar argument of an exact type, as the compiled kernel would receive it
    (the interpreter leaves Python floats untyped and guesses integer widths)."""
    from triton.runtime.interpreter import TensorHandle
    return tl.tensor(TensorHandle(np.array([value], dtype=np_dtype), tl_dtype), tl_dtype)


# The per-head term off_zh * Max_seqlen_q * stride is a product of 32-bit integers in the
# reference (dropout_rng.py:110, fwd_kernel.py:405-407) and wraps at 2**31 before it is added
# to the 64-bit base.  This case drives it there with a small tensor: only the first 64-row
# tile of each head is launched (grid.x = 1) while Max_seqlen_q is 2**27, so head 1's term
# is 2**31 (wraps to -2**31) and head 2's is 2**32 (wraps to 0).
# (B, H, rows written, Max_seqlen_q, Sk, p, seed, offset1, offset2)
WRAP_CASE = (1, 3, 64, 1 << 27, 64, 0.5, 0x1234, 0, 1 << 40)


def reference_wrap_case(dropout_rng):
    B, H, rows, max_sq, Sk, p, seed, off1, off2 = WRAP_CASE
    r = torch.zeros(B, H, rows, Sk, dtype=torch.float32)
    seed_t = torch.tensor([seed], dtype=torch.uint64)
    off1_t = torch.tensor([off1], dtype=torch.uint64)
    with np.errstate(over='ignore'):
        dropout_rng.debug_simulate_encoded_softmax[(1, H, B)](
            r, r.stride(0), r.stride(1), r.stride(2), r.stride(3),
            scalar(p, np.float32, tl.float32), H, max_sq, Sk, seed_t, off1_t,
            scalar(off2, np.uint64, tl.uint64), BLOCK_M=tl.constexpr(64), BLOCK_N=tl.constexpr(32))
    assert torch.all(r.abs() == 0.5)
    return {
        'wrap_params': np.array([B, H, rows, max_sq, Sk], dtype=np.int64),
        'wrap_p': np.array([p], dtype=np.float64),
        'wrap_rng': np.array([seed, off1, off2], dtype=np.uint64),
        'wrap_keep': np.packbits((r >= 0).numpy().reshape(-1)),
    }


def reference_masks():
    sys.path.insert(0, REF_KERNELS)
    import dropout_rng  # the reference's kernel file
    out = reference_wrap_case(dropout_rng)
    for i, (B, H, Sq, Sk, p, seed, off1, off2) in enumerate(CASES):
        r = torch.zeros(B, H, Sq, Sk, dtype=torch.float32)
        seed_t = torch.tensor([seed], dtype=torch.uint64)
        off1_t = torch.tensor([off1], dtype=torch.uint64)
        grid = (triton.cdiv(Sq, 64), H, B)
        dropout_rng.debug_simulate_encoded_softmax[grid](
            r, r.stride(0), r.stride(1), r.stride(2), r.stride(3),
            scalar(p, np.float32, tl.float32), H, Sq, Sk, seed_t, off1_t,
            scalar(off2, np.uint64, tl.uint64), BLOCK_M=tl.constexpr(64), BLOCK_N=tl.constexpr(32))
        assert torch.all(r.abs() == 0.5), 'every element must be written as +-0.5'
        out[f'case{i}_params'] = np.array([B, H, Sq, Sk], dtype=np.int64)
        out[f'case{i}_p'] = np.array([p], dtype=np.float64)
        out[f'case{i}_rng'] = np.array([seed, off1, off2], dtype=np.uint64)
        out[f'case{i}_keep'] = np.packbits((r >= 0).numpy().reshape(-1))
    return out


@triton.jit
def _probe(out_ptr, raw_ptr, thr_ptr, seed, ctr_ptr, p, N: tl.constexpr):
    ctr = tl.load(ctr_ptr + tl.arange(0, N))[None, :]
    r0, r1, r2, r3 = tl.randint4x(seed, ctr)
    row = tl.join(tl.join(r0, r1), tl.join(r2, r3)).reshape(1, N * 4)
    tl.store(out_ptr + tl.arange(0, N * 4)[None, :], row)
    tl.store(raw_ptr + tl.arange(0, N)[None, :] * 4 + 0, r0)
    tl.store(raw_ptr + tl.arange(0, N)[None, :] * 4 + 1, r1)
    tl.store(raw_ptr + tl.arange(0, N)[None, :] * 4 + 2, r2)
    tl.store(raw_ptr + tl.arange(0, N)[None, :] * 4 + 3, r3)
    tl.store(thr_ptr, ((p - 0.5) * 0xFFFFFFFF).to(tl.int32))


def library_probe():
    ctrs = [0, 1, 7, 8]
    ctr_t = torch.tensor(ctrs, dtype=torch.uint64)
    rows = torch.zeros(len(ctrs) * 4, dtype=torch.uint32)
    raw = torch.zeros(len(ctrs) * 4, dtype=torch.uint32)
    thr = {}
    for p in (0.1, 0.5, 0.2):
        t = torch.zeros(1, dtype=torch.int32)
        _probe[(1,)](rows, raw, t, scalar(0x1234, np.uint64, tl.uint64), ctr_t,
                     scalar(p, np.float32, tl.float32), N=len(ctrs))
        thr[str(p)] = int(t[0])
    hx = lambda xs: ['%08x' % int(x) for x in xs]
    rows = rows.view(len(ctrs), 4).numpy()
    raw = raw.view(len(ctrs), 4).numpy()
    return {
        '_comment': ("Words produced by Triton's tl.randint4x(seed=0x1234, counter) laid out by the "
                     "join/join/reshape idiom of the reference's dropout.py:37, recorded by "
                     "tests/golden/make_dropout_fixture.py from a CPU-interpreter probe of the Triton "
                     "library (not of the reference). Row order is the column order c%4 = 0,1,2,3. "
                     "'raw' is (w0,w1,w2,w3) before the permutation for counter 0."),
        'seed': 0x1234,
        'raw_counter0': hx(raw[0]),
        'rows': {str(c): hx(rows[i]) for i, c in enumerate(ctrs)},
        'idropout_p': thr,
        'random123_kat': [
            {'ctr': ['00000000'] * 4, 'key': ['00000000'] * 2,
             'out': ['6627e8d5', 'e169c58d', 'bc57ac4c', '9b00dbd8']},
            {'ctr': ['ffffffff'] * 4, 'key': ['ffffffff'] * 2,
             'out': ['408f276d', '41c83b0e', 'a20bc7c6', '6d5451fd']},
            {'ctr': ['243f6a88', '85a308d3', '13198a2e', '03707344'], 'key': ['a4093822', '299f31d0'],
             'out': ['d16cfe09', '94fdcceb', '5001e420', '24126ea1']},
        ],
    }


if __name__ == '__main__':
    probe = library_probe()
    with open(os.path.join(HERE, 'philox_seed1234.json'), 'w') as f:
        json.dump(probe, f, indent=1)
        f.write('\n')
    print('wrote philox_seed1234.json')
    masks = reference_masks()
    np.savez_compressed(os.path.join(HERE, 'dropout_mask_reference.npz'), **masks)
    print('wrote dropout_mask_reference.npz:', {k: v.shape for k, v in masks.items() if k.endswith('_keep')})
