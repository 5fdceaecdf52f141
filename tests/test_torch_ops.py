"""torch.library ops over the flash operators: shape-only (fake) implementations on the
CPU, and on the GPU the registration checks of torch.library.opcheck, equality with the
autograd Function path (same kernels, so bit-identical) and a trace through AOTAutograd."""
import math

import pytest
import torch

DEV = 'cuda'


def test_fake_implementations_give_the_operator_shapes():
    from aotriton_amd import torch_ops  # noqa: F401  (registers the ops)
    mk = lambda *s, dt=torch.bfloat16: torch.empty(*s, dtype=dt, device='meta')
    q, k, v = mk(2, 4, 128, 64), mk(2, 2, 96, 64), mk(2, 2, 96, 32)
    b = mk(2, 4, 128, 96)
    s = mk(1, dt=torch.uint64)
    o, lse = torch.ops.aotriton_amd.flash_attention_forward(q, k, v, b, 0.0, 3, 1, 2, 0.1, s, s)
    assert o.shape == (2, 4, 128, 32) and o.dtype == torch.bfloat16         # Out takes V's head dim
    assert lse.shape == (8, 128) and lse.dtype == torch.float32
    for need_db in (False, True):
        dq, dk, dv, db = torch.ops.aotriton_amd.flash_attention_backward(
            o, q, k, v, b, o, lse, 0.0, 3, 1, 2, 0.1, s, s, need_db, -1)
        assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
        assert db.shape == (b.shape if need_db else (0,))
    seed, off = torch.ops.aotriton_amd.philox_state(q, 10)
    assert seed.shape == (1,) and seed.dtype == torch.uint64 and off.dtype == torch.uint64


def _inputs(B=2, Hq=4, Hk=2, Sq=150, Sk=170, D=64, dtype=torch.bfloat16, bias=False, seed=0):
    from tests._util import make_inputs
    return make_inputs(B, Hq, Hk, Sq, Sk, D, dtype, DEV, seed=seed, bias=bias)


def _u64(x):
    return torch.tensor([x], device=DEV, dtype=torch.int64).view(torch.uint64)


@pytest.mark.gpu
@pytest.mark.parametrize('bias', [False, True])
@pytest.mark.parametrize('dropout_p', [0.0, 0.25])
def test_ops_equal_the_autograd_function(bias, dropout_p):
    from aotriton_amd import torch_ops  # noqa: F401
    from aotriton_amd.autograd import attention, AttentionExtraArgs
    q, k, v, b, do = _inputs(bias=bias)
    sm = 1.0 / math.sqrt(q.shape[-1])
    ext = AttentionExtraArgs(return_logsumexp=True)
    req = lambda t: None if t is None else t.detach().clone().requires_grad_()
    q1, k1, v1, b1 = req(q), req(k), req(v), req(b)
    o1, _, l1 = attention(q1, k1, v1, b1, (20, 3), sm, dropout_p, ext)
    o1.backward(do)
    q2, k2, v2, b2 = req(q), req(k), req(v), req(b)
    # the Function passes offset1 and offset2 separately; the kernels add them
    o2, l2 = torch.ops.aotriton_amd.flash_attention_forward(
        q2, k2, v2, b2, dropout_p, 3, 20, 3, sm, _u64(ext.philox_seed), _u64(ext.philox_offset1 + ext.philox_offset2))
    o2.backward(do)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
    assert torch.equal(q1.grad, q2.grad) and torch.equal(k1.grad, k2.grad) and torch.equal(v1.grad, v2.grad)
    if bias:
        assert torch.equal(b1.grad, b2.grad)


@pytest.mark.gpu
def test_opcheck_registrations():
    from aotriton_amd import torch_ops  # noqa: F401
    q, k, v, b, do = _inputs(Sq=64, Sk=80, bias=True)
    sm = 0.125
    seed, off = _u64(7), _u64(12)
    req = lambda t: t.detach().clone().requires_grad_()
    args = (req(q), req(k), req(v), req(b), 0.0, 3, 5, 2, sm, seed, off)
    torch.library.opcheck(torch.ops.aotriton_amd.flash_attention_forward.default, args,
                          test_utils=('test_schema', 'test_faketensor', 'test_autograd_registration',
                                      'test_aot_dispatch_dynamic'))
    o, lse = torch.ops.aotriton_amd.flash_attention_forward(q, k, v, b, 0.0, 3, 5, 2, sm, seed, off)
    torch.library.opcheck(torch.ops.aotriton_amd.flash_attention_backward.default,
                          (do, q, k, v, b, o, lse, 0.0, 3, 5, 2, sm, seed, off, True, -1),
                          test_utils=('test_schema', 'test_faketensor'))


@pytest.mark.gpu
@pytest.mark.parametrize('mode', ['causal', 'mask', 'gqa'])
def test_sdpa_on_ops_matches_torch_math_eager_and_traced(mode):
    from aotriton_amd.torch_ops import scaled_dot_product_attention as sdpa
    from torch.nn.attention import sdpa_kernel, SDPBackend
    Hk = 2 if mode == 'gqa' else 4
    q, k, v, _, do = _inputs(Hq=4, Hk=Hk, D=128, dtype=torch.float16, seed=3)
    kw = dict(is_causal=(mode == 'causal'), enable_gqa=(mode == 'gqa'))
    if mode == 'mask':
        g = torch.Generator(device='cpu').manual_seed(5)
        kw['attn_mask'] = (torch.randn(q.shape[0], 1, q.shape[2], k.shape[2], generator=g) * 0.5).to(q.dtype).to(DEV)
    req = lambda t: t.detach().clone().requires_grad_()

    def run(fn, dtype=None):
        a, b_, c = [req(t if dtype is None else t.to(dtype)) for t in (q, k, v)]
        kw2 = dict(kw)
        if dtype is not None and 'attn_mask' in kw2:
            kw2['attn_mask'] = kw2['attn_mask'].to(dtype)
        o = fn(a, b_, c, **kw2)
        o.backward(do.to(o.dtype))
        return [t.float() for t in (o, a.grad, b_.grad, c.grad)]

    with sdpa_kernel(SDPBackend.MATH):
        ref = run(torch.nn.functional.scaled_dot_product_attention, torch.float32)
        low = run(torch.nn.functional.scaled_dot_product_attention)
    eager = run(sdpa)
    traced = run(torch.compile(sdpa, backend='aot_eager', fullgraph=True))
    for name, fudge, r, l, e, t in zip(('out', 'dq', 'dk', 'dv'), (3.0, 148.0, 48.0, 36.0), ref, low, eager, traced):
        thr = max(1e-5, fudge * (l - r).abs().max().item())      # the reference's tolerance model
        assert (e - r).abs().max().item() <= thr, name
        assert torch.equal(e, t), name + ': traced run differs from eager'


@pytest.mark.gpu
def test_sdpa_dropout_follows_torch_generator():
    from aotriton_amd.torch_ops import scaled_dot_product_attention as sdpa
    q, k, v, _, _ = _inputs(Hk=4, D=64)
    torch.manual_seed(11)
    a = sdpa(q, k, v, dropout_p=0.3)
    b = sdpa(q, k, v, dropout_p=0.3)          # the generator moved on
    torch.manual_seed(11)
    c = sdpa(q, k, v, dropout_p=0.3)
    torch.cuda.synchronize()
    assert torch.equal(a, c) and not torch.equal(a, b)
    # and the mask is the operators' Philox stream at that seed and offset
    from oracle import philox, fa_ref
    B, H, Sq, Sk = q.shape[0], q.shape[1], q.shape[2], k.shape[2]
    keep = torch.from_numpy(philox.dropout_keep_mask(B, H, Sq, Sk, 0.3, 11, 0)).to(DEV)
    ro, _, _ = fa_ref.attn_fwd_ref(q.float(), k.float(), v.float(), None, 1.0 / 8, 0, 0, 0, 0.3, keep)
    assert (a.float() - ro).abs().max().item() < 0.05


@pytest.mark.gpu
@pytest.mark.parametrize('dropout_p', [0.0, 0.2])
def test_forward_and_backward_replay_from_a_hip_graph(dropout_p, recomputing_backward):
    """The operators launch on the caller's stream and, under stream capture, allocate nothing (the
    backward then leaves its dS workspace alone and recomputes), so a forward + backward can be
    captured into a graph.  Every replay (with eager work and synchronisation between replays)
    must reproduce the eager result bit for bit; the eager runs use the recomputing kernels too,
    which is what a capture records."""
    from aotriton_amd import torch_ops  # noqa: F401
    q, k, v, _, do = _inputs(B=2, Hq=4, Hk=2, Sq=300, Sk=300, D=128, seed=9)
    sm = 1.0 / math.sqrt(128)
    seed, off = _u64(0x5EED), _u64(64)
    args = (dropout_p, 3, -2147483647, -2147483647, sm, seed, off)

    def run():
        o, lse = torch.ops.aotriton_amd.flash_attention_forward(q, k, v, None, *args)
        dq, dk, dv, _ = torch.ops.aotriton_amd.flash_attention_backward(do, q, k, v, None, o, lse, *args, False, -1)
        return o, lse, dq, dk, dv

    eager = [t.clone() for t in run()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()                                   # warm-up on the capture stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = run()
    for rep in range(3):
        for t in captured:
            t.fill_(float('nan'))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, e, c in zip(('out', 'lse', 'dq', 'dk', 'dv'), eager, captured):
            assert torch.equal(e, c), f'replay {rep}: {name} differs from the eager run'
        again = run()                           # eager work between replays
        torch.cuda.synchronize()
        assert torch.equal(again[0], eager[0])


def test_router_leaves_cpu_calls_to_torch():
    """The hooks only take CUDA tensors: on the CPU F.scaled_dot_product_attention stays torch's own."""
    import torch.nn.functional as F
    from aotriton_amd import torch_ops
    q = torch.randn(1, 2, 8, 16)
    ref = F.scaled_dot_product_attention(q, q, q, is_causal=True)
    with torch_ops.sdpa_router():
        assert torch.equal(F.scaled_dot_product_attention(q, q, q, is_causal=True), ref)
    torch_ops.install()
    try:
        assert F.scaled_dot_product_attention is not torch_ops._torch_sdpa
        assert torch.equal(F.scaled_dot_product_attention(q, q, q, is_causal=True), ref)
    finally:
        torch_ops.uninstall()
    assert F.scaled_dot_product_attention is torch_ops._torch_sdpa


@pytest.mark.gpu
def test_sdpa_head_dim_that_is_no_multiple_of_8():
    """Any head dim up to 512 is taken (the reference pads it, modules/flash/csrc/attn_fwd.cc:76-82); against
    torch's math backend."""
    import torch.nn.functional as F
    from aotriton_amd import torch_ops
    q, k, v, _, do = _inputs(B=2, Hq=4, Hk=4, Sq=90, Sk=90, D=37)
    req = lambda t: t.detach().clone().requires_grad_()
    a, b, c = req(q), req(k), req(v)
    o = torch_ops.scaled_dot_product_attention(a, b, c, is_causal=True)
    o.backward(do)
    a2, b2, c2 = req(q.float()), req(k.float()), req(v.float())
    with torch.nn.attention.sdpa_kernel(torch.nn.attention.SDPBackend.MATH):
        o2 = F.scaled_dot_product_attention(a2, b2, c2, is_causal=True)
    o2.backward(do.float())
    for x, y in ((o, o2), (a.grad, a2.grad), (b.grad, b2.grad), (c.grad, c2.grad)):
        assert (x.float() - y).abs().max().item() < 6e-2


@pytest.mark.gpu
@pytest.mark.parametrize('hook', ['mode', 'install'])
def test_f_sdpa_routes_to_the_library(hook):
    """F.scaled_dot_product_attention itself, unchanged call sites: under the router the library's
    kernels run (LSE-free check: the result equals the library's own entry point bit for bit and
    torch's math backend within tolerance), gradients included."""
    import torch.nn.functional as F
    from aotriton_amd import torch_ops
    q, k, v, _, do = _inputs(B=2, Hq=4, Hk=2, Sq=200, Sk=200, D=64)
    req = lambda t: t.detach().clone().requires_grad_()

    def run(fn):
        a, b, c = req(q), req(k), req(v)
        o = fn(a, b, c, is_causal=True, enable_gqa=True)
        o.backward(do)
        return o, a.grad, b.grad, c.grad

    own = run(torch_ops.scaled_dot_product_attention)
    if hook == 'mode':
        with torch_ops.sdpa_router():
            routed = run(F.scaled_dot_product_attention)
    else:
        torch_ops.install()
        try:
            routed = run(F.scaled_dot_product_attention)
        finally:
            torch_ops.uninstall()
    for a, b in zip(own, routed):
        assert torch.equal(a, b)
    with torch.nn.attention.sdpa_kernel(torch.nn.attention.SDPBackend.MATH):
        ref = run(lambda a, b, c, **kw: F.scaled_dot_product_attention(a.float(), b.float(), c.float(), **kw))
    for a, b in zip(routed, ref):
        assert (a.float() - b).abs().max().item() < 6e-2


def test_router_only_takes_what_the_operators_accept():
    """unequal head counts without enable_gqa, unequal batch sizes, key and value of different
    lengths and a mask on another device fall through to torch (which raises its own error or
    broadcasts); checked on the predicate, with meta tensors standing in for CUDA ones"""
    from aotriton_amd import torch_ops

    class Fake(torch.Tensor):
        """a tensor that says it is on the GPU: only the predicate looks at it"""
        @property
        def is_cuda(self):
            return True

    mk = lambda *s: torch.empty(*s, dtype=torch.bfloat16, device='meta').as_subclass(Fake)
    q, k, v = mk(2, 8, 16, 64), mk(2, 8, 24, 64), mk(2, 8, 24, 64)
    assert torch_ops._routable(q, k, v, None, 0.0)
    k2, v2 = mk(2, 2, 24, 64), mk(2, 2, 24, 64)
    assert not torch_ops._routable(q, k2, v2, None, 0.0)                    # grouped heads, not asked for
    assert torch_ops._routable(q, k2, v2, None, 0.0, enable_gqa=True)
    assert not torch_ops._routable(q, mk(1, 8, 24, 64), mk(1, 8, 24, 64), None, 0.0)     # batch sizes
    assert not torch_ops._routable(q, k, mk(2, 8, 20, 64), None, 0.0)       # key and value lengths
    assert not torch_ops._routable(q, k, v, torch.zeros(16, 24), 0.0)        # mask elsewhere
