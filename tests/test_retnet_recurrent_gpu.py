"""RetNet recurrent form on the GPU, through the library's C entry points and the PyTorch wrapper, against
the oracle (oracle/ref_op.py closed form for small cases, oracle/brute.c sequential recurrence for larger
ones).  Tolerance: |err| <= 2e-5 * max|ref| -- fp32 arithmetic in a different association order than the
oracle's fp64 (the reference's own block scan reassociates too, reference recurrent.h:110-131)."""
import ctypes

import numpy as np
import pytest
import torch

import attention_autotuner_amd as aat
from attention_autotuner_amd.autotuner import codegen, library
from attention_autotuner_amd.autotuner.configs import RetRecurrentConfig
from attention_autotuner_amd.ops import retnet_recurrent
from oracle import brute, ref_op

pytestmark = pytest.mark.gpu
ARCH = aat.MI355X()
RTOL_OF_MAX = 2e-5


def _inputs(seed, b, h, kdim, vdim, seqlen, lo=0.0, hi=1.0):
    g = torch.Generator().manual_seed(seed)
    q = torch.rand(b, h, kdim, seqlen, generator=g) * 2 - 1
    k = torch.rand(b, h, kdim, seqlen, generator=g) * 2 - 1
    v = torch.rand(b, h, vdim, seqlen, generator=g) * 2 - 1
    decay = torch.rand(h, seqlen, generator=g) * (hi - lo) + lo
    return q, k, v, decay


def _close(got, ref):
    err = (got.cpu().double() - ref.double()).abs().max().item()
    scale = ref.abs().max().item()
    assert err <= RTOL_OF_MAX * scale, (err, scale)


# value slices of 64 and 128 dims, 64 and 128 key dims, few and many blocks (both launch shapes), ragged
# chunk counts (odd number of 32-position chunks), a single chunk, more than 128 key dims (passes that add)
@pytest.mark.parametrize("b,h,kdim,vdim,seqlen", [(1, 2, 128, 128, 256), (1, 3, 64, 256, 96), (2, 1, 128, 64, 32),
                                                   (1, 2, 64, 64, 160), (2, 2, 64, 192, 64), (1, 2, 256, 64, 96),
                                                   (1, 1, 192, 128, 64)])
def test_matches_the_closed_form(b, h, kdim, vdim, seqlen):
    q, k, v, decay = _inputs(0, b, h, kdim, vdim, seqlen, 0.5, 1.0)
    out = aat.retnet_recurrent_fwd(q.cuda(), k.cuda(), v.cuda(), decay.cuda())
    _close(out, ref_op.retnet_recurrent_ref(q, k, v, decay))


def test_zero_negative_and_vanishing_decays():
    """Zeros cut the history, negative values flip signs, long runs of small decays drive the carried
    product out of range (the state is then rescaled): all as in the recurrence."""
    q, k, v, decay = _inputs(1, 1, 4, 64, 64, 256, -1.0, 1.0)
    decay[0, 5] = 0.0
    decay[0, 64] = 0.0
    decay[1] = 0.05                      # 0.05^32 per chunk: leaves the range at once
    decay[2] = 1.0
    decay[3, :128] = 1.5                 # growth: leaves the range upwards after three chunks
    out = aat.retnet_recurrent_fwd(q.cuda(), k.cuda(), v.cuda(), decay.cuda())
    ref = torch.from_numpy(brute.retnet_recurrent(q.numpy(), k.numpy(), v.numpy(), decay.numpy()))
    for head in range(4):
        _close(out[:, head], ref[:, head])


def test_many_blocks_take_the_wide_value_slice_and_agree_with_the_narrow_one():
    """192 or more (batch, head, 128-dim slice) blocks launch the 128-wide kernel, fewer the 64-wide one."""
    q, k, v, decay = _inputs(2, 24, 8, 64, 128, 64, 0.9, 1.0)
    out = aat.retnet_recurrent_fwd(q.cuda(), k.cuda(), v.cuda(), decay.cuda())
    ref = torch.from_numpy(brute.retnet_recurrent(q.numpy(), k.numpy(), v.numpy(), decay.numpy()))
    _close(out, ref)
    narrow = aat.retnet_recurrent_fwd(q[:2].cuda(), k[:2].cuda(), v[:2].cuda(), decay.cuda())
    _close(narrow, ref[:2])


def test_block_kdim_limits_the_contraction():
    q, k, v, decay = _inputs(3, 1, 2, 128, 64, 128, 0.8, 1.0)
    out = aat.retnet_recurrent_fwd(q.cuda(), k.cuda(), v.cuda(), decay.cuda(), block_kdim=64)
    _close(out, ref_op.retnet_recurrent_ref(q, k, v, decay, block_kdim=64))


def test_reference_signature_entry_point_and_error_codes():
    """retnet_recurrent_fwd (reference recurrent.h:427: void, null stream, no workspace argument) gives the
    same result as the extended entry point; unsupported shapes and a short workspace are refused."""
    lib = library.load_recurrent(codegen.compile_config(RetRecurrentConfig(), ARCH))
    b, h, kdim, vdim, seqlen = 1, 2, 64, 64, 128
    q, k, v, decay = [t.cuda() for t in _inputs(4, b, h, kdim, vdim, seqlen, 0.7, 1.0)]
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    out_ref_sig = torch.zeros_like(v)
    torch.cuda.synchronize()
    lib.retnet_recurrent_fwd(ptr(q), ptr(k), ptr(v), ptr(decay), ptr(out_ref_sig), b, h, kdim, vdim, seqlen, kdim)
    torch.cuda.synchronize()
    out_ex = aat.retnet_recurrent_fwd(q, k, v, decay)
    assert torch.equal(out_ref_sig, out_ex)
    # a second, larger call: still within what the library's static array holds, so nothing is allocated
    q2, k2, v2, decay2 = [t.cuda() for t in _inputs(5, 1, 4, 64, 64, 256, 0.7, 1.0)]
    out2 = torch.zeros_like(v2)
    want2 = aat.retnet_recurrent_fwd(q2, k2, v2, decay2)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    lib.retnet_recurrent_fwd(ptr(q2), ptr(k2), ptr(v2), ptr(decay2), ptr(out2), 1, 4, 64, 64, 256, 64)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(out2, want2)
    # more than 128 key dims per pass need a second output-sized buffer: the entry point allocates one and keeps it
    q3, k3, v3, decay3 = [t.cuda() for t in _inputs(6, 1, 2, 256, 64, 128, 0.7, 1.0)]
    out3 = torch.zeros_like(v3)
    lib.retnet_recurrent_fwd(ptr(q3), ptr(k3), ptr(v3), ptr(decay3), ptr(out3), 1, 2, 256, 64, 128, 256)
    torch.cuda.synchronize()
    assert torch.equal(out3, aat.retnet_recurrent_fwd(q3, k3, v3, decay3, block_kdim=256))

    need = lib.workspace_size(b, h, seqlen, seqlen)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out = torch.empty_like(v)
    args = [ptr(q), ptr(k), ptr(v), ptr(decay), ptr(out)]
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    call = lambda dims, w, nbytes: lib.retnet_recurrent_fwd_ex(*args, *dims, w, ctypes.c_size_t(nbytes), stream)
    assert call((b, h, kdim, vdim, seqlen, kdim), ptr(ws), need) == 0
    assert call((b, h, kdim, vdim, seqlen, kdim), ptr(ws), need - 1) == -3
    assert call((b, h, kdim, vdim, seqlen, kdim), ctypes.c_void_p(0), 0) == -3
    assert call((b, h, kdim, vdim, 100, kdim), ptr(ws), need) == -2         # l not a multiple of 32
    assert call((b, h, kdim, vdim, seqlen, 32), ptr(ws), need) == -2        # block_kdim
    assert call((b, h, kdim, vdim, seqlen, 128), ptr(ws), need) == -2       # block_kdim > kdim
    assert call((b, h, kdim, 32, seqlen, kdim), ptr(ws), need) == -2        # vdim
    assert call((0, h, kdim, vdim, seqlen, kdim), ptr(ws), need) == -2
    torch.cuda.synchronize()
    with pytest.raises(RuntimeError, match="unsupported shape"):
        aat.retnet_recurrent_fwd(q[..., :100].contiguous(), k[..., :100].contiguous(), v[..., :100].contiguous(),
                                 decay[:, :100].contiguous())


def test_deterministic_and_profile_entry():
    q, k, v, decay = [t.cuda() for t in _inputs(6, 2, 2, 128, 128, 192, 0.9, 1.0)]
    a = aat.retnet_recurrent_fwd(q, k, v, decay)
    b = aat.retnet_recurrent_fwd(q, k, v, decay)
    assert torch.equal(a, b)
    lib = library.load_recurrent(codegen.compile_config(RetRecurrentConfig(), ARCH))
    ws = torch.empty(retnet_recurrent.workspace_size(2, 192), dtype=torch.uint8, device="cuda")
    out = torch.empty_like(v)
    ms = lib.retnet_recurrent_profile(*[ctypes.c_void_p(t.data_ptr()) for t in (q, k, v, decay, out)], 2, 2, 128, 128, 192, 128,
                                      ctypes.c_void_p(ws.data_ptr()), ctypes.c_size_t(ws.numel()),
                                      ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert 0 < ms < 50
    assert torch.equal(out, a)


def test_full_size_through_size_independent_properties():
    """Benchmark shape (8, 32, 128, 128, 2048): too large for the oracle, so linearity in v, a decay-zero
    closed form and one (batch, head) slice against the sequential recurrence."""
    b, h, kdim, vdim, seqlen = 8, 32, 128, 128, 2048
    g = torch.Generator(device="cuda").manual_seed(7)
    q = torch.rand(b, h, kdim, seqlen, generator=g, device="cuda") * 2 - 1
    k = torch.rand(b, h, kdim, seqlen, generator=g, device="cuda") * 2 - 1
    v = torch.rand(b, h, vdim, seqlen, generator=g, device="cuda") * 2 - 1
    v2 = torch.rand(b, h, vdim, seqlen, generator=g, device="cuda") * 2 - 1
    gamma = 1.0 - 2.0 ** (-5.0 - torch.arange(h, dtype=torch.float32, device="cuda"))
    decay = gamma.unsqueeze(1).expand(h, seqlen).contiguous()
    o1 = aat.retnet_recurrent_fwd(q, k, v, decay)
    o2 = aat.retnet_recurrent_fwd(q, k, v2, decay)
    o12 = aat.retnet_recurrent_fwd(q, k, v + v2, decay)
    scale = o12.abs().max().item()
    assert (o12 - (o1 + o2)).abs().max().item() <= 1e-5 * scale
    o0 = aat.retnet_recurrent_fwd(q, k, v, torch.zeros_like(decay))
    expect0 = (q * k).sum(dim=2, keepdim=True) * v
    assert (o0 - expect0).abs().max().item() <= 1e-5 * expect0.abs().max().item()
    sl = (slice(3, 4), slice(17, 18))
    ref = brute.retnet_recurrent(q[sl].cpu().numpy(), k[sl].cpu().numpy(), v[sl].cpu().numpy(), decay[17:18].cpu().numpy())
    _close(o1[sl], torch.from_numpy(ref))


def test_long_sequence_and_side_stream():
    """128 chunks per head (the carried product leaves its range several times), launched on a side stream."""
    q, k, v, decay = _inputs(8, 1, 2, 64, 64, 4096, 0.6, 1.0)
    side = torch.cuda.Stream()
    qc, kc, vc, dc = q.cuda(), k.cuda(), v.cuda(), decay.cuda()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        out = aat.retnet_recurrent_fwd(qc, kc, vc, dc)
    side.synchronize()
    ref = torch.from_numpy(brute.retnet_recurrent(q.numpy(), k.numpy(), v.numpy(), decay.numpy()))
    _close(out, ref)


def test_graph_capture_replays():
    """The extended entry point allocates nothing and launches two kernels: a captured graph of it replays
    correctly with eager work and synchronisations in between, and follows new inputs written in place."""
    b, h, kdim, vdim, seqlen = 2, 2, 128, 64, 256
    q, k, v, decay = [t.cuda() for t in _inputs(9, b, h, kdim, vdim, seqlen, 0.8, 1.0)]
    out = torch.empty_like(v)
    ws = torch.empty(retnet_recurrent.workspace_size(h, seqlen, batch=b, kdim=kdim, vdim=vdim), dtype=torch.uint8, device="cuda")
    eager = aat.retnet_recurrent_fwd(q, k, v, decay)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        aat.retnet_recurrent_fwd(q, k, v, decay, out=out, workspace=ws)          # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        aat.retnet_recurrent_fwd(q, k, v, decay, out=out, workspace=ws)
    for rep in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), rep
        _ = (q * 2).sum().item()                                              # eager work between replays
    q2, k2, v2, decay2 = [t.cuda() for t in _inputs(10, b, h, kdim, vdim, seqlen, 0.8, 1.0)]
    q.copy_(q2), k.copy_(k2), v.copy_(v2), decay.copy_(decay2)
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, aat.retnet_recurrent_fwd(q2, k2, v2, decay2))
