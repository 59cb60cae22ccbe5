"""The entry point that allocates nothing (retnet_recurrent_fwd_noalloc) against the entry point it is a
variant of (retnet_recurrent_fwd_ex, which takes its workspace from the caller), through the C ABI.

Both run the same two kernels on the same inputs and differ only in where the decay factors live, so their
outputs are compared bit for bit.  Two calls in a row share the library's static device array; the second
one is smaller, so it finds the first call's records still in place behind and under its own."""
import ctypes

import pytest
import torch

import attention_autotuner_amd as aat
from attention_autotuner_amd.autotuner import codegen, library
from attention_autotuner_amd.autotuner.configs import RetRecurrentConfig

pytestmark = pytest.mark.gpu
ARCH = aat.MI355X()
ERR_SHAPE, ERR_LIMIT = -2, -4
MAX_RECORDS = 3072


def _lib():
    lib = library.load_recurrent(codegen.compile_config(RetRecurrentConfig(), ARCH))
    # the first call on a device looks the static array up (and makes the runtime load the kernels): done here,
    # so that the calls under test find everything in place
    q, k, v, decay = _inputs(99, 1, 1, 64, 64, 32)
    out = torch.empty(1, 1, 64, 32, device="cuda")
    assert lib.retnet_recurrent_fwd_noalloc(*_ptrs(q, k, v, decay, out), 1, 1, 64, 64, 32, 64, ctypes.c_void_p(0)) == 0
    torch.cuda.synchronize()
    return lib


def _inputs(seed, b, h, kdim, vdim, seqlen):
    g = torch.Generator().manual_seed(seed)
    q, k = (torch.rand(b, h, kdim, seqlen, generator=g) * 2 - 1 for _ in range(2))
    v = torch.rand(b, h, vdim, seqlen, generator=g) * 2 - 1
    decay = torch.rand(h, seqlen, generator=g) * 0.5 + 0.5
    return [t.cuda() for t in (q, k, v, decay)]


def _ptrs(*tensors):
    return [ctypes.c_void_p(t.data_ptr()) for t in tensors]


def _both(lib, q, k, v, decay, block_kdim):
    b, h, kdim, seqlen = q.shape
    vdim = v.shape[2]
    dims = (b, h, kdim, vdim, seqlen, block_kdim)
    need = lib.retnet_recurrent_workspace_size(*dims)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    want = torch.full((b, h, vdim, seqlen), float("nan"), device="cuda")
    got = torch.full_like(want, float("nan"))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.retnet_recurrent_fwd_ex(*_ptrs(q, k, v, decay, want), *dims, ctypes.c_void_p(ws.data_ptr()), need, stream) == 0
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()          # the driver's view: an allocation by the library would show here
    assert lib.retnet_recurrent_fwd_noalloc(*_ptrs(q, k, v, decay, got), *dims, stream) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after >= free_before, (free_before, free_after)
    return got, want


def test_two_calls_in_a_row_match_the_workspace_entry_point_bit_for_bit():
    lib = _lib()
    # first call: 4 heads x 12 chunks of factors; second: 2 heads x 3 chunks, over the first call's leftovers
    for seed, (b, h, kdim, vdim, seqlen, bk) in enumerate([(2, 4, 128, 128, 384, 128), (1, 2, 64, 64, 96, 64)]):
        q, k, v, decay = _inputs(seed, b, h, kdim, vdim, seqlen)
        got, want = _both(lib, q, k, v, decay, bk)
        assert torch.isfinite(want).all()
        assert torch.equal(got, want), (seed, (got - want).abs().max().item())


def test_limits_are_refused_before_anything_is_launched():
    lib = _lib()
    q, k, v, decay = _inputs(7, 1, 1, 256, 64, 64)
    out = torch.zeros(1, 1, 64, 64, device="cuda")
    null = ctypes.c_void_p(0)
    assert lib.retnet_recurrent_fwd_noalloc(*_ptrs(q, k, v, decay, out), 1, 1, 256, 64, 64, 256, null) == ERR_LIMIT      # two passes need a second buffer
    assert lib.retnet_recurrent_fwd_noalloc(*_ptrs(q, k, v, decay, out), 1, 1, 256, 64, 48, 128, null) == ERR_SHAPE      # l % 32
    # one record too many: heads * (l / 32) = 3073 (nothing is read: the check comes first)
    assert lib.retnet_recurrent_fwd_noalloc(*_ptrs(q, k, v, decay, out), 1, MAX_RECORDS + 1, 64, 64, 32, 64, null) == ERR_LIMIT
    torch.cuda.synchronize()
    assert out.abs().max().item() == 0


def test_capacity_is_usable_to_the_last_record():
    """heads * chunks == the maximum: the last record of the array is written and read."""
    lib = _lib()
    q, k, v, decay = _inputs(9, 1, 96, 64, 64, 1024)          # 96 heads x 32 chunks = 3072 records
    got, want = _both(lib, q, k, v, decay, 64)
    assert torch.equal(got, want)
