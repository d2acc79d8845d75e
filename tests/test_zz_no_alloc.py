"""xmc_fp8_forward_static, the entry point that takes no workspace (its operand images of X live in a static device array
of the library), against xmc_fp8_forward on the same inputs: bit-identical logits, on two calls in a row of which the
second is smaller, so that what the first call left in the array must not show in the second.  Both are called
through the C ABI with buffers allocated beforehand; the static call itself allocates nothing."""
import ctypes

import numpy as np
import pytest

import helpers as H
from elmo_amd import _lib, ops, synth

pytestmark = pytest.mark.gpu


def _forward_pair(gpu, nc, rows, batch, num_labels, seed):
    import torch
    lib = _lib.load()
    case = H.make_case(nc, rows, 16, seed, std=0.3)
    chunks, _, _ = H.to_device_case(case, gpu)
    x = torch.from_numpy(synth.make_x(batch, 768, seed + 1)).to(gpu).to(torch.bfloat16).contiguous()
    arr, _ = ops._chunk_array(chunks)
    stride = nc * rows
    ws = ops.alloc_workspace(nc, rows, gpu)
    want = torch.full((batch, stride), 7.0, dtype=torch.bfloat16, device=gpu)
    got = torch.full((batch, stride), -7.0, dtype=torch.bfloat16, device=gpu)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    # the first call on a device looks the static array's address up (and the runtime may load the code object): it is
    # made once before anything is measured
    st = lib.xmc_fp8_forward_static(arr, nc, rows, x.data_ptr(), batch, 768, 1.0, 1.0, got.data_ptr(), stride, num_labels, stream)
    assert st == 0, lib.xmc_error_string(st)
    torch.cuda.synchronize()
    got.fill_(-7.0)
    torch.cuda.synchronize()
    # torch's counter sees only its own caching allocator; the free device memory the driver reports would also show a
    # hipMalloc made by the library itself
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]
    st = lib.xmc_fp8_forward_static(arr, nc, rows, x.data_ptr(), batch, 768, 1.0, 1.0, got.data_ptr(), stride, num_labels, stream)
    assert st == 0, lib.xmc_error_string(st)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    st = lib.xmc_fp8_forward(arr, nc, rows, x.data_ptr(), batch, 768, 1.0, 1.0, want.data_ptr(), stride, num_labels,
                             ws.data_ptr(), ws.numel(), stream)
    assert st == 0, lib.xmc_error_string(st)
    torch.cuda.synchronize()
    g = got[:, :num_labels].view(torch.int16).cpu().numpy()
    w = want[:, :num_labels].view(torch.int16).cpu().numpy()
    assert np.array_equal(g, w)
    assert np.abs(want[:, :num_labels].float().cpu().numpy()).max() > 0.1      # real logits, not a cleared buffer
    # columns past num_labels are written by neither
    if num_labels < stride:
        assert bool((got[:, num_labels:] == -7.0).all()) and bool((want[:, num_labels:] == 7.0).all())


def test_static_forward_matches_workspace_forward_twice(gpu):
    _forward_pair(gpu, 3, 2048, 128, 6000, 91)     # the largest batch the array holds
    _forward_pair(gpu, 2, 208, 32, 400, 93)        # then a smaller one: fewer batch rows, fewer labels


def test_static_forward_rejects_what_the_array_cannot_hold(gpu):
    import torch
    lib = _lib.load()
    case = H.make_case(1, 64, 16, 95)
    chunks, _, _ = H.to_device_case(case, gpu)
    arr, _ = ops._chunk_array(chunks)
    x = torch.zeros(144, 768, dtype=torch.bfloat16, device=gpu)
    out = torch.zeros(144, 64, dtype=torch.bfloat16, device=gpu)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert lib.xmc_fp8_forward_static(arr, 1, 64, x.data_ptr(), 144, 768, 1.0, 1.0, out.data_ptr(), 64, 64, stream) == -2
    assert lib.xmc_fp8_forward_static(arr, 1, 64, x.data_ptr(), 16, 1024, 1.0, 1.0, out.data_ptr(), 64, 64, stream) == -2
    assert b"128" in lib.xmc_error_string(-2)
