"""The entry point that allocates nothing (`lq_argmax_no_alloc`, csrc/lq_no_alloc.h), called through
ctypes as a caller without this package would, against the arg-max that takes its scratch as an
argument: two calls in a row, the second with a smaller input; ties, bad rows, and the size limit."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu
MAX_ROWS = 1024  # LQ_ARGMAX_NO_ALLOC_MAX_ROWS


@pytest.fixture(scope="module")
def lib():
    from longbow_quarrel_amd import build

    lib = ctypes.CDLL(build.ensure_built())
    lib.lq_last_error.restype = ctypes.c_char_p
    lib.lq_argmax_no_alloc.restype = ctypes.c_int
    lib.lq_argmax_no_alloc.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                       ctypes.c_void_p]
    return lib


def no_alloc(lib, logits, out):
    torch.cuda.set_device(logits.device)
    stream = torch.cuda.current_stream(logits.device).cuda_stream
    return lib.lq_argmax_no_alloc(logits.data_ptr(), logits.stride(0), logits.shape[0], logits.shape[1],
                                  out.data_ptr(), stream)


def with_scratch(logits):
    from longbow_quarrel_amd.kernels.hip import HipKernels

    rows = logits.shape[0]
    out = torch.full((rows,), -5, dtype=torch.int32, device=logits.device)
    scratch = torch.zeros(32 * rows, dtype=torch.int64, device=logits.device)
    HipKernels().argmax(logits, out, scratch)
    return out


def test_two_calls_in_a_row_the_second_smaller_agree_with_the_arg_max_that_takes_its_scratch(lib):
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(3)
    big = (torch.randn((37, 128256), generator=g) * 4).to(dev)
    big[3, 100:105] = 99.0  # a tie: the first maximal index wins
    big[5, 128255] = float("nan")  # a row that cannot be sampled from
    big[6, 0] = float("inf")
    small = (torch.randn((4, 331), generator=g) * 4).to(dev)
    small[2, 330] = 50.0
    out_big = torch.full((37,), -5, dtype=torch.int32, device=dev)
    out_small = torch.full((4,), -5, dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    # what the driver itself has handed out on this GPU, to anyone: an allocation that goes past torch's
    # allocator (a hipMalloc inside the entry point) shows here and not in torch's own count
    free_before, _ = torch.cuda.mem_get_info(dev)
    torch_before = torch.cuda.memory_allocated(dev)
    assert no_alloc(lib, big, out_big) == 0, lib.lq_last_error()
    assert no_alloc(lib, small, out_small) == 0, lib.lq_last_error()  # finds the first call's leftovers in the scratch
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before and torch.cuda.memory_allocated(dev) == torch_before
    want_big, want_small = with_scratch(big), with_scratch(small)
    assert torch.equal(out_big, want_big) and torch.equal(out_small, want_small)
    assert out_big[3].item() == 100 and out_big[5].item() == -1 and out_big[6].item() == -1
    assert out_small[2].item() == 330
    plain = big.cpu().clone()
    rows_ok = [r for r in range(37) if r not in (5, 6)]
    assert out_big.cpu()[rows_ok].tolist() == plain[rows_ok].argmax(dim=-1).tolist()
    # a view whose rows lie further apart than they are long, and the largest batch the array holds
    wide = (torch.randn((MAX_ROWS, 700), generator=g)).to(dev)
    view = wide[:, :513]
    out = torch.full((MAX_ROWS,), -5, dtype=torch.int32, device=dev)
    assert no_alloc(lib, view, out) == 0, lib.lq_last_error()
    assert out.cpu().tolist() == view.cpu().argmax(dim=-1).tolist()
    assert no_alloc(lib, small, out_small) == 0 and torch.equal(out_small, want_small)


def test_sizes_beyond_the_fixed_array_are_refused_with_a_clear_error(lib):
    dev = torch.device("cuda:0")
    logits = torch.zeros((MAX_ROWS + 1, 8), device=dev)
    out = torch.full((MAX_ROWS + 1,), -5, dtype=torch.int32, device=dev)
    assert no_alloc(lib, logits, out) != 0
    message = lib.lq_last_error().decode()
    assert str(MAX_ROWS) in message and "rows" in message
    torch.cuda.synchronize()
    assert out.eq(-5).all()  # nothing ran
    assert lib.lq_argmax_no_alloc(None, 8, 1, 8, out.data_ptr(), None) != 0
    assert lib.lq_argmax_no_alloc(logits.data_ptr(), 4, 1, 8, out.data_ptr(), None) != 0  # rows closer than they are long
