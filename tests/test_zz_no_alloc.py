"""The sampler's entry point that allocates nothing, called through ctypes like a foreign caller would."""
import ctypes
from ctypes import c_float, c_int, c_int64, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def load(name):
    from vosti_amd.kernels import build
    lib = ctypes.CDLL(str(build.ensure(name)))
    lib.vk_last_error.restype = ctypes.c_char_p
    lib.vk_sample.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_void_p]
    lib.vk_sample.restype = c_int
    lib.vk_sample_static.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_void_p]
    lib.vk_sample_static.restype = c_int
    lib.vk_sample_scratch_words.argtypes = [c_int]
    lib.vk_sample_scratch_words.restype = c_int
    lib.vk_sample_static_max_rows.restype = c_int
    return lib


@pytest.mark.parametrize("name,dtype", [("bf16", torch.bfloat16), ("f32", torch.float32)])
def test_sample_static_equals_sample_on_two_calls_in_a_row(name, dtype):
    """Two calls in a row, the second with a smaller input (fewer rows, a shorter vocabulary), so that
    what the first call left in the library's scratch lies beside and behind what the second one uses:
    both give the tokens of the entry point whose scratch the caller brings."""
    lib = load(name)
    stream = c_void_p(torch.cuda.current_stream().cuda_stream)
    g = torch.Generator().manual_seed(3)
    for R, V in ((40, 5003), (3, 1000)):
        logits = (torch.randn(R, V, generator=g) * 3).to(dtype).cuda()
        temps = torch.tensor([0.0 if r % 3 == 0 else 0.7 + 0.1 * r for r in range(R)], dtype=torch.float32).cuda()
        unis = torch.rand(R, generator=g).cuda()
        want = torch.full((R,), -1, dtype=torch.int32, device="cuda")
        got = torch.full((R,), -2, dtype=torch.int32, device="cuda")
        scratch = torch.empty(lib.vk_sample_scratch_words(R), dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        assert lib.vk_sample(want.data_ptr(), logits.data_ptr(), temps.data_ptr(), unis.data_ptr(), scratch.data_ptr(),
                             R, V, V, stream) == 0, lib.vk_last_error()
        # One call first (the library asks for its array's address once per GPU, and the runtime loads the kernels),
        # then the device's own count of free memory must not move over a call: the allocator of torch would not see
        # a hipMalloc inside the library, the device does.
        assert lib.vk_sample_static(got.data_ptr(), logits.data_ptr(), temps.data_ptr(), unis.data_ptr(), R, V, V,
                                    stream) == 0, lib.vk_last_error()
        torch.cuda.synchronize()
        got.fill_(-2)
        before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        assert lib.vk_sample_static(got.data_ptr(), logits.data_ptr(), temps.data_ptr(), unis.data_ptr(), R, V, V,
                                    stream) == 0, lib.vk_last_error()
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == free_before
        assert torch.equal(got, want) and int(got.min()) >= 0 and int(got.max()) < V
        # Greedy for every row (no temperatures).
        assert lib.vk_sample(want.data_ptr(), logits.data_ptr(), None, None, scratch.data_ptr(), R, V, V, stream) == 0
        assert lib.vk_sample_static(got.data_ptr(), logits.data_ptr(), None, None, R, V, V, stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        row_max = logits.float().max(dim=1).values
        assert torch.equal(logits.float()[torch.arange(R), got.long()], row_max)
    # More rows than the library's scratch holds: a clear error, nothing launched.
    too_many = lib.vk_sample_static_max_rows() + 1
    assert lib.vk_sample_static(got.data_ptr(), logits.data_ptr(), None, None, too_many, V, V, stream) != 0
    assert b"more than" in lib.vk_last_error()
