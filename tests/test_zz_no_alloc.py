"""`akv_linear_packed_static`: the product of up to 64 rows whose repacked activations live in static device memory
of the library, for callers that cannot allocate.  Called through ctypes, as such a caller would, and held to the
existing entry points (`akv_pack_rows` into a buffer of the caller's, then `akv_linear_packed`) bit for bit - on two
calls in a row, the second with a smaller input, so that what the first call left in the static memory must not
reach the second's result."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _pointer(tensor):
    return ctypes.c_void_p(tensor.data_ptr())


def test_the_product_without_allocation_equals_the_one_with_a_buffer():
    from ampere_kv_engine_amd.csrc.build import ensure_built
    from ampere_kv_engine_amd.kernels.hip import PackedWeight
    lib = ctypes.CDLL(ensure_built())
    for name in ("akv_pack_rows", "akv_linear_packed", "akv_linear_packed_static"):
        getattr(lib, name).restype = ctypes.c_int
    torch.cuda.set_device(0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    generator = torch.Generator().manual_seed(5)
    for rows, outs, k in ((61, 328, 1032), (19, 40, 72)):          # the second call is the smaller one
        x = (torch.randn(rows, k, generator=generator) * 0.5).to(torch.bfloat16).cuda()
        weight = PackedWeight((torch.randn(outs, k, generator=generator) * 0.05).to(torch.bfloat16).cuda())
        for code, dtype in ((1, torch.bfloat16), (0, torch.float32)):
            staged = torch.full(((rows + 15) // 16 * 16 * k,), float("nan"), dtype=torch.bfloat16, device="cuda")
            want = torch.full((rows, outs), float("nan"), dtype=dtype, device="cuda")
            got = torch.full((rows, outs), float("nan"), dtype=dtype, device="cuda")
            assert lib.akv_pack_rows(_pointer(x), _pointer(staged), rows, k, stream) == 0
            assert lib.akv_linear_packed(_pointer(staged), _pointer(weight.data), _pointer(want), code, rows, outs, k,
                                         weight.n_tiles, weight.k_tiles, 1, None, stream) == 0
            torch.cuda.synchronize()
            before = torch.cuda.memory_stats()["allocation.all.allocated"]
            assert lib.akv_linear_packed_static(_pointer(x), _pointer(weight.data), _pointer(got), code, rows, outs, k,
                                                weight.n_tiles, weight.k_tiles, stream) == 0
            torch.cuda.synchronize()
            assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
            assert not torch.isnan(want.float()).any()
            assert torch.equal(got, want), f"{rows} x {k} -> {outs} ({dtype}): the two entry points differ"
            reference = x.float() @ weight.unpack().float().T
            torch.testing.assert_close(got.float(), reference, rtol=1.6e-2, atol=1e-3)
    # sizes beyond the static memory are refused, by the entry point itself and by its wrapper with a message
    big = PackedWeight(torch.zeros(16, 40000, dtype=torch.bfloat16, device="cuda"))
    x = torch.zeros(64, 40000, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(64, 16, dtype=torch.bfloat16, device="cuda")
    assert lib.akv_linear_packed_static(_pointer(x), _pointer(big.data), _pointer(out), 1, 64, 16, 40000, big.n_tiles,
                                        big.k_tiles, stream) == -3
    assert lib.akv_linear_packed_static(_pointer(x), _pointer(big.data), _pointer(out), 1, 65, 16, 40000, big.n_tiles,
                                        big.k_tiles, stream) == -3
    from ampere_kv_engine_amd.kernels.hip import HipKernels, KernelError
    with pytest.raises(KernelError, match="do not fit the static memory"):
        HipKernels("cuda:0").linear_without_allocation(x, big, out)
    small = PackedWeight((torch.randn(48, 64, generator=generator) * 0.05).to(torch.bfloat16).cuda())
    x = torch.randn(5, 64, generator=generator).to(torch.bfloat16).cuda()
    out = torch.empty(5, 48, dtype=torch.bfloat16, device="cuda")
    HipKernels("cuda:0").linear_without_allocation(x, small, out)
    torch.testing.assert_close(out.float(), x.float() @ small.unpack().float().T, rtol=1.6e-2, atol=1e-3)
