"""t2fw_cast through the C ABI: several arrays of different lengths converted in one launch, against torch's
own conversion (round to nearest even in both), bit for bit; lengths around the eight-element pieces a lane
converts, an empty array in the list, and the argument checks."""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("narrow", [torch.float16, torch.bfloat16])
def test_cast_matches_torch_both_ways(narrow):
    from t2fw_amd import _lib
    g = torch.Generator().manual_seed(3)
    sizes = [1, 7, 8, 9, 0, 4096 + 5, 96 * 1024 * 64, 33]
    wide = [(torch.randn(n, generator=g) * 10 ** float(torch.randint(-6, 5, (1,), generator=g))).cuda() for n in sizes]
    wide[1][:3] = torch.tensor([float("inf"), -0.0, 65520.0])          # overflow of float16, signed zero
    out = [torch.empty(n, dtype=narrow, device="cuda") for n in sizes]
    st = _lib.current_stream_handle(out[0].device)
    _lib.cast_tensors(wide, out, st)
    torch.cuda.synchronize()
    for w, o in zip(wide, out):
        assert torch.equal(o, w.to(narrow))
    back = [torch.empty(n, dtype=torch.float32, device="cuda") for n in sizes]
    _lib.cast_tensors(out, back, st)
    torch.cuda.synchronize()
    for o, b in zip(out, back):
        assert torch.equal(b, o.float())


def test_cast_refuses_what_it_cannot_do():
    from t2fw_amd import _lib
    lib = _lib.load()
    a = torch.zeros(16, dtype=torch.float32, device="cuda")
    b = torch.zeros(16, dtype=torch.float32, device="cuda")
    sp, dp, cnt = (ctypes.c_void_p * 1)(_lib.ptr(a)), (ctypes.c_void_p * 1)(_lib.ptr(b)), (ctypes.c_int64 * 1)(16)
    f32, f16 = _lib.DTYPE_CODE[torch.float32], _lib.DTYPE_CODE[torch.float16]
    assert lib.t2fw_cast(sp, dp, cnt, 1, f32, f32, None) != 0           # not a conversion it has
    assert lib.t2fw_cast(sp, dp, cnt, 9, f32, f16, None) != 0           # too many arrays
    odd = (ctypes.c_void_p * 1)(a.data_ptr() + 4)
    assert lib.t2fw_cast(odd, dp, cnt, 1, f32, f16, None) != 0          # misaligned
    neg = (ctypes.c_int64 * 1)(-1)
    assert lib.t2fw_cast(sp, dp, neg, 1, f32, f16, None) != 0
