"""Host-side logic that needs no device: the autograd wrapper's argument checks (the asserts of
t2fw/functional_lfw.py:42-49,71-72 of the reference), the cached shape queries, the workspace layout
arithmetic of the C ABI and the choice of the backward path from the forward's hints."""
import ctypes

import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def lib():
    from t2fw_amd import _lib
    return _lib.load()


def _inputs(B=2, T=3, D=4, K=5, dtype=torch.float32):
    x, f = torch.randn(B, T, D, dtype=dtype), torch.rand(B, T, D, dtype=dtype)
    q, k, fk = torch.randn(B, T, K, dtype=dtype), torch.randn(B, T, K, dtype=dtype), torch.rand(B, T, K, dtype=dtype)
    return [x, f, q, k, fk, torch.randn(B, D, K, dtype=dtype)]


@pytest.mark.parametrize("which,bad", [
    (1, lambda t: t[:, :2]),                        # forget.shape != value.shape
    (3, lambda t: t[:, :, :4]),                     # key.shape != query.shape
    (4, lambda t: t[:1]),                           # f_key.shape != query.shape
    (1, lambda t: t.double()), (2, lambda t: t.half()), (4, lambda t: t.double()),
    (5, lambda t: t.double()), (3, lambda t: t.half()),          # dtypes must equal value.dtype
])
def test_wrapper_asserts_like_the_reference(which, bad):
    from t2fw.functional_lfw import LFWFunction
    ins = _inputs()
    ins[which] = bad(ins[which])
    with pytest.raises(AssertionError):
        LFWFunction.apply(*ins)


def test_wrapper_checks_device_and_contiguity_after_the_asserts():
    """CHECK_INPUT of t2fw/csrc/lfw.cpp:24-26: a RuntimeError, raised once the shapes and dtypes are fine"""
    from t2fw.functional_lfw import LFWFunction
    from t2fw.functional_dfw import DFWFunction
    with pytest.raises(RuntimeError, match="CUDA"):
        LFWFunction.apply(*_inputs())
    q, k, v, s = torch.randn(2, 3, 5), torch.randn(2, 3, 5), torch.randn(2, 3, 4), torch.randn(2, 4, 5)
    with pytest.raises(RuntimeError, match="CUDA"):
        DFWFunction.apply(q, k, v, s)


def test_shape_queries_are_cached_per_shape(lib):
    from t2fw_amd import functional_lfw as F
    F._sizes.cache_clear()
    a = F._sizes(96, 1024, 64, 64, 64, 1, 0)
    b = F._sizes(96, 1024, 64, 64, 64, 1, 0)
    assert a is b and F._sizes.cache_info().hits == 1 and F._sizes.cache_info().misses == 1
    nc, fwd_bytes, both_bytes, regions = a
    assert nc == 16 and fwd_bytes == lib.t2fw_lfw_forward_workspace_bytes(96, 1024, 64, 64, 64, 1, 0)
    assert both_bytes == lib.t2fw_lfw_workspace_bytes(96, 1024, 64, 64, 64, 1, 0) and len(regions) == 6


def _regions(lib, *a):
    r = (ctypes.c_int64 * 6)()
    assert lib.t2fw_lfw_flag_regions(*a, r) == 0
    return list(r)


@pytest.mark.parametrize("B", [1, 7, 8, 96, 100, 300])
def test_flag_regions_lie_inside_the_workspace_and_do_not_overlap(lib, B):
    T, C = 1000, 64
    pad = (B + 7) // 8 * 8
    fwd_ws = lib.t2fw_lfw_forward_workspace_bytes(B, T, 64, 64, C, 1, 0)
    r = _regions(lib, B, T, 64, 64, C, 1, 0)
    assert r[0] == 0 and r[1] == 2 * pad                   # forward verdicts: two slots per row
    assert r[3] == 2 * pad and r[2] >= 4 * r[1] and r[2] % 256 == 0      # hints: the next aligned region
    assert r[2] + 4 * r[3] <= fwd_ws                        # both inside the forward's workspace
    assert (r[4], r[5]) == (r[2], B)                        # chunk-parallel backward: one slot per row, second region
    both = lib.t2fw_lfw_workspace_bytes(B, T, 64, 64, C, 1, 0)
    nc = lib.t2fw_lfw_num_ckpt(T, C)
    scratch = B * nc * (4 + 6 * 64 * 4 + 64 * 64 * 2)       # per chunk: flag, six vectors, one bf16 matrix
    assert 2 * r[2] + scratch <= both <= 2 * r[2] + scratch + 512
    # block-wise backward: verdicts in the first region, no per-chunk scratch
    rb = _regions(lib, B, T, 64, 64, C, 1, 8)
    assert (rb[4], rb[5]) == (0, 2 * pad) and lib.t2fw_lfw_workspace_bytes(B, T, 64, 64, C, 1, 8) == fwd_ws


def test_flag_regions_of_paths_without_flags(lib):
    assert _regions(lib, 4, 100, 33, 17, 64, 1, 0) == [0] * 6           # exact kernels
    assert _regions(lib, 4, 100, 64, 64, 64, 0, 0) == [0] * 6           # fp32
    assert _regions(lib, 4, 100, 64, 64, 64, 1, 1) == [0] * 6           # exact kernels forced
    r = _regions(lib, 4, 100, 64, 64, 48, 1, 0)                         # an interval only the forward takes
    assert r[1] == 16 and r[3] == 16 and r[5] == 0
    assert lib.t2fw_lfw_flag_regions(4, 100, 64, 64, 64, 9, 0, (ctypes.c_int64 * 6)()) == 2
    assert lib.t2fw_lfw_flag_regions(4, 100, 64, 64, 64, 1, 0, None) == 1


def test_hinted_rows_are_counted_over_both_slots():
    from t2fw_amd.path_hint import count_hinted_rows
    h = np.zeros(2 * 8, dtype=np.int32)
    assert count_hinted_rows(h, 5) == 0
    h[1] = 1; h[8 + 1] = 1; h[8 + 4] = 1; h[7] = 1          # row 1 in both slots, row 4, and a padding slot
    assert count_hinted_rows(h, 5) == 2
    assert count_hinted_rows(h, 8) == 3


def test_choice_of_the_backward_path():
    from t2fw_amd import _lib
    from t2fw_amd.path_hint import choose_backward_flags as choose
    assert choose(0, None, 96) == 0                                  # hints not there: the device decides
    assert choose(0, 0, 96) == _lib.FLAG_NO_FIXUP                    # nothing can be flagged: no extra launch
    assert choose(0, 96, 96) == _lib.FLAG_BLOCKWISE                  # the reference test's gates: every row
    assert choose(0, 1, 96) == _lib.FLAG_BLOCKWISE                   # one round of the block-wise kernel either way
    assert choose(0, 3, 4096) == 0                                   # a few rows of many: redo only those
    assert choose(0, 4096, 4096) == _lib.FLAG_BLOCKWISE
    for caller in (_lib.FLAG_FORCE_SCAN, _lib.FLAG_BLOCKWISE, _lib.FLAG_FP16_OPERANDS, _lib.FLAG_NO_FIXUP):
        assert choose(caller, 0, 96) == caller and choose(caller, 50, 96) == caller       # the caller chose
