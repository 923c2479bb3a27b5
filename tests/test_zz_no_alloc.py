"""The decode attention entry point that allocates nothing (``fl_attn_decode_static``), called
through ctypes as a caller outside Python would: its output equals that of ``fl_attn_decode`` with a
workspace of the caller's, on two calls in a row (the second with a smaller input, so that it finds
the first call's partial results in the shared array), and it refuses what the array cannot hold."""
import ctypes
import math

import pytest
import torch

from test_kernels_gpu import DEV, build_attention_case, decode_rows

pytestmark = pytest.mark.gpu

P, I, F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float


def _library():
    from flambeau_amd.csrc import build
    path = build.library_path()
    assert path.exists(), "build the kernel library first (python __graft_entry__.py)"
    lib = ctypes.CDLL(str(path))
    lib.fl_last_error.restype = ctypes.c_char_p
    lib.fl_attn_decode.argtypes = [P, P, P, P, P, P, I, P, I, I, I, I, I, I, F, I, I, P]
    lib.fl_attn_decode.restype = I
    lib.fl_attn_decode_static.argtypes = [P, P, P, P, I, P, I, I, I, I, I, I, F, I, I, P]
    lib.fl_attn_decode_static.restype = I
    lib.fl_attn_decode_static_capacity.restype = ctypes.c_long
    return lib


def _both(lib, case, rows, nh, nkv, hd, ps, window, n_split):
    """Outputs of the two entry points for the same inputs (NaN where nothing is written)."""
    n = case["n"]
    scale = 1.0 / math.sqrt(hd)
    q = case["q"].reshape(n, nh * hd).contiguous()
    pool, table = case["cache"].pool, case["table"]
    hdp = -(-hd // 32) * 32
    n_items = rows.shape[0]
    part_o = torch.empty(n_items * nh * n_split * hdp, dtype=torch.float32, device=DEV)
    part_ml = torch.empty(n_items * nh * n_split * 2, dtype=torch.float32, device=DEV)
    want = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    got = torch.full((n, nh * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.fl_attn_decode(q.data_ptr(), want.data_ptr(), part_o.data_ptr(), part_ml.data_ptr(), pool.data_ptr(),
                            rows.data_ptr(), n_items, table.data_ptr(), table.shape[1], nh, nkv, hd, ps, pool.shape[0],
                            scale, window, n_split, stream)
    assert rc == 0, lib.fl_last_error()
    torch.cuda.synchronize()
    # from here on nothing may be allocated: the static entry point gets pointers only
    before = torch.cuda.memory_allocated()
    rc = lib.fl_attn_decode_static(q.data_ptr(), got.data_ptr(), pool.data_ptr(), rows.data_ptr(), n_items,
                                   table.data_ptr(), table.shape[1], nh, nkv, hd, ps, pool.shape[0], scale, window,
                                   n_split, stream)
    assert rc == 0, lib.fl_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    return got, want


def test_static_entry_point_equals_the_one_with_a_workspace():
    lib = _library()
    nh, nkv, hd, ps, window = 32, 8, 128, 16, 0
    # first call: 8 rows over long contexts in 6 splits; second call: fewer rows, fewer splits, other
    # contexts, so that its slots hold the first call's partial results when it starts
    big = build_attention_case(torch.bfloat16, nh, nkv, hd, ps, [(700, 1), (333, 1), (48, 1), (1, 1), (257, 3), (90, 1)], seed=3)
    rows = decode_rows(big, range(big["n"]))
    got, want = _both(lib, big, rows, nh, nkv, hd, ps, window, n_split=6)
    assert not torch.isnan(want.float()).any()
    assert torch.equal(got, want)
    small = build_attention_case(torch.bfloat16, nh, nkv, hd, ps, [(130, 1), (500, 2)], seed=5)
    rows = decode_rows(small, range(small["n"]))
    got, want = _both(lib, small, rows, nh, nkv, hd, ps, window, n_split=3)
    assert not torch.isnan(want.float()).any()
    assert torch.equal(got, want)
    # one split needs no scratch at all; other head sizes, a window
    other = build_attention_case(torch.bfloat16, 6, 1, 24, 16, [(70, 1), (33, 2)], seed=6)
    rows = decode_rows(other, range(other["n"]))
    for n_split in (1, 4):
        got, want = _both(lib, other, rows, 6, 1, 24, 16, 11, n_split=n_split)
        assert torch.equal(got, want)


def test_static_entry_point_refuses_what_its_array_cannot_hold():
    lib = _library()
    cap = lib.fl_attn_decode_static_capacity()
    assert cap == 2 << 20
    nh, nkv, hd, ps = 32, 8, 128, 16
    case = build_attention_case(torch.bfloat16, nh, nkv, hd, ps, [(40, 1)], seed=1)
    n_items = cap // (nh * 64 * (128 + 2)) + 1            # one row too many for 64 splits
    rows = decode_rows(case, [0] * n_items)
    out = torch.zeros(1, nh * hd, dtype=torch.bfloat16, device=DEV)
    q = case["q"].reshape(1, nh * hd).contiguous()
    pool, table = case["cache"].pool, case["table"]
    rc = lib.fl_attn_decode_static(q.data_ptr(), out.data_ptr(), pool.data_ptr(), rows.data_ptr(), n_items,
                                   table.data_ptr(), table.shape[1], nh, nkv, hd, ps, pool.shape[0], 0.1, 0, 64,
                                   torch.cuda.current_stream().cuda_stream)
    assert rc != 0
    assert b"static array holds" in lib.fl_last_error()
    torch.cuda.synchronize()
    assert (out == 0).all()
