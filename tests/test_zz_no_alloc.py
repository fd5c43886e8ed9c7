"""The entry point that allocates nothing (helix_a2a_alltoall_loopback_static), through the C ABI: bit-exact
against the oracle's closed form and against helix_a2a_alltoall_loopback, on calls in a row that share the
built-in workspace (the second smaller than the first, then other cp_sizes up to the limit of 11, then a
reset), and with no change in the device's free memory across warm calls."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import helix_oracle as ho

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hx():
    import helix_a2a

    assert torch.cuda.is_available(), "these tests need the MI355X"
    return helix_a2a


@pytest.fixture(scope="module")
def ops(hx):
    from helix_a2a import _ops

    return _ops


def _inputs(cp, entries, x, s, seed):
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    ins_o = [torch.randint(-32768, 32767, (entries, cp, x), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
             for _ in range(cp)]
    ins_s = [torch.randint(-2**31, 2**31 - 1, (entries, cp, s), generator=g, dtype=torch.int32).view(torch.float32).cuda()
             for _ in range(cp)]
    return ins_o, ins_s


def _bits_equal(a, b):
    view = {2: torch.int16, 4: torch.int32}[a.element_size()]
    return torch.equal(a.view(view), b.view(view))


def _both(hx, ops, ws, cp, entries, x, s, seed, reset=False):
    ins_o, ins_s = _inputs(cp, entries, x, s, seed)
    got_o = [torch.full_like(t, 7.0) for t in ins_o]
    got_s = [torch.full_like(t, 7.0) for t in ins_s]
    torch.cuda.synchronize()
    ops.alltoall_loopback_static(ins_o, ins_s, (got_o, got_s), reset=reset)
    torch.cuda.synchronize()
    assert ops.device_status() == 0
    # first against the oracle: out[r][e, s, :] = in[s][e, r, :] on raw bits
    want_o = ho.exchange_closed_form([ho.torch_bits(t) for t in ins_o])
    want_s = ho.exchange_closed_form([ho.torch_bits(t) for t in ins_s])
    for r in range(cp):
        assert np.array_equal(ho.torch_bits(got_o[r]), want_o[r]), f"partial_o of rank {r} differs from the oracle (cp={cp}, entries={entries})"
        assert np.array_equal(ho.torch_bits(got_s[r]), want_s[r]), f"softmax_stats of rank {r} differs from the oracle (cp={cp}, entries={entries})"
    # then against the entry point it is a variant of
    if ws is not None:
        ws_o, ws_s = hx.alltoall_loopback(ins_o, ins_s, ws)
        torch.cuda.synchronize()
        for r in range(cp):
            assert _bits_equal(got_o[r], ws_o[r]) and _bits_equal(got_s[r], ws_s[r]), f"rank {r} differs from the workspace entry point"


def _workspace(hx, cp):
    ws = hx.allocate_workspace(cp, 0)
    for r in range(cp):
        hx.init_workspace(ws, r, cp)
    return ws


def test_static_loopback_matches_the_oracle_and_the_workspace_entry_point(hx, ops):
    cp = 4
    ws = _workspace(hx, cp)
    _both(hx, ops, ws, cp, 64, 32 * 128, 64, seed=1)      # c2's shape
    _both(hx, ops, ws, cp, 37, 6 * 96, 12, seed=2)        # smaller, ragged: the array still holds the first call's lines
    _both(hx, ops, ws, cp, 3, 64, 2, seed=3)              # a few tiny messages
    for i in range(6):                                    # the FIFO entries wrap (four per stream)
        _both(hx, ops, ws, cp, 5 + i, 256, 4, seed=10 + i)
    _both(hx, ops, ws, cp, 2000, 512, 4, seed=4)          # 8 channels x 4 entries cannot hold it: rounds
    del ws
    # another cp_size lays the array out again
    cp = 8
    ws = _workspace(hx, cp)
    _both(hx, ops, ws, cp, 256, 8 * 128, 16, seed=5)      # c3's shape on 2 channels
    _both(hx, ops, ws, cp, 9, 128, 2, seed=6)
    _both(hx, ops, ws, cp, 9, 128, 2, seed=7, reset=True)
    del ws
    cp = 2
    ws = _workspace(hx, cp)
    _both(hx, ops, ws, cp, 8, 4 * 128, 8, seed=8)
    del ws
    torch.cuda.empty_cache()


def test_static_loopback_at_its_largest_cp_size(hx, ops):
    # cp_size = 11: 121 of the 128 FIFOs, one channel; compared with the oracle alone and with a workspace
    cp = 11
    _both(hx, ops, None, cp, 40, 2 * 128, 4, seed=21)
    _both(hx, ops, None, cp, 7, 64, 2, seed=22)           # smaller, in a row
    ws = _workspace(hx, cp)
    _both(hx, ops, ws, cp, 23, 3 * 96, 6, seed=23)
    del ws
    torch.cuda.empty_cache()


def test_static_loopback_leaves_free_memory_alone(hx, ops):
    # outputs preallocated, a warm call behind us: further calls must not change what the device reports as
    # free (no hipMalloc / hipFree by the library; torch allocates nothing either on this path)
    cp = 4
    ins_o, ins_s = _inputs(cp, 48, 512, 8, seed=31)
    out = ([torch.empty_like(t) for t in ins_o], [torch.empty_like(t) for t in ins_s])
    arr = (ops._Params * cp)()
    for r in range(cp):
        arr[r] = ops._make_params(ins_o[r], ins_s[r], out[0][r], out[1][r], None, r, cp, 0)
    stream = ops._stream_handle()
    assert ops._lib.helix_a2a_alltoall_loopback_static(arr, cp, 0, stream) == 0
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    reserved_before = torch.cuda.memory_reserved()
    for i in range(5):
        assert ops._lib.helix_a2a_alltoall_loopback_static(arr, cp, 1 if i == 3 else 0, stream) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before and torch.cuda.memory_reserved() == reserved_before
    assert ops.device_status() == 0
    want_o = ho.exchange_closed_form([ho.torch_bits(t) for t in ins_o])
    for r in range(cp):
        assert np.array_equal(ho.torch_bits(out[0][r]), want_o[r])


def test_static_loopback_limits(hx, ops):
    cp = 12  # 144 FIFOs: more than the built-in workspace holds
    ins_o, ins_s = _inputs(cp, 2, 64, 2, seed=9)
    out = ([torch.empty_like(t) for t in ins_o], [torch.empty_like(t) for t in ins_s])
    with pytest.raises(RuntimeError, match="built-in workspace holds 128 FIFOs"):
        ops.alltoall_loopback_static(ins_o, ins_s, out)
    # a workspace pointer is refused: the call would silently ignore it otherwise
    cp = 2
    ins_o, ins_s = _inputs(cp, 2, 64, 2, seed=10)
    out = ([torch.empty_like(t) for t in ins_o], [torch.empty_like(t) for t in ins_s])
    arr = (ops._Params * cp)()
    for r in range(cp):
        arr[r] = ops._make_params(ins_o[r], ins_s[r], out[0][r], out[1][r], None, r, cp, 0)
        arr[r].workspace = ins_o[0].data_ptr()
    assert ops._lib.helix_a2a_alltoall_loopback_static(arr, cp, 0, ops._stream_handle()) == 1
    assert b"built-in workspace" in ops._lib.helix_a2a_last_error()
    assert isinstance(ctypes.CDLL(ops.library_path()).helix_a2a_alltoall_loopback_static, ctypes._CFuncPtr)
