"""GPU parity tests of the exchange: the HIP path, called through the C ABI, against the oracle.

Bit-exact everywhere: the exchange moves opaque bytes.
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from helix_testing import FIFO_BYTES, torch_bits
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


_WORKSPACES = {}


@pytest.fixture
def unchecked(ops):
    """For tests that make a kernel fail on purpose and read the status word themselves: checked mode off,
    whatever HELIX_A2A_CHECKED says, and back to what it says afterwards."""
    import os
    ops.set_checked_mode(False)
    yield
    ops.set_checked_mode(os.environ.get("HELIX_A2A_CHECKED", "") not in ("", "0"))


@pytest.fixture(params=[False, True], ids=["fused-at-last-rank", "eager-send"])
def send_policy(request, ops):
    """Both ways a per-rank exchange can be issued: all of it with the last rank's call (default), or every
    rank's send half at its own call."""
    ops.set_eager_send(request.param)
    yield request.param
    ops.set_eager_send(False)


def get_workspace(hx, cp, fresh=False):
    """One workspace per cp for the whole module (4.3 GB at cp = 8), initialised on first use."""
    ws = _WORKSPACES.get(cp)
    if ws is None:
        ws = _WORKSPACES[cp] = hx.allocate_workspace(cp, 0)
        fresh = True
    if fresh:
        for r in range(cp):
            hx.init_workspace(ws, r, cp)
    return ws


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    view = {2: torch.int16, 4: torch.int32}[a.element_size()]
    return torch.equal(a.contiguous().view(view), b.contiguous().view(view))


def expected_on_device(ins):
    """The oracle's single-copy form of the closed form, evaluated on the tensors' device."""
    return ho.exchange_single_copy(ins)


def check_against_oracle(ins_o, ins_s, outs_o, outs_s, with_numpy=True):
    cp = len(ins_o)
    want_o, want_s = expected_on_device(ins_o), expected_on_device(ins_s)
    for r in range(cp):
        assert bits_equal(outs_o[r].view(ins_o[r].shape), want_o[r]), f"partial_o of rank {r} differs"
        assert bits_equal(outs_s[r].view(ins_s[r].shape), want_s[r]), f"softmax_stats of rank {r} differs"
    if with_numpy:  # the same comparison on the host against the numpy closed form, on raw bits
        np_o = ho.exchange_closed_form([torch_bits(t) for t in ins_o])
        np_s = ho.exchange_closed_form([torch_bits(t) for t in ins_s])
        for r in range(cp):
            assert np.array_equal(torch_bits(outs_o[r]).reshape(np_o[r].shape), np_o[r])
            assert np.array_equal(torch_bits(outs_s[r]).reshape(np_s[r].shape), np_s[r])


def assert_clean(ops):
    assert ops.device_status() == 0, "a kernel reported a timed-out wait"


# ---------------------------------------------------------------------------
# the reference's single-GPU tests (tests/test_build.py, tests/test_phase2.py)
# ---------------------------------------------------------------------------

def _max_channels(cp_size):
    cu = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
    max_group = min(cp_size, 8)
    blocks_per_ch = ((cp_size + max_group - 1) // max_group) * 2
    return max(cu // blocks_per_ch, 1)


def test_workspace_size_matches_manual_computation(hx):
    for cp_size in (2, 4, 8):
        ch = _max_channels(cp_size)
        expected = 512 * 1024 * cp_size * ch + 256 * cp_size * ch * 2
        actual = hx.workspace_size(cp_size)
        assert isinstance(actual, int) and actual == expected
    assert hx.workspace_size(4) != 16_778_240


def test_init_workspace_pattern(hx):
    cp = 4
    ws = hx.allocate_workspace(cp_size=cp, cp_rank=0)
    assert ws.dtype == torch.int64 and ws.dim() == 2 and ws.shape[0] == cp and ws.shape[1] > 0
    ws.fill_(0x1234)
    hx.init_workspace(ws, cp_rank=2, cp_size=cp)
    fifo_elems = 512 * 1024 * cp * _max_channels(cp) // 8
    assert bool((ws[2, :fifo_elems] == -1).all())
    assert bool((ws[2, fifo_elems:] == 0).all())
    for other in (0, 1, 3):
        assert bool((ws[other] == 0x1234).all())
    del ws
    torch.cuda.empty_cache()


def test_input_validation(hx):
    cp = 4
    ws = get_workspace(hx, cp)
    good_o = torch.randn(2, cp, 128, dtype=torch.bfloat16, device="cuda")
    good_s = torch.randn(2, cp, 2, dtype=torch.float32, device="cuda")
    bad = [
        (good_o.float(), good_s, ws, 0, cp),                                        # partial_o dtype
        (good_o, good_s.half(), ws, 0, cp),                                         # stats dtype
        (torch.randn(2, 3, 128, dtype=torch.bfloat16, device="cuda"), good_s, ws, 0, cp),  # cp dimension
        (good_o, torch.randn(2, cp, 3, device="cuda"), ws, 0, cp),                  # odd stats width
        (good_o, torch.randn(3, cp, 2, device="cuda"), ws, 0, cp),                  # leading dims differ
        (torch.randn(2, cp, 100, dtype=torch.bfloat16, device="cuda"), good_s, ws, 0, cp),  # 200-byte rows
        (good_o.transpose(0, 1), good_s, ws, 0, cp),                                # not contiguous
        (good_o, good_s, ws.int(), 0, cp),                                          # workspace dtype
        (good_o, good_s, ws[0], 0, cp),                                             # workspace rank
        (good_o, good_s, ws[:2], 0, cp),                                            # workspace rows
        (good_o, good_s, ws, cp, cp),                                               # rank out of range
        (good_o, good_s, ws, -1, cp),
        (good_o.cpu(), good_s, ws, 0, cp),
    ]
    for args in bad:
        with pytest.raises(RuntimeError):
            hx.alltoall(*args)
    with pytest.raises(RuntimeError):
        hx.init_workspace(ws, cp, cp)
    with pytest.raises(RuntimeError):
        hx.init_workspace(ws[:, :1000], 0, cp)
    # nothing was enqueued by the rejected calls
    from helix_a2a import _ops
    assert not any(g.pending for g in _ops._groups.values())


# ---------------------------------------------------------------------------
# loopback parity on the benchmark workloads
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("name", ["c1", "c2", "c5b", "c3", "c4", "c5a"])
def test_loopback_workloads(hx, ops, name):
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS[name]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws)
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(ins_o, ins_s, outs_o, outs_s, with_numpy=name in ("c1", "c2", "c5b", "c3"))


@pytest.mark.parametrize("name", ["c3", "c4", "c5a"])
def test_exchange_twice_is_the_identity(hx, ops, name):
    # out[r][e, s] = in[s][e, r], so exchanging the result again returns every rank its own input; and the
    # exchange only moves bytes: sums of the 64-bit words (plain and shifted) over all ranks do not change
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS[name]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    once_o, once_s = hx.alltoall_loopback(ins_o, ins_s, ws)
    back_o, back_s = hx.alltoall_loopback(once_o, once_s, ws)
    torch.cuda.synchronize()
    assert_clean(ops)
    for r in range(w.cp):
        assert bits_equal(back_o[r], ins_o[r]) and bits_equal(back_s[r], ins_s[r])

    def digest(ts):
        words = torch.cat([t.contiguous().view(torch.int64).reshape(-1) for t in ts])
        return tuple(int((words >> shift).sum()) for shift in (0, 8, 16, 32))

    assert digest(ins_o) == digest(once_o) and digest(ins_s) == digest(once_s)


@pytest.mark.parametrize("name", ["c1", "c5b", "c2"])
def test_loopback_against_reference_model(hx, ops, ref_model, name):
    # the C restatement of the reference kernel, run on the same bits
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS[name]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws)
    torch.cuda.synchronize()
    assert_clean(ops)
    np_o, np_s = [torch_bits(t) for t in ins_o], [torch_bits(t) for t in ins_s]
    model_ws = ref_model.new_workspace(w.cp, 8)
    for r in range(w.cp):
        ref_model.init_workspace(model_ws, r, w.cp, 8)
    ref_o, ref_s = ref_model.alltoall_all_ranks(np_o, np_s, model_ws, sm_count=8)
    for r in range(w.cp):
        assert np.array_equal(torch_bits(outs_o[r]), ref_o[r])
        assert np.array_equal(torch_bits(outs_s[r]), ref_s[r])


@pytest.mark.parametrize("name", ["c2", "c5b", "c3"])
def test_per_head_layout(hx, ops, name):
    # the layout the serving integration passes: one entry per (token, head), stats are one float2
    from helix_workloads import WORKLOADS, as_head_layout, make_inputs

    w = WORKLOADS[name]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    pairs = [as_head_layout(w, o, s) for o, s in zip(ins_o, ins_s)]
    h_o, h_s = [p[0] for p in pairs], [p[1] for p in pairs]
    assert h_s[0].shape[-1] == 2
    outs_o, outs_s = hx.alltoall_loopback(h_o, h_s, ws)
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(h_o, h_s, outs_o, outs_s, with_numpy=name != "c3")


@pytest.mark.parametrize("channels", [1, 2, 3, 4, 8, 16, 32, 64, 128, 0])
def test_channel_sweep(hx, ops, channels):
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS["c3"]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws, channel_count=channels)
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(ins_o, ins_s, outs_o, outs_s, with_numpy=False)


def test_channel_count_limits(hx, ops):
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS["c1"]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    with pytest.raises(RuntimeError, match="channel_count"):
        hx.alltoall_loopback(ins_o, ins_s, ws, channel_count=ops.max_channel_count(w.cp) + 1)
    os.environ["HELIX_A2A_CHANNEL_COUNT"] = "3"
    try:
        outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws)
        torch.cuda.synchronize()
    finally:
        del os.environ["HELIX_A2A_CHANNEL_COUNT"]
    assert_clean(ops)
    check_against_oracle(ins_o, ins_s, outs_o, outs_s)


@pytest.mark.parametrize("cp,entries,x,s", [
    (4, 37, 48, 2),     # 104 bytes: a single partial line
    (3, 11, 8, 6),      # 40 bytes, odd cp, stats row of 24 bytes
    (2, 1, 8, 2),       # smallest legal message: 24 bytes
    (5, 13, 136, 10),   # 312 bytes: 2.6 lines, straddling units
    (7, 3, 2048, 62),   # 4344 bytes
    (2, 4, 61440, 2),   # 122888 bytes: 1025 lines, more than a FIFO entry holds -> rejected
    (1, 9, 64, 2),      # a single rank talking to itself
    (16, 2, 64, 2),
    (24, 5, 200, 4),    # more than sixteen ranks: three workgroup columns of eight in the reference's terms
    (32, 40, 128, 2),   # the largest rank count of an exchange (16 GiB of workspace)
    (4, 0, 64, 2),      # nothing to send
])
def test_ragged_shapes(hx, ops, cp, entries, x, s):
    ws = get_workspace(hx, cp)
    g = torch.Generator().manual_seed(cp * 1000 + entries)
    ins_o = [torch.randint(-32768, 32767, (entries, cp, x), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
             for _ in range(cp)]
    ins_s = [torch.randint(-2**31, 2**31 - 1, (entries, cp, s), generator=g, dtype=torch.int32).view(torch.float32).cuda()
             for _ in range(cp)]
    if 2 * x + 4 * s > 1024 * 120:
        with pytest.raises(RuntimeError, match="FIFO entry"):
            hx.alltoall_loopback(ins_o, ins_s, ws)
        return
    outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws)
    torch.cuda.synchronize()
    assert_clean(ops)
    if entries:
        check_against_oracle(ins_o, ins_s, outs_o, outs_s)
    else:
        assert outs_o[0].shape == ins_o[0].shape


def _seeded_cases(count, seed):
    """(cp, entries, x, s, channels, team_units, units_per_wavefront) drawn from one seed: ragged sizes, every
    rank count up to eight and sixteen, channel counts from one to all the layout provides, every sharing rule."""
    import random
    rng = random.Random(seed)
    cases = []
    while len(cases) < count:
        cp = rng.choice([1, 2, 3, 4, 5, 6, 7, 8, 16])
        x = 8 * rng.choice([1, 2, 3, 5, 8, 17, 32, 33, 64, 100, 128, 255, 256, 512, 1000, 2048])
        s = rng.choice([2, 2, 2, 4, 6, 8, 14, 16, 32, 62])
        entries = rng.choice([1, 2, 3, 7, 16, 33, 64, 100, 129, 256, 300])
        if cp * cp * entries * (2 * x + 4 * s) > 96 << 20:   # keeps the whole test within seconds
            continue
        channels = rng.choice([0, 0, 1, 2, 3, 5, 8, 16, 31, 64, 128])
        cases.append((cp, entries, x, s, channels, rng.choice([-1, -1, 0, 2, 6]), rng.choice([-1, -1, 0, 3])))
    return cases


def test_seeded_random_shapes_on_shared_workspaces(hx, ops):
    # sixty exchanges of unrelated shapes, one after the other on the workspaces of their rank counts: whatever
    # a launch leaves in the counters and the FIFO slots is what the next one, with another placement of its
    # runs, starts from; every result bit-exact against the closed form
    try:
        for i, (cp, entries, x, s, channels, team_units, units) in enumerate(_seeded_cases(60, 20240607)):
            ws = get_workspace(hx, cp)
            channels = min(channels, _max_channels(cp))
            g = torch.Generator().manual_seed(7000 + i)
            ins_o = [torch.randint(-32768, 32767, (entries, cp, x), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
                     for _ in range(cp)]
            ins_s = [torch.randint(-2**31, 2**31 - 1, (entries, cp, s), generator=g, dtype=torch.int32).view(torch.float32).cuda()
                     for _ in range(cp)]
            ops.set_team_units(team_units)
            ops.set_units_per_wavefront(units)
            outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws, channel_count=channels)
            torch.cuda.synchronize()
            assert ops.device_status() == 0, (i, cp, entries, x, s, channels, team_units, units)
            want_o, want_s = expected_on_device(ins_o), expected_on_device(ins_s)
            for r in range(cp):
                assert bits_equal(outs_o[r], want_o[r]) and bits_equal(outs_s[r], want_s[r]), \
                    (i, r, cp, entries, x, s, channels, team_units, units)
    finally:
        ops.set_team_units(-1)
        ops.set_units_per_wavefront(-1)


@pytest.mark.parametrize("entries,units_in_flight", [(1, 1), (3, 2), (5, 3), (7, 4), (9, 5), (11, 6), (12, 4), (33, 6)])
def test_every_units_in_flight_variant(hx, ops, entries, units_in_flight):
    # one channel, 520-byte messages (65 pieces): the run of `entries` messages, packed piece by piece into
    # ceil(65 * entries / 15) lines of 8 units, makes the host pick the kernel instantiation with that many
    # units in flight per lane
    cp, x = 3, 256
    ws = get_workspace(hx, cp)
    g = torch.Generator().manual_seed(4000 + entries)
    ins_o = [torch.randint(-32768, 32767, (entries, cp, x), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
             for _ in range(cp)]
    ins_s = [torch.randint(-2**31, 2**31 - 1, (entries, cp, 2), generator=g, dtype=torch.int32).view(torch.float32).cuda()
             for _ in range(cp)]
    per_lane = -(-(-(-entries * 65 // 15) * 8) // 64)
    passes = -(-per_lane // 6)
    assert -(-per_lane // passes) == units_in_flight          # the case is what its label says
    outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws, channel_count=1)
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(ins_o, ins_s, outs_o, outs_s)


@pytest.mark.parametrize("cp,entries,x,s,channels", [
    (3, 40, 136, 10, 2),    # 312 bytes = 39 pieces (odd), 20 messages per stream: two passes
    (2, 400, 8, 6, 2),      # 40 bytes = 5 pieces: three messages per line, 200 per stream
    (5, 26, 600, 2, 2),     # 1208 bytes = 151 pieces, the pass boundary falls inside a message
    (4, 12, 1016, 14, 1),   # 2088 bytes = 261 pieces with 56 bytes of statistics astride two lines
    (2, 9, 61432, 2, 1),    # 122872 bytes = 15 360 pieces: one message per FIFO entry, 22 passes each
    (16, 64, 264, 2, 4),    # 536 bytes = 67 pieces, 16 ranks
    (8, 2048, 128, 2, 128), # the benchmark shape passed per head: 264 bytes = 33 pieces, 16 per stream
])
def test_runs_of_several_passes(hx, ops, cp, entries, x, s, channels):
    # runs longer than one pass go through the kernels whose receivers realign the payload to 16-byte stores
    ws = get_workspace(hx, cp)
    g = torch.Generator().manual_seed(cp * 977 + entries)
    ins_o = [torch.randint(-32768, 32767, (entries, cp, x), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
             for _ in range(cp)]
    ins_s = [torch.randint(-2**31, 2**31 - 1, (entries, cp, s), generator=g, dtype=torch.int32).view(torch.float32).cuda()
             for _ in range(cp)]
    pieces = (2 * x + 4 * s) // 8
    run_units = -(-min(-(-entries // channels), 15360 // pieces) * pieces // 15) * 8
    assert run_units > 6 * 64 or entries == 2048
    outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws, channel_count=channels)
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(ins_o, ins_s, outs_o, outs_s)


@pytest.mark.parametrize("units", [0, 1, 2, 3, 4, 5])
def test_runs_shared_by_several_wavefronts(hx, ops, units):
    # every split of a stream's runs over wavefronts gives the same bits, on one workspace, call after call:
    # the step counters of all parts of a stream move in lockstep whatever the number of parts of a call
    shapes = [(3, 7, 1096, 6, 2), (8, 256, 1024, 16, 128), (2, 9, 61432, 2, 1), (4, 12, 1016, 14, 1), (16, 64, 264, 2, 4)]
    try:
        for cp, entries, x, s, channels in shapes:
            ws = get_workspace(hx, cp)
            g = torch.Generator().manual_seed(cp * 31 + entries + units)
            ins_o = [torch.randint(-32768, 32767, (entries, cp, x), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
                     for _ in range(cp)]
            ins_s = [torch.randint(-2**31, 2**31 - 1, (entries, cp, s), generator=g, dtype=torch.int32).view(torch.float32).cuda()
                     for _ in range(cp)]
            for u in (units, 6, units):
                ops.set_units_per_wavefront(u)
                outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws, channel_count=channels)
                torch.cuda.synchronize()
                assert_clean(ops)
                check_against_oracle(ins_o, ins_s, outs_o, outs_s, with_numpy=False)
    finally:
        ops.set_units_per_wavefront(-1)
    with pytest.raises(RuntimeError, match="units per wavefront"):
        ops.set_units_per_wavefront(7)


def test_special_values_survive(hx, ops):
    # NaN payloads, infinities, denormals and negative zero are bytes like any other
    cp, entries = 2, 4
    ws = get_workspace(hx, cp)
    specials = torch.tensor([float("nan"), float("inf"), float("-inf"), -0.0, 1e-45, 3.0e38, 0.0, -1.0])
    ins_o = [specials.to(torch.bfloat16).repeat(entries, cp, 16).cuda() for _ in range(cp)]
    ins_s = [specials.repeat(entries, cp, 1).contiguous().cuda() for _ in range(cp)]
    ins_s[1] = ins_s[1].view(torch.int32).bitwise_xor(0x00400001).view(torch.float32)  # a signalling-NaN pattern among them
    outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws)
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(ins_o, ins_s, outs_o, outs_s)


# ---------------------------------------------------------------------------
# FIFO state across calls
# ---------------------------------------------------------------------------

def test_repeated_calls_wrap_the_fifo(hx, ops):
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS["c2"]
    ws = get_workspace(hx, w.cp, fresh=True)
    ins_o, ins_s = make_inputs(w, "cuda")
    for call in range(11):  # every stream consumes one FIFO entry per call: entries are reused from call 4 on
        rolled_o = [t.roll(call, 0) for t in ins_o]
        rolled_s = [t.roll(call, 0) for t in ins_s]
        outs_o, outs_s = hx.alltoall_loopback(rolled_o, rolled_s, ws, channel_count=(call % 5) * 7 + 1)
        check_against_oracle(rolled_o, rolled_s, outs_o, outs_s, with_numpy=False)
    assert_clean(ops)


def test_reinit_between_calls(hx, ops):
    # tests/test_mnnvl.py:100-161 re-initialises the workspace before every call
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS["c1"]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    for _ in range(3):
        for r in range(w.cp):
            hx.init_workspace(ws, r, w.cp)
        outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws)
        check_against_oracle(ins_o, ins_s, outs_o, outs_s)
    assert_clean(ops)


def test_many_calls_back_to_back_without_sync(hx, ops):
    # a torn or stale line would show up as a mismatch in one of many asynchronous iterations
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS["c3"]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    want_o, want_s = expected_on_device(ins_o), expected_on_device(ins_s)
    bad = torch.zeros((), dtype=torch.int64, device="cuda")
    for it in range(60):
        src_o = [t.bitwise_xor(it) for t in (x.view(torch.int16) for x in ins_o)]
        outs_o, outs_s = hx.alltoall_loopback([t.view(torch.bfloat16) for t in src_o], ins_s, ws)
        for r in range(w.cp):
            bad += (outs_o[r].view(torch.int16) != want_o[r].view(torch.int16).bitwise_xor(it)).sum()
            bad += (outs_s[r].view(torch.int32) != want_s[r].view(torch.int32)).sum()
    torch.cuda.synchronize()
    assert_clean(ops)
    assert int(bad.item()) == 0


def test_exchange_beside_a_competing_kernel(hx, ops):
    # Sender wavefronts come first in a launch's dispatch order, and receivers rely on that to find their
    # senders running. Here the device is shared with long unrelated kernels on a second stream of the same
    # (default) priority, which take wavefront slots away from the exchange at arbitrary moments: the
    # exchanges must still complete, bit for bit, with no wait running into its limit.
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS["c3"]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    want_o, want_s = expected_on_device(ins_o), expected_on_device(ins_s)
    side = torch.cuda.Stream()
    noise = torch.randn(1 << 26, device="cuda")             # 256 MB: every launch fills the device for a while
    small = torch.randn(1 << 16, device="cuda")             # and short ones in between
    bad = torch.zeros((), dtype=torch.int64, device="cuda")
    torch.cuda.synchronize()
    plan = ops.LoopbackPlan(ins_o, ins_s, ws)
    for it in range(40):
        with torch.cuda.stream(side):
            noise.mul_(1.0001).sin_()
            for _ in range(4):
                small.add_(1.0)
        outs_o, outs_s = plan.run()
        for r in range(w.cp):
            bad += (outs_o[r].view(torch.int16) != want_o[r].view(torch.int16)).sum()
            bad += (outs_s[r].view(torch.int32) != want_s[r].view(torch.int32)).sum()
        if it % 10 == 9:
            torch.cuda.synchronize()
            assert ops.device_status() == 0, f"a wait gave up in iterations {it - 9}..{it}"
            assert int(bad.item()) == 0, f"wrong output in iterations {it - 9}..{it}"
    side.synchronize()
    torch.cuda.synchronize()
    assert ops.device_status() == 0 and int(bad.item()) == 0


# ---------------------------------------------------------------------------
# the per-rank call (the reference's signature)
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_per_rank_calls_seeded_full_tensor(hx, ops, dtype, send_policy):
    # tests/test_alltoall.py:303-360 on logical ranks: rank r sends full[:, :, r, :] and receives full[:, r, :, :]
    cp, b, d, s = 4, 4, 128, 2
    ws = get_workspace(hx, cp)
    torch.manual_seed(42)
    full_o = torch.randn(b, cp, cp, d, dtype=dtype, device="cuda")
    full_s = torch.randn(b, cp, cp, s, dtype=torch.float32, device="cuda")
    results = []
    for rank in range(cp):
        send_o = full_o[:, :, rank, :].contiguous()
        send_s = full_s[:, :, rank, :].contiguous()
        results.append(hx.alltoall(send_o.clone(), send_s.clone(), ws, cp_rank=rank, cp_size=cp))
    torch.cuda.synchronize()
    assert_clean(ops)
    for rank, (recv_o, recv_s) in enumerate(results):
        assert bits_equal(recv_o, full_o[:, rank, :, :])
        assert bits_equal(recv_s, full_s[:, rank, :, :])


def test_per_rank_calls_fill_vectors(hx, ops, send_policy):
    # tests/test_mnnvl.py:164-219: rank r sends the constant r+1; slot j of every result holds j+1
    cp, n, d = 4, 4, 64
    ws = get_workspace(hx, cp)
    results = []
    for rank in reversed(range(cp)):  # any call order works
        po = torch.full((n, cp, d), float(rank + 1), dtype=torch.bfloat16, device="cuda")
        ss = torch.full((n, cp, 2), float(rank + 1) * 0.1, dtype=torch.float32, device="cuda")
        results.append((rank, *hx.alltoall(po, ss, ws, cp_rank=rank, cp_size=cp)))
    torch.cuda.synchronize()
    assert_clean(ops)
    for rank, po_out, ss_out in results:
        assert po_out.shape == (n, cp, d) and ss_out.shape == (n, cp, 2)
        for j in range(cp):
            assert bool((po_out[:, j, :].float() == float(j + 1)).all())
            assert bool((ss_out[:, j, :] == torch.tensor(float(j + 1) * 0.1, dtype=torch.float32)).all())


def test_per_rank_calls_4d_and_leading_dims(hx, ops):
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS["c2"]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    hp = w.heads_per_rank
    outs = [hx.alltoall(o.view(w.tokens, w.cp, hp, w.head_dim), s.view(w.tokens, w.cp, hp, 2), ws, r, w.cp)
            for r, (o, s) in enumerate(zip(ins_o, ins_s))]
    torch.cuda.synchronize()
    assert_clean(ops)
    assert outs[0][0].shape == (w.tokens, w.cp, hp, w.head_dim)
    check_against_oracle(ins_o, ins_s, [o[0] for o in outs], [o[1] for o in outs], with_numpy=False)
    # extra leading dimensions are flattened into the entry count: [2, T/2, cp, X]
    outs = [hx.alltoall(o.view(2, w.tokens // 2, w.cp, -1), s.view(2, w.tokens // 2, w.cp, -1), ws, r, w.cp)
            for r, (o, s) in enumerate(zip(ins_o, ins_s))]
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(ins_o, ins_s, [o[0] for o in outs], [o[1] for o in outs], with_numpy=False)


def test_per_rank_calls_with_temporary_workspace_views(hx, ops, send_policy):
    # every rank hands over a fresh view of the workspace that dies with its call: the exchange must not
    # be forgotten (nor its workspace freed) between the first rank's call and the last one's
    cp, entries = 4, 24
    ws = get_workspace(hx, cp)
    g = torch.Generator().manual_seed(77)
    for rep in range(3):
        ins_o = [torch.randn(entries, cp, 256, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
        ins_s = [torch.randn(entries, cp, 4, generator=g).cuda() for _ in range(cp)]
        outs = [hx.alltoall(ins_o[r], ins_s[r], ws.view(cp, -1) if r % 2 else ws[:], cp_rank=r, cp_size=cp)
                for r in range(cp)]
        torch.cuda.synchronize()
        assert_clean(ops)
        check_against_oracle(ins_o, ins_s, [a for a, _ in outs], [b for _, b in outs], with_numpy=False)
    assert not any(g_.pending for g_ in ops._groups.values())


def test_eager_send_lets_a_rank_reuse_its_input_buffer(hx, ops):
    # with eager sends a rank's inputs are read in stream order at its call, as with the reference: one
    # buffer refilled for every rank works. (The default issues everything with the last rank's call and
    # asks the ranks to leave their inputs alone until then.)
    cp, entries = 4, 32
    ws = get_workspace(hx, cp)
    g = torch.Generator().manual_seed(78)
    ins_o = [torch.randn(entries, cp, 128, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
    ins_s = [torch.randn(entries, cp, 2, generator=g).cuda() for _ in range(cp)]
    buf_o, buf_s = torch.empty_like(ins_o[0]), torch.empty_like(ins_s[0])
    ops.set_eager_send(True)
    try:
        outs = []
        for r in range(cp):
            buf_o.copy_(ins_o[r])
            buf_s.copy_(ins_s[r])
            outs.append(hx.alltoall(buf_o, buf_s, ws, cp_rank=r, cp_size=cp))
        buf_o.zero_()
        buf_s.zero_()
    finally:
        ops.set_eager_send(False)
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(ins_o, ins_s, [a for a, _ in outs], [b for _, b in outs], with_numpy=False)


def test_per_rank_call_twice_is_an_error(hx, ops):
    cp = 2
    ws = get_workspace(hx, cp)
    o = torch.zeros(2, cp, 64, dtype=torch.bfloat16, device="cuda")
    s = torch.zeros(2, cp, 2, device="cuda")
    hx.alltoall(o, s, ws, 0, cp)
    with pytest.raises(RuntimeError, match="again"):
        hx.alltoall(o, s, ws, 0, cp)
    hx.alltoall(o, s, ws, 1, cp)  # completes the group
    torch.cuda.synchronize()
    assert_clean(ops)


# ---------------------------------------------------------------------------
# what the sender leaves in the FIFO
# ---------------------------------------------------------------------------

def test_fifo_image_matches_host_model(hx, ops, host_model):
    import ctypes

    cp, entries, x, s = 2, 300, 512, 8  # 9-line messages, 113 per FIFO entry: 3 entries per stream on one channel
    cu = torch.cuda.get_device_properties(0).multi_processor_count
    ws = get_workspace(hx, cp, fresh=True)
    g = torch.Generator().manual_seed(5)
    ins_o = [torch.randint(-32768, 32767, (entries, cp, x), generator=g, dtype=torch.int16) for _ in range(cp)]
    ins_s = [torch.randint(-2**31, 2**31 - 1, (entries, cp, s), generator=g, dtype=torch.int32) for _ in range(cp)]
    dev_o = [t.view(torch.bfloat16).cuda() for t in ins_o]
    dev_s = [t.view(torch.float32).cuda() for t in ins_s]
    out_o = [torch.empty_like(t) for t in dev_o]
    out_s = [torch.empty_like(t) for t in dev_s]
    arr = (ops._Params * cp)()
    for r in range(cp):
        arr[r] = ops._make_params(dev_o[r], dev_s[r], out_o[r], out_s[r], ws, r, cp, 1)
    ops._check(ops._lib.helix_a2a_alltoall_send(arr, cp, ops._stream_handle()), "send")
    torch.cuda.synchronize()
    assert_clean(ops)

    host_ws = host_model.new_workspace(cp, cu)
    np_o = [t.numpy().view(np.uint16) for t in ins_o]
    np_s = [t.numpy().view(np.uint32) for t in ins_s]
    _, _, rc, msg = host_model.alltoall(np_o, np_s, host_ws, cu, 1, send=True, recv=False)
    assert rc == 0, msg
    max_ch = host_model.max_channel_count(cp, cu)
    fifo_region_elems = FIFO_BYTES * cp * max_ch // 8
    for row in range(cp):
        # the whole FIFO region: the lines of every stream where the launch packed them, 0xFF everywhere else
        assert np.array_equal(ws[row, :fifo_region_elems].cpu().numpy(), host_ws[row, :fifo_region_elems]), f"FIFO region of row {row} differs"
        assert np.array_equal(ws[row, fifo_region_elems:].cpu().numpy(), host_ws[row, fifo_region_elems:])
    # finish the exchange so the workspace is consistent again
    ops._check(ops._lib.helix_a2a_alltoall_recv(arr, cp, ops._stream_handle()), "recv")
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(dev_o, dev_s, out_o, out_s)


def test_launches_of_different_sizes_alternate_on_one_workspace(hx, ops):
    # the lines of a launch are packed by its own shape, and a launch too large for the memory-side cache rewrites
    # one or two positions instead of rotating through four: launches of all three kinds follow each other on one
    # workspace, fresh payload every time, exchange and fused combine
    cp = 8
    ws = get_workspace(hx, cp)
    g = torch.Generator().manual_seed(91)
    shapes = [(512, 1024, 16), (64, 1024, 16), (384, 1024, 16), (512, 1024, 16), (5, 256, 4), (384, 1024, 16), (512, 1024, 16)]
    for rep, (entries, x, s) in enumerate(shapes):
        ins_o = [torch.randint(-32768, 32767, (entries, cp, x), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
                 for _ in range(cp)]
        ins_s = [torch.randint(-2**31, 2**31 - 1, (entries, cp, s), generator=g, dtype=torch.int32).view(torch.float32).cuda()
                 for _ in range(cp)]
        for _ in range(2):   # twice in a row: the second call rewrites (one position) or moves on (two, four)
            outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws)
        torch.cuda.synchronize()
        assert_clean(ops)
        check_against_oracle(ins_o, ins_s, outs_o, outs_s, with_numpy=False)
        if rep % 2 == 0:
            vals = [torch.randn(entries, cp, x, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
            lse = [torch.randn(entries, cp, s, generator=g).cuda() for _ in range(cp)]
            combined = hx.alltoall_combine_loopback(vals, lse, ws, hx.STATS_LSE)
            torch.cuda.synchronize()
            assert_clean(ops)
            heads = s // 2
            recv_o = ho.exchange_closed_form([torch_bits(t) for t in vals])
            recv_s = ho.exchange_closed_form([torch_bits(t) for t in lse])
            for r in (0, cp - 1):
                with np.errstate(all="ignore"):
                    want, _ = ho.combine_after_exchange(ho.bf16_bits_to_f32(recv_o[r]), recv_s[r].view(np.float32), heads, 0)
                got = combined[r].float().cpu().numpy()
                assert (np.abs(got - want) <= 2e-2 + 2e-2 * np.abs(want)).all()


# ---------------------------------------------------------------------------
# bounded waits and back-pressure
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("units", [1, 2, 3, 5, 6])
def test_runs_walked_by_teams(hx, ops, units):
    # the wavefronts of a workgroup walk one stream's run together (slices of at most `units` units per lane),
    # sharing its counters through the first of them: same bits as one wavefront per stream, call after call
    # on one workspace, for runs of one and of many passes, several runs per launch, ragged message sizes
    shapes = [(3, 7, 1096, 6, 2), (8, 256, 1024, 16, 128), (2, 9, 61432, 2, 1), (4, 12, 1016, 14, 1), (16, 64, 264, 2, 4),
              (2, 400, 8, 6, 2), (5, 26, 600, 2, 2)]
    try:
        ops.set_units_per_wavefront(0)  # one part per stream: the launches teams apply to
        for cp, entries, x, s, channels in shapes:
            ws = get_workspace(hx, cp)
            g = torch.Generator().manual_seed(cp * 37 + entries + units)
            ins_o = [torch.randint(-32768, 32767, (entries, cp, x), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
                     for _ in range(cp)]
            ins_s = [torch.randint(-2**31, 2**31 - 1, (entries, cp, s), generator=g, dtype=torch.int32).view(torch.float32).cuda()
                     for _ in range(cp)]
            for u in (units, 0, units):
                ops.set_team_units(u)
                outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws, channel_count=channels)
                torch.cuda.synchronize()
                assert_clean(ops)
                check_against_oracle(ins_o, ins_s, outs_o, outs_s, with_numpy=False)
    finally:
        ops.set_team_units(-1)
        ops.set_units_per_wavefront(-1)
    with pytest.raises(RuntimeError, match="units per team wavefront"):
        ops.set_team_units(7)


def test_team_whose_wait_gives_up_leaves_together(hx, ops, unchecked):
    # receivers without senders, as teams: the first wavefront of each team gives up its wait and every
    # wavefront of the team leaves with it; the kernel ends normally and reports the time-out
    cp = 2
    ws = get_workspace(hx, cp, fresh=True)
    o = [torch.zeros(3, cp, 2048, dtype=torch.bfloat16, device="cuda") for _ in range(cp)]
    s = [torch.zeros(3, cp, 2, device="cuda") for _ in range(cp)]
    out_o = [torch.empty_like(t) for t in o]
    out_s = [torch.empty_like(t) for t in s]
    arr = (ops._Params * cp)()
    for r in range(cp):
        arr[r] = ops._make_params(o[r], s[r], out_o[r], out_s[r], ws, r, cp, 1)
    ops.set_spin_limit_us(0)  # every wait gives up at its first clock check
    ops.set_units_per_wavefront(0)
    ops.set_team_units(2)
    try:
        ops._check(ops._lib.helix_a2a_alltoall_recv(arr, cp, ops._stream_handle()), "recv")
        torch.cuda.synchronize()
        status = ops.device_status()
    finally:
        ops.set_spin_limit_us(2_000_000)
        ops.set_team_units(-1)
        ops.set_units_per_wavefront(-1)
    assert status & 1, "the receiving teams should have reported a timed-out wait"
    for r in range(cp):
        hx.init_workspace(ws, r, cp)
    ins_o = [torch.randn(3, cp, 2048, device="cuda").to(torch.bfloat16) for _ in range(cp)]
    outs_o, outs_s = hx.alltoall_loopback(ins_o, s, ws, channel_count=1)
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(ins_o, s, outs_o, outs_s, with_numpy=False)


@pytest.mark.parametrize("teams", [False, True])
def test_corrupt_line_is_reported(hx, ops, teams, unchecked):
    # a line whose flag word does not carry the step once the token says the run is complete: the receiver
    # reports a corrupt workspace (status bit 4), the kernel ends normally, and the workspace stays out of use
    # (bit 8) until it is initialised again -- for single wavefronts and for teams alike
    cp, entries, channels = 2, 3, 1
    ws = get_workspace(hx, cp, fresh=True)
    g = torch.Generator().manual_seed(5)
    o = [torch.randint(-32768, 32767, (entries, cp, 2048), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
         for _ in range(cp)]
    s = [torch.zeros(entries, cp, 2, device="cuda") for _ in range(cp)]
    out_o = [torch.zeros_like(t) for t in o]
    out_s = [torch.zeros_like(t) for t in s]
    arr = (ops._Params * cp)()
    for r in range(cp):
        arr[r] = ops._make_params(o[r], s[r], out_o[r], out_s[r], ws, r, cp, channels)
    try:
        if teams:
            ops.set_units_per_wavefront(0)
            ops.set_team_units(2)
        ops._check(ops._lib.helix_a2a_alltoall_send(arr, cp, ops._stream_handle()), "send")
        torch.cuda.synchronize()
        assert ops.device_status() == 0
        # the FIFO of stream (sender 0 -> receiver 1, channel 0) starts receiver 1's row; a fresh workspace is at
        # step 0, entry 0; the flag word is the last 8 bytes of a 128-byte line
        line = 37
        assert int(ws[1, line * 16 + 15]) == 0, "the flag word of a line of step 0"
        ws[1, line * 16 + 15] = 12345
        ops._check(ops._lib.helix_a2a_alltoall_recv(arr, cp, ops._stream_handle()), "recv")
        torch.cuda.synchronize()
        status = ops.device_status()
        assert status & ops.STATUS_INTERNAL, status
        if teams:
            # 3 messages of 513 pieces on one channel: a run of 103 lines walked by 7 wavefronts, 16 lines each,
            # one pass per wavefront. The wavefront that owns lines 32..47 stores its pass as it came and reports;
            # its team-mates store their slices; the stream's counters stay put
            assert bits_equal(out_o[1][2, 0], o[0][2, 1])
            max_ch = _max_channels(cp)
            receiver_info = (512 * 1024 * cp * max_ch + 256 * cp * max_ch) // 8
            assert int(ws[1, receiver_info + 1]) == 0, "the receiver's counter of the corrupt stream was released"
        hx.alltoall_loopback(o, s, ws, channel_count=channels)
        torch.cuda.synchronize()
        assert ops.device_status() & ops.STATUS_BROKEN_WORKSPACE
    finally:
        ops.set_team_units(-1)
        ops.set_units_per_wavefront(-1)
        for r in range(cp):
            hx.init_workspace(ws, r, cp)
    outs_o, outs_s = hx.alltoall_loopback(o, s, ws, channel_count=channels)
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(o, s, outs_o, outs_s, with_numpy=False)


def test_receive_without_send_times_out_cleanly(hx, ops, unchecked):
    cp = 2
    ws = get_workspace(hx, cp, fresh=True)
    o = [torch.zeros(3, cp, 64, dtype=torch.bfloat16, device="cuda") for _ in range(cp)]
    s = [torch.zeros(3, cp, 2, device="cuda") for _ in range(cp)]
    out_o = [torch.empty_like(t) for t in o]
    out_s = [torch.empty_like(t) for t in s]
    arr = (ops._Params * cp)()
    for r in range(cp):
        arr[r] = ops._make_params(o[r], s[r], out_o[r], out_s[r], ws, r, cp, 1)
    ops.set_spin_limit_us(0)  # every wait gives up at its first clock check: the kernel still exits normally
    try:
        ops._check(ops._lib.helix_a2a_alltoall_recv(arr, cp, ops._stream_handle()), "recv")
        torch.cuda.synchronize()
        status = ops.device_status()
    finally:
        ops.set_spin_limit_us(2_000_000)
    assert status & 1, "the receiver should have reported a timed-out wait"
    assert ops.device_status() == 0  # reading clears it
    for r in range(cp):
        hx.init_workspace(ws, r, cp)


def test_exchange_after_a_timeout_does_nothing_until_reinit(hx, ops, unchecked):
    # a wait that gives up marks the workspace broken: the exchanges queued behind it write nothing and say so
    cp = 4
    ws = get_workspace(hx, cp, fresh=True)
    g = torch.Generator().manual_seed(77)
    o = [torch.randint(-32768, 32767, (24, cp, 256), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda() for _ in range(cp)]
    s = [torch.randint(-2**31, 2**31 - 1, (24, cp, 4), generator=g, dtype=torch.int32).view(torch.float32).cuda() for _ in range(cp)]
    out_o = [torch.empty_like(t) for t in o]
    out_s = [torch.empty_like(t) for t in s]
    arr = (ops._Params * cp)()
    for r in range(cp):
        arr[r] = ops._make_params(o[r], s[r], out_o[r], out_s[r], ws, r, cp, 0)
    ops.set_spin_limit_us(0)  # the receivers' wait gives up at its first clock check; every kernel still exits normally
    try:
        ops._check(ops._lib.helix_a2a_alltoall_recv(arr, cp, ops._stream_handle()), "recv")
        torch.cuda.synchronize()
    finally:
        ops.set_spin_limit_us(2_000_000)
    assert ops.device_status() & ops.STATUS_RECV_TIMEOUT
    # a complete exchange on the same workspace, with normal limits, without re-initialising
    sentinel_o = [torch.full_like(t, 3.0) for t in o]
    sentinel_s = [torch.full_like(t, 3.0) for t in s]
    hx.alltoall_loopback(o, s, ws, out=(sentinel_o, sentinel_s))
    comb = torch.full((24, 256), 5.0, dtype=torch.bfloat16, device="cuda")
    plan = ops.CombinePlan(o, s, ws, ops.STATS_LSE, False, 0)
    for c in plan.combined:
        c.fill_(5.0)
    plan.run()
    torch.cuda.synchronize()
    status = ops.device_status()
    assert status == ops.STATUS_BROKEN_WORKSPACE, f"status {status:#x}"
    for r in range(cp):
        assert (sentinel_o[r] == 3.0).all() and (sentinel_s[r] == 3.0).all(), "a broken workspace must not produce output"
        assert torch.equal(plan.combined[r], comb)
    # checked mode turns the same condition into an error of the call
    ops.set_checked_mode(True)
    try:
        with pytest.raises(RuntimeError, match="workspace broken by an earlier failure"):
            hx.alltoall_loopback(o, s, ws)
    finally:
        ops.set_checked_mode(False)
    assert ops.device_status() == 0  # the checked call has read and cleared it
    for r in range(cp):
        hx.init_workspace(ws, r, cp)
    outs_o, outs_s = hx.alltoall_loopback(o, s, ws)
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(o, s, outs_o, outs_s)
    # and checked mode is silent on a healthy exchange
    ops.set_checked_mode(True)
    try:
        outs_o, outs_s = hx.alltoall_loopback(o, s, ws)
        check_against_oracle(o, s, outs_o, outs_s, with_numpy=False)
    finally:
        ops.set_checked_mode(False)


def test_send_capacity_is_checked_for_split_phases(hx, ops):
    # 17-piece messages on one channel: 4 x 903 fit the four FIFO entries; a send-only launch of more is refused
    cp, entries = 2, 3613
    ws = get_workspace(hx, cp)
    o = torch.zeros(entries, cp, 64, dtype=torch.bfloat16, device="cuda")
    s = torch.zeros(entries, cp, 2, device="cuda")
    oo, so = torch.empty_like(o), torch.empty_like(s)
    p = ops._make_params(o, s, oo, so, ws, 0, cp, 1)
    assert ops._lib.helix_a2a_alltoall_send(ctypes.byref(p), 1, ops._stream_handle()) == 3  # HELIX_A2A_ERR_CAPACITY
    assert b"FIFO entries in flight" in ops._lib.helix_a2a_last_error()
    assert ops._lib.helix_a2a_alltoall_recv(ctypes.byref(p), 1, ops._stream_handle()) == 3
    torch.cuda.synchronize()
    assert_clean(ops)


def test_per_rank_calls_beyond_fifo_capacity(hx, ops, send_policy):
    # the reference accepts any entry count (its senders wait for their receivers); per-rank calls of logical
    # ranks hold such an exchange back until the last rank has called and issue it in stream-ordered rounds
    cp, entries = 3, 7300  # one channel: 3612 messages per round
    ws = get_workspace(hx, cp)
    g = torch.Generator().manual_seed(123)
    ins_o = [torch.randint(-32768, 32767, (entries, cp, 64), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
             for _ in range(cp)]
    ins_s = [torch.randint(-2**31, 2**31 - 1, (entries, cp, 2), generator=g, dtype=torch.int32).view(torch.float32).cuda()
             for _ in range(cp)]
    os.environ["HELIX_A2A_CHANNEL_COUNT"] = "1"
    try:
        results = [hx.alltoall(ins_o[r], ins_s[r], ws, r, cp) for r in range(cp)]
    finally:
        del os.environ["HELIX_A2A_CHANNEL_COUNT"]
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(ins_o, ins_s, [x[0] for x in results], [x[1] for x in results], with_numpy=False)
    # an exchange that fits goes back to sending at once, on the same workspace
    small_o = [t[:100].contiguous() for t in ins_o]
    small_s = [t[:100].contiguous() for t in ins_s]
    results = [hx.alltoall(small_o[r], small_s[r], ws, r, cp) for r in range(cp)]
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(small_o, small_s, [x[0] for x in results], [x[1] for x in results], with_numpy=False)


def test_channel_count_of_an_exchange_is_settled_by_its_first_rank(hx, ops, send_policy):
    # the send halves and the receive half of one per-rank exchange are separate launches; the environment
    # may change between them without the halves disagreeing
    cp, entries = 4, 40
    ws = get_workspace(hx, cp)
    g = torch.Generator().manual_seed(321)
    ins_o = [torch.randint(-32768, 32767, (entries, cp, 128), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
             for _ in range(cp)]
    ins_s = [torch.randint(-2**31, 2**31 - 1, (entries, cp, 4), generator=g, dtype=torch.int32).view(torch.float32).cuda()
             for _ in range(cp)]
    results = []
    try:
        for r in range(cp):
            os.environ["HELIX_A2A_CHANNEL_COUNT"] = str(3 + 2 * r)
            results.append(hx.alltoall(ins_o[r], ins_s[r], ws, r, cp))
    finally:
        del os.environ["HELIX_A2A_CHANNEL_COUNT"]
    torch.cuda.synchronize()
    assert_clean(ops)
    check_against_oracle(ins_o, ins_s, [x[0] for x in results], [x[1] for x in results], with_numpy=False)


def test_abandoned_per_rank_exchange_expires(hx, ops, send_policy):
    # a group whose last ranks never call does not pin its tensors for ever: the next call after the expiry
    # time gives the exchange up and says what to do
    cp = 2
    ws = get_workspace(hx, cp, fresh=True)
    o = torch.zeros(4, cp, 64, dtype=torch.bfloat16, device="cuda")
    s = torch.zeros(4, cp, 2, device="cuda")
    ops.set_pending_expiry(0.0)
    try:
        hx.alltoall(o, s, ws, 0, cp)
        with pytest.raises(RuntimeError, match="waited more than"):
            hx.alltoall(o, s, ws, 0, cp)
    finally:
        ops.set_pending_expiry(120.0)
    assert not any(g.pending for g in ops._groups.values())
    torch.cuda.synchronize()
    for r in range(cp):   # with eager sends rank 0's lines sit in the FIFOs unreceived
        hx.init_workspace(ws, r, cp)
    # a group is found by its workspace's address and rank count
    ws2 = hx.allocate_workspace(cp, 0)
    for r in range(cp):
        hx.init_workspace(ws2, r, cp)
    hx.alltoall(o, s, ws2, 0, cp)
    key = (ws2.data_ptr(), cp)
    assert key in ops._groups
    torch.cuda.synchronize()
    # ... and keeps that workspace alive while ranks are waiting, whatever the caller does with its handle
    del ws2
    import gc
    gc.collect()
    assert ops._groups[key].pending and ops._groups[key].workspace is not None
    ops.reset_logical_ranks()
    assert not ops._groups


@pytest.mark.parametrize("single_round", [False, True])
def test_traffic_beyond_fifo_capacity(hx, ops, single_round):
    # 9000 messages of 17 pieces per stream on one channel = 10 FIFO entries. Default: three stream-ordered
    # rounds. single_round: one launch, senders wait in-kernel until receivers release entries.
    cp, entries = 2, 9000
    ws = get_workspace(hx, cp, fresh=True)
    g = torch.Generator().manual_seed(9)
    ins_o = [torch.randint(-32768, 32767, (entries, cp, 64), generator=g, dtype=torch.int16).view(torch.bfloat16).cuda()
             for _ in range(cp)]
    ins_s = [torch.randn(entries, cp, 2, generator=g).cuda() for _ in range(cp)]
    ops.set_single_round(single_round)
    try:
        outs_o, outs_s = hx.alltoall_loopback(ins_o, ins_s, ws, channel_count=1)
        torch.cuda.synchronize()
    finally:
        ops.set_single_round(False)
    assert_clean(ops)
    check_against_oracle(ins_o, ins_s, outs_o, outs_s)


@pytest.mark.parametrize("channels", [8, 16])
def test_receivers_overlapping_their_senders(hx, ops, channels):
    # With few channels every wavefront of the launch is resident at once and receivers poll FIFO
    # lines while their senders are still writing them. A receiver that consumed a line on the
    # strength of a flag it had read in the same pass as the payload could see a half-written line.
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS["c3"]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    want_o = expected_on_device(ins_o).view(torch.int16)
    want_s = expected_on_device(ins_s).view(torch.int32)
    plan = ops.LoopbackPlan(ins_o, ins_s, ws, channels)
    bad = torch.zeros((), dtype=torch.int64, device="cuda")
    for _ in range(150):
        for t in plan.out_o:
            t.zero_()
        outs_o, outs_s = plan.run()
        for r in range(w.cp):
            bad += (outs_o[r].view(torch.int16) != want_o[r]).sum() + (outs_s[r].view(torch.int32) != want_s[r]).sum()
    torch.cuda.synchronize()
    assert_clean(ops)
    assert int(bad.item()) == 0


# ---------------------------------------------------------------------------
# graph capture
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("name", ["c2", "c4"])
def test_exchange_and_combine_replay_from_a_captured_graph(hx, ops, name):
    # The FIFO step counters live in the workspace, not in the kernel arguments, so a captured
    # launch can be replayed: every replay walks on to the next FIFO entry. Replays are interleaved
    # with eager work and synchronisations, and every one of them is checked. c2: single-pass runs;
    # c4: long runs, whose wavefronts read every counter they start from -- their own and, at first,
    # their sender's -- through the scalar cache, which must not hold what the kernel before left there.
    from helix_workloads import WORKLOADS, make_inputs

    w = WORKLOADS[name]
    ws = get_workspace(hx, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    plan = ops.LoopbackPlan(ins_o, ins_s, ws)
    fused = ops.CombinePlan(ins_o, ins_s, ws, ops.STATS_MAX_SUM, return_lse=True)
    plan.run()
    fused.run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan.run()
        fused.run()
    torch.cuda.synchronize()
    assert_clean(ops)
    base_o = [t.clone() for t in ins_o]
    for replay in range(7):
        for r in range(w.cp):  # eager work between replays: new payload in the captured buffers
            ins_o[r].copy_((base_o[r].float() * (1.0 + 0.25 * replay)).to(torch.bfloat16))
        for t in plan.out_o + plan.out_s + fused.combined:
            t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert_clean(ops)
        check_against_oracle(ins_o, ins_s, plan.out_o, plan.out_s, with_numpy=False)
        # the same graph also ran the fused combine: compare with an eager fused call on the same inputs
        got = [c.clone() for c in fused.combined]
        got_lse = [l.clone() for l in fused.lse]
        eager_c, eager_l = hx.alltoall_combine_loopback(ins_o, ins_s, ws, hx.STATS_MAX_SUM, return_lse=True)
        torch.cuda.synchronize()
        for r in range(w.cp):
            assert torch.equal(got[r], eager_c[r]) and torch.equal(got_lse[r], eager_l[r]), f"replay {replay}, rank {r}"
    for r in range(w.cp):
        ins_o[r].copy_(base_o[r])


# ---------------------------------------------------------------------------
# helix_a2a_alltoall: both halves of one rank in one launch (what one process per GPU would call)
# ---------------------------------------------------------------------------

def test_single_rank_call_both_halves(hx, ops, unchecked):
    import ctypes

    # cp_size 1: the rank is its own peer, the launch sends and receives its own traffic
    ws = get_workspace(hx, 1)
    g = torch.Generator().manual_seed(17)
    o = torch.randn(50, 1, 256, generator=g).to(torch.bfloat16).cuda()
    s = torch.randn(50, 1, 4, generator=g).cuda()
    out_o, out_s = torch.empty_like(o), torch.empty_like(s)
    p = ops._make_params(o, s, out_o, out_s, ws, 0, 1, 0)
    ops._check(ops._lib.helix_a2a_alltoall(ctypes.byref(p), ops._stream_handle()), "alltoall")
    torch.cuda.synchronize()
    assert_clean(ops)
    assert bits_equal(out_o, o) and bits_equal(out_s, s)

    # cp_size 2 with only rank 0 calling: its receive half waits for rank 1, which never sends;
    # the bounded wait gives up, the kernel ends normally and the status word says so
    ws2 = get_workspace(hx, 2, fresh=True)
    o2 = torch.zeros(3, 2, 64, dtype=torch.bfloat16, device="cuda")
    s2 = torch.zeros(3, 2, 2, device="cuda")
    p2 = ops._make_params(o2, s2, torch.empty_like(o2), torch.empty_like(s2), ws2, 0, 2, 1)
    ops.set_spin_limit_us(0)
    try:
        ops._check(ops._lib.helix_a2a_alltoall(ctypes.byref(p2), ops._stream_handle()), "alltoall")
        torch.cuda.synchronize()
        status = ops.device_status()
    finally:
        ops.set_spin_limit_us(2_000_000)
    assert status & 1
    for r in range(2):
        hx.init_workspace(ws2, r, 2)


# ---------------------------------------------------------------------------
# nothing to exchange: zero entries is a valid call that launches nothing
# ---------------------------------------------------------------------------

def test_plain_c_host_drives_the_exchange(hx, ops):
    # tests/c_abi/gpu_host.c: hipMalloc + include/helix_a2a.h, no torch -- what a native binding would do
    import subprocess

    from helix_testing import C_ABI_HOST_EXE

    assert C_ABI_HOST_EXE.exists(), "build it with __graft_entry__.build() (tests/helix_testing.py::build_c_abi_host)"
    torch.cuda.synchronize()
    run = subprocess.run([str(C_ABI_HOST_EXE)], capture_output=True, text=True, timeout=100)
    assert run.returncode == 0 and "gpu_host ok" in run.stdout, run.stdout + run.stderr
    for what in ("loopback:", "loopback again:", "send halves + receive half:", "loopback through the built-in workspace:"):
        assert f"{what} 0 wrong element(s)" in run.stdout, run.stdout


def test_empty_inputs(hx, ops):
    cp = 4
    ws = get_workspace(hx, cp)
    o = [torch.empty(0, cp, 256, dtype=torch.bfloat16, device="cuda") for _ in range(cp)]
    s = [torch.empty(0, cp, 2, device="cuda") for _ in range(cp)]
    out_o, out_s = hx.alltoall_loopback(o, s, ws)
    assert all(t.shape == (0, cp, 256) for t in out_o) and all(t.shape == (0, cp, 2) for t in out_s)
    outs = [hx.alltoall(o[r], s[r], ws, cp_rank=r, cp_size=cp) for r in range(cp)]
    assert all(a.shape == (0, cp, 256) and b.shape == (0, cp, 2) for a, b in outs)
    combined = hx.alltoall_combine_loopback(o, s, ws, hx.STATS_LSE_PACKED)
    assert all(t.shape[0] == 0 for t in combined)
    torch.cuda.synchronize()
    assert_clean(ops)
    # the workspace was not touched: a real exchange right after still works
    g = torch.Generator().manual_seed(3)
    o1 = [torch.randn(5, cp, 256, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
    s1 = [torch.randn(5, cp, 2, generator=g).cuda() for _ in range(cp)]
    got_o, got_s = hx.alltoall_loopback(o1, s1, ws)
    torch.cuda.synchronize()
    check_against_oracle(o1, s1, got_o, got_s)


def test_per_rank_calls_on_separate_streams(hx, ops, send_policy):
    # every logical rank calls on a stream of its own and waits for that stream only
    cp, entries = 4, 96
    ws = get_workspace(hx, cp)
    g = torch.Generator().manual_seed(23)
    ins_o = [torch.randn(entries, cp, 1024, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
    ins_s = [torch.randn(entries, cp, 16, generator=g).cuda() for _ in range(cp)]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(cp)]
    for _ in range(3):
        outs = [None] * cp
        for r in (2, 0, 3, 1):
            with torch.cuda.stream(streams[r]):
                outs[r] = hx.alltoall(ins_o[r], ins_s[r], ws, cp_rank=r, cp_size=cp)
        snap = []
        for r in range(cp):
            streams[r].synchronize()          # only the rank's own stream
            snap.append((outs[r][0].clone(), outs[r][1].clone()))
        torch.cuda.synchronize()
        check_against_oracle(ins_o, ins_s, [a for a, _ in snap], [b for _, b in snap])
    assert_clean(ops)


def test_per_rank_calls_replay_from_a_captured_graph(hx, ops, send_policy):
    # the reference's signature, one call per logical rank, captured once and replayed on fresh payload
    cp, entries = 4, 64
    ws = get_workspace(hx, cp)
    g = torch.Generator().manual_seed(29)
    ins_o = [torch.randn(entries, cp, 512, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
    ins_s = [torch.randn(entries, cp, 8, generator=g).cuda() for _ in range(cp)]

    def run():
        return [hx.alltoall(ins_o[r], ins_s[r], ws, cp_rank=r, cp_size=cp) for r in range(cp)]

    for _ in range(2):
        run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run()
    torch.cuda.synchronize()
    for _ in range(4):
        for a, b in outs:
            a.zero_()
            b.zero_()
        for t in ins_o:
            t.add_(1.0)
        eager = run()                     # eager work between the replays, on the same workspace
        graph.replay()
        torch.cuda.synchronize()
        check_against_oracle(ins_o, ins_s, [a for a, _ in outs], [b for _, b in outs], with_numpy=False)
        check_against_oracle(ins_o, ins_s, [a for a, _ in eager], [b for _, b in eager], with_numpy=False)
    assert_clean(ops)


def test_reference_environment_switches(hx, ops, monkeypatch, send_policy):
    # HELIX_A2A_ENABLE_PDL (csrc/helix_alltoall.cu:541-548) is accepted and changes nothing: ordering between
    # calls is stream order. HELIX_A2A_CHANNEL_COUNT (csrc/torch_binding.cpp:25-32) is honoured, re-read per call.
    cp = 4
    ws = get_workspace(hx, cp)
    g = torch.Generator().manual_seed(31)
    ins_o = [torch.randn(40, cp, 256, generator=g).to(torch.bfloat16).cuda() for _ in range(cp)]
    ins_s = [torch.randn(40, cp, 4, generator=g).cuda() for _ in range(cp)]
    for pdl in ("0", "1"):
        monkeypatch.setenv("HELIX_A2A_ENABLE_PDL", pdl)
        for channels in ("", "3", "40", "1"):
            if channels:
                monkeypatch.setenv("HELIX_A2A_CHANNEL_COUNT", channels)
            else:
                monkeypatch.delenv("HELIX_A2A_CHANNEL_COUNT", raising=False)
            outs = [hx.alltoall(ins_o[r], ins_s[r], ws, cp_rank=r, cp_size=cp) for r in range(cp)]
            torch.cuda.synchronize()
            check_against_oracle(ins_o, ins_s, [a for a, _ in outs], [b for _, b in outs], with_numpy=False)
    monkeypatch.setenv("HELIX_A2A_CHANNEL_COUNT", "100000")      # more than the layout provides
    with pytest.raises(RuntimeError, match="max_channel_count"):
        hx.alltoall(ins_o[0], ins_s[0], ws, cp_rank=0, cp_size=cp)
    ops.reset_logical_ranks()
    assert_clean(ops)
