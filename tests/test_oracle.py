"""Pins the CPU oracle (oracle/) before anything is compared with it.

Every check here is independent of the oracle's own formulas: the reference's
test-held closed forms and vectors, hand-derived known answers for the LL128
block shuffling, library routines (scipy) for the combine, brute force on tiny
inputs, and invariants a plausible mistake would break.
"""
import numpy as np
import pytest

from helix_testing import coded_inputs, random_inputs
from oracle import helix_oracle as ho

H100 = 132


# ---------------------------------------------------------------------------
# sizes
# ---------------------------------------------------------------------------

def _size_like_reference_test(cp_size, sm_count):
    # the computation of the reference's own test, tests/test_phase2.py:13-35
    max_group = min(cp_size, 8)
    blocks_per_ch = ((cp_size + max_group - 1) // max_group) * 2
    max_channels = max(sm_count // blocks_per_ch, 1)
    fifo = 512 * 1024 * cp_size * max_channels
    info = 256 * cp_size * max_channels * 2
    return fifo + info, max_channels


@pytest.mark.parametrize("sm_count", [1, 2, 3, 108, 132, 256, 304])
@pytest.mark.parametrize("cp_size", [1, 2, 4, 8, 9, 16])
def test_workspace_size_closed_form(ref_model, cp_size, sm_count):
    want, want_ch = _size_like_reference_test(cp_size, sm_count)
    assert ref_model.workspace_size(cp_size, sm_count) == want
    assert ref_model.max_channel_count(cp_size, sm_count) == want_ch
    assert ho.workspace_size(cp_size, sm_count) == want
    assert ho.max_channel_count(cp_size, sm_count) == want_ch


def test_workspace_size_known_values(ref_model):
    # 256 compute units: (524288 + 512) * cp * 128 for cp <= 8, 64 channels at cp = 16
    assert ref_model.workspace_size(2, 256) == 134_348_800
    assert ref_model.workspace_size(4, 256) == 268_697_600
    assert ref_model.workspace_size(8, 256) == 537_395_200
    assert ref_model.workspace_size(16, 256) == 537_395_200
    # 132 SMs, cp = 8: 66 channels
    assert ref_model.workspace_size(8, H100) == 524_800 * 8 * 66
    # the stale stub value the reference's test rejects (tests/test_phase2.py:38-45)
    assert ref_model.workspace_size(4, H100) != 16_778_240
    assert ref_model.workspace_size(4, 256) != 16_778_240


def test_init_pattern(ref_model):
    # tests/test_phase2.py:48-62: FIFO region all ones, the rest of the row zero, other rows untouched
    cp, sm = 4, 8
    ws = ref_model.new_workspace(cp, sm)
    ws[:] = 0x5A5A5A5A
    ref_model.init_workspace(ws, 1, cp, sm)
    fifo_elems = 512 * 1024 * cp * _size_like_reference_test(cp, sm)[1] // 8
    assert fifo_elems == ho.fifo_region_elems(cp, sm)
    assert (ws[1, :fifo_elems] == -1).all()
    assert (ws[1, fifo_elems:] == 0).all()
    for other in (0, 2, 3):
        assert (ws[other] == 0x5A5A5A5A).all()
    assert ws.shape[1] * 8 == ref_model.workspace_size(cp, sm)


# message sizes on the reference wire: (field0, field1) -> (unpacked, proto, messages per 128 KiB entry)
# hand-derived: unpacked = align128(f0 + f1), proto = unpacked + 128 * ceil(unpacked / 1920)
WIRE = {
    (1024, 32): (1152, 1280, 102),
    (2048, 64): (2176, 2432, 53),
    (16384, 128): (16512, 17664, 7),
    (512, 16): (640, 768, 170),
    (1152, 48): (1280, 1408, 93),
    (256, 8): (384, 512, 256),
    (192, 8): (256, 384, 341),
}


@pytest.mark.parametrize("fields,want", WIRE.items())
def test_wire_sizes(ref_model, fields, want):
    unpacked = ref_model.unpacked_size(*fields)
    proto = ref_model.proto_size(unpacked)
    assert (unpacked, proto, 131072 // proto) == want


def test_channel_and_group_count(ref_model):
    # 8 warps of 2432 B fit easily: 2 blocks per channel on 132 SMs -> 66 channels
    assert ref_model.channel_and_group_count(8, 2048, 64, 132, 232448) == (66, 8)
    assert ref_model.channel_and_group_count(16, 512, 16, 132, 232448) == (33, 8)
    assert ref_model.channel_and_group_count(2, 1024, 32, 132, 232448) == (66, 2)
    # 17664 B per warp with 48 KiB of shared memory: 2 warps per block, 8 blocks per channel
    assert ref_model.channel_and_group_count(8, 16384, 128, 132, 49152) == (16, 2)
    # nothing fits
    assert ref_model.channel_and_group_count(8, 16384, 128, 132, 1024)[0] == -1


# ---------------------------------------------------------------------------
# LL128 block shuffling of the reference layout
# ---------------------------------------------------------------------------

STEP = 0x0123456789ABCDEF


def _blocks(p_blocks, tails, seed=0):
    rng = np.random.default_rng(seed)
    shm = np.zeros((p_blocks + tails) * 16, dtype=np.uint64)
    shm[: p_blocks * 16] = rng.integers(1, 1 << 62, size=p_blocks * 16, dtype=np.uint64)
    return shm


def test_pack_known_answer_one_block(ref_model):
    # P = 1, base = 0: block 0 gives up word 0; tail block 1 has its flag in word (0+1)%16 = 1,
    # so the displaced word lands in tail word 0 and everything else in the tail is the step.
    shm = _blocks(1, 1)
    orig = shm.copy()
    ref_model.proto_pack(shm, STEP, 1, 0)
    want = orig.copy()
    want[0] = STEP
    want[16] = orig[0]
    want[17:32] = STEP
    assert (shm == want).all()


def test_pack_known_answer_two_blocks_offset_base(ref_model):
    # P = 2, base = 5: flags in block0[5], block1[6]; tail is block 2 with flag word (5+2)%16 = 7
    shm = _blocks(2, 1)
    orig = shm.copy()
    ref_model.proto_pack(shm, STEP, 2, 5)
    want = orig.copy()
    want[5] = STEP
    want[16 + 6] = STEP
    tail = np.full(16, STEP, dtype=np.uint64)
    tail[0] = orig[5]
    tail[1] = orig[16 + 6]
    want[32:48] = tail
    assert (shm == want).all()


def test_pack_known_answer_two_tail_blocks(ref_model):
    # P = 16, base = 3: blocks 0..14 use tail block 16 (flag word (3+16)%16 = 3),
    # block 15 uses tail block 17 (flag word 4)
    shm = _blocks(16, 2)
    orig = shm.copy().reshape(18, 16)
    ref_model.proto_pack(shm, STEP, 16, 3)
    got = shm.reshape(18, 16)
    tail16 = np.full(16, STEP, dtype=np.uint64)
    for j in range(15):
        tail16[j + 1 if j >= 3 else j] = orig[j, (3 + j) % 16]
    tail17 = np.full(16, STEP, dtype=np.uint64)
    tail17[0] = orig[15, (3 + 15) % 16]
    assert (got[16] == tail16).all()
    assert (got[17] == tail17).all()
    for b in range(16):
        row = orig[b].copy()
        row[(3 + b) % 16] = STEP
        assert (got[b] == row).all()


@pytest.mark.parametrize("p_blocks", [1, 2, 9, 14, 15, 16, 17, 29, 30, 31, 45, 129])
@pytest.mark.parametrize("base", [0, 1, 7, 15, 16, 1000])
def test_pack_flags_roundtrip_and_conservation(ref_model, p_blocks, base):
    tails = -(-p_blocks // 15)
    shm = _blocks(p_blocks, tails, seed=p_blocks * 31 + base)
    orig = shm.copy()
    ref_model.proto_pack(shm, STEP, p_blocks, base)
    total = p_blocks + tails
    # every block on the wire carries the step in word (base + b) % 16
    for b in range(total):
        assert shm[b * 16 + (base + b) % 16] == STEP
    assert ref_model.check_received(shm, STEP, total, base, 0) == total
    # nothing is lost: the data words are all still there, the rest is the step value
    data_words = np.sort(orig[: p_blocks * 16])
    wire_words = shm[shm != STEP]
    assert (np.sort(wire_words) == data_words).all()
    # unpack restores the data blocks exactly
    ref_model.proto_unpack(shm, p_blocks, base)
    assert (shm[: p_blocks * 16] == orig[: p_blocks * 16]).all()


def test_check_received_is_prefix_length(ref_model):
    p_blocks, base = 40, 9
    tails = 3
    shm = _blocks(p_blocks, tails, seed=5)
    ref_model.proto_pack(shm, STEP, p_blocks, base)
    total = p_blocks + tails
    for hole in (0, 1, 31, 32, 33, 42):
        broken = shm.copy()
        broken[hole * 16 + (base + hole) % 16] = STEP ^ 1
        assert ref_model.check_received(broken, STEP, total, base, 0) == hole
        assert ref_model.check_received(broken, STEP, total, base, min(hole, 5)) == hole - min(hole, 5)
    # all-ones (the initial FIFO content) never matches a step counter
    ones = np.full_like(shm, np.uint64(0xFFFFFFFFFFFFFFFF))
    assert ref_model.check_received(ones, 0, total, base, 0) == 0


# ---------------------------------------------------------------------------
# the exchange
# ---------------------------------------------------------------------------

def _brute_force(ins):
    cp = len(ins)
    outs = [np.zeros_like(a) for a in ins]
    for r in range(cp):
        for s in range(cp):
            for e in range(ins[0].shape[0]):
                for i in range(ins[0].shape[2]):
                    outs[r][e, s, i] = ins[s][e, r, i]
    return outs


def test_closed_form_matches_brute_force():
    ins_o, ins_s = coded_inputs(cp=3, entries=4, x=8, s=2)
    for ins in (ins_o, ins_s):
        got = ho.exchange_closed_form(ins)
        want = _brute_force(ins)
        for g, w in zip(got, want):
            assert (g == w).all()


def test_closed_form_is_an_involution_and_a_permutation():
    ins_o, _ = random_inputs(cp=4, entries=6, x=16, s=2, seed=3)
    once = ho.exchange_closed_form(ins_o)
    twice = ho.exchange_closed_form(once)
    for a, b in zip(ins_o, twice):
        assert (a == b).all()
    assert (np.sort(np.concatenate([a.ravel() for a in ins_o])) ==
            np.sort(np.concatenate([a.ravel() for a in once]))).all()
    # cp = 1 is a copy
    solo, _ = random_inputs(cp=1, entries=5, x=8, s=2, seed=4)
    assert (ho.exchange_closed_form(solo)[0] == solo[0]).all()


def _run_model(ref_model, ins_o, ins_s, sm, channel_count=0, schedule=0, workspace=None, init=True):
    cp = len(ins_o)
    ws = workspace if workspace is not None else ref_model.new_workspace(cp, sm)
    if init:
        for r in range(cp):
            ref_model.init_workspace(ws, r, cp, sm)
    outs = ref_model.alltoall_all_ranks(ins_o, ins_s, ws, sm_count=sm, channel_count=channel_count, schedule=schedule)
    return outs, ws


@pytest.mark.parametrize("schedule", [0, 1])
@pytest.mark.parametrize("cp,entries,x,s", [
    (2, 8, 512, 8),      # the CPU-runnable config: H/cp = 4 heads of D = 128
    (4, 5, 64, 2),       # per-head layout, field 1 is one float2
    (3, 7, 8, 6),        # field 1 not a multiple of 16 bytes
    (8, 3, 1024, 16),
    (4, 37, 576, 12),    # 1200-byte payload, the tail shape
    (1, 4, 64, 2),
])
def test_model_equals_closed_form(ref_model, cp, entries, x, s, schedule):
    ins_o, ins_s = random_inputs(cp, entries, x, s, seed=cp * 100 + entries)
    (got_o, got_s), _ = _run_model(ref_model, ins_o, ins_s, sm=8, schedule=schedule)
    for r in range(cp):
        assert (got_o[r] == ho.exchange_closed_form(ins_o)[r]).all()
        assert (got_s[r] == ho.exchange_closed_form(ins_s)[r]).all()


def test_model_coded_payload_tiny(ref_model):
    ins_o, ins_s = coded_inputs(cp=2, entries=3, x=8, s=2)
    (got_o, got_s), _ = _run_model(ref_model, ins_o, ins_s, sm=4)
    want_o, want_s = _brute_force(ins_o), _brute_force(ins_s)
    for r in range(2):
        assert (got_o[r] == want_o[r]).all() and (got_s[r] == want_s[r]).all()


@pytest.mark.parametrize("schedule", [0, 1])
def test_model_backpressure_and_fifo_wrap(ref_model, schedule):
    # one channel, 1280-byte wire messages: 102 per entry, so 900 entries need 9 FIFO entries per
    # stream, more than the 4 that exist: senders must wait for receivers, entries are reused
    cp, entries = 2, 900
    ins_o, ins_s = random_inputs(cp, entries, 512, 8, seed=11)
    (got_o, got_s), ws = _run_model(ref_model, ins_o, ins_s, sm=2, channel_count=1, schedule=schedule)
    want_o, want_s = ho.exchange_closed_form(ins_o), ho.exchange_closed_form(ins_s)
    for r in range(cp):
        assert (got_o[r] == want_o[r]).all() and (got_s[r] == want_s[r]).all()
    # counters: 9 entries consumed by every stream, head == tail on both sides
    fifo_elems = ho.fifo_region_elems(cp, 2)
    info = ws[:, fifo_elems:].reshape(cp, 2, cp, 1, 32)  # [row, sender/receiver info, peer, channel, 256 B]
    assert (info[:, 0, :, 0, 0] == 9).all()  # sender head
    assert (info[:, 0, :, 0, 1] == 9).all()  # sender's copy of tail
    assert (info[:, 1, :, 0, 1] == 9).all()  # receiver tail


def test_model_repeated_calls_and_reinit(ref_model):
    cp, sm = 4, 16
    ws = ref_model.new_workspace(cp, sm)
    for r in range(cp):
        ref_model.init_workspace(ws, r, cp, sm)
    for call in range(6):  # more calls than FIFO entries: every entry is reused with a new step value
        ins_o, ins_s = random_inputs(cp, 9, 128, 4, seed=call)
        (got_o, got_s), _ = _run_model(ref_model, ins_o, ins_s, sm, workspace=ws, init=(call == 3))
        want_o, want_s = ho.exchange_closed_form(ins_o), ho.exchange_closed_form(ins_s)
        for r in range(cp):
            assert (got_o[r] == want_o[r]).all() and (got_s[r] == want_s[r]).all()


def test_model_fill_vectors(ref_model):
    # tests/test_mnnvl.py:177-213: rank r sends the constant r+1 (bf16) and 0.1*(r+1); slot j holds j+1
    import torch

    cp, n, d = 4, 4, 64
    ins_o = [torch.full((n, cp, d), float(r + 1), dtype=torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
             for r in range(cp)]
    ins_s = [np.full((n, cp, 2), 0.1 * (r + 1), dtype=np.float32).view(np.uint32) for r in range(cp)]
    (got_o, got_s), _ = _run_model(ref_model, ins_o, ins_s, sm=8)
    for r in range(cp):
        o = torch.from_numpy(got_o[r].view(np.int16)).view(torch.bfloat16).float()
        for j in range(cp):
            assert (o[:, j, :] == float(j + 1)).all()
            assert (got_s[r].view(np.float32)[:, j, :] == np.float32(0.1 * (j + 1))).all()
        assert got_o[r].shape == (n, cp, d) and got_s[r].shape == (n, cp, 2)


@pytest.mark.parametrize("dtype_name", ["bfloat16", "float16"])
def test_seeded_full_tensor_construction(ref_model, dtype_name):
    # tests/test_alltoall.py:303-360: all ranks derive their send buffer from one seeded tensor
    # full[B, cp, cp, D]; rank r sends full[:, :, r, :] and must receive full[:, r, :, :]
    import torch

    dtype = getattr(torch, dtype_name)
    cp, b, d, s = 4, 4, 128, 2
    torch.manual_seed(42)
    full_o = torch.randn(b, cp, cp, d, dtype=dtype)
    full_s = torch.randn(b, cp, cp, s, dtype=torch.float32)
    sends_o = [full_o[:, :, r, :].contiguous() for r in range(cp)]
    sends_s = [full_s[:, :, r, :].contiguous() for r in range(cp)]
    ins_o = [t.view(torch.int16).numpy().view(np.uint16) for t in sends_o]
    ins_s = [t.numpy().view(np.uint32) for t in sends_s]
    (got_o, got_s), _ = _run_model(ref_model, ins_o, ins_s, sm=8)
    via_transposes_o = ho.exchange_transpose_style(sends_o)
    via_transposes_s = ho.exchange_transpose_style(sends_s)
    for r in range(cp):
        want_o = full_o[:, r, :, :].contiguous()
        want_s = full_s[:, r, :, :].contiguous()
        assert (got_o[r] == want_o.view(torch.int16).numpy().view(np.uint16)).all()
        assert (got_s[r] == want_s.numpy().view(np.uint32)).all()
        assert torch.equal(via_transposes_o[r], want_o) and torch.equal(via_transposes_s[r], want_s)


def test_transpose_style_and_single_copy_equal_closed_form():
    import torch

    ins_o, ins_s = random_inputs(cp=4, entries=6, x=32, s=4, seed=8)
    want = ho.exchange_closed_form(ins_s)
    tens = [torch.from_numpy(a.view(np.int32)) for a in ins_s]
    got = ho.exchange_transpose_style(tens)
    single = ho.exchange_single_copy(tens)
    for r in range(4):
        assert (got[r].numpy().view(np.uint32) == want[r]).all()
        assert (single[r].numpy().view(np.uint32) == want[r]).all()


# ---------------------------------------------------------------------------
# combine
# ---------------------------------------------------------------------------

def test_combine_against_scipy():
    from scipy.special import logsumexp, softmax

    rng = np.random.default_rng(0)
    n, b, h, d = 5, 3, 4, 8
    o = rng.standard_normal((n, b, h, d))
    lse = rng.standard_normal((n, b, h)) * 3
    got, glse = ho.lse_combine(o, lse, dtype=np.float64)
    w = softmax(lse, axis=0)
    want = (o * w[..., None]).sum(axis=0)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    assert np.allclose(glse, logsumexp(lse, axis=0), rtol=1e-12, atol=1e-12)


def test_combine_special_cases():
    rng = np.random.default_rng(1)
    n, b, h, d = 4, 2, 3, 8
    o = rng.standard_normal((n, b, h, d)).astype(np.float32)
    # one shard: identity, global lse is that shard's lse
    c, g = ho.lse_combine(o[:1], np.full((1, b, h), 0.7, np.float32))
    assert np.array_equal(c, o[0]) and np.allclose(g, 0.7)
    # equal lse: arithmetic mean, global lse = lse + ln n
    c, g = ho.lse_combine(o, np.full((n, b, h), -1.25, np.float32))
    assert np.allclose(c, o.mean(axis=0), atol=1e-6) and np.allclose(g, -1.25 + np.log(n), atol=1e-6)
    # a shard at -inf (fully masked) or NaN or +inf is excluded
    for bad in (-np.inf, np.nan, np.inf):
        lse = np.zeros((n, b, h), np.float32)
        lse[2] = bad
        c, _ = ho.lse_combine(o, lse)
        assert np.allclose(c, o[[0, 1, 3]].mean(axis=0), atol=1e-6)
    # everything masked: zeros, global lse -inf
    c, g = ho.lse_combine(o, np.full((n, b, h), -np.inf, np.float32))
    assert (c == 0).all() and np.isneginf(g).all()
    # a shift of all lses does not change the weights
    lse = rng.standard_normal((n, b, h)).astype(np.float32)
    c1, g1 = ho.lse_combine(o, lse)
    c2, g2 = ho.lse_combine(o, lse + 10)
    assert np.allclose(c1, c2, atol=1e-5) and np.allclose(g1 + 10, g2, atol=1e-5)


def test_combine_brute_force_and_stats_modes():
    rng = np.random.default_rng(2)
    e, cp, heads, d = 3, 4, 2, 4
    o = rng.standard_normal((e, cp, heads * d)).astype(np.float32)
    mx = rng.standard_normal((e, cp, heads)).astype(np.float32) * 2
    sm = (1 + rng.random((e, cp, heads)) * 63).astype(np.float32)
    stats = np.stack((mx, sm), axis=-1).reshape(e, cp, 2 * heads)
    got, glse = ho.combine_after_exchange(o, stats, heads, mode=1, dtype=np.float64)
    for t in range(e):
        for hh in range(heads):
            num = np.zeros(d)
            den = 0.0
            for s in range(cp):
                wgt = float(sm[t, s, hh]) * np.exp(float(mx[t, s, hh]))
                num += wgt * o[t, s, hh * d:(hh + 1) * d].astype(np.float64)
                den += wgt
            assert np.allclose(got[t, hh * d:(hh + 1) * d], num / den, rtol=1e-6, atol=1e-9)
            assert np.isclose(glse[t, hh], np.log(den), rtol=1e-6)
    # mode 0 reads slot 0 as the lse and ignores slot 1
    lse_stats = stats.copy()
    lse_stats[..., 1::2] = 12345.0
    got0, _ = ho.combine_after_exchange(o, lse_stats, heads, mode=0, dtype=np.float64)
    lse = mx.transpose(1, 0, 2)
    want0, _ = ho.lse_combine(o.reshape(e, cp, heads, d).transpose(1, 0, 2, 3), lse, dtype=np.float64)
    assert np.allclose(got0, want0.reshape(e, heads * d))


def test_bf16_widening():
    import torch

    t = torch.randn(257, dtype=torch.float32).to(torch.bfloat16)
    bits = t.view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ho.bf16_bits_to_f32(bits), t.float().numpy())
    h = torch.randn(257).to(torch.float16)
    assert np.array_equal(ho.f16_bits_to_f32(h.view(torch.int16).numpy().view(np.uint16)), h.float().numpy())


def test_combine_packed_lse_mode_equals_padded_mode():
    rng = np.random.default_rng(4)
    e, cp, heads, d = 3, 4, 6, 8
    o = rng.standard_normal((e, cp, heads * d)).astype(np.float32)
    lse = (rng.standard_normal((e, cp, heads)) * 3).astype(np.float32)
    padded = np.stack((lse, np.zeros_like(lse)), axis=-1).reshape(e, cp, 2 * heads)
    got2, l2 = ho.combine_after_exchange(o, lse, heads, mode=2)
    got0, l0 = ho.combine_after_exchange(o, padded, heads, mode=0)
    assert np.array_equal(got2, got0) and np.array_equal(l2, l0)
