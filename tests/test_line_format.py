"""CPU checks of the build's own LL128 line format and workspace geometry.

They run the bounds-checked host walk-through of the GPU wave programs
(tests/host_model, built on csrc/helix_ll128.hpp) and compare its result with
the oracle, and they inspect the FIFO image it leaves behind.
"""
import numpy as np
import pytest

from helix_testing import FIFO_BYTES, FIFO_ENTRY_BYTES, INFO_BYTES, coded_inputs, random_inputs
from oracle import helix_oracle as ho

CU = 8  # a small device: 4 channels at cp <= 8 keeps host workspaces small


def _exchange(host_model, ins_o, ins_s, channels, cu=CU, ws=None):
    cp = len(ins_o)
    ws = ws if ws is not None else host_model.new_workspace(cp, cu)
    out_o, out_s, rc, msg = host_model.alltoall(ins_o, ins_s, ws, cu, channels)
    assert rc == 0, msg
    return out_o, out_s, ws


@pytest.mark.parametrize("cp,entries,x,s,channels", [
    (2, 8, 512, 8, 4),     # 1056-byte payload: 8.8 lines
    (2, 8, 512, 8, 1),
    (4, 64, 64, 2, 3),     # per-head layout, 136-byte payload: 2 lines, the second nearly empty
    (8, 5, 1024, 16, 4),   # 2112 bytes: 17.6 lines
    (4, 37, 576, 12, 4),   # 1200 bytes: exactly 10 lines
    (4, 37, 48, 2, 2),     # 104 bytes: less than one line
    (3, 11, 8, 6, 1),      # 40 bytes, odd cp, stats not a multiple of 16 bytes
    (1, 9, 64, 2, 2),
    (16, 3, 256, 4, 2),
    (2, 2, 8192, 32, 1),   # 16512 bytes: 138 lines
    # runs of several passes: receivers realign the payload to 16-byte stores
    (3, 40, 136, 10, 2),   # 312 bytes = 3 lines (odd), 20 messages per stream
    (2, 200, 8, 6, 2),     # 40 bytes = one line per message, 100 messages per stream
    (5, 26, 600, 2, 2),    # 1208 bytes = 11 lines, the pass boundary falls inside a message
    (4, 12, 1016, 14, 1),  # 2088 bytes = 18 lines with 56 bytes of statistics astride two lines
    (2, 3, 61432, 2, 1),   # 122872 bytes = 1024 lines: one message per FIFO entry
    (16, 64, 264, 2, 2),   # 536 bytes = 5 lines, 16 ranks
    (32, 3, 64, 2, 1),     # the largest rank count of an exchange
    (24, 7, 200, 4, 1),
])
def test_host_model_matches_oracle(host_model, cp, entries, x, s, channels):
    ins_o, ins_s = random_inputs(cp, entries, x, s, seed=cp + entries + x)
    out_o, out_s, _ = _exchange(host_model, ins_o, ins_s, channels)
    want_o, want_s = ho.exchange_closed_form(ins_o), ho.exchange_closed_form(ins_s)
    for r in range(cp):
        assert (out_o[r] == want_o[r]).all()
        assert (out_s[r] == want_s[r]).all()


def test_host_model_matches_reference_model(host_model, ref_model):
    # same inputs through the reference algorithm (its own wire format) and through this build's
    ins_o, ins_s = coded_inputs(cp=4, entries=6, x=64, s=4)
    out_o, out_s, _ = _exchange(host_model, ins_o, ins_s, channels=2)
    ws = ref_model.new_workspace(4, 8)
    for r in range(4):
        ref_model.init_workspace(ws, r, 4, 8)
    ref_o, ref_s = ref_model.alltoall_all_ranks(ins_o, ins_s, ws, sm_count=8)
    for r in range(4):
        assert (out_o[r] == ref_o[r]).all() and (out_s[r] == ref_s[r]).all()


def test_line_layout_in_fifo(host_model):
    # one message of 1056 bytes = 132 pieces -> 9 lines; look at what the sender wrote
    cp, entries, x, s = 2, 1, 512, 8
    ins_o, ins_s = random_inputs(cp, entries, x, s, seed=1)
    ws = host_model.new_workspace(cp, CU)
    _, _, rc, msg = host_model.alltoall(ins_o, ins_s, ws, CU, 1, send=True, recv=False)
    assert rc == 0, msg
    max_ch = host_model.max_channel_count(cp, CU)
    assert host_model.lib.hm_msg_lines(2 * x, 4 * s) == 9
    fifo_region = FIFO_BYTES * cp * max_ch
    for receiver in range(cp):
        region = ws[receiver].view(np.uint64)[: fifo_region // 8]
        untouched = np.ones(region.size, dtype=bool)
        for sender in range(cp):
            # a launch packs its streams: runs shorter than 8 KiB sit 16 KiB apart, in the quarter of step & 3
            off = host_model.stream_fifo_offset(sender, 0, 1, 9, cp, CU)
            assert off == sender * 16384
            lines = region[off // 8: off // 8 + 9 * 16].reshape(9, 16)
            untouched[off // 8: off // 8 + 9 * 16] = False
            payload = np.concatenate([ins_o[sender][0, receiver].view(np.uint64), ins_s[sender][0, receiver].view(np.uint64)])
            assert payload.size == 132
            padded = np.zeros(9 * 15, dtype=np.uint64)
            padded[:132] = payload
            assert (lines[:, :15] == padded.reshape(9, 15)).all()   # 15 payload words per line, in order
            assert (lines[:, 15] == 0).all()                        # flag word = step 0 of a fresh workspace
        assert (region[untouched] == np.uint64(0xFFFFFFFFFFFFFFFF)).all()  # nothing else was touched
    # counters: each sender stream consumed one FIFO entry; the receiver has not run
    for sender in range(cp):
        for receiver in range(cp):
            so = host_model.lib.hm_sender_info_offset(cp, max_ch, receiver, 0)
            assert so == fifo_region + (receiver * max_ch) * INFO_BYTES
            head, tail = ws[sender][so // 8], ws[sender][so // 8 + 1]
            assert (head, tail) == (1, 0)
            ro = host_model.lib.hm_receiver_info_offset(cp, max_ch, sender, 0)
            assert ro == fifo_region + INFO_BYTES * cp * max_ch + (sender * max_ch) * INFO_BYTES
            assert ws[receiver][ro // 8 + 1] == 0


def test_packed_layout_keeps_the_streams_of_a_launch_apart(host_model):
    # a launch packs its streams inside a quarter of the FIFO region: every slot holds the largest run, no two
    # streams overlap, everything stays inside the quarter, and the four positions are a quarter apart
    assert host_model.lib.hm_packed_slot_bytes(8) == 16384                 # one line
    assert host_model.lib.hm_packed_slot_bytes(36 * 8) == 16384            # 4.5 KiB: short runs sit 16 KiB apart
    assert host_model.lib.hm_packed_slot_bytes(63 * 8) == 16384
    assert host_model.lib.hm_packed_slot_bytes(64 * 8) == 8192             # from 8 KiB on: whole KiB
    assert host_model.lib.hm_packed_slot_bytes(71 * 8) == 9216
    assert host_model.lib.hm_packed_slot_bytes(138 * 8) == 18432
    assert host_model.lib.hm_packed_slot_bytes(1024 * 8) == FIFO_ENTRY_BYTES  # the longest run there is
    for cu in (16, 256):
        for cp in (1, 2, 3, 8, 16, 32):
            max_ch = host_model.max_channel_count(cp, cu)
            quarter = FIFO_ENTRY_BYTES * cp * max_ch
            for run_channels in sorted({1, 2, max_ch}):
                for lines in (1, 36, 63, 64, 71, 138, 1000, 1024):
                    slot = host_model.lib.hm_packed_slot_bytes(lines * 8)
                    assert slot >= lines * 128
                    offs = sorted(host_model.stream_fifo_offset(s, ch, run_channels, lines, cp, cu)
                                  for s in range(cp) for ch in range(run_channels))
                    assert offs[0] == 0 and all(b - a >= slot for a, b in zip(offs, offs[1:]))
                    assert offs[-1] + slot <= quarter
                    positions = host_model.lib.hm_fifo_positions(cp, run_channels, lines * 8, 1)
                    assert positions in (1, 2, 4)
                    for step in range(9):
                        assert (host_model.stream_fifo_offset(cp - 1, run_channels - 1, run_channels, lines, cp, cu, step)
                                == offs[-1] + (step % positions) * quarter)
                        assert (host_model.stream_fifo_offset(cp - 1, run_channels - 1, run_channels, lines, cp, cu, step, 3)
                                == offs[-1] + (step % 4) * quarter)     # several entries per stream: all four
            assert 4 * quarter == FIFO_BYTES * cp * max_ch      # the four quarters are the reference's FIFO region
    # positions: all four while the lines of four positions and the tensors fit the memory-side cache, then two, then one;
    # a launch in which a stream opens several entries always rotates through four
    pos = host_model.lib.hm_fifo_positions
    assert pos(8, 128, 36 * 8, 1) == 4          # c3: 37.7 MB of lines per launch
    assert pos(8, 128, 54 * 8, 1) == 2          # cp = 8, T = 384: 56.6 MB
    assert pos(8, 128, 71 * 8, 1) == 1          # cp = 8, T = 512: 74.4 MB
    assert pos(8, 128, 138 * 8, 1) == 1         # c4: 144.7 MB
    assert pos(16, 64, 71 * 8, 1) == 1          # c5a: 148.9 MB
    assert pos(8, 128, 138 * 8, 2) == 4 and pos(2, 1, 1024 * 8, 4) == 4
    assert pos(2, 8, 9 * 8, 1) == 4             # c1
    big = host_model.stream_fifo_offset(1, 2, 128, 138, 8, 256, step=7)
    assert big == host_model.stream_fifo_offset(1, 2, 128, 138, 8, 256, step=0)   # one position: every step in place


def test_unit_to_piece_map_covers_every_piece_once(host_model):
    for lines in (1, 2, 9, 18, 138):
        seen = []
        for g in range(8 * lines):
            p0 = host_model.lib.hm_unit_first_piece(g)
            seen.append(p0)
            if g % 8 != 7:
                seen.append(p0 + 1)
        assert seen == list(range(15 * lines))


def test_piece_division_is_exact(host_model):
    # the multiply-high that replaces g / np must be exact for every run piece of a FIFO entry (g < 15 360)
    # and every message size that fits one (3 <= np <= 15 360); every np up to 2048, then a sample
    sizes = list(range(1, 2049)) + list(range(2049, 15361, 97)) + [15359, 15360]
    for d in sizes:
        assert host_model.lib.hm_div_mismatches(d) == 0, d
    assert [host_model.lib.hm_div(g, 33) for g in (0, 32, 33, 65, 66, 15359)] == [0, 0, 1, 1, 2, 465]


def test_statistics_pieces_of_a_pass_fit_the_senders_gather(host_model):
    # A sender fetches the statistics pieces of a pass -- K * 120 consecutive run pieces -- with at most two loads of
    # 64 lanes, lane j taking the j-th of them. The count of statistics pieces before a run piece must be what
    # counting them one by one gives, and the K the launch rule allows a shape must keep every pass within 128.
    lib = host_model.lib
    shapes = [(5, 2), (3, 2), (2, 1), (33, 32), (66, 64), (264, 256), (2064, 2048), (129, 128), (9, 8), (24, 8), (100, 3),
              (15360, 15359), (15360, 15000), (300, 172), (7, 1), (120, 60), (121, 1)]
    for np, np0 in shapes:
        ns = np - np0
        run_pieces = (15360 // np) * np
        before = [0] * (run_pieces + 1)          # statistics pieces before run piece P, counted one by one
        for P in range(run_pieces):
            before[P + 1] = before[P] + (1 if P % np >= np0 else 0)
        for P in list(range(0, min(run_pieces, 3 * np) + 1)) + list(range(0, run_pieces + 1, 120)) + [run_pieces]:
            assert lib.hm_stats_ordinal_at(P, np, np0) == before[P], (np, np0, P)
        k = lib.hm_max_units_for_statistics(np, np0)
        assert 1 <= k <= 6
        most = max(before[min(P + k * 120, run_pieces)] - before[P] for P in range(0, run_pieces, 120))
        assert most <= 128, (np, np0, k, most)
        if k < 6:   # the rule is not needlessly strict: one more unit per lane could overflow some shape's window bound
            assert ((k + 1) * 120 // np + 2) * ns > 128
    assert lib.hm_max_units_for_statistics(264, 256) == 6 and lib.hm_max_units_for_statistics(5, 2) == 1


def test_messages_of_a_run_are_packed_piece_by_piece(host_model):
    # per-head layout of the benchmark shape: 264-byte messages = 33 pieces = 2.2 lines each. Five of them
    # are 165 pieces = exactly 11 lines, where one message per three lines would take 15.
    cp, entries, x, s = 2, 5, 128, 2
    assert host_model.lib.hm_msg_lines(2 * x, 4 * s) == 3
    assert host_model.lib.hm_run_lines(5, 2 * x, 4 * s) == 11
    assert host_model.lib.hm_run_lines(16, 2 * x, 4 * s) == 36
    assert host_model.lib.hm_msgs_per_entry(2 * x, 4 * s) == 15360 // 33
    assert host_model.lib.hm_msgs_per_entry(2048, 64) == 58          # 264 pieces
    assert host_model.lib.hm_msgs_per_entry(122872, 8) == 1          # 15 360 pieces: the largest message
    ins_o, ins_s = random_inputs(cp, entries, x, s, seed=2)
    ws = host_model.new_workspace(cp, CU)
    _, _, rc, msg = host_model.alltoall(ins_o, ins_s, ws, CU, 1, send=True, recv=False)
    assert rc == 0, msg
    max_ch = host_model.max_channel_count(cp, CU)
    for receiver in range(cp):
        region = ws[receiver].view(np.uint64)[: FIFO_BYTES * cp * max_ch // 8]
        untouched = np.ones(region.size, dtype=bool)
        for sender in range(cp):
            off = host_model.stream_fifo_offset(sender, 0, 1, 11, cp, CU)
            lines = region[off // 8: off // 8 + 11 * 16].reshape(11, 16)
            untouched[off // 8: off // 8 + 11 * 16] = False
            run = np.concatenate([np.concatenate([ins_o[sender][e, receiver].view(np.uint64),
                                                  ins_s[sender][e, receiver].view(np.uint64)]) for e in range(entries)])
            assert run.size == 165
            assert (lines[:, :15].reshape(-1) == run).all()          # message after message, no gaps
            assert (lines[:, 15] == 0).all()                         # every line carries the step
        assert (region[untouched] == np.uint64(0xFFFFFFFFFFFFFFFF)).all()
    # six messages: 198 pieces = 13.2 lines -> 14 lines, the last one zero padded
    ins_o, ins_s = random_inputs(cp, 6, x, s, seed=3)
    ws = host_model.new_workspace(cp, CU)
    out_o, out_s, rc, msg = host_model.alltoall(ins_o, ins_s, ws, CU, 1)
    assert rc == 0, msg
    fifo = ws[1].view(np.uint64)[: 16384 // 8]                       # sender 0 -> receiver 1: the first 16 KiB slot
    last = fifo[13 * 16: 14 * 16]
    assert (last[3:15] == 0).all() and last[15] == 0 and (fifo[14 * 16:] == np.uint64(0xFFFFFFFFFFFFFFFF)).all()
    want_o, want_s = ho.exchange_closed_form(ins_o), ho.exchange_closed_form(ins_s)
    for r in range(cp):
        assert np.array_equal(out_o[r], want_o[r]) and np.array_equal(out_s[r], want_s[r])


def test_units_in_flight_rule(host_model):
    # fewest passes of at most 6 units per lane, then the smallest count that keeps that many passes
    f = host_model.lib.hm_units_in_flight
    known = {0: 1, 1: 1, 64: 1, 65: 2, 144: 3, 288: 5, 384: 6, 385: 4, 640: 5, 768: 6, 769: 5, 1104: 6, 8192: 6}
    assert {u: f(u) for u in known} == known
    for units in range(1, 8193, 7):
        k = f(units)
        per_lane = -(-units // 64)
        passes = -(-per_lane // 6)
        assert 1 <= k <= 6
        assert k * passes >= per_lane          # the run is covered in the minimal number of passes
        assert (k - 1) * passes < per_lane     # and no smaller count would do


def test_repeated_calls_reuse_entries_with_new_steps(host_model):
    cp = 2
    ws = host_model.new_workspace(cp, CU)
    for call in range(9):
        ins_o, ins_s = random_inputs(cp, 5, 64, 2, seed=call)
        out_o, out_s, _ = _exchange(host_model, ins_o, ins_s, channels=2, ws=ws)
        want_o, want_s = ho.exchange_closed_form(ins_o), ho.exchange_closed_form(ins_s)
        for r in range(cp):
            assert (out_o[r] == want_o[r]).all() and (out_s[r] == want_s[r]).all()
    max_ch = host_model.max_channel_count(cp, CU)
    so = host_model.lib.hm_sender_info_offset(cp, max_ch, 1, 1)
    assert ws[0][so // 8] == 9 and ws[0][so // 8 + 1] == 9  # one entry per call and stream
    # the flag of the first line of FIFO entry 9 % 4 == 1 ... entry 0 was last written at step 8
    # (5 entries over 2 channels: channel 0 carries 3 messages of 17 pieces = 4 lines, the largest run of the launch)
    row1 = ws[1].view(np.uint64)
    assert row1[host_model.stream_fifo_offset(0, 1, 2, 4, cp, CU, step=8) // 8 + 15] == 8
    assert row1[host_model.stream_fifo_offset(0, 1, 2, 4, cp, CU, step=5) // 8 + 15] == 5
    assert (host_model.stream_fifo_offset(0, 1, 2, 4, cp, CU, step=5) - host_model.stream_fifo_offset(0, 1, 2, 4, cp, CU, step=8)
            == FIFO_ENTRY_BYTES * cp * max_ch)   # a quarter of the FIFO region between consecutive positions


def test_rounds_when_traffic_exceeds_the_fifo(host_model):
    # 17-piece messages, one channel: 903 messages per entry, 3612 per round; 9000 entries need 3 rounds
    cp, entries = 2, 9000
    ins_o, ins_s = random_inputs(cp, entries, 64, 2, seed=7)
    out_o, out_s, ws = _exchange(host_model, ins_o, ins_s, channels=1)
    want_o, want_s = ho.exchange_closed_form(ins_o), ho.exchange_closed_form(ins_s)
    for r in range(cp):
        assert (out_o[r] == want_o[r]).all() and (out_s[r] == want_s[r]).all()
    so = host_model.lib.hm_sender_info_offset(cp, host_model.max_channel_count(cp, CU), 0, 0)
    assert ws[0][so // 8] == 4 + 4 + 2  # entries consumed: 3612 + 3612 + 1776 messages


def test_receiver_rejects_stale_lines(host_model):
    # a receive without the matching send finds no token (the sender's counter has not moved) ...
    cp = 2
    ins_o, ins_s = random_inputs(cp, 3, 64, 2, seed=2)
    ws = host_model.new_workspace(cp, CU)
    _, _, rc, msg = host_model.alltoall(ins_o, ins_s, ws, CU, 1, send=False, recv=True)
    assert rc > 0 and "token" in msg
    # ... and with a forged token, no valid flag: a fresh FIFO holds all ones
    max_ch = host_model.max_channel_count(cp, CU)
    for sender in range(cp):
        for receiver in range(cp):
            ws[sender][host_model.lib.hm_sender_info_offset(cp, max_ch, receiver, 0) // 8] = 1
    _, _, rc, msg = host_model.alltoall(ins_o, ins_s, ws, CU, 1, send=False, recv=True)
    assert rc > 0 and "flag" in msg


def test_stream_of_a_wavefront_without_a_divide(host_model):
    # wavefronts find (part, peer, channel, rank) from their index with a multiply-high, an add and a shift per
    # divisor; exact for every index below 2^31 and every divisor a launch can have (parts, cp, channels)
    lib = host_model.lib
    for d in list(range(1, 4100)) + [4999, 65535, 65536, 65537, 10**6 + 3, 2**20, 2**24 - 1, 2**30, 2**30 + 1, 2**31 - 1]:
        assert lib.hm_fast_div_mismatches(d, 200) == 0, d
    assert [lib.hm_fast_div(n, 7) for n in (0, 6, 7, 13, 14, 2**31 - 1)] == [0, 0, 1, 1, 2, (2**31 - 1) // 7]
    assert lib.hm_fast_div(12345, 1) == 12345


def test_workgroups_regrouped_by_xcd(host_model):
    # workgroup i runs on XCD i mod 8; within tiles of 8 * group workgroups the regrouping is a permutation that
    # gives every XCD `group` consecutive places, and it leaves a launch alone when group is 0
    f = host_model.lib.hm_xcd_grouped
    for group in (2, 4, 8, 16):
        tile = 8 * group
        n = 5 * tile
        places = [f(b, group) for b in range(n)]
        assert sorted(places) == list(range(n))
        for t in range(0, n, tile):
            assert sorted(places[t:t + tile]) == list(range(t, t + tile))      # a tile stays a tile
            for xcd in range(8):
                mine = sorted(places[b] for b in range(t, t + tile) if b % 8 == xcd)
                assert mine == list(range(t + xcd * group, t + (xcd + 1) * group))  # consecutive places per XCD
    assert [f(b, 0) for b in range(20)] == list(range(20))


def test_split_rule(host_model):
    # wavefronts per stream: as many as leave each at most `units per part` units per lane (16 at most);
    # units in flight: the slice of a part in the fewest passes of at most 6, then the smallest such count
    f = host_model.split_for_run
    assert f(144) == (1, 3)      # c2's run: 18 lines
    assert f(288) == (1, 5)      # c3: 36 lines, 4.5 units per lane
    assert f(584) == (2, 5)      # c5a: 73 lines
    assert f(1104) == (3, 6)     # c4: 138 lines
    assert f(8192) == (16, 4)    # a full FIFO entry: 128 units per lane, 8 per part in two passes of 4
    assert f(288, 3) == (2, 3)
    assert f(0) == (1, 1)
    assert f(8192, 6, 1) == (1, 6) and f(8192, 6, 4) == (4, 6) and f(1104, 6, 2) == (2, 5)
    for units in range(0, 8193, 17):      # one wavefront per stream: the units-in-flight rule alone
        assert f(units, 6, 1) == (1, host_model.lib.hm_units_in_flight(units))
    for units in range(1, 8193, 13):
        for per_part in (1, 2, 3, 4, 5, 6):
            parts, k = f(units, per_part)
            per_lane = -(-units // 64)
            slice_per_lane = -(-per_lane // parts)
            passes = -(-slice_per_lane // 6)
            assert 1 <= parts <= 16 and 1 <= k <= 6
            assert parts == min(-(-per_lane // per_part), 16)
            assert k * passes >= slice_per_lane and (k - 1) * passes < slice_per_lane


@pytest.mark.parametrize("units_per_part", [0, 1, 2, 3, 6])
def test_runs_shared_by_several_wavefronts(host_model, units_per_part):
    # the same exchange whatever the number of wavefronts per stream, also when calls on one workspace
    # differ in it: a call brings the counters of its parts level before it starts
    cp, entries, x, s = 3, 7, 1096, 6        # 277 pieces per message; channel 0 carries 4 messages = 74 lines
    ins_o, ins_s = random_inputs(cp, entries, x, s, seed=11)
    host_model.set_units_per_part(units_per_part)
    try:
        out_o, out_s, ws = _exchange(host_model, ins_o, ins_s, channels=2)
        # a second call on the same workspace with the default split: counters of all parts are in step
        host_model.set_units_per_part(6)
        out_o2, out_s2, _ = _exchange(host_model, ins_o, ins_s, channels=2, ws=ws)
    finally:
        host_model.set_units_per_part(-1)
    want_o, want_s = ho.exchange_closed_form(ins_o), ho.exchange_closed_form(ins_s)
    for r in range(cp):
        assert (out_o[r] == want_o[r]).all() and (out_s[r] == want_s[r]).all()
        assert (out_o2[r] == want_o[r]).all() and (out_s2[r] == want_s[r]).all()
    max_ch = host_model.max_channel_count(cp, CU)
    parts = {0: 1, 1: 10, 2: 5, 3: 4, 6: 2}[units_per_part]      # 74 lines = 592 units = 10 units per lane
    for a in range(cp):
        for b in range(cp):
            for ch in range(2):
                so = host_model.lib.hm_sender_info_offset(cp, max_ch, b, ch) // 8
                ro = host_model.lib.hm_receiver_info_offset(cp, max_ch, b, ch) // 8
                # head and tail count both calls; so do the counters of the parts the second call had (two);
                # parts only the first call had stay where that call left them
                assert ws[a][so] == 2 and ws[a][so + 1] == 2 and ws[a][ro + 1] == 2 and ws[a][ro] == 0
                for p in range(1, 16):
                    want = 2 if p < 2 else (1 if p < parts else 0)
                    assert ws[a][so + p + 1] == want and ws[a][ro + p + 1] == want, (p, parts)


def test_bounds_checker_catches_short_buffers(host_model):
    # the walk-through refuses an access outside its buffer instead of performing it:
    # a workspace laid out for 4 channels, addressed as if it had 8
    cp = 2
    ins_o, ins_s = random_inputs(cp, 4, 64, 2, seed=3)
    ws = host_model.new_workspace(cp, CU)
    _, _, rc, _ = host_model.alltoall(ins_o, ins_s, ws, 2 * CU, 4)
    assert rc > 0 and host_model.lib.hm_last_out_of_extent() > 0
    # and is silent for the layout it was made for
    ws = host_model.new_workspace(cp, CU)
    _, _, rc, _ = host_model.alltoall(ins_o, ins_s, ws, CU, 4)
    assert rc == 0 and host_model.lib.hm_last_out_of_extent() == 0
