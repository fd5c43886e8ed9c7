// helix_host_model.cpp -- CPU walk-through of the GPU kernels' wave programs.
//
// Test fixture (never loaded by the product). It executes, lane by lane and
// in plain C++, the same sequence of loads and stores the gfx950 kernels
// issue, using the index arithmetic of csrc/helix_ll128.hpp, on host memory,
// and checks every single access against the extent of the buffer it
// belongs to. CPU tests use it to show that the index math stays in bounds
// for a shape before that shape is ever launched on a GPU, and to produce the
// expected FIFO image (line layout, flags, counters) that GPU tests compare
// the real FIFO contents with.
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "../../include/helix_a2a.h"
#include "../../helix-a2a_amd/csrc/helix_ll128.hpp"

using namespace helix;

namespace {

struct Extent {
  const uint8_t* base;
  uint64_t bytes;
};

struct Checker {
  int violations = 0;
  int outOfExtent = 0;
  char first[256] = "";
  bool ok(const Extent& e, const void* p, uint64_t n, const char* what) {
    const uint8_t* q = static_cast<const uint8_t*>(p);
    if (q >= e.base && q + n <= e.base + e.bytes) return true;
    outOfExtent++;
    if (violations++ == 0)
      snprintf(first, sizeof(first), "%s: access of %llu bytes at offset %lld outside extent %llu", what,
               (unsigned long long)n, (long long)(q - e.base), (unsigned long long)e.bytes);
    return false;
  }
};

thread_local char g_msg[256] = "";
thread_local int g_outOfExtent = 0;

struct Ctx {
  const helix_a2a_params_t* ranks;
  int cp, maxCh, channels, entryBegin, entryEnd;
  MsgShape sh;
  Extent ws;
  Checker chk;
  int unitsInFlight;   // per round, by the library's rule
  int parts;           // wavefronts that share a stream's runs, by the library's rule
  bool alignedStores;  // receivers of long runs store realigned 16-byte pieces
  uint32_t positionMask;              // positions the round's entries rotate through - 1 (fifo_positions)
  uint32_t slotBytes, positionBytes;  // where the round's streams put their lines (packed_slot_bytes, fifo_position_bytes)
  // the FIFO region of rank r's row
  Extent fifoRegion(int r) const {
    return Extent{reinterpret_cast<const uint8_t*>(ranks[0].workspace) + r * ranks[0].workspace_stride_u64 * 8,
                  fifo_region_bytes(cp, maxCh)};
  }
};

int g_unitsPerPart = -1;  // the library's knob: -1 automatic, 0 one wavefront per stream, 1..6 share runs longer than that per lane

Extent field_extent(const helix_a2a_field_t& f, int entries, int cp) {
  return Extent{static_cast<const uint8_t*>(f.data), static_cast<uint64_t>(entries) * cp * f.stride_bytes};
}

// Offsets of the two payload pieces of run unit U, computed in 32-bit
// arithmetic exactly as the kernels do; kNone where the piece is not in that field.
constexpr uint32_t kNone = 0x80000000u;
struct UnitOffsets {
  uint32_t a0, b0, a1, b1;
  bool flag;
};

UnitOffsets unit_offsets(const Ctx& c, uint32_t firstRow, uint32_t rowStep, uint32_t stride0, uint32_t stride1,
                         uint32_t firstMsg, uint32_t runMsgs, uint32_t U, RunUnit* decoded = nullptr) {
  const uint32_t np0 = static_cast<uint32_t>(c.sh.np0), np = static_cast<uint32_t>(c.sh.np);
  RunUnit d = decode_run_unit(U, np, div_magic(np));
  uint32_t rowA = firstRow + (firstMsg + d.msgA) * rowStep;
  uint32_t rowB = firstRow + (firstMsg + d.msgB) * rowStep;
  const bool aLive = d.msgA < runMsgs;
  const bool bLive = !d.flag && d.msgB < runMsgs;
  UnitOffsets o;
  o.flag = d.flag;
  o.a0 = (aLive && d.pieceA < np0) ? rowA * stride0 + d.pieceA * kPieceBytes : kNone;
  o.b0 = (bLive && d.pieceB < np0) ? rowB * stride0 + d.pieceB * kPieceBytes : kNone;
  o.a1 = (aLive && d.pieceA >= np0) ? rowA * stride1 + (d.pieceA - np0) * kPieceBytes : kNone;
  o.b1 = (bLive && d.pieceB >= np0) ? rowB * stride1 + (d.pieceB - np0) * kPieceBytes : kNone;
  if (decoded) *decoded = d;
  return o;
}

// part `part` of the sender waves of stream (s -> r, ch): one run per FIFO entry, its slice of the units walked flat
void run_sender(Ctx& c, int s, int r, int ch, int part) {
  const helix_a2a_params_t& p = c.ranks[s];
  uint8_t* wsBase = reinterpret_cast<uint8_t*>(p.workspace);
  uint64_t rowStride = p.workspace_stride_u64 * 8;
  uint8_t* senderRow = wsBase + s * rowStride;
  uint8_t* receiverRow = wsBase + r * rowStride;
  int64_t* info = reinterpret_cast<int64_t*>(senderRow + sender_info_offset(c.cp, c.maxCh, r, ch));
  uint8_t* fifo = receiverRow + stream_fifo_offset(s, ch, c.channels, c.slotBytes);
  if (!c.chk.ok(c.ws, info, kFifoInfoBytes, "sender info")) return;
  int64_t* token = info + sender_counter_slot(part);
  Extent e0 = field_extent(p.send_fields[0], p.entry_count, c.cp);
  Extent e1 = field_extent(p.send_fields[1], p.entry_count, c.cp);
  const int msgs = stream_msg_count(c.entryBegin, c.entryEnd, ch, c.channels);
  if (msgs == 0) return;
  const int perEntry = msgs_per_fifo_entry(c.sh);
  const uint32_t firstRow = static_cast<uint32_t>(c.entryBegin + ch) * c.cp + r;
  const uint32_t rowStep = static_cast<uint32_t>(c.channels) * c.cp;
  int64_t step = *token;
  for (int firstMsg = 0; firstMsg < msgs; firstMsg += perEntry) {
    int runMsgs = perEntry < msgs - firstMsg ? perEntry : msgs - firstMsg;
    uint32_t runUnits = static_cast<uint32_t>(run_units(runMsgs, c.sh));
    const Slice slice = slice_of_run(runUnits, part, c.parts);
    if (firstMsg > 0) {
      step += 1;
      *token = step;
    }
    // the model runs senders to completion first: room must already be there
    if (info[1] + kFifoDepth <= step) {
      c.chk.violations++;
      snprintf(c.chk.first, sizeof(c.chk.first), "sender %d->%d ch %d would block at step %lld", s, r, ch,
               (long long)step);
      return;
    }
    uint32_t entryOffset = (static_cast<uint32_t>(step) & c.positionMask) * c.positionBytes;
    // tighter than the GPU's descriptor: every access must stay inside the stream's slot of this step's quarter
    Extent fifoExt{fifo + entryOffset, c.slotBytes};
    if (!c.chk.ok(c.fifoRegion(r), fifoExt.base, c.slotBytes, "fifo slot")) return;
    // one pass = unitsInFlight accesses of 64 lanes. The statistics pieces of the pass are gathered first, lane j
    // of gather g taking the pass's statistics piece number g * 64 + j in run order; the lanes that store a
    // statistics piece take it from there.
    const uint32_t np = static_cast<uint32_t>(c.sh.np), np0 = static_cast<uint32_t>(c.sh.np0), ns = np - np0;
    const uint32_t passUnits = static_cast<uint32_t>(c.unitsInFlight) * kWaveLanes;
    for (uint32_t U0 = slice.begin; U0 < slice.end; U0 += passUnits) {
      const uint32_t passFirst = (U0 / kUnitsPerLine) * kPiecesPerLine;
      uint32_t passEnd = passFirst + static_cast<uint32_t>(c.unitsInFlight) * (kWaveLanes / kUnitsPerLine) * kPiecesPerLine;
      if (passEnd > static_cast<uint32_t>(runMsgs) * np) passEnd = static_cast<uint32_t>(runMsgs) * np;
      if (passEnd > (slice.end / kUnitsPerLine) * kPiecesPerLine) passEnd = (slice.end / kUnitsPerLine) * kPiecesPerLine;
      const uint32_t ordFirst = stats_ordinal_at(passFirst, np, np0, div_magic(np));
      const uint32_t ordEnd = passEnd > passFirst ? stats_ordinal_at(passEnd, np, np0, div_magic(np)) : ordFirst;
      if (ordEnd - ordFirst > static_cast<uint32_t>(kStatsGathers * kWaveLanes)) {
        c.chk.violations++;
        snprintf(c.chk.first, sizeof(c.chk.first), "sender %d->%d ch %d: %u statistics pieces in one pass", s, r, ch, ordEnd - ordFirst);
        return;
      }
      uint64_t gathered[kStatsGathers * kWaveLanes] = {0};
      for (uint32_t ord = ordFirst; ord < ordEnd; ++ord) {
        const uint32_t m = div_by_magic(ord, div_magic(ns));
        const uint32_t index = ord - m * ns;
        const uint32_t off = (firstRow + (firstMsg + m) * rowStep) * p.send_fields[1].stride_bytes + index * kPieceBytes;
        if (c.chk.ok(e1, e1.base + off, 8, "send field 1")) memcpy(&gathered[ord - ordFirst], e1.base + off, 8);
      }
      for (uint32_t U = U0; U < U0 + passUnits && U < slice.end; ++U) {  // every lane of every wave access
        RunUnit d;
        UnitOffsets o = unit_offsets(c, firstRow, rowStep, p.send_fields[0].stride_bytes, p.send_fields[1].stride_bytes,
                                     firstMsg, runMsgs, U, &d);
        uint64_t words[2] = {0, 0};
        const uint32_t offs0[2] = {o.a0, o.b0}, offs1[2] = {o.a1, o.b1};
        const uint32_t ords[2] = {d.msgA * ns + (d.pieceA - np0), d.msgB * ns + (d.pieceB - np0)};
        for (int k = 0; k < 2; ++k) {
          if (offs0[k] != kNone && c.chk.ok(e0, e0.base + offs0[k], 8, "send field 0")) memcpy(&words[k], e0.base + offs0[k], 8);
          if (offs1[k] != kNone) {
            if (ords[k] < ordFirst || ords[k] >= ordEnd) {
              c.chk.violations++;
              snprintf(c.chk.first, sizeof(c.chk.first), "sender %d->%d ch %d unit %u: statistics piece %u outside the pass's [%u, %u)",
                       s, r, ch, U, ords[k], ordFirst, ordEnd);
              return;
            }
            words[k] = gathered[ords[k] - ordFirst];
          }
        }
        if (o.flag) words[1] = static_cast<uint64_t>(step);
        uint8_t* dst = fifo + entryOffset + U * kUnitBytes;
        if (c.chk.ok(fifoExt, dst, 16, "fifo store")) memcpy(dst, words, 16);
      }
    }
  }
  *token = step + 1;
}

// part `part` of the receiver waves of stream (s -> r, ch); a missing token or a line whose flag is not there
// counts as a violation
void run_receiver(Ctx& c, int r, int s, int ch, int part) {
  const helix_a2a_params_t& p = c.ranks[r];
  uint8_t* wsBase = reinterpret_cast<uint8_t*>(p.workspace);
  uint64_t rowStride = p.workspace_stride_u64 * 8;
  uint8_t* senderRow = wsBase + s * rowStride;
  uint8_t* receiverRow = wsBase + r * rowStride;
  int64_t* sinfo = reinterpret_cast<int64_t*>(senderRow + sender_info_offset(c.cp, c.maxCh, r, ch));
  int64_t* info = reinterpret_cast<int64_t*>(receiverRow + receiver_info_offset(c.cp, c.maxCh, s, ch));
  uint8_t* fifo = receiverRow + stream_fifo_offset(s, ch, c.channels, c.slotBytes);
  if (!c.chk.ok(c.ws, info, kFifoInfoBytes, "receiver info") || !c.chk.ok(c.ws, sinfo, kFifoInfoBytes, "sender info")) return;
  const int64_t* token = sinfo + sender_counter_slot(part);
  int64_t* mine = info + receiver_counter_slot(part);
  Extent e0 = field_extent(p.recv_fields[0], p.entry_count, c.cp);
  Extent e1 = field_extent(p.recv_fields[1], p.entry_count, c.cp);
  const int msgs = stream_msg_count(c.entryBegin, c.entryEnd, ch, c.channels);
  if (msgs == 0) return;
  const int perEntry = msgs_per_fifo_entry(c.sh);
  const uint32_t firstRow = static_cast<uint32_t>(c.entryBegin + ch) * c.cp + s;
  const uint32_t rowStep = static_cast<uint32_t>(c.channels) * c.cp;
  int64_t step = *mine;
  for (int firstMsg = 0; firstMsg < msgs; firstMsg += perEntry) {
    int runMsgs = perEntry < msgs - firstMsg ? perEntry : msgs - firstMsg;
    uint32_t runUnits = static_cast<uint32_t>(run_units(runMsgs, c.sh));
    const Slice slice = slice_of_run(runUnits, part, c.parts);
    if (firstMsg > 0) {
      step += 1;
      *mine = step;
      if (part == 0) sinfo[1] = step;
    }
    if (*token <= step) {  // the sending part has not closed this step: the GPU receiver would wait here
      if (c.chk.violations++ == 0)
        snprintf(c.chk.first, sizeof(c.chk.first), "stream %d->%d ch %d part %d: token %lld not beyond step %lld", s, r, ch,
                 part, (long long)*token, (long long)step);
      return;
    }
    uint32_t entryOffset = (static_cast<uint32_t>(step) & c.positionMask) * c.positionBytes;
    Extent fifoExt{fifo + entryOffset, c.slotBytes};
    if (!c.chk.ok(c.fifoRegion(r), fifoExt.base, c.slotBytes, "fifo slot")) return;
    uint8_t* base0 = const_cast<uint8_t*>(e0.base);
    uint8_t* base1 = const_cast<uint8_t*>(e1.base);
    const uint32_t stride0 = p.recv_fields[0].stride_bytes, stride1 = p.recv_fields[1].stride_bytes;
    // one pass = unitsInFlight accesses of 64 lanes, all loaded before anything is stored
    const uint32_t passUnits = static_cast<uint32_t>(c.unitsInFlight) * kWaveLanes;
    for (uint32_t U0 = slice.begin; U0 < slice.end; U0 += passUnits) {
      const uint32_t passEnd = U0 + passUnits < slice.end ? U0 + passUnits : slice.end;
      uint64_t words[kMaxUnitsInFlight][kWaveLanes][2];
      bool landed[kMaxUnitsInFlight][kWaveLanes];
      for (int i = 0; i < c.unitsInFlight; ++i) {
        for (int lane = 0; lane < kWaveLanes; ++lane) {
          const uint32_t U = U0 + i * kWaveLanes + lane;
          landed[i][lane] = false;
          words[i][lane][0] = words[i][lane][1] = 0;  // what an out-of-range load returns
          if (U >= passEnd) continue;
          const uint8_t* src = fifo + entryOffset + U * kUnitBytes;
          if (!c.chk.ok(fifoExt, src, 16, "fifo load")) continue;
          memcpy(words[i][lane], src, 16);
          uint64_t flag;  // flag of this lane's line
          memcpy(&flag, fifo + entryOffset + (U | 7u) * kUnitBytes + 8, 8);
          if (flag != static_cast<uint64_t>(step)) {
            if (c.chk.violations++ == 0)
              snprintf(c.chk.first, sizeof(c.chk.first), "stream %d->%d ch %d unit %u: flag %llx != step %llx", s, r, ch,
                       U, (unsigned long long)flag, (unsigned long long)step);
            continue;
          }
          landed[i][lane] = true;
        }
      }
      for (int i = 0; i < c.unitsInFlight; ++i) {
        for (int lane = 0; lane < kWaveLanes; ++lane) {
          if (!landed[i][lane]) continue;
          const uint32_t U = U0 + i * kWaveLanes + lane;
          RunUnit d;
          UnitOffsets o = unit_offsets(c, firstRow, rowStep, stride0, stride1, firstMsg, runMsgs, U, &d);
          const uint64_t* w = words[i][lane];
          if (c.alignedStores) {
            // the aligned 16 bytes that start at whichever word is an even partial_o piece; second half from the next unit
            const bool haveNext = U + 1 < passEnd;
            const uint64_t nextFirst = lane < kWaveLanes - 1 ? words[i][lane + 1][0] : (i + 1 < c.unitsInFlight ? words[i + 1][0][0] : 0);
            const bool startsAtA = o.a0 != kNone && (d.pieceA & 1u) == 0;
            const bool startsAtB = o.b0 != kNone && (d.pieceB & 1u) == 0;
            const bool takesNext = startsAtB || (startsAtA && d.flag);
            if ((startsAtA || startsAtB) && (!takesNext || haveNext)) {
              const uint64_t chunk[2] = {startsAtB ? w[1] : w[0], takesNext ? nextFirst : w[1]};
              uint8_t* dst = base0 + (startsAtB ? o.b0 : o.a0);
              if (c.chk.ok(e0, dst, 16, "recv field 0 (16 bytes)")) memcpy(dst, chunk, 16);
            }
            const bool alone = o.a0 != kNone && ((U + 1 == passEnd && startsAtA && d.flag) || (U == U0 && (d.pieceA & 1u) != 0));
            if (alone) {
              uint8_t* dst = base0 + o.a0;
              if (c.chk.ok(e0, dst, 8, "recv field 0 (lone piece)")) memcpy(dst, &w[0], 8);
            }
          } else {
            const uint32_t offs0[2] = {o.a0, o.b0};
            for (int k = 0; k < 2; ++k)
              if (offs0[k] != kNone && c.chk.ok(e0, base0 + offs0[k], 8, "recv field 0")) memcpy(base0 + offs0[k], &w[k], 8);
          }
          const uint32_t offs1[2] = {o.a1, o.b1};
          for (int k = 0; k < 2; ++k)
            if (offs1[k] != kNone && c.chk.ok(e1, base1 + offs1[k], 8, "recv field 1")) memcpy(base1 + offs1[k], &w[k], 8);
        }
      }
    }
  }
  *mine = step + 1;
  if (part == 0) sinfo[1] = step + 1;
}

// what the library does ahead of a launch that shares runs between wavefronts: the counters of
// parts 1.. of every stream of the launch take the value of part 0's
void level_part_counters(Ctx& c, bool send, bool recv) {
  for (int local = 0; local < c.cp; ++local)
    for (int ch = 0; ch < c.channels; ++ch)
      for (int peer = 0; peer < c.cp; ++peer) {
        uint8_t* row = reinterpret_cast<uint8_t*>(c.ranks[0].workspace) + local * c.ranks[0].workspace_stride_u64 * 8;
        int64_t* si = reinterpret_cast<int64_t*>(row + sender_info_offset(c.cp, c.maxCh, peer, ch));
        int64_t* ri = reinterpret_cast<int64_t*>(row + receiver_info_offset(c.cp, c.maxCh, peer, ch));
        if (!c.chk.ok(c.ws, si, kFifoInfoBytes, "sender info") || !c.chk.ok(c.ws, ri, kFifoInfoBytes, "receiver info")) return;
        for (int p = 1; p < c.parts; ++p) {
          if (send) si[sender_counter_slot(p)] = si[0];
          if (recv) ri[receiver_counter_slot(p)] = ri[1];
        }
      }
}

}  // namespace

extern "C" {

const char* hm_last_message(void) { return g_msg; }
// accesses the last hm_alltoall refused because they left their buffer
int hm_last_out_of_extent(void) { return g_outOfExtent; }

// Run the send and/or receive programs of all cp ranks (per_rank[r].cp_rank == r)
// for entries [0, entry_count) split in rounds exactly like the library does.
// Returns the number of violations (out-of-extent accesses, missing flags,
// blocked senders); 0 means the walk-through was clean.
int hm_alltoall(const helix_a2a_params_t* per_rank, int cp, int cu_count, int channels, int do_send, int do_recv) {
  g_msg[0] = 0;
  Ctx c;
  c.ranks = per_rank;
  c.cp = cp;
  c.maxCh = max_channel_count(cp, cu_count);
  c.channels = channels;
  const helix_a2a_params_t& p0 = per_rank[0];
  c.sh = make_msg_shape(p0.send_fields[0].element_count * p0.send_fields[0].element_size,
                        p0.send_fields[1].element_count * p0.send_fields[1].element_size);
  c.ws = Extent{reinterpret_cast<const uint8_t*>(p0.workspace), p0.workspace_stride_u64 * 8 * cp};
  if (channels < 1 || channels > c.maxCh || c.sh.lines > kFifoEntryLines) {
    snprintf(g_msg, sizeof(g_msg), "bad channel count or message size");
    return -1;
  }
  long perStream = static_cast<long>(kFifoDepth) * msgs_per_fifo_entry(c.sh);
  long roundEntries = perStream * channels;
  for (long begin = 0; begin < p0.entry_count; begin += roundEntries) {
    c.entryBegin = static_cast<int>(begin);
    long end = begin + roundEntries;
    c.entryEnd = end > p0.entry_count ? p0.entry_count : static_cast<int>(end);
    {  // what launch_exchange derives from the round's largest run (channel 0's first)
      const int msgs0 = stream_msg_count(c.entryBegin, c.entryEnd, 0, channels);
      const int perEntry = msgs_per_fifo_entry(c.sh);
      const long maxRun = run_units(msgs0 < perEntry ? msgs0 : perEntry, c.sh);
      const RunSplit split = g_unitsPerPart == 0  ? split_for_run(maxRun, kMaxUnitsInFlight, 1)
                             : g_unitsPerPart > 0 ? split_for_run(maxRun, g_unitsPerPart, kMaxStreamParts)
                                                  : split_for_run(maxRun, kMaxUnitsInFlight, auto_max_parts(cp, channels, cu_count));
      c.parts = split.parts;
      c.unitsInFlight = split.unitsInFlight;
      if (c.unitsInFlight > max_units_in_flight_for_statistics(c.sh.np, c.sh.np0)) c.unitsInFlight = max_units_in_flight_for_statistics(c.sh.np, c.sh.np0);
      c.alignedStores = maxRun > static_cast<long>(kMaxUnitsInFlight) * kWaveLanes;
      const int msgsMax = stream_msg_count(c.entryBegin, c.entryEnd, 0, channels);
      c.positionMask = static_cast<uint32_t>(fifo_positions(exchange_lines_bytes(cp, channels, maxRun), entries_for_msgs(msgsMax, c.sh))) - 1u;
      c.slotBytes = packed_slot_bytes(maxRun);
      c.positionBytes = fifo_position_bytes(cp, c.maxCh);
    }
    if (c.parts > 1) level_part_counters(c, do_send != 0, do_recv != 0);
    if (do_send)
      for (int s = 0; s < cp; ++s)
        for (int ch = 0; ch < channels; ++ch)
          for (int r = 0; r < cp; ++r)
            for (int part = 0; part < c.parts; ++part) run_sender(c, s, r, ch, part);
    if (do_recv)
      for (int r = 0; r < cp; ++r)
        for (int ch = 0; ch < channels; ++ch)
          for (int s = 0; s < cp; ++s)
            for (int part = 0; part < c.parts; ++part) run_receiver(c, r, s, ch, part);
  }
  if (c.chk.violations) snprintf(g_msg, sizeof(g_msg), "%s", c.chk.first);
  g_outOfExtent = c.chk.outOfExtent;
  return c.chk.violations;
}

// the library's knob (helix_a2a_set_units_per_wavefront): -1 automatic, 0 never share, 1..6 always beyond that
void hm_set_units_per_part(int units) { g_unitsPerPart = units; }
// what the launch rule makes of a largest run of `runUnits` units: parts * 256 + units in flight
int hm_split_for_run(long runUnits, int unitsPerPart, int maxParts) {
  const RunSplit r = split_for_run(runUnits, unitsPerPart, maxParts);
  return r.parts * 256 + r.unitsInFlight;
}

// geometry probes for tests
// byte offset, inside the receiver's row, of the lines stream (sender, channel) writes under step `step` in a launch
// over `run_channels` channels whose largest run has `largest_run_units` units
// (`positions`: fifo_positions of the launch)
uint64_t hm_stream_fifo_offset(int sender, int channel, int run_channels, long largest_run_units, int cp, int max_ch, long step,
                               int positions) {
  return stream_fifo_offset(sender, channel, run_channels, packed_slot_bytes(largest_run_units)) +
         static_cast<uint64_t>(step & (positions - 1)) * fifo_position_bytes(cp, max_ch);
}
int hm_fifo_positions(int cp, int run_channels, long largest_run_units, int entries_per_stream) {
  return fifo_positions(exchange_lines_bytes(cp, run_channels, largest_run_units), entries_per_stream);
}
uint32_t hm_packed_slot_bytes(long largest_run_units) { return packed_slot_bytes(largest_run_units); }
uint64_t hm_sender_info_offset(int cp, int max_ch, int receiver, int channel) {
  return sender_info_offset(cp, max_ch, receiver, channel);
}
uint64_t hm_receiver_info_offset(int cp, int max_ch, int sender, int channel) {
  return receiver_info_offset(cp, max_ch, sender, channel);
}
int hm_msg_lines(int f0, int f1) { return make_msg_shape(f0, f1).lines; }
int hm_unit_first_piece(int g) { return unit_first_piece(g); }
// floor(g / d) the way the kernels compute it
uint32_t hm_div(uint32_t g, uint32_t d) { return div_by_magic(g, div_magic(d)); }
// number of run piece indices g of a FIFO entry for which that differs from g / d
int hm_div_mismatches(uint32_t d) {
  int bad = 0;
  const uint32_t magic = div_magic(d);
  for (uint32_t g = 0; g < static_cast<uint32_t>(kFifoEntryLines * kPiecesPerLine) + 16u; ++g)
    bad += div_by_magic(g, magic) != g / d;
  return bad;
}
// the place workgroup `block` takes when `group` consecutive workgroups' worth of streams go to one XCD
int hm_xcd_grouped(int block, int group) { return xcd_grouped(block, group); }
// floor(n / d) the way wavefronts find their stream from their index (any n < 2^31)
uint32_t hm_fast_div(uint32_t n, uint32_t d) { return fast_div_by(n, fast_div(d)); }
// number of n among multiples of d, their neighbours, small values, 2^31 - 1 and `samples` pseudo-random values for
// which that differs from n / d
int hm_fast_div_mismatches(uint32_t d, int samples) {
  int bad = 0;
  const FastDiv f = fast_div(d);
  auto check = [&](uint64_t n) {
    if (n < (1ull << 31)) bad += fast_div_by(static_cast<uint32_t>(n), f) != static_cast<uint32_t>(n) / d;
  };
  for (uint64_t n = 0; n < 300; ++n) check(n);
  for (uint64_t k = 1; k < 300; ++k) {
    check(k * d - 1);
    check(k * d);
    check(k * d + 1);
  }
  const uint64_t top = ((1ull << 31) - 1) / d * d;
  check(top - 1);
  check(top);
  check(top + 1);
  check((1ull << 31) - 1);
  uint64_t x = 88172645463325252ull + d;
  for (int i = 0; i < samples; ++i) {
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    check(x & 0x7fffffffull);
  }
  return bad;
}
// Statistics pieces of a run of messages of np pieces (np0 of them payload) that sit before run piece P, and the
// most units per lane a pass may take so that its statistics pieces fit the senders' gather.
uint32_t hm_stats_ordinal_at(uint32_t P, int np, int np0) { return stats_ordinal_at(P, np, np0, div_magic(np)); }
int hm_max_units_for_statistics(int np, int np0) { return max_units_in_flight_for_statistics(np, np0); }
// lines of a run of `msgs` messages and messages per FIFO entry for a message of the two field sizes
int hm_run_lines(int msgs, int field0_bytes, int field1_bytes) { return run_lines(msgs, make_msg_shape(field0_bytes, field1_bytes)); }
int hm_msgs_per_entry(int field0_bytes, int field1_bytes) { return msgs_per_fifo_entry(make_msg_shape(field0_bytes, field1_bytes)); }
// units a lane keeps in flight per pass for a launch whose largest run has `runUnits` units
int hm_units_in_flight(long runUnits) { return units_in_flight_for_run(runUnits); }

}  // extern "C"
