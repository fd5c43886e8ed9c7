// helix_ll128.hpp -- the CDNA4 LL128 line format and the workspace geometry.
//
// Pure integer arithmetic, usable from device code (hipcc) and from host code
// (g++): the host model used by the CPU tests includes this very file, so the
// index math the kernels run is the index math those tests bound-check.
//
// Line format (new for wave64; the reference rotates its flag through the
// line and displaces payload words into tail blocks, csrc/ll128_proto.cuh:73-139):
//
//   one line  = 128 bytes = 16 words of 8 bytes
//   words 0..14  payload pieces 15*l .. 15*l+14 of the message (l = line index)
//   word  15     flag = the FIFO step counter under which the line was written
//
//   one unit  = 16 bytes = words (2u, 2u+1) of a line, u = 0..7. A lane moves
//   one unit per access, so 8 consecutive lanes cover a line, a 64-lane
//   wavefront covers 8 lines (1 KiB), and the lane with u == 7 carries
//   {payload piece 15*l+14, flag} in a single 16-byte store.
//
// A message is field 0 followed by field 1, cut into 8-byte pieces; the last
// line is zero padded.
//
// Workspace geometry (one row per rank, unchanged from the reference so that
// workspace_size and the init pattern stay drop-in,
// csrc/helix_alltoall.cu:61-75,194-242,605-614):
//
//   [ FIFO region : cp senders x maxCh channels x 4 entries x 128 KiB ]
//   [ sender info : cp receivers x maxCh x 256 B  {int64 head; int64 tail} ]
//   [ receiver info: cp senders  x maxCh x 256 B  {int64 head; int64 tail} ]
//
//   FIFO of (sender s -> receiver r, channel c) lives in row r at
//   (s*maxCh + c) * 512 KiB; the sender's counters live in row s indexed by r,
//   the receiver's counters in row r indexed by s.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define HELIX_HD __host__ __device__ __forceinline__
#else
#define HELIX_HD inline
#endif

namespace helix {

constexpr int kMaxCpSize = 16;

// ---- line format ---------------------------------------------------------
constexpr int kPieceBytes = 8;
constexpr int kLineBytes = 128;
constexpr int kWordsPerLine = 16;
constexpr int kPiecesPerLine = 15;
constexpr int kFlagWord = 15;
constexpr int kUnitBytes = 16;
constexpr int kUnitsPerLine = 8;
constexpr int kWaveLanes = 64;
constexpr int kLinesPerWaveAccess = kWaveLanes / kUnitsPerLine;  // 8

// ---- FIFO geometry (csrc/helix_alltoall.cu:70-75) -------------------------
constexpr int kFifoDepth = 4;
constexpr int kFifoEntryBytes = 128 * 1024;
constexpr int kFifoEntryLines = kFifoEntryBytes / kLineBytes;  // 1024
constexpr int kFifoBytes = kFifoDepth * kFifoEntryBytes;       // 512 KiB
constexpr int kFifoInfoBytes = 256;                            // sizeof(HelixFifoInfo), 256-aligned
constexpr int kMaxGroupsPerBlock = 8;                          // csrc/helix_common.h:35

HELIX_HD int ceil_div_i(int a, int b) { return (a + b - 1) / b; }

// csrc/helix_alltoall.cu:590-603 with the CU count in place of the SM count.
HELIX_HD int max_channel_count(int cpSize, int cuCount) {
  int blocksPerChannel = 2 * ceil_div_i(cpSize, kMaxGroupsPerBlock);
  int c = cuCount / blocksPerChannel;
  return c > 1 ? c : 1;
}

HELIX_HD uint64_t fifo_region_bytes(int cpSize, int maxCh) {
  return static_cast<uint64_t>(kFifoBytes) * cpSize * maxCh;
}
HELIX_HD uint64_t info_region_bytes(int cpSize, int maxCh) {
  return static_cast<uint64_t>(kFifoInfoBytes) * cpSize * maxCh;  // one of the two
}
// csrc/helix_alltoall.cu:605-614
HELIX_HD uint64_t workspace_bytes(int cpSize, int maxCh) {
  return fifo_region_bytes(cpSize, maxCh) + 2 * info_region_bytes(cpSize, maxCh);
}

// byte offset inside the RECEIVER's row (csrc/helix_alltoall.cu:194-206)
HELIX_HD uint64_t fifo_offset(int sender, int channel, int maxCh) {
  return (static_cast<uint64_t>(sender) * maxCh + channel) * kFifoBytes;
}
// byte offset inside the SENDER's row (csrc/helix_alltoall.cu:208-223)
HELIX_HD uint64_t sender_info_offset(int cpSize, int maxCh, int receiver, int channel) {
  return fifo_region_bytes(cpSize, maxCh) +
         (static_cast<uint64_t>(receiver) * maxCh + channel) * kFifoInfoBytes;
}
// byte offset inside the RECEIVER's row (csrc/helix_alltoall.cu:225-242)
HELIX_HD uint64_t receiver_info_offset(int cpSize, int maxCh, int sender, int channel) {
  return fifo_region_bytes(cpSize, maxCh) + info_region_bytes(cpSize, maxCh) +
         (static_cast<uint64_t>(sender) * maxCh + channel) * kFifoInfoBytes;
}

// ---- message shape ----------------------------------------------------------
struct MsgShape {
  int np0;    // 8-byte pieces of field 0
  int np;     // pieces of field 0 + field 1
  int lines;  // LL128 lines on the wire
  int units;  // 16-byte units on the wire = 8 * lines
};

HELIX_HD MsgShape make_msg_shape(int field0Bytes, int field1Bytes) {
  MsgShape s;
  s.np0 = field0Bytes / kPieceBytes;
  s.np = s.np0 + field1Bytes / kPieceBytes;
  s.lines = (s.np + kPiecesPerLine - 1) / kPiecesPerLine;
  s.units = s.lines * kUnitsPerLine;
  return s;
}

HELIX_HD int msgs_per_fifo_entry(const MsgShape& s) { return kFifoEntryLines / s.lines; }

// first payload piece carried by unit g (= line*8 + u) of a message; the
// second word of the unit is piece+1, or the flag when (g & 7) == 7.
HELIX_HD int unit_first_piece(int g) { return (g >> 3) * kPiecesPerLine + 2 * (g & 7); }
HELIX_HD bool unit_has_flag(int g) { return (g & 7) == 7; }

// byte offset of unit g of a message that starts at line `lineBase` of FIFO
// entry `entry` (0..3), relative to the FIFO base.
HELIX_HD uint32_t fifo_unit_offset(int entry, int lineBase, int g) {
  return static_cast<uint32_t>(entry) * kFifoEntryBytes +
         static_cast<uint32_t>(lineBase) * kLineBytes + static_cast<uint32_t>(g) * kUnitBytes;
}

// ---- per-stream schedule ------------------------------------------------------
// Entries e = entryBegin + channel, + runChannels, ... < entryEnd belong to the
// stream of `channel` (csrc/helix_alltoall.cu:368-369,417-418).
HELIX_HD int stream_msg_count(int entryBegin, int entryEnd, int channel, int runChannels) {
  int first = entryBegin + channel;
  if (first >= entryEnd) return 0;
  return (entryEnd - first + runChannels - 1) / runChannels;
}

// Division of a line index x < 1024 by the lines-per-message count L <= 1024
// without an integer divide: floor(x / L) == (x * M) >> 20 with
// M = ceil(2^20 / L). Exact on that range: the excess x * (M - 2^20/L) / 2^20
// stays below 2^-10 <= 1/L (and is zero for L = 1024).
constexpr int kLineDivShift = 20;
HELIX_HD uint32_t line_div_magic(int lines) {
  return static_cast<uint32_t>(((1u << kLineDivShift) + lines - 1) / lines);
}
HELIX_HD uint32_t line_div(uint32_t x, uint32_t magic) { return (x * magic) >> kLineDivShift; }

// Where unit U of a run lives. A run is the sequence of messages a stream
// puts into one FIFO entry; it starts at line 0 of the entry and its messages
// follow each other without gaps, so unit U sits at byte U*16 of the entry.
struct RunUnit {
  uint32_t msg;     // message index inside the run
  uint32_t piece0;  // first payload piece of the unit inside its message
  bool flag;        // second word of the unit is the flag word
};
HELIX_HD RunUnit decode_run_unit(uint32_t U, uint32_t lines, uint32_t magic) {
  RunUnit d;
  uint32_t x = U >> 3;
  uint32_t u = U & 7u;
  d.msg = line_div(x, magic);
  uint32_t line = x - d.msg * lines;
  d.piece0 = line * kPiecesPerLine + 2u * u;
  d.flag = u == 7u;
  return d;
}

// Head index of payload piece p when a head spans `piecesPerHead` pieces
// (head_dim * 2 bytes / 8): floor(p / piecesPerHead) as a multiply-high by
// M = floor(2^32 / piecesPerHead) + 1. Exact for p < 2^16 and
// 2 <= piecesPerHead < 2^16 (the excess p * (M - 2^32/d) / 2^32 is below
// 2^-16 <= 1/d); piecesPerHead == 1 is the identity and uses magic 0.
HELIX_HD uint32_t head_div_magic(uint32_t piecesPerHead) {
  return piecesPerHead <= 1 ? 0u : static_cast<uint32_t>((1ull << 32) / piecesPerHead) + 1u;
}
HELIX_HD uint32_t head_of_piece(uint32_t p, uint32_t magic) {
  return magic == 0u ? p : static_cast<uint32_t>((static_cast<uint64_t>(p) * magic) >> 32);
}

// Number of FIFO entries a stream of `msgs` messages consumes in one call.
HELIX_HD int entries_for_msgs(int msgs, const MsgShape& s) {
  if (msgs <= 0) return 0;
  int per = msgs_per_fifo_entry(s);
  return (msgs + per - 1) / per;
}

// Units a lane keeps in flight per pass when the largest run of a launch has
// `runUnits` units: the fewest passes of at most kMaxUnitsInFlight units per
// lane, then the smallest count that still makes that number of passes (a run
// of 4.5 units per lane takes one pass of 5, not one of 6 with a wasted slot;
// one of 10 takes two passes of 5, not 6 + 4).
constexpr int kMaxUnitsInFlight = 6;
HELIX_HD int units_in_flight_for_run(long runUnits) {
  long perLane = (runUnits + kWaveLanes - 1) / kWaveLanes;
  if (perLane < 1) perLane = 1;
  long passes = (perLane + kMaxUnitsInFlight - 1) / kMaxUnitsInFlight;
  return static_cast<int>((perLane + passes - 1) / passes);
}

}  // namespace helix
