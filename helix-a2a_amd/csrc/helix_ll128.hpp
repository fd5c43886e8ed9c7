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
//   words 0..14  payload pieces 15*l .. 15*l+14 of the run (l = line index)
//   word  15     flag = the FIFO step counter under which the line was written
//
//   one unit  = 16 bytes = words (2u, 2u+1) of a line, u = 0..7. A lane moves
//   one unit per access, so 8 consecutive lanes cover a line, a 64-lane
//   wavefront covers 8 lines (1 KiB), and the lane with u == 7 carries
//   {payload piece 15*l+14, flag} in a single 16-byte store.
//
// A message is field 0 followed by field 1, cut into 8-byte pieces. A run is
// the messages a stream puts into one FIFO entry, piece after piece without
// gaps: message j of the run is run pieces j*np .. (j+1)*np - 1, wherever the
// line boundaries fall (a 264-byte message is 33 pieces = 2.2 lines, not 3).
// Only the last line of a run is zero padded.
//
// Workspace geometry (one row per rank; the regions, their sizes and the init
// pattern are the reference's, so that workspace_size and init_workspace stay
// drop-in, csrc/helix_alltoall.cu:61-75,194-242,605-614):
//
//   [ FIFO region : cp senders x maxCh channels x 4 entries x 128 KiB ]
//   [ sender info : cp receivers x maxCh x 256 B  {int64 head; int64 tail} ]
//   [ receiver info: cp senders  x maxCh x 256 B  {int64 head; int64 tail} ]
//
//   The sender's counters of stream (s -> r, channel c) live in row s indexed by
//   r, the receiver's counters in row r indexed by s, as in the reference.
//   Where the stream's lines live inside row r's FIFO region is this build's
//   own (nothing outside the kernels reads them): the region is four quarters,
//   one per position a stream's entry rotates through (step & 3; launches too
//   large for the memory-side cache use fewer, see fifo_positions), and inside a
//   quarter a launch packs its streams side by side, a slot of
//   packed_slot_bytes(largest run of the launch) each -- see stream_fifo_offset.
//   (The reference gives every stream four 128 KiB entries of its own,
//   512 KiB apart: a launch's lines are then spread thinly over the whole
//   region, which measured 3-9 % slower on MI355X wherever runs are long or a
//   wavefront reads the lines of many senders.)
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define HELIX_HD __host__ __device__ __forceinline__
#else
#define HELIX_HD inline
#endif

namespace helix {

constexpr int kMaxCpSize = 32;         // ranks of one exchange (size of the kernel argument block)
constexpr int kMaxCombineCpSize = 32;  // ranks of one fused combine (lanes per slot of its sideways pass)

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

// ---- where a launch puts its runs inside the receiver row's FIFO region ----------
// A stream's entry of step k sits in quarter k & (positions - 1) of the region (fifo_positions below); a quarter is cp * maxCh * 128 KiB, room for a
// full 128 KiB entry of every stream the layout provides for. Within the quarter the streams of a launch are
// packed: stream (sender, channel) of a launch over runChannels channels starts at
// (sender * runChannels + channel) * slotBytes, and slotBytes is the launch's largest run (every launch knows it:
// channel 0's first run) rounded up to whole KiB -- but runs shorter than 8 KiB are kept 16 KiB apart (4.5 KiB
// runs packed closer than that measured 2-16 % slower). Sender and receiver of a launch derive the same
// slotBytes from the same launch shape; between launches nothing but the counters is carried over, so launches
// of different shapes may place their lines differently.
HELIX_HD uint32_t fifo_position_bytes(int cpSize, int maxCh) {
  return static_cast<uint32_t>(static_cast<uint64_t>(kFifoEntryBytes) * cpSize * maxCh);  // a quarter of the region, < 2^32
}
HELIX_HD uint32_t packed_slot_bytes(long largestRunUnits) {
  const long bytes = largestRunUnits * kUnitBytes;
  if (bytes < 8192) return 16384;
  return static_cast<uint32_t>((bytes + 1023) / 1024 * 1024);  // at most kFifoEntryBytes: a run is at most 1024 lines
}
// How many of the four quarters the entries of a launch rotate through (1, 2 or 4; the entry of step k sits in
// quarter k & (positions - 1)). Lines are dead once they have been received, but a cache does not know that:
// every position a launch writes for the first time in a while pushes as many dead bytes of an older position
// out of the 256 MB memory-side cache to DRAM. A launch whose lines of all four positions, with the tensors it
// reads and writes (about as many bytes each as the lines), fit that cache keeps all four (24.2 us at cp = 8,
// T = 256, against 27.5 us rewriting one position: lines that small are still in the L2s of the XCDs that read
// them last); a larger one rewrites the same two, or the same one, every time (cp = 8, T = 512: 54.7 -> 44.9 us;
// T = 768: 86.9 -> 65.8 us; c4: 99.4 -> 90.0 us). `linesBytes`: what the whole exchange writes into the FIFOs
// of all ranks under one step, so that launches that carry a part of an exchange (one rank's send half) agree
// with the others. A launch in which a stream opens more than one entry rotates through all four.
constexpr uint64_t kMemorySideCacheBytes = 256ull << 20;
HELIX_HD int fifo_positions(uint64_t linesBytes, int entriesPerStream) {
  if (entriesPerStream > 1) return kFifoDepth;
  const uint64_t budget = kMemorySideCacheBytes / 16 * 15;
  if (6 * linesBytes <= budget) return 4;  // four positions of lines + tensors in + tensors out
  if (4 * linesBytes <= budget) return 2;
  return 1;
}
// bytes the streams of all cp * cp * runChannels (sender, receiver, channel) triples write under one step, at most
HELIX_HD uint64_t exchange_lines_bytes(int cpSize, int runChannels, long largestRunUnits) {
  return static_cast<uint64_t>(cpSize) * cpSize * runChannels * static_cast<uint64_t>(largestRunUnits) * kUnitBytes;
}
// byte offset of the stream's slot inside a quarter of the RECEIVER's row
HELIX_HD uint64_t stream_fifo_offset(int sender, int channel, int runChannels, uint32_t slotBytes) {
  return (static_cast<uint64_t>(sender) * runChannels + channel) * slotBytes;
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
  int lines;  // LL128 lines of a message on its own (what must fit one FIFO entry)
};

HELIX_HD MsgShape make_msg_shape(int field0Bytes, int field1Bytes) {
  MsgShape s;
  s.np0 = field0Bytes / kPieceBytes;
  s.np = s.np0 + (field1Bytes + kPieceBytes - 1) / kPieceBytes;  // a row of an odd number of floats: the last piece is half empty
  s.lines = (s.np + kPiecesPerLine - 1) / kPiecesPerLine;
  return s;
}

// messages one FIFO entry (1024 lines = 15 360 pieces) holds
HELIX_HD int msgs_per_fifo_entry(const MsgShape& s) { return kFifoEntryLines * kPiecesPerLine / s.np; }
// lines and 16-byte units of a run of `msgs` messages
HELIX_HD int run_lines(int msgs, const MsgShape& s) { return (msgs * s.np + kPiecesPerLine - 1) / kPiecesPerLine; }
HELIX_HD int run_units(int msgs, const MsgShape& s) { return run_lines(msgs, s) * kUnitsPerLine; }

// first payload piece carried by unit g (= line*8 + u) of a run; the second
// word of the unit is piece+1, or the flag when (g & 7) == 7.
HELIX_HD int unit_first_piece(int g) { return (g >> 3) * kPiecesPerLine + 2 * (g & 7); }

// ---- per-stream schedule ------------------------------------------------------
// Entries e = entryBegin + channel, + runChannels, ... < entryEnd belong to the
// stream of `channel` (csrc/helix_alltoall.cu:368-369,417-418).
HELIX_HD int stream_msg_count(int entryBegin, int entryEnd, int channel, int runChannels) {
  int first = entryBegin + channel;
  if (first >= entryEnd) return 0;
  return (entryEnd - first + runChannels - 1) / runChannels;
}

// floor(p / d) for p < 2^16 and 1 <= d < 2^16 without an integer divide: a
// multiply-high by M = floor(2^32 / d) + 1. Exact on that range (the excess
// p * (M - 2^32/d) / 2^32 is below 2^-16 <= 1/d); d == 1 is the identity and
// uses magic 0. Run pieces (< 15 360) are divided by the pieces per message
// with it, pieces of a message by the pieces per head.
HELIX_HD uint32_t div_magic(uint32_t d) { return d <= 1 ? 0u : static_cast<uint32_t>((1ull << 32) / d) + 1u; }
HELIX_HD uint32_t div_by_magic(uint32_t p, uint32_t magic) {
#if defined(__HIP_DEVICE_COMPILE__)
  return magic == 0u ? p : __umulhi(p, magic);
#else
  return magic == 0u ? p : static_cast<uint32_t>((static_cast<uint64_t>(p) * magic) >> 32);
#endif
}

// floor(n / d) for any n < 2^31 and 1 <= d < 2^31 without a divide and without a branch:
// q = (mulhi(n, m) + n) >> s with s = ceil(log2 d) and m = floor(2^32 * (2^s - d) / d) + 1, that is a
// multiplication by M = 2^32 + m = floor(2^(32+s) / d) + 1 (exact because 2^(32+s) < M*d <= 2^(32+s) + 2^s;
// the sum cannot overflow for n < 2^31; d == 1 gives m = 1, s = 0, the identity). The host works the pair
// out once per launch; wavefronts find their stream from their index with it.
struct FastDiv {
  uint32_t magic;
  uint32_t shift;
};
HELIX_HD FastDiv fast_div(uint32_t d) {
  FastDiv f;
  if (d < 1u) d = 1u;
  uint32_t s = 0;
  while ((1ull << s) < d) ++s;
  f.magic = static_cast<uint32_t>((((1ull << s) - d) << 32) / d) + 1u;
  f.shift = s;
  return f;
}
HELIX_HD uint32_t fast_div_by(uint32_t n, FastDiv f) {
#if defined(__HIP_DEVICE_COMPILE__)
  return (__umulhi(n, f.magic) + n) >> f.shift;
#else
  return (static_cast<uint32_t>((static_cast<uint64_t>(n) * f.magic) >> 32) + n) >> f.shift;
#endif
}

// Where unit U of a run lives: the message and the piece inside that message
// of each of its two words. Unit U sits at byte U*16 of the FIFO entry.
struct RunUnit {
  uint32_t msgA, pieceA;  // first word
  uint32_t msgB, pieceB;  // second word (the next piece of the run; may start the next message)
  bool flag;              // ... unless it is the line's flag word
};
HELIX_HD RunUnit decode_run_unit(uint32_t U, uint32_t np, uint32_t npMagic) {
  RunUnit d;
  const uint32_t g = (U >> 3) * kPiecesPerLine + 2u * (U & 7u);
  d.msgA = div_by_magic(g, npMagic);
  d.pieceA = g - d.msgA * np;
  const bool wraps = d.pieceA + 1u == np;
  d.msgB = d.msgA + (wraps ? 1u : 0u);
  d.pieceB = wraps ? 0u : d.pieceA + 1u;
  d.flag = (U & 7u) == 7u;
  return d;
}

// ---- the statistics pieces of a run, counted ----------------------------------
// Message m of a run holds its statistics in its last ns = np - np0 pieces; its i-th statistics piece is the
// run's statistics piece number ("ordinal") m * ns + i. A sender fetches the statistics pieces of one pass with
// one load -- lane j takes the j-th of them -- and hands every piece to the lane that stores it, instead of one
// load of a few live lanes per wave access that touches the end of a message.
// Statistics pieces of the run that sit before run piece P:
HELIX_HD uint32_t stats_ordinal_at(uint32_t P, uint32_t np, uint32_t np0, uint32_t npMagic) {
  const uint32_t m = div_by_magic(P, npMagic);
  const uint32_t q = P - m * np;
  return m * (np - np0) + (q > np0 ? q - np0 : 0u);
}
// Head index of payload piece p when a head spans `piecesPerHead` pieces (head_dim * 2 bytes / 8).
HELIX_HD uint32_t head_div_magic(uint32_t piecesPerHead) { return div_magic(piecesPerHead); }
HELIX_HD uint32_t head_of_piece(uint32_t p, uint32_t magic) { return div_by_magic(p, magic); }

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

// A pass of `unitsInFlight` units per lane covers unitsInFlight * 120 consecutive pieces of the run; a sender
// gathers its statistics pieces in at most kStatsGathers loads of 64. Whatever the shape, a pass of one unit
// per lane (120 pieces) fits; launches whose messages are mostly statistics take fewer units per pass.
constexpr int kStatsGathers = 2;
HELIX_HD int max_units_in_flight_for_statistics(int np, int np0) {
  const int ns = np - np0;
  for (int k = kMaxUnitsInFlight; k > 1; --k) {
    const int pieces = k * (kWaveLanes / kUnitsPerLine) * kPiecesPerLine;
    int most = (pieces / np + 2) * ns;   // message ends a pass can touch, all of their statistics
    if (most > pieces) most = pieces;
    if (most <= kStatsGathers * kWaveLanes) return k;
  }
  return 1;
}



// ---- runs shared by several wavefronts ---------------------------------------
// A long run can be cut into `parts` slices of whole wave accesses (64 units),
// one wavefront per slice and direction. A launch that would leave most of the
// device idle (few streams, long runs) is spread over more wavefronts that way;
// a launch that fills the device anyway is not split (measured on MI355X: more,
// shorter wavefronts for the same bytes are slower once every slot is taken).
//
// Every part of a stream keeps a step counter of its own in the stream's
// 256-byte counter blocks (32 slots of 8 bytes; the reference uses two,
// csrc/helix_alltoall.cu:61-64): part 0 uses the reference's head (sender
// block, slot 0) and tail (receiver block, slot 1; its copy for the sender's
// back-pressure in the sender block, slot 1), part p >= 1 uses slot p + 1 of
// either block. A sender part moves its counter beyond a step once its stores
// of that step are acknowledged: that is the token its receiver part waits for.
// A launch moves the counters of the parts it has; a launch with more than one
// part first brings the counters of its parts 1.. level with part 0's, so
// launches may differ in their number of parts.
constexpr int kCounterSlots = kFifoInfoBytes / 8;     // 32
constexpr int kMaxStreamParts = 16;
// The last slot of the very first sender counter block of row 0 (receiver 0, channel 0) is the workspace's
// "broken" word: a kernel whose wait gave up, or that met a corrupt line, leaves its status bits there,
// and every later wavefront that finds it non-zero does nothing. Initialising row 0 clears it.
constexpr int kBrokenSlot = kCounterSlots - 1;
HELIX_HD uint64_t broken_word_offset(int cpSize, int maxCh) { return sender_info_offset(cpSize, maxCh, 0, 0) + kBrokenSlot * 8ull; }
HELIX_HD int sender_counter_slot(int part) { return part == 0 ? 0 : part + 1; }
HELIX_HD int receiver_counter_slot(int part) { return part + 1; }

struct RunSplit {
  int parts;          // wavefronts per stream and direction
  int unitsInFlight;  // units a lane keeps in flight per pass over its slice
};
// For the largest run of a launch: as many parts (at most maxParts, at most kMaxStreamParts) as leave each
// at most unitsPerPart units per lane; then the slice of a part in the fewest passes of at most
// kMaxUnitsInFlight units per lane, with the smallest count that still makes that number of passes.
HELIX_HD RunSplit split_for_run(long runUnits, int unitsPerPart, int maxParts) {
  if (unitsPerPart < 1) unitsPerPart = 1;
  if (unitsPerPart > kMaxUnitsInFlight) unitsPerPart = kMaxUnitsInFlight;
  if (maxParts > kMaxStreamParts) maxParts = kMaxStreamParts;
  if (maxParts < 1) maxParts = 1;
  long perLane = (runUnits + kWaveLanes - 1) / kWaveLanes;
  if (perLane < 1) perLane = 1;
  long parts = (perLane + unitsPerPart - 1) / unitsPerPart;
  if (parts > maxParts) parts = maxParts;
  long slicePerLane = (perLane + parts - 1) / parts;
  long passes = (slicePerLane + kMaxUnitsInFlight - 1) / kMaxUnitsInFlight;
  RunSplit r;
  r.parts = static_cast<int>(parts);
  r.unitsInFlight = static_cast<int>((slicePerLane + passes - 1) / passes);
  return r;
}
// Wavefronts per stream the automatic rule allows: as many as the wavefront slots of the device (four per
// SIMD, sixteen per compute unit) leave room for when every stream of the exchange -- both directions of
// all cp ranks, whatever part of it a launch carries -- takes that many.
HELIX_HD int auto_max_parts(int cpSize, int runChannels, int cuCount) {
  const long slots = static_cast<long>(cuCount) * 16;
  const long streams = 2L * cpSize * cpSize * runChannels;
  const long parts = streams > 0 ? slots / streams : 1;
  return parts < 1 ? 1 : (parts > kMaxStreamParts ? kMaxStreamParts : static_cast<int>(parts));
}

// units [begin, end) of a run of `runUnits` units that part `part` of `parts` walks
struct Slice {
  uint32_t begin, end;
};
HELIX_HD Slice slice_of_run(uint32_t runUnits, int part, int parts, FastDiv byParts) {
  const uint32_t perLane = (runUnits + kWaveLanes - 1) / kWaveLanes;
  const uint32_t slice = fast_div_by(perLane + parts - 1, byParts) * kWaveLanes;
  Slice s;
  s.begin = static_cast<uint32_t>(part) * slice;
  if (s.begin > runUnits) s.begin = runUnits;
  s.end = s.begin + slice;
  if (s.end > runUnits) s.end = runUnits;
  return s;
}
HELIX_HD Slice slice_of_run(uint32_t runUnits, int part, int parts) {
  return slice_of_run(runUnits, part, parts, fast_div(static_cast<uint32_t>(parts)));
}

// ---- which XCD serves which streams -------------------------------------------
// Workgroup i of a launch runs on XCD i mod 8, each XCD behind an L2 of its own. The wavefronts that send
// to, or receive from, the peers of one (rank, channel) touch rows that are neighbours in memory -- their
// statistics rows are 8 to 64 bytes apart, several to a cache line -- and with consecutive workgroups on
// consecutive XCDs every such line was fetched by up to eight L2s and written in pieces by as many.
// Within tiles of 8 * group workgroups, workgroup 8 * j + x (on XCD x) therefore takes the place group * x + j:
// `group` consecutive workgroups' worth of streams run on one XCD, while the launch as a whole still sweeps
// the tensors in order (dealing whole eighths of the launch to the XCDs instead costs c4 and c5a 12-14 %).
// Measured on MI355X: c5a 111.3 -> 108.0 us, the per-head layout of c3 26.4 -> 25.3 us, of c5a 113.7 -> 111.2 us;
// launches whose statistics rows fill whole lines (c3 and c4 in the per-token layout) are left as dispatched.
HELIX_HD int xcd_grouped(int block, int group) {
  if (group <= 0) return block;
  const int pos = block & (8 * group - 1);  // group is a power of two
  return block - pos + (pos & 7) * group + (pos >> 3);
}

}  // namespace helix
