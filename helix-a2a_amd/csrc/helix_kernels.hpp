// helix_kernels.hpp -- launch descriptors shared by the kernels and the host
// side of the library (internal; the public boundary is include/helix_a2a.h).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "helix_ll128.hpp"

namespace helix {

// Field pointers of one logical rank.
struct RankPtrs {
  const uint8_t* send0;  // partial_o     [E, cp, field0Bytes]
  const uint8_t* send1;  // softmax_stats [E, cp, field1Bytes]
  uint8_t* recv0;        // exchange: partial_o out; combine: combined out [E, field0Bytes]
  uint8_t* recv1;        // exchange: softmax_stats out; combine: lse out [E, heads] or null
};

// Kernel argument block. `rank` is indexed by logical rank id; only ids in
// [rankBegin, rankBegin + rankCount) are dereferenced by a launch.
struct KernelArgs {
  RankPtrs rank[kMaxCpSize];
  uint8_t* workspace;       // base of the [cp, rowStrideBytes] workspace
  uint64_t rowStrideBytes;
  int cpSize;
  int maxChannels;          // layout constant of the workspace
  int runChannels;          // channels this launch deals entries over
  int entryBegin, entryEnd; // entries [entryBegin, entryEnd) of the call
  int field0Bytes, field1Bytes;  // field1Bytes is a multiple of 8, or of 4 for the packed per-head statistics of the combine
  int sendStride0, sendStride1;  // bytes between consecutive (entry, peer) rows
  int recvStride0, recvStride1;
  uint32_t sendBytes0, sendBytes1;  // extent of each tensor (< 2 GiB), the range of its buffer descriptor
  uint32_t recvBytes0, recvBytes1;
  uint32_t npMagic;                 // div_magic(pieces per message)
  uint32_t nsMagic;                 // div_magic(statistics pieces per message)
  int rankBegin, rankCount;
  int doSend, doRecv;
  int unitsInFlight;        // units_in_flight_for_run(largest run of the launch), 1..kMaxUnitsInFlight
  int alignedStores;        // receivers realign payload to 16-byte stores: set when runs take several passes
  int longRuns;             // the largest run of the launch takes several passes (combine kernel: receivers first look at the senders' counters through the scalar cache)
  int parts;                // wavefronts that share one stream's runs (per direction), 1..kMaxStreamParts
  int team;                 // exchange kernel: wavefronts of a workgroup that walk one stream's run together (parts == 1), 1..kMaxTeamWavefronts
  // Worked out by the launch functions from the fields above, so that no wavefront divides:
  int np0, np;              // 8-byte pieces of field 0, of a message
  int msgsPerEntry;         // messages one FIFO entry holds
  int baseMsgs, extraChannels;  // channel c has baseMsgs + (c < extraChannels) messages in this launch
  int entriesBase, entriesExtra;  // FIFO entries that baseMsgs and baseMsgs + 1 messages take
  FastDiv byParts, byTeam, byCp, byChannels;
  int sendBlocks;           // combine kernel: workgroups that send (the rest receive)
  int wavesPerBlock;        // wavefronts of a workgroup of the launch
  int dirBlocks;            // workgroups per direction (combine kernel: that send)
  int xcdGroup;             // consecutive workgroups' worth of streams that one XCD serves (xcd_grouped), 0: as dispatched
  uint32_t slotBytes;       // packed_slot_bytes(largest run of the launch): the streams of the launch sit this far apart
  uint32_t positionMask;    // fifo_positions(...) - 1: the entry of step k sits in quarter k & positionMask
  uint32_t positionBytes;   // fifo_position_bytes: between the four positions (quarters of the FIFO region) an entry rotates through
  uint64_t spinLimitTicks;  // bound of one in-kernel wait, in 100 MHz ticks
  uint32_t* status;         // device status word (HELIX_A2A_STATUS_* bits)
  // combine only
  int heads, headDim;
  int statsMode, dtype;
  int lseBase2;        // the statistics are base-2 logarithms, and so is the combined log-sum-exp that is stored
  uint32_t headMagic;  // head_div_magic(pieces per head)
  uint32_t np0Magic;   // div_magic(pieces of field 0)
};

// Wavefronts of a workgroup of the exchange kernel are independent unless they form a team (no LDS, no barrier); small
// workgroups dispatch and retire at a finer grain (2 measured best of 1..16 on launches that queue).
constexpr int kWavesPerBlock = 2;
constexpr int kMaxWavesPerBlock = 4;       // ... four when the whole launch is resident at once
constexpr int kResidentWavefronts = 4096;  // 256 CUs x 4 SIMDs x 4 wavefronts: what runs at once

// streams one direction of a launch serves: one per (local rank, channel, peer)
inline int waves_per_direction(const KernelArgs& a) { return a.rankCount * a.runChannels * a.cpSize; }

// A stream's runs are shared by as many wavefronts (at most maxParts) as leave each at most
// unitsPerPart units per lane; maxParts = 1: one wavefront per stream.
// Teams (launches with one part per stream only): the wavefronts of a workgroup walk one stream's run together,
// each a slice, sharing the stream's counters through the first of them. teamUnits -1: a launch whose wavefronts
// queue for slots gives runs of three or more passes to teams, one pass per wavefront; 0: never; 1..6: always,
// with at most that many units per lane and wavefront.
constexpr int kMaxTeamWavefronts = 8;
hipError_t launch_exchange(const KernelArgs& a, int unitsPerPart, int maxParts, int teamUnits, hipStream_t stream);
// exchange fused with the LSE-weighted combine, all ranks of the launch; `parts` wavefronts share
// the units of one (receiver, channel)
constexpr int kMaxCombineParts = 8;
hipError_t launch_combine(const KernelArgs& a, int parts, hipStream_t stream);
hipError_t launch_init_row(uint8_t* row, uint64_t fifoBytes, uint64_t infoBytes, hipStream_t stream);

}  // namespace helix
