// helix_kernels.hip -- gfx950 kernels of the Helix all-to-all.
//
// One wavefront owns one stream = (sender rank, receiver rank, channel) in one
// direction, the role a warp has in the reference kernel
// (csrc/helix_alltoall.cu:315-474). A long run is shared by several wavefronts,
// each with a slice of its own: wavefronts with counters of their own ("parts")
// in a launch that leaves the device under-filled, the wavefronts of one
// workgroup behind one set of counters (a "team") in a launch that fills it.
// A sender wavefront reads its messages from the send tensors, turns them into
// LL128 lines in registers, stores the lines into the receiver's FIFO and, once
// those stores are acknowledged, moves its step counter: that is the token its
// receiver waits for. A receiver wavefront then reads the lines in one pass,
// checks that their flags carry the step, and stores the payload into the
// receive tensors. There is no staging copy: data moves
// global -> registers -> FIFO -> registers -> global, 16 bytes per lane on
// the FIFO side. Nothing but a team's step goes through LDS, and only teams
// meet at a barrier.
//
// No wavefront divides: what follows from the shape of a launch (pieces per
// message, messages per channel, the divisors that turn a wavefront's index
// into its stream) is worked out by the host and travels in the argument
// block, which every wavefront fetches with a few wide scalar loads at its
// very start. Before that, a wavefront spent a dozen dependent trips to the
// scalar cache and six software divisions ahead of its first payload load.
//
// Why the token and not the flags alone: a 64-lane 16-byte load of eight lines
// is served in 64-byte halves, and the flag word of a line sits in its second
// half. A receiver that reads a line while it is being written can see a
// valid flag next to a stale first half. The counter moves only after the
// sender has waited for every store of the step (s_waitcnt vmcnt(0) on
// write-through stores), so a line is never read before all of it is in
// memory, whatever the granularity of the memory system. Measured on MI355X
// the token costs nothing against polling the flags (within 0.5 % on every
// workload): sender wavefronts are dispatched first, so receivers rarely start
// before their run is complete. The flags stay in the line format and are
// still compared: a mismatch after the token means a corrupt workspace.
//
// The messages a stream puts into one FIFO entry form a "run": they follow
// each other without gaps from line 0 of the entry, so a wavefront walks a
// run as one flat sequence of 16-byte units, in passes of up to six units per
// lane, regardless of message boundaries. All loads of a pass are issued
// before its first store, and loads return in the order they were issued, so
// the store of a wave access goes as soon as the loads of that access are back.
// What a pass holds of the second, small field (the statistics at the end of
// every message) is fetched by one load per pass and handed to the lanes that
// store it, not by one sparse load per wave access: the load pipeline charges
// per instruction, whatever the number of live lanes.
//
// Every global access goes through a buffer descriptor that spans exactly the
// tensor it belongs to (for FIFO lines: the stream's slots, first quarter of
// the FIFO region to last): the hardware returns zero for loads
// and drops stores that would fall outside, and an offset of kOutOfRange is
// how a lane opts out of an access without a branch.
//
// FIFO lines and counters are written and read with the sc1 cache policy
// (device-scope coherence: every XCD has its own L2, and the sender and the
// receiver of a stream may run on different XCDs).
#include "helix_kernels.hpp"

#include <hip/hip_fp16.h>

namespace helix {
namespace {

using u32x2 = uint32_t __attribute__((ext_vector_type(2)));
using u32x4 = uint32_t __attribute__((ext_vector_type(4)));

// gfx940+ buffer cache-policy immediates: bit 0 sc0, bit 1 nt, bit 4 sc1.
// sc1 alone is device scope. (The compiler's "volatile" bit 31 would widen
// the access to system scope; polling loops use a compiler barrier instead.)
constexpr int kAuxNone = 0;
constexpr int kAuxNt = 2;  // streaming: received payload is written once and not read again by this kernel
constexpr int kAuxSc1 = 16;
constexpr uint32_t kRsrcWord3 = 0x00020000u;   // raw buffer, 32-bit data format
constexpr uint32_t kOutOfRange = 0x80000000u;  // beyond any descriptor (extents are < 2 GiB)

// Launches of independent wavefronts and the combine kernel are held to four
// wavefronts per SIMD (16 per CU): with more resident wavefronts the same
// traffic takes 1-5 % longer on MI355X, on every shape measured, whatever the
// register count would allow. (Teams of the exchange kernel run at six, see there.)
#define HELIX_WAVES_PER_SIMD __attribute__((amdgpu_waves_per_eu(4, 4)))

constexpr int kDppWaveShl1 = 0x130;  // DPP control: lane i reads lane i + 1 of the wavefront

constexpr uint32_t kStatusRecvTimeout = 1u;
constexpr uint32_t kStatusSendTimeout = 2u;
constexpr uint32_t kStatusInternal = 4u;
constexpr uint32_t kStatusBrokenWorkspace = 8u;

// Units a lane keeps in flight per pass over a run: at most kMaxUnitsInFlight
// (6 x 16 B x 64 lanes = 6 KiB per wavefront), and no more than the runs of a
// launch need -- the host picks the count (units_in_flight_for_run) so that a
// run takes the fewest passes and no pass issues accesses that every lane
// opts out of. The count is a template parameter of the wave programs, so the
// units stay in registers; the kernels branch once, wave-uniformly, on
// KernelArgs::unitsInFlight.

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), kRsrcWord3);
}

__device__ __forceinline__ int64_t ld_counter(const int64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_counter(int64_t* p, int64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Phase stamps. A build with -DHELIX_A2A_TIMELINE (build.py --timeline, a separate library file) makes
// every wavefront record the 100 MHz clock at four points of its program: 0 start, 1 its input is in
// registers (sender: payload and counters; receiver: token seen and lines loaded), 2 its stores are
// issued, 3 done (sender: stores acknowledged). The stamped build waits for outstanding memory
// operations at points 1 and 3, which the product build does not; it is a measuring tool only.
#ifdef HELIX_A2A_TIMELINE
constexpr int kTimelineWaves = 1 << 16;
__device__ uint64_t g_timeline[kTimelineWaves * 4];
#define HELIX_MARK(wave, k, drain)                                                                 \
  do {                                                                                             \
    if (drain) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                    \
    if (lane == 0 && (wave) >= 0 && (wave) < kTimelineWaves)                                       \
      g_timeline[(wave) * 4 + (k)] = __builtin_amdgcn_s_memrealtime();                             \
  } while (0)
#else
#define HELIX_MARK(wave, k, drain) \
  do {                            \
  } while (0)
#endif

// Bounded wait bookkeeping. Every 64th spin reads the clock and the workspace's broken word: a wait
// ends when its time is up or when another wavefront has given up on this workspace already, so that
// a failed launch drains at once instead of one time limit after the other.
struct SpinGuard {
  uint64_t limit;
  uint64_t start;
  const uint64_t* broken;
  uint32_t spins;
  __device__ __forceinline__ SpinGuard(uint64_t limitTicks, const uint64_t* brokenWord)
      : limit(limitTicks), start(0), broken(brokenWord), spins(0) {}
  __device__ __forceinline__ bool expired() {
    spins += 1;
    if ((spins & 63u) != 1u) return false;
    uint64_t now = __builtin_amdgcn_s_memrealtime();
    if (start == 0) {
      start = now;
      return limit == 0;
    }
    if (__hip_atomic_load(broken, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) return true;
    return now - start > limit;
  }
};

// Wait until every store this wavefront has issued is acknowledged. Used by a
// sender before it moves `head`: FIFO lines are stored write-through (sc1), so
// a `head` beyond a step tells any reader that the lines of that step are in
// memory, all of them.
__device__ __forceinline__ void wait_stores_acknowledged() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ __forceinline__ uint32_t lane_value(uint32_t v, int q) {
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), q));
}

__device__ __forceinline__ uint64_t* broken_word(const KernelArgs& a) {
  return reinterpret_cast<uint64_t*>(a.workspace + broken_word_offset(a.cpSize, a.maxChannels));
}

// How far a wavefront's descriptor of its stream's lines reaches: from the stream's slot in the first quarter of
// the FIFO region to the end of its slot in the last one (the entry of a step sits in quarter step & 3).
__device__ __forceinline__ uint32_t fifo_extent(const KernelArgs& a) { return (kFifoDepth - 1) * a.positionBytes + a.slotBytes; }

// Whether the workspace was broken before this launch started. A wave-uniform read through the scalar
// cache (which starts every launch empty): it costs no vector memory instruction, and it need not see
// what the running launch does to the word -- the bounded waits look at that themselves.
__device__ __forceinline__ uint64_t broken_at_launch(const KernelArgs& a) {
  using ConstWord = const __attribute__((address_space(4))) uint64_t;
  return *reinterpret_cast<ConstWord*>(reinterpret_cast<uintptr_t>(broken_word(a)));
}

// A counter as it stood when this launch started (what the launches before it left), read through the scalar
// cache like the broken word: wave-uniform, off the vector memory pipeline, so that it neither takes vector
// registers nor sits in the queue of vector loads that the payload loads and their waits go through. Only for
// counters that nothing in the running launch moves before this wavefront is done reading them (a stream's own
// step, the tail a sender starts from); everything a wavefront polls goes through ld_counter.
__device__ __forceinline__ int64_t counter_at_launch(const int64_t* p) {
  using ConstWord = const __attribute__((address_space(4))) int64_t;
  return *reinterpret_cast<ConstWord*>(reinterpret_cast<uintptr_t>(p));
}

// A failure: the status word of the device tells the host, the broken word of the workspace tells every
// wavefront that comes later (of this launch and of the launches behind it).
__device__ __forceinline__ void raise_status(const KernelArgs& a, uint32_t bits, int lane) {
  if (lane == 0) {
    atomicOr(a.status, bits);
    __hip_atomic_fetch_or(broken_word(a), static_cast<uint64_t>(bits), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}
// The workspace was broken before this wavefront started: it reports that and does nothing.
__device__ __forceinline__ void report_broken(const KernelArgs& a, int lane) {
  if (lane == 0) atomicOr(a.status, kStatusBrokenWorkspace);
}

// A team: the wavefronts of one workgroup that walk one stream's run together, each a slice of it. Only
// the first wavefront (the leader) touches the stream's counters; it hands the step (or -1: give up) to
// the others through this word of LDS. Launches whose wavefronts queue for slots anyway use teams for
// runs of several passes: the same bytes move in more, shorter wavefronts without one more counter.
struct TeamLds {
  int64_t step;
  int bad;  // a wavefront of the team met a corrupt line: the leader leaves the stream's counters where they are
};
// A barrier of the workgroup that waits for this wavefront's LDS traffic only (not, as __syncthreads
// does, for its outstanding loads and stores to memory).
__device__ __forceinline__ void team_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
// The leader's step, or -1, for every wavefront of the team.
__device__ __forceinline__ int64_t team_share_step(TeamLds* lds, bool leader, int lane, int64_t step) {
  if (leader && lane == 0) *reinterpret_cast<volatile int64_t*>(&lds->step) = step;
  team_barrier();
  return *reinterpret_cast<volatile int64_t*>(&lds->step);
}
// A wavefront of a team that met a corrupt line says so before the team's next barrier; the leader looks after it.
__device__ __forceinline__ void team_report_bad(TeamLds* lds, int lane) {
  if (lane == 0) *reinterpret_cast<volatile int*>(&lds->bad) = 1;
}
__device__ __forceinline__ bool team_is_bad(TeamLds* lds) { return *reinterpret_cast<volatile int*>(&lds->bad) != 0; }

// Every scalar of the argument block a wavefront needs before its first memory access, asked for at once:
// the compiler then fetches the block in a few wide scalar loads and one wait at the top of the kernel,
// instead of one small load and one wait wherever a field is first used (a dozen dependent trips to the
// scalar cache before the first payload load otherwise).
__device__ __forceinline__ void fetch_scalars_up_front(const KernelArgs& a) {
  asm volatile("" ::"s"(a.workspace), "s"(a.rowStrideBytes), "s"(a.cpSize), "s"(a.maxChannels), "s"(a.runChannels),
               "s"(a.entryBegin), "s"(a.field0Bytes), "s"(a.field1Bytes), "s"(a.sendStride0), "s"(a.sendStride1),
               "s"(a.recvStride0), "s"(a.recvStride1), "s"(a.sendBytes0), "s"(a.sendBytes1), "s"(a.recvBytes0),
               "s"(a.recvBytes1), "s"(a.npMagic), "s"(a.nsMagic), "s"(a.rankBegin), "s"(a.rankCount), "s"(a.doSend), "s"(a.doRecv));
  asm volatile("" ::"s"(a.parts), "s"(a.team), "s"(a.np0), "s"(a.np), "s"(a.msgsPerEntry), "s"(a.baseMsgs),
               "s"(a.extraChannels), "s"(a.byParts.magic), "s"(a.byParts.shift), "s"(a.byTeam.magic), "s"(a.byTeam.shift),
               "s"(a.byCp.magic), "s"(a.byCp.shift), "s"(a.byChannels.magic), "s"(a.byChannels.shift), "s"(a.sendBlocks), "s"(a.wavesPerBlock), "s"(a.dirBlocks), "s"(a.xcdGroup),
               "s"(a.spinLimitTicks), "s"(a.slotBytes), "s"(a.positionBytes), "s"(a.positionMask));
}

// What a stream's wavefront needs to know, all wave-uniform.
struct Stream {
  __amdgpu_buffer_rsrc_t fifo;    // the 512 KiB FIFO of the stream
  __amdgpu_buffer_rsrc_t field0;  // partial_o tensor of the local rank (send or recv side)
  __amdgpu_buffer_rsrc_t field1;  // softmax_stats tensor of the local rank
  uint32_t stride0, stride1;      // row strides in bytes
  uint32_t firstRow;              // row of the stream's first message of this launch
  uint32_t rowStep;               // rows between consecutive messages of the stream
  uint32_t np0, np, npMagic;       // pieces of field 0, of a message, div_magic(np)
  uint32_t ns, nsMagic;           // statistics pieces of a message (np - np0), div_magic(ns)
  int msgs;                       // messages of the stream in this launch
  int msgsPerEntry;
};

__device__ __forceinline__ void setup_stream(Stream& st, const KernelArgs& a, int peer, int ch) {
  st.np0 = static_cast<uint32_t>(a.np0);
  st.np = static_cast<uint32_t>(a.np);
  st.npMagic = a.npMagic;
  st.ns = st.np - st.np0;
  st.nsMagic = a.nsMagic;
  st.msgsPerEntry = a.msgsPerEntry;
  st.msgs = a.baseMsgs + (ch < a.extraChannels ? 1 : 0);  // stream_msg_count(a.entryBegin, a.entryEnd, ch, a.runChannels)
  st.firstRow = static_cast<uint32_t>(a.entryBegin + ch) * a.cpSize + peer;
  st.rowStep = static_cast<uint32_t>(a.runChannels) * a.cpSize;
}

// 16-byte units of a run of `msgs` messages of this stream's shape
__device__ __forceinline__ uint32_t stream_run_units(const Stream& st, int msgs) {
  const uint32_t pieces = static_cast<uint32_t>(msgs) * st.np;
  return (pieces + kPiecesPerLine - 1) / kPiecesPerLine * kUnitsPerLine;
}

// Byte offsets of the two payload pieces of run unit U inside the field
// tensors; kOutOfRange where a piece is not in that field (or is the flag
// word, padding, or beyond the run).
struct UnitOffsets {
  uint32_t a0, b0;  // pieces a (first word) and b (second word) in field 0
  uint32_t a1, b1;  // ... in field 1
};

// `runMsgs` bounds the run: pieces of later messages are padding of the last line.
__device__ __forceinline__ UnitOffsets unit_offsets(const Stream& st, uint32_t firstMsg, uint32_t runMsgs, uint32_t U,
                                                    bool live, RunUnit* decoded = nullptr) {
  const RunUnit d = decode_run_unit(U, st.np, st.npMagic);
  const uint32_t rowA = st.firstRow + (firstMsg + d.msgA) * st.rowStep;
  const uint32_t rowB = d.msgB == d.msgA ? rowA : rowA + st.rowStep;
  const uint32_t baseA0 = rowA * st.stride0, baseA1 = rowA * st.stride1;
  const uint32_t baseB0 = rowB * st.stride0, baseB1 = rowB * st.stride1;
  const bool aLive = live && d.msgA < runMsgs;
  const bool bLive = live && !d.flag && d.msgB < runMsgs;
  const uint32_t pa = d.pieceA, pb = d.pieceB;
  UnitOffsets o;
  o.a0 = (aLive && pa < st.np0) ? baseA0 + pa * kPieceBytes : kOutOfRange;
  o.b0 = (bLive && pb < st.np0) ? baseB0 + pb * kPieceBytes : kOutOfRange;
  o.a1 = (aLive && pa >= st.np0) ? baseA1 + (pa - st.np0) * kPieceBytes : kOutOfRange;
  o.b1 = (bLive && pb >= st.np0) ? baseB1 + (pb - st.np0) * kPieceBytes : kOutOfRange;
  if (decoded) *decoded = d;
  return o;
}

// ---------------------------------------------------------------------------
// sender
// ---------------------------------------------------------------------------
// Part `part` of the a.parts wavefronts that send stream (s -> r, ch): it walks its slice of every run.
// With kTeam the parts are the a.team wavefronts of this workgroup and share part 0's counters.
// kOddStats: the statistics rows are an odd number of floats (the combine's packed log-sum-exps); the exchange
// kernel never sees such rows, and a compile-time switch keeps their loads out of its instruction stream.
template <int kAux, int kUnitsInFlight, bool kTeam = false, bool kOddStats = false>
__device__ __forceinline__ void run_sender(const KernelArgs& a, int s, int r, int ch, int part, int lane, int wave,
                                           TeamLds* lds = nullptr) {
  HELIX_MARK(wave, 0, false);
  const bool leader = !kTeam || part == 0;
  const int sliceCount = kTeam ? a.team : a.parts;
  Stream st;
  setup_stream(st, a, r, ch);
  if (st.msgs == 0) return;
  uint8_t* senderRow = a.workspace + static_cast<uint64_t>(s) * a.rowStrideBytes;
  uint8_t* receiverRow = a.workspace + static_cast<uint64_t>(r) * a.rowStrideBytes;
  int64_t* info = reinterpret_cast<int64_t*>(senderRow + sender_info_offset(a.cpSize, a.maxChannels, r, ch));
  int64_t* token = info + sender_counter_slot(kTeam ? 0 : part);
  st.fifo = make_rsrc(receiverRow + stream_fifo_offset(s, ch, a.runChannels, a.slotBytes), fifo_extent(a));
  st.field0 = make_rsrc(a.rank[s].send0, a.sendBytes0);
  st.field1 = make_rsrc(a.rank[s].send1, a.sendBytes1);
  st.stride0 = a.sendStride0;
  st.stride1 = a.sendStride1;

  // the counters are only needed once the first payload loads are in flight
  int64_t step = 0, tail = 0;
  uint64_t broken = 0;
  if (leader) {
    step = counter_at_launch(token);
    tail = counter_at_launch(&info[1]);
    broken = broken_at_launch(a);
  }

  for (int firstMsg = 0; firstMsg < st.msgs; firstMsg += st.msgsPerEntry) {
    const int runMsgs = min(st.msgsPerEntry, st.msgs - firstMsg);
    const uint32_t runUnits = stream_run_units(st, runMsgs);
    const Slice slice = slice_of_run(runUnits, part, sliceCount, kTeam ? a.byTeam : a.byParts);
    bool opened = false;
    // open the FIFO entry of this run (csrc/helix_alltoall.cu:377-390); false when the wait for room gave up
    auto leader_opens = [&]() -> bool {
      if (broken != 0) {
        report_broken(a, lane);
        return false;
      }
      if (firstMsg > 0) {
        step += 1;
        if (!kTeam) wait_stores_acknowledged();
        if (lane == 0) st_counter(token, step);
      }
      SpinGuard guard(a.spinLimitTicks, broken_word(a));
      while (tail + kFifoDepth <= step) {  // the entry is free once the receiver released step - 4
        tail = ld_counter(&info[1]);
        if (tail + kFifoDepth > step) break;
        if (guard.expired()) {
          raise_status(a, kStatusSendTimeout, lane);
          return false;
        }
        __builtin_amdgcn_s_sleep(4);
      }
      return true;
    };
    auto open_entry = [&]() -> bool {
      opened = true;
      if (!kTeam) return leader_opens();
      if (firstMsg > 0) {  // the leader closes the previous entry once every wavefront's lines of it are in memory
        wait_stores_acknowledged();
        team_barrier();
      }
      bool ok = true;
      if (leader) ok = leader_opens();
      step = team_share_step(lds, leader, lane, ok ? step : -1);
      return step >= 0;
    };
    for (uint32_t U0 = slice.begin; U0 < slice.end; U0 += kUnitsInFlight * kWaveLanes) {
      // Statistics first: the statistics pieces of the whole pass in one load (two, beyond 64 pieces), lane j
      // taking the j-th of them in run order; the lanes that store them pick them up below. One load per wave
      // access that touches the end of a message, a few live lanes each, cost a sender as much as its payload
      // loads did. Loads return in the order they were issued, so with these first every store below waits for
      // the payload of its own access only.
      const uint32_t passFirst = (U0 / kUnitsPerLine) * kPiecesPerLine;
      uint32_t passEnd = passFirst + kUnitsInFlight * (kWaveLanes / kUnitsPerLine) * kPiecesPerLine;
      passEnd = min(passEnd, min(static_cast<uint32_t>(runMsgs) * st.np, (slice.end / kUnitsPerLine) * kPiecesPerLine));
      const uint32_t ordFirst = stats_ordinal_at(passFirst, st.np, st.np0, st.npMagic);
      const uint32_t ordEnd = passEnd > passFirst ? stats_ordinal_at(passEnd, st.np, st.np0, st.npMagic) : ordFirst;
      u32x2 gathered[kStatsGathers];
#pragma unroll
      for (int c = 0; c < kStatsGathers; ++c) {
        gathered[c] = u32x2{0u, 0u};
        if (ordFirst + c * kWaveLanes < ordEnd) {  // wave-uniform
          const uint32_t ord = ordFirst + c * kWaveLanes + lane;
          const uint32_t m = div_by_magic(ord, st.nsMagic);
          const uint32_t index = ord - m * st.ns;
          const uint32_t row = st.firstRow + (firstMsg + m) * st.rowStep;
          const uint32_t off = ord < ordEnd ? row * st.stride1 + index * kPieceBytes : kOutOfRange;
          if (!kOddStats) {
            gathered[c] = __builtin_amdgcn_raw_buffer_load_b64(st.field1, off, 0, kAuxNone);
          } else {
            // rows of an odd number of floats (one log-sum-exp per head): 4-byte aligned, and the upper
            // half of a row's last piece is not part of the row -- it travels as zero
            gathered[c].x = __builtin_amdgcn_raw_buffer_load_b32(st.field1, off, 0, kAuxNone);
            gathered[c].y = __builtin_amdgcn_raw_buffer_load_b32(st.field1, (off != kOutOfRange && index + 1u != st.ns) ? off + 4u : kOutOfRange, 0, kAuxNone);
          }
        }
      }
      u32x2 wa[kUnitsInFlight], wb[kUnitsInFlight];
      unsigned long long needField1[kUnitsInFlight];  // wave-uniform: lanes of access i that hold statistics pieces
#pragma unroll
      for (int i = 0; i < kUnitsInFlight; ++i) {
        uint32_t U = U0 + i * kWaveLanes + lane;
        UnitOffsets o = unit_offsets(st, firstMsg, runMsgs, U, U < slice.end);
        wa[i] = __builtin_amdgcn_raw_buffer_load_b64(st.field0, o.a0, 0, kAuxNone);
        wb[i] = __builtin_amdgcn_raw_buffer_load_b64(st.field0, o.b0, 0, kAuxNone);
        needField1[i] = __ballot((o.a1 != kOutOfRange) | (o.b1 != kOutOfRange));
      }
      // A wavefront that gives up here still runs through the stores of the pass, every lane out of range, and
      // leaves after them: an exit between the loads and the stores leaves through the end of this loop in the
      // compiled code, which then counts the loads as still in flight when the next pass starts and makes every
      // pass wait for registers that are long back.
      const bool open = opened || open_entry();
      if (U0 == slice.begin && firstMsg == 0) HELIX_MARK(wave, 1, true);
      const uint32_t entryOffset = (static_cast<uint32_t>(step) & a.positionMask) * a.positionBytes;
      const uint32_t stepLo = static_cast<uint32_t>(step);
      const uint32_t stepHi = static_cast<uint32_t>(static_cast<uint64_t>(step) >> 32);
      // the statistics piece with ordinal `ord`, from the lane that loaded it
      auto statistics_piece = [&](uint32_t ord) -> u32x2 {
        const uint32_t rel = ord - ordFirst;
        const int from = static_cast<int>((rel & (kWaveLanes - 1)) * 4u);
        u32x2 v = {static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(gathered[0].x))),
                   static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(gathered[0].y)))};
        if (ordFirst + kWaveLanes < ordEnd) {  // wave-uniform: a second load was needed
          const u32x2 w = {static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(gathered[1].x))),
                           static_cast<uint32_t>(__builtin_amdgcn_ds_bpermute(from, static_cast<int>(gathered[1].y)))};
          if (rel >= static_cast<uint32_t>(kWaveLanes)) v = w;
        }
        return v;
      };
#pragma unroll
      for (int i = 0; i < kUnitsInFlight; ++i) {
        uint32_t U = U0 + i * kWaveLanes + lane;
        bool flag = (U & 7u) == 7u;
        u32x2 pa = wa[i], pb = wb[i];
        if (needField1[i] != 0ull) {  // a piece comes from one of the two tensors; the payload load gave zeros elsewhere
          RunUnit d;
          UnitOffsets o = unit_offsets(st, firstMsg, runMsgs, U, U < slice.end, &d);
          const u32x2 sa = statistics_piece(d.msgA * st.ns + (d.pieceA - st.np0));
          const u32x2 sb = statistics_piece(d.msgB * st.ns + (d.pieceB - st.np0));
          if (o.a1 != kOutOfRange) pa = sa;
          if (o.b1 != kOutOfRange) pb = sb;
        }
        u32x4 v = {pa.x, pa.y, flag ? stepLo : pb.x, flag ? stepHi : pb.y};
        uint32_t off = (open && U < slice.end) ? entryOffset + U * kUnitBytes : kOutOfRange;
        __builtin_amdgcn_raw_buffer_store_b128(v, st.fifo, off, 0, kAux);
      }
      if (!open) return;
    }
    if (!opened && !open_entry()) return;  // nothing of this run falls to this part: the step still counts
  }
  // Close the last entry (csrc/helix_alltoall.cu:409-412): once this part's stores are acknowledged its
  // counter moves beyond the step, which tells the receiving part that every line of the slice is in memory.
  HELIX_MARK(wave, 2, false);
  wait_stores_acknowledged();
  HELIX_MARK(wave, 3, false);
  if (kTeam) team_barrier();
  if (leader && lane == 0) st_counter(token, step + 1);
}

// ---------------------------------------------------------------------------
// receiver
// ---------------------------------------------------------------------------
// Part `part` of the wavefronts that receive stream (s -> r, ch). It waits for the token of the sending
// part (that part's counter beyond the step: all its lines of the step are in memory), reads its slice
// in passes of kUnitsInFlight units per lane and stores the payload. Line flags are still compared: one
// that disagrees after the token means the workspace is corrupt.
// `stage`: kStatsGathers * 64 pieces of LDS of this wavefront's own.
template <int kAux, int kUnitsInFlight, bool kAlignedStores, bool kTeam = false>
__device__ __forceinline__ void run_receiver(const KernelArgs& a, int r, int s, int ch, int part, int lane, int wave,
                                             u32x2* stage, TeamLds* lds = nullptr) {
  HELIX_MARK(wave, 0, false);
  const bool leader = !kTeam || part == 0;
  const int sliceCount = kTeam ? a.team : a.parts;
  const int counterPart = kTeam ? 0 : part;
  Stream st;
  setup_stream(st, a, s, ch);
  if (st.msgs == 0) return;
  uint8_t* senderRow = a.workspace + static_cast<uint64_t>(s) * a.rowStrideBytes;
  uint8_t* receiverRow = a.workspace + static_cast<uint64_t>(r) * a.rowStrideBytes;
  int64_t* senderInfo = reinterpret_cast<int64_t*>(senderRow + sender_info_offset(a.cpSize, a.maxChannels, r, ch));
  int64_t* info = reinterpret_cast<int64_t*>(receiverRow + receiver_info_offset(a.cpSize, a.maxChannels, s, ch));
  int64_t* token = senderInfo + sender_counter_slot(counterPart);
  int64_t* mine = info + receiver_counter_slot(counterPart);
  st.fifo = make_rsrc(receiverRow + stream_fifo_offset(s, ch, a.runChannels, a.slotBytes), fifo_extent(a));
  st.field0 = make_rsrc(a.rank[r].recv0, a.recvBytes0);
  st.field1 = make_rsrc(a.rank[r].recv1, a.recvBytes1);
  st.stride0 = a.recvStride0;
  st.stride1 = a.recvStride1;

  int64_t step = 0, head = 0;
  bool broken = false;
  if (leader) {
    step = counter_at_launch(mine);
    // The first look at the sender's counter. Senders come first in a launch, so most receivers find their run
    // closed already. In launches of long runs (several passes per run, teams) that look goes through the scalar
    // cache too, and the vector loads of the lines do not queue behind a vector load of the counter. Such a look
    // can only be older than memory, never newer (a line this CU's scalar cache or this XCD's L2 took in earlier
    // in the launch): a run that looks open is polled through coherent vector loads below, a run that looks
    // closed is closed, and its lines -- stored and acknowledged before the counter moved -- are read past the
    // caches. (Measured on MI355X: c4 87.6 -> 83.3 us, c5a 99.3 -> 97.9; launches of single-pass runs gain
    // nothing from it hot and lose 1 % on rotating tensors -- c3 26.7 -> 27.05 us -- and keep the vector load.)
    head = (kAlignedStores || kTeam) ? counter_at_launch(token) : ld_counter(token);
    broken = broken_at_launch(a) != 0;
    if (kTeam && lane == 0) *reinterpret_cast<volatile int*>(&lds->bad) = 0;  // ahead of the team's first barrier
  }
  bool corrupt = false;  // this wavefront met a line whose flag disagrees with the token: it stores nothing from then on

  for (int firstMsg = 0; firstMsg < st.msgs; firstMsg += st.msgsPerEntry) {
    const int runMsgs = min(st.msgsPerEntry, st.msgs - firstMsg);
    const uint32_t runUnits = stream_run_units(st, runMsgs);
    const Slice slice = slice_of_run(runUnits, part, sliceCount, kTeam ? a.byTeam : a.byParts);
    // the leader releases the previous entry and waits for the token of this one; false when it gave up
    auto leader_acquires = [&]() -> bool {
      if (broken) {
        report_broken(a, lane);
        return false;
      }
      if (firstMsg > 0) {
        // the lines of the previous entry have been consumed (csrc/helix_alltoall.cu:427-449);
        // part 0's counter is the tail the sender's back-pressure reads
        step += 1;
        if (lane == 0) {
          st_counter(mine, step);
          if (counterPart == 0) st_counter(&senderInfo[1], step);
        }
      }
      if (head <= step) {
        SpinGuard guard(a.spinLimitTicks, broken_word(a));
        for (;;) {
          head = ld_counter(token);
          if (head > step) break;
          if (guard.expired()) {
            raise_status(a, kStatusRecvTimeout, lane);
            return false;
          }
          __builtin_amdgcn_s_sleep(1);
        }
      }
      return true;
    };
    if (!kTeam) {
      if (!leader_acquires()) return;
    } else {
      if (firstMsg > 0) team_barrier();  // every wavefront of the team has its lines of the previous entry in registers
      bool ok = true;
      if (leader) ok = !team_is_bad(lds) && leader_acquires();  // after a corrupt line the team leaves, counters untouched
      step = team_share_step(lds, leader, lane, ok ? step : -1);
      if (step < 0) return;
    }
    asm volatile("" ::: "memory");  // no line is read before the token was seen
    const uint32_t entryOffset = (static_cast<uint32_t>(step) & a.positionMask) * a.positionBytes;
    const uint32_t stepLo = static_cast<uint32_t>(step);
    const uint32_t stepHi = static_cast<uint32_t>(static_cast<uint64_t>(step) >> 32);
    for (uint32_t U0 = slice.begin; U0 < slice.end; U0 += kUnitsInFlight * kWaveLanes) {
      const uint32_t passEnd = min(U0 + kUnitsInFlight * kWaveLanes, slice.end);
      u32x4 v[kUnitsInFlight];
#pragma unroll
      for (int i = 0; i < kUnitsInFlight; ++i) {
        uint32_t U = U0 + i * kWaveLanes + lane;
        uint32_t off = U < passEnd ? entryOffset + U * kUnitBytes : kOutOfRange;
        v[i] = __builtin_amdgcn_raw_buffer_load_b128(st.fifo, off, 0, kAux);
      }
      // Loads return in the order they were issued and the stores of access i need nothing but the load of access
      // i (the realigned variant: and of i + 1), so every store goes out as soon as its own lines are back, while
      // the later ones are still in flight. Every line carries its flag in the very load that brought its last
      // unit; the flags are compared on the way, without a branch, and looked at once the pass is stored.
      if (U0 == slice.begin && firstMsg == 0) HELIX_MARK(wave, 1, false);
      bool flagsAgree = true;
      // where the statistics pieces of the pass sit among those of the run (see run_sender)
      const uint32_t piecesFirst = (U0 / kUnitsPerLine) * kPiecesPerLine;
      const uint32_t piecesEnd = (kTeam && corrupt) ? piecesFirst
                                                    : min((passEnd / kUnitsPerLine) * kPiecesPerLine, static_cast<uint32_t>(runMsgs) * st.np);
      const uint32_t ordFirst = stats_ordinal_at(piecesFirst, st.np, st.np0, st.npMagic);
      const uint32_t ordEnd = piecesEnd > piecesFirst ? stats_ordinal_at(piecesEnd, st.np, st.np0, st.npMagic) : ordFirst;
#pragma unroll
      for (int i = 0; i < kUnitsInFlight; ++i) {
        uint32_t U = U0 + i * kWaveLanes + lane;
        flagsAgree &= U >= passEnd || (U & 7u) != 7u || (v[i].z == stepLo && v[i].w == stepHi);
        RunUnit d;
        UnitOffsets o = unit_offsets(st, firstMsg, runMsgs, U, U < passEnd && !(kTeam && corrupt), &d);
        u32x2 wa = {v[i].x, v[i].y};
        u32x2 wb = {v[i].z, v[i].w};
        if (kAlignedStores) {
          // Messages follow each other piece by piece and a line carries 15 of
          // them, so the two pieces of a unit sit astride a 16-byte boundary
          // of the output row about half of the time, and the two 8-byte stores
          // of an access then each write every other 8 bytes. With the whole
          // pass in registers every lane stores the aligned 16 bytes ("chunk")
          // that start at whichever of its words is an even partial_o piece:
          //   first word even:   both own words, or -- in the flag unit -- the
          //                      own word + the first word of the next unit;
          //   second word even:  that word + the first word of the next unit;
          // the next unit being the next lane (for lane 63, lane 0 of the next
          // access). An odd first word belongs to the previous unit's chunk.
          // Where the pass ends between the halves of a chunk, both are stored
          // alone. (Costs a dozen vector instructions per unit and halves the
          // store instructions: measured on MI355X it is 5-6 % faster on long
          // runs and 2 % slower on runs of one short pass, hence a template
          // parameter the host sets through KernelArgs::alignedStores.)
          uint32_t nx = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v[i].x), kDppWaveShl1, 0xF, 0xF, false));
          uint32_t ny = static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v[i].y), kDppWaveShl1, 0xF, 0xF, false));
          const bool haveNext = U + 1u < passEnd;
          if (i + 1 < kUnitsInFlight) {
            const uint32_t fx = lane_value(v[i + 1 < kUnitsInFlight ? i + 1 : i].x, 0);
            const uint32_t fy = lane_value(v[i + 1 < kUnitsInFlight ? i + 1 : i].y, 0);
            if (lane == kWaveLanes - 1) {
              nx = fx;
              ny = fy;
            }
          }
          const bool startsAtA = o.a0 != kOutOfRange && (d.pieceA & 1u) == 0u;
          const bool startsAtB = o.b0 != kOutOfRange && (d.pieceB & 1u) == 0u;
          const bool takesNext = startsAtB || (startsAtA && d.flag);
          const bool store16 = (startsAtA || startsAtB) && (!takesNext || haveNext);
          u32x4 chunk = {startsAtB ? v[i].z : v[i].x, startsAtB ? v[i].w : v[i].y, takesNext ? nx : v[i].z,
                         takesNext ? ny : v[i].w};
          __builtin_amdgcn_raw_buffer_store_b128(chunk, st.field0, store16 ? (startsAtB ? o.b0 : o.a0) : kOutOfRange, 0,
                                                 kAuxNt);
          // the halves of a chunk the pass boundary separates: the last unit's lone first word (a flag
          // unit: passes end on line boundaries), the first unit's odd first word
          const bool alone = o.a0 != kOutOfRange && ((U + 1u == passEnd && startsAtA && d.flag) ||
                                                     (U == U0 && (d.pieceA & 1u) != 0u));
          if (__ballot(alone) != 0ull)
            __builtin_amdgcn_raw_buffer_store_b64(wa, st.field0, alone ? o.a0 : kOutOfRange, 0, kAuxNt);
        } else {
          __builtin_amdgcn_raw_buffer_store_b64(wa, st.field0, o.a0, 0, kAuxNt);
          __builtin_amdgcn_raw_buffer_store_b64(wb, st.field0, o.b0, 0, kAuxNt);
        }
        // Statistics sit at the end of a message: few accesses hold pieces of the second tensor. Each such piece
        // is put where the lane that stores it will look: slot "number of the piece among the statistics pieces of
        // the pass" of this wavefront's staging row in LDS.
        // (kernels of long runs only: where a run is one short pass, the trip through LDS at the end of the
        // wavefront's only pass costs more than the few stores it saves -- c2 5.5 -> 5.9 us)
        if (__ballot((o.a1 != kOutOfRange) | (o.b1 != kOutOfRange)) != 0ull) {
          if (kAlignedStores) {
            if (o.a1 != kOutOfRange) stage[d.msgA * st.ns + (d.pieceA - st.np0) - ordFirst] = wa;
            if (o.b1 != kOutOfRange) stage[d.msgB * st.ns + (d.pieceB - st.np0) - ordFirst] = wb;
          } else {
            // (no streaming hint: a statistics row can be as small as 8 bytes, and the rows of the
            // cp senders share 64-byte sectors that the L2 should merge before they go to memory)
            __builtin_amdgcn_raw_buffer_store_b64(wa, st.field1, o.a1, 0, kAuxNone);
            __builtin_amdgcn_raw_buffer_store_b64(wb, st.field1, o.b1, 0, kAuxNone);
          }
        }
      }
      // The statistics pieces of the whole pass go out in one store (two, beyond 64 pieces), lane j taking the j-th
      // of them in run order. One store of a few live lanes per wave access that touches the end of a message cost
      // a receiver as much as its payload stores did.
#pragma unroll
      for (int c = 0; c < (kAlignedStores ? kStatsGathers : 0); ++c) {
        if (ordFirst + c * kWaveLanes < ordEnd) {  // wave-uniform
          const uint32_t ord = ordFirst + c * kWaveLanes + lane;
          const uint32_t m = div_by_magic(ord, st.nsMagic);
          const uint32_t index = ord - m * st.ns;
          const uint32_t row = st.firstRow + (firstMsg + m) * st.rowStep;
          const u32x2 piece = stage[c * kWaveLanes + lane];
          // (no streaming hint: a statistics row can be as small as 8 bytes, and the rows of the
          // cp senders share 64-byte sectors that the L2 should merge before they go to memory)
          __builtin_amdgcn_raw_buffer_store_b64(piece, st.field1, ord < ordEnd ? row * st.stride1 + index * kPieceBytes : kOutOfRange,
                                                0, kAuxNone);
        }
      }
      if (__ballot(!flagsAgree) != 0ull) {
        // a line of this pass did not carry the step: the pass went out as it came, nothing goes out after it
        raise_status(a, kStatusInternal, lane);
        if (!kTeam) return;
        // a wavefront of a team stays with its team to the next barrier, where the leader learns of it; it
        // stores nothing any more, and the workspace is marked broken
        if (!corrupt) team_report_bad(lds, lane);
        corrupt = true;
      }
    }
  }
  HELIX_MARK(wave, 2, false);
  if (kTeam) team_barrier();  // every wavefront of the team has the lines of the last entry in registers
  if (kTeam && leader && team_is_bad(lds)) return;
  if (leader && lane == 0) {  // close the last entry (csrc/helix_alltoall.cu:468-472)
    st_counter(mine, step + 1);
    if (counterPart == 0) st_counter(&senderInfo[1], step + 1);
  }
  HELIX_MARK(wave, 3, true);
}

// The one wave-uniform branch on the units-in-flight count of the launch.
template <int kAux, bool kOddStats>
__device__ __forceinline__ void run_sender_any(const KernelArgs& a, int s, int r, int ch, int part, int lane, int wave) {
  switch (a.unitsInFlight) {
    case 1: run_sender<kAux, 1, false, kOddStats>(a, s, r, ch, part, lane, wave); break;
    case 2: run_sender<kAux, 2, false, kOddStats>(a, s, r, ch, part, lane, wave); break;
    case 3: run_sender<kAux, 3, false, kOddStats>(a, s, r, ch, part, lane, wave); break;
    case 4: run_sender<kAux, 4, false, kOddStats>(a, s, r, ch, part, lane, wave); break;
    case 5: run_sender<kAux, 5, false, kOddStats>(a, s, r, ch, part, lane, wave); break;
    default: run_sender<kAux, kMaxUnitsInFlight, false, kOddStats>(a, s, r, ch, part, lane, wave); break;
  }
}
// Wavefront w of a launch: sender wavefronts come first in dispatch order so
// that no receiver can occupy a slot a not-yet-started sender needs.
// Within a direction, w = ((local rank * runChannels + channel) * cp + peer) * parts + part:
// neighbouring wavefronts touch neighbouring slices, then neighbouring rows of the same entry.
// With kTeam a workgroup is one team: workgroup b serves stream b of the launch (parts = 1).
// (Teams run six wavefronts per SIMD instead of four: a workgroup is then a team of 3..8 wavefronts, and sixteen
// slots per CU hold only five teams of three, or three of five; with 24 slots c4's teams of three measured 88.5 ->
// 85.4 us, teams of five 140 -> 101 us. Launches of independent wavefronts stay at four, where 5, 6 and 8 are slower.)
template <int kUnitsInFlight, bool kAlignedStores, bool kTeam>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(kTeam ? 6 : 4, kTeam ? 6 : 4))) void helix_exchange_kernel(KernelArgs a) {
  __shared__ TeamLds teamLds;
  // a row per wavefront, for the receivers of long runs
  __shared__ u32x2 statisticsStage[!kAlignedStores ? 1 : kTeam ? kMaxTeamWavefronts : kMaxWavesPerBlock][kAlignedStores ? kStatsGathers * kWaveLanes : 1];
  fetch_scalars_up_front(a);
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWaveLanes);
  const int lane = static_cast<int>(threadIdx.x) % kWaveLanes;
  const int probe = static_cast<int>(blockIdx.x) * a.wavesPerBlock + wave;  // index of the wavefront in the launch
  // Workgroups of the sending direction come first, a.dirBlocks of them, then as many that receive.
  const bool isSender = a.doSend != 0 && static_cast<int>(blockIdx.x) < a.dirBlocks;
  int block = static_cast<int>(blockIdx.x) - (a.doSend != 0 && !isSender ? a.dirBlocks : 0);
  block = xcd_grouped(block, a.xcdGroup);
  const int w = kTeam ? block : block * a.wavesPerBlock + wave;
  const int perDirection = a.rankCount * a.runChannels * a.cpSize * a.parts;
  if (w >= perDirection) return;
  const int q = static_cast<int>(fast_div_by(static_cast<uint32_t>(w), a.byParts));
  const int part = kTeam ? wave : w - q * a.parts;
  const int t = static_cast<int>(fast_div_by(static_cast<uint32_t>(q), a.byCp));
  const int peer = q - t * a.cpSize;
  const int localIndex = static_cast<int>(fast_div_by(static_cast<uint32_t>(t), a.byChannels));
  const int ch = t - localIndex * a.runChannels;
  const int local = a.rankBegin + localIndex;
  if (isSender) {
    run_sender<kAuxSc1, kUnitsInFlight, kTeam>(a, local, peer, ch, part, lane, probe, &teamLds);
  } else {
    run_receiver<kAuxSc1, kUnitsInFlight, kAlignedStores, kTeam>(a, local, peer, ch, part, lane, probe, statisticsStage[kAlignedStores ? wave : 0], &teamLds);
  }
}

// ---------------------------------------------------------------------------
// exchange fused with the LSE-weighted combine
// ---------------------------------------------------------------------------
// Element conversions of partial_o (4 elements per 8-byte piece).
template <int kDtype>
__device__ __forceinline__ void widen4(u32x2 piece, float (&f)[4]);
template <>
__device__ __forceinline__ void widen4<0>(u32x2 piece, float (&f)[4]) {  // bf16: the upper half of an fp32
  f[0] = __uint_as_float(piece.x << 16);
  f[1] = __uint_as_float(piece.x & 0xFFFF0000u);
  f[2] = __uint_as_float(piece.y << 16);
  f[3] = __uint_as_float(piece.y & 0xFFFF0000u);
}
template <>
__device__ __forceinline__ void widen4<1>(u32x2 piece, float (&f)[4]) {  // fp16
  f[0] = __half2float(__ushort_as_half(static_cast<unsigned short>(piece.x & 0xFFFFu)));
  f[1] = __half2float(__ushort_as_half(static_cast<unsigned short>(piece.x >> 16)));
  f[2] = __half2float(__ushort_as_half(static_cast<unsigned short>(piece.y & 0xFFFFu)));
  f[3] = __half2float(__ushort_as_half(static_cast<unsigned short>(piece.y >> 16)));
}

// Receive half of the fused form. The workgroup of one (receiver, channel) walks the payload of the
// run in output order: its wavefronts take turns at accesses of 64 consecutive 8-byte pieces of the
// combined output, a lane owns one piece (four elements of one head of one entry), finds that piece
// in the run (message j, piece p -> run piece j*np + p -> line and word: the same place in every
// sender's FIFO, since all streams of a channel share one layout), loads it from each sender's
// FIFO, and reduces over the senders in registers:
//   out[e, h, :] = sum_s w[s, h] * partial_o_s[e, h, :],  w = softmax_s(lse[s, h])
// (patches/dcp_alltoall_helix.py:142-207). The output goes out as one coalesced 8-byte store per
// lane. The wavefront first acquires the run from every sender through that sender's step counter,
// so every line it touches afterwards is complete (the flag words are not loaded here at all).
//
// Weights are computed once per wavefront and (message, head), not once per lane: the pieces of an
// access cover a few heads. The lanes that start a head enter it in a slot table (LDS), then the
// wavefront turns sideways -- lane i serves slot i / G and sender i % G, loads that sender's
// statistics of that head, and a softmax over the G lanes of a slot gives the weight -- and the
// weights go back through LDS to the lanes that own pieces of the head. (G = 4, 8, 16 or 32 lanes
// per slot for cpSize <= 4, 8, 16, 32.) With up to sixteen senders a lane handles two accesses per
// turn (sixteen loads in flight with eight senders, thirty-two with sixteen: c5a -1 % against one
// access), with more senders one.
constexpr int kCombineSlots = 32;  // distinct (message, head) pairs one turn may touch (head_dim >= 32: at most 18)

struct CombineCtx {
  __amdgpu_buffer_rsrc_t fifos;  // the whole FIFO region of the receiver's row
  uint32_t channelBase;          // byte offset of sender 0's FIFO of this channel
  uint32_t senderStride;         // bytes between the FIFOs of consecutive senders
  uint32_t stepLo;               // lane q: step counter (low word) of sender q's stream
  uint32_t positionBytes;        // bytes between the positions an entry of a stream rotates through
  uint32_t positionMask;         // positions of this launch - 1
};

template <int kLanesPerSlot>
struct CombineLds {
  uint32_t slot[kMaxCombineParts][kCombineSlots][4];  // {first run piece of the message, head, entry, -}
  float __attribute__((aligned(16))) weight[kMaxCombineParts][kCombineSlots][kLanesPerSlot];  // softmax weight per sender
};

__device__ __forceinline__ float shuffle_xor(float v, int mask) { return __shfl_xor(v, mask, kWaveLanes); }

// byte offset of sender q's open FIFO entry inside the receiver's FIFO region
__device__ __forceinline__ uint32_t entry_base(const CombineCtx& cx, int q, uint32_t stepLo) {
  return cx.channelBase + static_cast<uint32_t>(q) * cx.senderStride + (stepLo & cx.positionMask) * cx.positionBytes;
}

// byte offset of run piece g inside a FIFO entry: line g / 15, word g % 15
__device__ __forceinline__ uint32_t run_piece_offset(uint32_t g) {
  const uint32_t line = __umulhi(g, 0x11111112u);  // floor(g / 15) for g < 2^16 (div_magic(15))
  return line * kLineBytes + (g - line * kPiecesPerLine) * kPieceBytes;
}

// exp and ln on the hardware's base-2 units (v_exp_f32 / v_log_f32, about 1 ulp):
// the result is rounded to 8 or 11 mantissa bits anyway. exp(-inf) = 0,
// ln(0) = -inf, ln(x < 0) = NaN hold.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ __forceinline__ float fast_log(float x) { return __builtin_amdgcn_logf(x) * 0.6931471805599453f; }

// log-sum-exp of head h from the 8-byte statistics piece {s0, s1} that holds it;
// NaN and +-inf count as "no contribution".
//   mode 0: piece h = {lse, unused}     mode 1: piece h = {running max, running sum}
//   mode 2: piece h/2 = {lse of head 2*(h/2), lse of head 2*(h/2)+1}
// With base2 the log-sum-exp values are base-2 logarithms (the is_lse_base_on_e=False of
// patches/dcp_alltoall_helix.py:183-186); they are brought to natural logarithms here.
__device__ __forceinline__ float lse_of_stats(uint32_t s0, uint32_t s1, int statsMode, uint32_t h, bool base2) {
  float x = __uint_as_float((statsMode == 2 && (h & 1u)) ? s1 : s0);
  if (statsMode == 1) x = x + fast_log(__uint_as_float(s1));  // running max + ln(running sum)
  else if (base2) x *= 0.6931471805599453f;
  return (isnan(x) || isinf(x)) ? -INFINITY : x;
}

// four fp32 -> one 8-byte piece of bf16 (v_cvt_pk_bf16_f32: round to nearest even, NaN stays NaN) or fp16
template <int kDtype>
__device__ __forceinline__ u32x2 narrow_piece(const float (&acc)[4]);
template <>
__device__ __forceinline__ u32x2 narrow_piece<0>(const float (&acc)[4]) {
  using f32x2 = float __attribute__((ext_vector_type(2)));
  using bf16x2 = __bf16 __attribute__((ext_vector_type(2)));
  const bf16x2 lo = __builtin_convertvector(f32x2{acc[0], acc[1]}, bf16x2);
  const bf16x2 hi = __builtin_convertvector(f32x2{acc[2], acc[3]}, bf16x2);
  u32x2 r = {__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi)};
  return r;
}
template <>
__device__ __forceinline__ u32x2 narrow_piece<1>(const float (&acc)[4]) {
  using f32x2 = float __attribute__((ext_vector_type(2)));
  using f16x2 = _Float16 __attribute__((ext_vector_type(2)));
  const f16x2 lo = __builtin_convertvector(f32x2{acc[0], acc[1]}, f16x2);  // round to nearest even
  const f16x2 hi = __builtin_convertvector(f32x2{acc[2], acc[3]}, f16x2);
  u32x2 r = {__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi)};
  return r;
}

template <int kDtype, int kLanesPerSlot>
__device__ __forceinline__ void run_combine_receiver(const KernelArgs& a, int r, int ch, int part, int parts,
                                                     int lane, CombineLds<kLanesPerSlot>& lds, int probe) {
  HELIX_MARK(probe, 0, false);
  constexpr int kSlotsPerPass = kWaveLanes / kLanesPerSlot;
  constexpr int kAccesses = kLanesPerSlot <= 16 ? 2 : 1;                  // accesses a lane handles per turn
  constexpr int kGroup = kLanesPerSlot <= 16 ? kLanesPerSlot : 16;       // senders whose pieces are in flight together
  Stream st;
  setup_stream(st, a, 0, ch);
  if (st.msgs == 0) return;  // uniform over the workgroup: same channel
  uint8_t* receiverRow = a.workspace + static_cast<uint64_t>(r) * a.rowStrideBytes;
  CombineCtx cx;
  cx.fifos = make_rsrc(receiverRow, static_cast<uint32_t>(fifo_region_bytes(a.cpSize, a.maxChannels)));
  cx.channelBase = static_cast<uint32_t>(stream_fifo_offset(0, ch, a.runChannels, a.slotBytes));
  cx.senderStride = static_cast<uint32_t>(stream_fifo_offset(1, 0, a.runChannels, a.slotBytes));
  cx.positionBytes = a.positionBytes;
  cx.positionMask = a.positionMask;
  __amdgpu_buffer_rsrc_t outRsrc = make_rsrc(a.rank[r].recv0, a.recvBytes0);
  const bool wantLse = a.rank[r].recv1 != nullptr;
  __amdgpu_buffer_rsrc_t lseRsrc = make_rsrc(a.rank[r].recv1, wantLse ? a.recvBytes1 : 0u);
  const unsigned long long lanesUpToMe = (2ull << lane) - 1ull;  // lanes 0..lane
  const uint32_t piecesPerHead = static_cast<uint32_t>(a.headDim) / 4u;

  // lane q owns the counters of sender q's stream
  int64_t myStep = 0;
  int64_t* myInfo = nullptr;
  int64_t* mySenderInfo = nullptr;
  if (lane < a.cpSize) {
    uint8_t* senderRow = a.workspace + static_cast<uint64_t>(lane) * a.rowStrideBytes;
    myInfo = reinterpret_cast<int64_t*>(receiverRow + receiver_info_offset(a.cpSize, a.maxChannels, lane, ch));
    mySenderInfo = reinterpret_cast<int64_t*>(senderRow + sender_info_offset(a.cpSize, a.maxChannels, r, ch));
    myStep = myInfo[1];
  }
  const bool broken = broken_at_launch(a) != 0;
  __syncthreads();  // every part has read the counters before part 0 moves them
  if (broken) {
    report_broken(a, lane);
    return;
  }
  if (part == 0 && lane < a.cpSize) {
    // rounds never put more than the four entries in flight, so the entries can
    // be handed back up front; nothing reads these counters before the launch ends
    int64_t done = myStep + (ch < a.extraChannels ? a.entriesExtra : a.entriesBase);  // entries_for_msgs(st.msgs)
    st_counter(&myInfo[1], done);
    st_counter(&mySenderInfo[1], done);
  }

  for (int firstMsg = 0; firstMsg < st.msgs; firstMsg += st.msgsPerEntry, myStep += 1) {
    const int runMsgs = min(st.msgsPerEntry, st.msgs - firstMsg);
    const uint32_t runPieces = static_cast<uint32_t>(runMsgs) * st.np0;  // payload pieces of the run = output pieces
    cx.stepLo = static_cast<uint32_t>(myStep);
    {
      // Acquire the run from every sender: a counter beyond the step says that all
      // lines of the step are in memory (the sender waits for its stores before
      // it moves it). Every piece needs all cpSize senders anyway.
      // In launches of long runs, a first look through the scalar cache, sender by sender (wave-uniform
      // addresses): it does not queue behind the vector loads of the device, and it can only be older than
      // memory, never newer (see run_receiver). Measured on MI355X: c4 71.9 -> 70.8 us, c5a 79.5 -> 78.5; launches
      // of single-pass runs lose by it (c3 20.9 -> 21.7 us) and go straight to the vector loads.
      bool allClosed = a.longRuns != 0;
      for (int q = 0; allClosed && q < a.cpSize; ++q) {
        const uint8_t* senderRow = a.workspace + static_cast<uint64_t>(q) * a.rowStrideBytes;
        const int64_t* tok = reinterpret_cast<const int64_t*>(senderRow + sender_info_offset(a.cpSize, a.maxChannels, r, ch));
        const uint32_t lo = lane_value(static_cast<uint32_t>(myStep), q);
        const uint32_t hi = lane_value(static_cast<uint32_t>(static_cast<uint64_t>(myStep) >> 32), q);
        const int64_t stepOfQ = static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
        allClosed = allClosed & (counter_at_launch(tok) > stepOfQ);
      }
      SpinGuard guard(a.spinLimitTicks, broken_word(a));
      while (!allClosed) {
        const bool closed = lane >= a.cpSize || ld_counter(&mySenderInfo[0]) > myStep;
        if (__ballot(!closed) == 0ull) break;
        if (guard.expired()) {
          raise_status(a, kStatusRecvTimeout, lane);
          return;
        }
        __builtin_amdgcn_s_sleep(8);
      }
      asm volatile("" ::: "memory");
    }
    if (firstMsg == 0) HELIX_MARK(probe, 1, false);
    for (uint32_t P0 = static_cast<uint32_t>(part) * (kAccesses * kWaveLanes); P0 < runPieces;
         P0 += static_cast<uint32_t>(parts) * (kAccesses * kWaveLanes)) {
      // ---- where this lane's pieces are: in the run (every sender's FIFO alike) and in the output
      bool live[kAccesses];
      uint32_t fifoOff[kAccesses], outOff[kAccesses], msg[kAccesses], head[kAccesses], entry[kAccesses], piece[kAccesses];
#pragma unroll
      for (int k = 0; k < kAccesses; ++k) {
        const uint32_t P = P0 + static_cast<uint32_t>(k) * kWaveLanes + lane;
        live[k] = P < runPieces;
        msg[k] = div_by_magic(P, a.np0Magic);
        piece[k] = P - msg[k] * st.np0;
        head[k] = head_of_piece(piece[k], a.headMagic);
        entry[k] = static_cast<uint32_t>(a.entryBegin + ch) + (firstMsg + msg[k]) * a.runChannels;
        fifoOff[k] = live[k] ? run_piece_offset(msg[k] * st.np + piece[k]) : kOutOfRange;
        outOff[k] = live[k] ? (entry[k] * st.np0 + piece[k]) * kPieceBytes : kOutOfRange;
      }

      // The pieces do not depend on the weights: their loads go out first, and that round trip
      // overlaps the one of the statistics. Senders beyond cpSize are read out of range (zeros, no
      // memory traffic), which keeps the sequence free of branches.
      u32x2 v[kAccesses][kGroup];
      auto load_group = [&](int g) {
#pragma unroll
        for (int jq = 0; jq < kGroup; ++jq) {
          const int q = g + jq;
          const int qs = q < a.cpSize ? q : 0;
          const uint32_t base = entry_base(cx, qs, lane_value(cx.stepLo, qs));
#pragma unroll
          for (int k = 0; k < kAccesses; ++k)
            v[k][jq] = __builtin_amdgcn_raw_buffer_load_b64(cx.fifos, q < a.cpSize ? base + fifoOff[k] : kOutOfRange, 0, kAuxSc1);
        }
      };
      load_group(0);

      // ---- slots: one per distinct (message, head) the lanes of this turn touch, in piece order
      int mySlot[kAccesses];
      int slotCount = 0;
#pragma unroll
      for (int k = 0; k < kAccesses; ++k) {
        const bool starts = live[k] && (lane == 0 || piece[k] == head[k] * piecesPerHead);
        const unsigned long long mask = __ballot(starts);
        mySlot[k] = slotCount + __popcll(mask & lanesUpToMe) - 1;
        if (starts) {
          lds.slot[part][mySlot[k]][0] = msg[k] * st.np;
          lds.slot[part][mySlot[k]][1] = head[k];
          lds.slot[part][mySlot[k]][2] = entry[k];
        }
        if (!live[k]) mySlot[k] = 0;
        slotCount += __popcll(mask);
      }
      if (slotCount > kCombineSlots) {  // excluded by the host's shape check (head_dim >= 32)
        raise_status(a, kStatusInternal, lane);
        return;
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

      // ---- weights: lane i serves slot base + i / G and sender i % G
      for (int base = 0; base < slotCount; base += kSlotsPerPass) {
        const int slot = base + lane / kLanesPerSlot;
        const int q = lane % kLanesPerSlot;
        const bool inSlot = slot < slotCount;
        const bool serving = inSlot && q < a.cpSize;
        const int slotSafe = inSlot ? slot : 0;
        const uint32_t msgPiece0 = lds.slot[part][slotSafe][0];
        const uint32_t h = lds.slot[part][slotSafe][1];
        const uint32_t slotEntry = lds.slot[part][slotSafe][2];
        const uint32_t gs = msgPiece0 + st.np0 + (a.statsMode == 2 ? h >> 1 : h);  // run piece that holds head h's statistics
        const uint32_t qStepLo = static_cast<uint32_t>(__shfl(static_cast<int>(cx.stepLo), q < a.cpSize ? q : 0, kWaveLanes));
        const uint32_t off = entry_base(cx, q, qStepLo) + run_piece_offset(gs);
        const u32x2 sv = __builtin_amdgcn_raw_buffer_load_b64(cx.fifos, serving ? off : kOutOfRange, 0, kAuxSc1);
        const float lse = serving ? lse_of_stats(sv.x, sv.y, a.statsMode, h, a.lseBase2 != 0) : -INFINITY;
        float m = lse;
#pragma unroll
        for (int x = 1; x < kLanesPerSlot; x <<= 1) m = fmaxf(m, shuffle_xor(m, x));
        if (m == -INFINITY) m = 0.0f;  // every sender masked: weights 0, lse -inf
        float e = fast_exp(lse - m);
        if (isnan(e)) e = 0.0f;
        float total = e;
#pragma unroll
        for (int x = 1; x < kLanesPerSlot; x <<= 1) total += shuffle_xor(total, x);
        // (senders beyond cpSize get weight 0: their pieces are read as zeros, and 0 * 0 stays 0)
        if (inSlot) lds.weight[part][slotSafe][q] = e * __builtin_amdgcn_rcpf(fmaxf(total, 1e-10f));
        // one lane per slot reports the head's combined log-sum-exp
        if (wantLse) {  // wave-uniform: a store that every lane opts out of still costs its place in the store queue
          const float combinedLse = fast_log(total) + m;
          __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(a.lseBase2 ? combinedLse * 1.4426950408889634f : combinedLse), lseRsrc,
                                                (serving && q == 0) ? (slotEntry * a.heads + h) * 4u : kOutOfRange, 0,
                                                kAuxNone);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

      // ---- the piece of every sender, weighted
      float acc[kAccesses][4];
#pragma unroll
      for (int k = 0; k < kAccesses; ++k)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[k][c] = 0.0f;
#pragma unroll 1  // thirty-two senders: one group of sixteen pieces in registers at a time
      for (int g = 0; g < kLanesPerSlot; g += kGroup) {
        if (g > 0) load_group(g);
#pragma unroll
        for (int k = 0; k < kAccesses; ++k) {
          const float* w = &lds.weight[part][mySlot[k]][g];
#pragma unroll
          for (int jq = 0; jq < kGroup; ++jq) {
            float f[4];
            widen4<kDtype>(v[k][jq], f);
            const float wq = w[jq];
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[k][c] += wq * f[c];
          }
        }
      }
#pragma unroll
      for (int k = 0; k < kAccesses; ++k)
        __builtin_amdgcn_raw_buffer_store_b64(narrow_piece<kDtype>(acc[k]), outRsrc, outOff[k], 0, kAuxNone);
      __builtin_amdgcn_wave_barrier();  // the tables are rewritten by the next turn
    }
  }
  HELIX_MARK(probe, 2, false);
  HELIX_MARK(probe, 3, true);
}

// Workgroups of `parts` wavefronts (blockDim.x / 64). The first
// ceil(senderStreams / parts) workgroups send, one stream per wavefront; the
// rest receive and combine, one workgroup per (receiver, channel).
template <int kDtype, int kLanesPerSlot>
__global__ __launch_bounds__(kMaxCombineParts * kWaveLanes) HELIX_WAVES_PER_SIMD void helix_combine_kernel(KernelArgs a) {
  __shared__ CombineLds<kLanesPerSlot> lds;
  fetch_scalars_up_front(a);
  const int parts = a.wavesPerBlock;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWaveLanes);
  const int lane = static_cast<int>(threadIdx.x) % kWaveLanes;
  const int senderStreams = a.doSend ? a.rankCount * a.runChannels * a.cpSize : 0;
  const int sendBlocks = a.doSend ? a.sendBlocks : 0;  // ceil(senderStreams / parts)
  int b = static_cast<int>(blockIdx.x);
  if (b < sendBlocks) {
    const int w = b * parts + wave;
    if (w >= senderStreams) return;
    const int t = static_cast<int>(fast_div_by(static_cast<uint32_t>(w), a.byCp));
    const int localIndex = static_cast<int>(fast_div_by(static_cast<uint32_t>(t), a.byChannels));
    if ((a.field1Bytes & 7) == 0)
      run_sender_any<kAuxSc1, false>(a, a.rankBegin + localIndex, w - t * a.cpSize, t - localIndex * a.runChannels, 0, lane, w);
    else
      run_sender_any<kAuxSc1, true>(a, a.rankBegin + localIndex, w - t * a.cpSize, t - localIndex * a.runChannels, 0, lane, w);
    return;
  }
  b -= sendBlocks;
  const int localIndex = static_cast<int>(fast_div_by(static_cast<uint32_t>(b), a.byChannels));
  const int r = a.rankBegin + localIndex;
  const int ch = b - localIndex * a.runChannels;
  run_combine_receiver<kDtype, kLanesPerSlot>(a, r, ch, wave, parts, lane, lds, senderStreams + b * parts + wave);
}

// Before a launch that shares runs between wavefronts: the step counters of parts 1.. of every stream
// the launch touches take the value of part 0's (head on the sending side, tail on the receiving
// side). Launches with one wavefront per stream move part 0's counters only, so the others may be
// behind; this brings them level. One thread per (local rank, channel, peer) and direction.
__global__ __launch_bounds__(256) void helix_level_part_counters_kernel(KernelArgs a) {
  const int perDirection = a.rankCount * a.runChannels * a.cpSize;
  int i = static_cast<int>(blockIdx.x * blockDim.x + threadIdx.x);
  const int senders = a.doSend ? perDirection : 0;
  const int total = senders + (a.doRecv ? perDirection : 0);
  if (i >= total) return;
  const bool sending = i < senders;
  if (!sending) i -= senders;
  const int peer = i % a.cpSize;
  const int t = i / a.cpSize;
  const int ch = t % a.runChannels;
  const int local = a.rankBegin + t / a.runChannels;
  uint8_t* row = a.workspace + static_cast<uint64_t>(local) * a.rowStrideBytes;
  int64_t* info = reinterpret_cast<int64_t*>(
      row + (sending ? sender_info_offset(a.cpSize, a.maxChannels, peer, ch) : receiver_info_offset(a.cpSize, a.maxChannels, peer, ch)));
  const int64_t v = sending ? info[0] : info[1];
  for (int p = 1; p < a.parts; ++p) info[sending ? sender_counter_slot(p) : receiver_counter_slot(p)] = v;
}

// FIFO region <- 0xFF bytes, info regions <- 0 (csrc/helix_alltoall.cu:637-643).
__global__ __launch_bounds__(256) void helix_init_row_kernel(u32x4* row, uint64_t fifoUnits, uint64_t totalUnits) {
  const u32x4 ones = {0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu};
  const u32x4 zeros = {0u, 0u, 0u, 0u};
  uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < totalUnits; i += stride) {
    row[i] = i < fifoUnits ? ones : zeros;
  }
}

}  // namespace

// The largest run of the launch is the first one of channel 0's streams.
static long largest_run_units(const KernelArgs& a) {
  const MsgShape sh = make_msg_shape(a.field0Bytes, a.field1Bytes);
  const int msgs = stream_msg_count(a.entryBegin, a.entryEnd, 0, a.runChannels);
  const int perEntry = msgs_per_fifo_entry(sh);
  return run_units(msgs < perEntry ? msgs : perEntry, sh);
}

// The `group` of xcd_grouped for a launch direction of `blocks` workgroups of `wavesPerBlock` wavefronts in which
// `wavesPerPeerSet` consecutive wavefronts serve the peers of one (rank, channel), `streamsPerBlock` of them to
// a workgroup: the workgroups of one peer set, if the statistics rows of different workgroups share 128-byte
// lines at all and the tiling fits; else 0 (as dispatched). A power of two.
static int xcd_group_for(int wavesPerPeerSet, int wavesPerBlock, int streamsPerBlock, int blocks, int field1Bytes) {
  if (field1Bytes * streamsPerBlock >= 128) return 0;  // the rows a workgroup touches fill whole lines
  if (wavesPerPeerSet % wavesPerBlock != 0) return 0;
  const int group = wavesPerPeerSet / wavesPerBlock;
  if (group < 2 || (group & (group - 1)) != 0 || blocks % (8 * group) != 0) return 0;
  return group;
}

// The fields of the argument block that follow from the others (see KernelArgs); a.parts, a.team and
// a.unitsInFlight are set.
static void set_launch_constants(KernelArgs& a) {
  const MsgShape sh = make_msg_shape(a.field0Bytes, a.field1Bytes);
  a.np0 = sh.np0;
  a.np = sh.np;
  a.msgsPerEntry = msgs_per_fifo_entry(sh);
  const int entries = a.entryEnd > a.entryBegin ? a.entryEnd - a.entryBegin : 0;
  a.baseMsgs = entries / a.runChannels;
  a.extraChannels = entries % a.runChannels;
  a.entriesBase = entries_for_msgs(a.baseMsgs, sh);
  a.entriesExtra = entries_for_msgs(a.baseMsgs + 1, sh);
  const int entriesPerStream = a.extraChannels > 0 ? a.entriesExtra : a.entriesBase;
  a.positionMask = static_cast<uint32_t>(fifo_positions(exchange_lines_bytes(a.cpSize, a.runChannels, largest_run_units(a)), entriesPerStream)) - 1u;
  a.slotBytes = packed_slot_bytes(largest_run_units(a));
  a.positionBytes = fifo_position_bytes(a.cpSize, a.maxChannels);
  a.byParts = fast_div(static_cast<uint32_t>(a.parts));
  a.byTeam = fast_div(static_cast<uint32_t>(a.team));
  a.byCp = fast_div(static_cast<uint32_t>(a.cpSize));
  a.byChannels = fast_div(static_cast<uint32_t>(a.runChannels));
  // messages that are mostly statistics: passes short enough for the senders' gather (a.unitsInFlight is set)
  const int forStatistics = max_units_in_flight_for_statistics(a.np, a.np0);
  if (a.unitsInFlight > forStatistics) a.unitsInFlight = forStatistics;
}

hipError_t launch_exchange(const KernelArgs& args, int unitsPerPart, int maxParts, int teamUnits, hipStream_t stream) {
  KernelArgs a = args;
  if (a.runChannels <= 0) return hipSuccess;
  const long runUnits = largest_run_units(a);
  const RunSplit split = split_for_run(runUnits, unitsPerPart, maxParts);
  a.parts = split.parts;
  a.unitsInFlight = split.unitsInFlight;
  a.team = 1;
  int directions = (a.doSend ? 1 : 0) + (a.doRecv ? 1 : 0);
  int waves = directions * waves_per_direction(a) * a.parts;
  if (waves <= 0) return hipSuccess;
  if (a.parts == 1 && teamUnits != 0) {
    // Wavefronts that queue for slots anyway: a run of three or more passes goes to a team, one pass per
    // wavefront (c4's three passes: -3 %; two passes, c5a: +2 %, so those stay with one wavefront).
    const long perLane = (runUnits + kWaveLanes - 1) / kWaveLanes;
    const long passes = (perLane + kMaxUnitsInFlight - 1) / kMaxUnitsInFlight;
    if (teamUnits > 0 || (waves > kResidentWavefronts && passes >= 3)) {
      const RunSplit team = split_for_run(runUnits, teamUnits > 0 ? teamUnits : kMaxUnitsInFlight, kMaxTeamWavefronts);
      if (team.parts > 1) {
        a.team = team.parts;
        a.unitsInFlight = team.unitsInFlight;
      }
    }
  }
  a.alignedStores = runUnits > static_cast<long>(kMaxUnitsInFlight) * kWaveLanes ? 1 : 0;
  a.longRuns = a.alignedStores;
  set_launch_constants(a);
  if (a.parts > 1) {
    const int threads = directions * waves_per_direction(a);
    hipLaunchKernelGGL(helix_level_part_counters_kernel, dim3((threads + 255) / 256), dim3(256), 0, stream, a);
  }
  // Wavefronts of a workgroup without teams are independent (no LDS, no barrier). Two per workgroup dispatch and
  // retire at the finest useful grain when wavefronts queue for slots; a launch that fits the device at once is
  // bound by how fast its workgroups are dispatched, and four per workgroup halve that (c2: 7.2 -> 6.6 us).
  const int wpb = a.team > 1 ? a.team : waves <= kResidentWavefronts ? kMaxWavesPerBlock : kWavesPerBlock;
  const int perDirection = waves / directions;
  a.dirBlocks = a.team > 1 ? perDirection : (perDirection + wpb - 1) / wpb;
  // (launches with teams stay as dispatched: regrouped, c4 in the per-head layout took 0.7 % longer)
  a.xcdGroup = a.team > 1 ? 0 : xcd_group_for(a.cpSize * a.parts, wpb, a.parts > 1 ? 1 : wpb, a.dirBlocks, a.field1Bytes);
  int blocks = directions * a.dirBlocks;
  a.wavesPerBlock = wpb;
  // Short runs: 1..6 units in flight, payload stored piece by piece. Long runs (more than one
  // pass of six; at least 4 units in flight by the rule): the instantiation whose receivers
  // realign the payload to 16-byte stores.
#define HELIX_LAUNCH_EXCHANGE(K, ALIGNED)                                                                                 \
  do {                                                                                                                    \
    if (a.team > 1)                                                                                                       \
      hipLaunchKernelGGL((helix_exchange_kernel<K, ALIGNED, true>), dim3(blocks), dim3(wpb * kWaveLanes), 0, stream, a);  \
    else                                                                                                                  \
      hipLaunchKernelGGL((helix_exchange_kernel<K, ALIGNED, false>), dim3(blocks), dim3(wpb * kWaveLanes), 0, stream, a); \
  } while (0)
  if (a.alignedStores && a.unitsInFlight >= 4) {
    switch (a.unitsInFlight) {
      case 4: HELIX_LAUNCH_EXCHANGE(4, true); break;
      case 5: HELIX_LAUNCH_EXCHANGE(5, true); break;
      default: HELIX_LAUNCH_EXCHANGE(kMaxUnitsInFlight, true); break;
    }
  } else {
    switch (a.unitsInFlight) {
      case 1: HELIX_LAUNCH_EXCHANGE(1, false); break;
      case 2: HELIX_LAUNCH_EXCHANGE(2, false); break;
      case 3: HELIX_LAUNCH_EXCHANGE(3, false); break;
      case 4: HELIX_LAUNCH_EXCHANGE(4, false); break;
      case 5: HELIX_LAUNCH_EXCHANGE(5, false); break;
      default: HELIX_LAUNCH_EXCHANGE(kMaxUnitsInFlight, false); break;
    }
  }
#undef HELIX_LAUNCH_EXCHANGE
  return hipGetLastError();
}

hipError_t launch_combine(const KernelArgs& args, int parts, hipStream_t stream) {
  KernelArgs a = args;
  if (a.rankCount * a.runChannels <= 0) return hipSuccess;
  if (parts < 1) parts = 1;
  if (parts > kMaxCombineParts) parts = kMaxCombineParts;
  a.parts = 1;  // the senders of this kernel walk whole runs
  a.team = 1;
  a.unitsInFlight = units_in_flight_for_run(largest_run_units(a));
  a.alignedStores = 0;  // exchange kernel only
  a.longRuns = largest_run_units(a) > static_cast<long>(kMaxUnitsInFlight) * kWaveLanes ? 1 : 0;
  set_launch_constants(a);
  const int senderStreams = a.doSend ? a.rankCount * a.runChannels * a.cpSize : 0;
  a.sendBlocks = (senderStreams + parts - 1) / parts;
  a.wavesPerBlock = parts;
  a.dirBlocks = a.sendBlocks;
  a.xcdGroup = 0;  // regrouping the sending workgroups of this kernel was measured: nothing at c3 / c5a, +1.3 % at c4
  const int blocks = a.sendBlocks + a.rankCount * a.runChannels;
  dim3 block(static_cast<unsigned>(parts * kWaveLanes));
  // lanes per slot of the sideways pass: the smallest of 4, 8, 16, 32 that holds every sender
  const int g = a.cpSize <= 4 ? 4 : a.cpSize <= 8 ? 8 : a.cpSize <= 16 ? 16 : 32;
#define HELIX_LAUNCH_COMBINE(DT, G) hipLaunchKernelGGL((helix_combine_kernel<DT, G>), dim3(blocks), block, 0, stream, a)
  if (a.dtype == 1) {
    if (g == 4) HELIX_LAUNCH_COMBINE(1, 4);
    else if (g == 8) HELIX_LAUNCH_COMBINE(1, 8);
    else if (g == 16) HELIX_LAUNCH_COMBINE(1, 16);
    else HELIX_LAUNCH_COMBINE(1, 32);
  } else {
    if (g == 4) HELIX_LAUNCH_COMBINE(0, 4);
    else if (g == 8) HELIX_LAUNCH_COMBINE(0, 8);
    else if (g == 16) HELIX_LAUNCH_COMBINE(0, 16);
    else HELIX_LAUNCH_COMBINE(0, 32);
  }
#undef HELIX_LAUNCH_COMBINE
  return hipGetLastError();
}

#ifdef HELIX_A2A_TIMELINE
// Copies the phase stamps of the first `waves` wavefronts of the launches so far to the host
// (four 100 MHz clock values per wavefront) and clears them. Stamped builds only.
extern "C" int helix_a2a_timeline_read(uint64_t* host, int waves) {
  if (waves < 0 || waves > kTimelineWaves) return 1;
  void* dev = nullptr;
  if (hipGetSymbolAddress(&dev, HIP_SYMBOL(g_timeline)) != hipSuccess) return 2;
  if (hipDeviceSynchronize() != hipSuccess) return 2;
  if (hipMemcpy(host, dev, static_cast<size_t>(waves) * 4 * sizeof(uint64_t), hipMemcpyDeviceToHost) != hipSuccess) return 2;
  if (hipMemset(dev, 0, static_cast<size_t>(kTimelineWaves) * 4 * sizeof(uint64_t)) != hipSuccess) return 2;
  return 0;
}
#endif

hipError_t launch_init_row(uint8_t* row, uint64_t fifoBytes, uint64_t infoBytes, hipStream_t stream) {
  uint64_t fifoUnits = fifoBytes / kUnitBytes;
  uint64_t totalUnits = (fifoBytes + infoBytes) / kUnitBytes;
  if (totalUnits == 0) return hipSuccess;
  uint64_t want = (totalUnits + 255) / 256;
  int blocks = static_cast<int>(want < 8192 ? want : 8192);
  hipLaunchKernelGGL(helix_init_row_kernel, dim3(blocks), dim3(256), 0, stream, reinterpret_cast<u32x4*>(row),
                     fifoUnits, totalUnits);
  return hipGetLastError();
}

}  // namespace helix
