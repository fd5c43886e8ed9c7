// helix_kernels.hip -- gfx950 kernels of the Helix all-to-all.
//
// One wavefront owns one stream = (sender rank, receiver rank, channel) in one
// direction, the role a warp has in the reference kernel
// (csrc/helix_alltoall.cu:315-474). A sender wavefront reads its messages from
// the send tensors, turns them into LL128 lines in registers and stores the
// lines into the receiver's FIFO; a receiver wavefront polls the FIFO lines
// until their flags carry the expected step, then stores the payload into the
// receive tensors. There is no staging copy and no barrier: data moves
// global -> registers -> FIFO -> registers -> global, 16 bytes per lane on
// the FIFO side.
//
// The messages a stream puts into one FIFO entry form a "run": they follow
// each other without gaps from line 0 of the entry, so a wavefront walks a
// run as one flat sequence of 16-byte units, kUnitsInFlight units per lane at
// a time, regardless of message boundaries. All loads of a chunk are issued
// before the first store.
//
// Every global access goes through a buffer descriptor that spans exactly the
// tensor (or the one FIFO) it belongs to: the hardware returns zero for loads
// and drops stores that would fall outside, and an offset of kOutOfRange is
// how a lane opts out of an access without a branch.
//
// FIFO lines are written and polled with the sc1 cache policy (device-scope
// coherence: every XCD has its own L2, and the sender and the receiver of a
// stream may run on different XCDs).
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
constexpr int kAuxSc1 = 16;
constexpr uint32_t kRsrcWord3 = 0x00020000u;   // raw buffer, 32-bit data format
constexpr uint32_t kOutOfRange = 0x80000000u;  // beyond any descriptor (extents are < 2 GiB)

constexpr uint32_t kStatusRecvTimeout = 1u;
constexpr uint32_t kStatusSendTimeout = 2u;

// units a lane keeps in flight per chunk of a run
// (6 x 16 B x 64 lanes = 6 KiB per wavefront; measured best of 3..10 on MI355X)
constexpr int kUnitsInFlight = 6;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), kRsrcWord3);
}

__device__ __forceinline__ int64_t ld_counter(const int64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_counter(int64_t* p, int64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Bounded wait bookkeeping. The clock is read every 64th spin only.
struct SpinGuard {
  uint64_t limit;
  uint64_t start;
  uint32_t spins;
  __device__ __forceinline__ explicit SpinGuard(uint64_t limitTicks) : limit(limitTicks), start(0), spins(0) {}
  __device__ __forceinline__ bool expired() {
    spins += 1;
    if ((spins & 63u) != 1u) return false;
    uint64_t now = __builtin_amdgcn_s_memrealtime();
    if (start == 0) {
      start = now;
      return limit == 0;
    }
    return now - start > limit;
  }
};

// Wait until every store this wavefront has issued is acknowledged. Used by a
// sender before it moves `head`: FIFO lines are stored write-through (sc1), so
// a `head` beyond a step tells any reader that the lines of that step are in
// memory, all of them.
__device__ __forceinline__ void wait_stores_acknowledged() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ __forceinline__ void raise_status(uint32_t* status, uint32_t bits, int lane) {
  if (lane == 0) atomicOr(status, bits);
}

// What a stream's wavefront needs to know, all wave-uniform.
struct Stream {
  __amdgpu_buffer_rsrc_t fifo;    // the 512 KiB FIFO of the stream
  __amdgpu_buffer_rsrc_t field0;  // partial_o tensor of the local rank (send or recv side)
  __amdgpu_buffer_rsrc_t field1;  // softmax_stats tensor of the local rank
  uint32_t stride0, stride1;      // row strides in bytes
  uint32_t firstRow;              // row of the stream's first message of this launch
  uint32_t rowStep;               // rows between consecutive messages of the stream
  uint32_t np0, np, lines, unitsPerMsg, magic;
  int msgs;                       // messages of the stream in this launch
  int msgsPerEntry;
};

__device__ __forceinline__ void setup_stream(Stream& st, const KernelArgs& a, int peer, int ch) {
  const MsgShape sh = make_msg_shape(a.field0Bytes, a.field1Bytes);
  st.np0 = sh.np0;
  st.np = sh.np;
  st.lines = sh.lines;
  st.unitsPerMsg = sh.units;
  st.magic = a.lineMagic;
  st.msgsPerEntry = msgs_per_fifo_entry(sh);
  st.msgs = stream_msg_count(a.entryBegin, a.entryEnd, ch, a.runChannels);
  st.firstRow = static_cast<uint32_t>(a.entryBegin + ch) * a.cpSize + peer;
  st.rowStep = static_cast<uint32_t>(a.runChannels) * a.cpSize;
}

// Byte offsets of the two payload pieces of run unit U inside the field
// tensors; kOutOfRange where a piece is not in that field (or is the flag
// word, padding, or beyond the run).
struct UnitOffsets {
  uint32_t a0, b0;  // pieces a (first word) and b (second word) in field 0
  uint32_t a1, b1;  // ... in field 1
};

__device__ __forceinline__ UnitOffsets unit_offsets(const Stream& st, uint32_t firstMsg, uint32_t U, bool live) {
  RunUnit d = decode_run_unit(U, st.lines, st.magic);
  uint32_t row = st.firstRow + (firstMsg + d.msg) * st.rowStep;
  uint32_t base0 = row * st.stride0;
  uint32_t base1 = row * st.stride1;
  uint32_t pa = d.piece0;
  uint32_t pb = d.piece0 + 1;
  bool bLive = live && !d.flag;
  UnitOffsets o;
  o.a0 = (live && pa < st.np0) ? base0 + pa * kPieceBytes : kOutOfRange;
  o.b0 = (bLive && pb < st.np0) ? base0 + pb * kPieceBytes : kOutOfRange;
  o.a1 = (live && pa >= st.np0 && pa < st.np) ? base1 + (pa - st.np0) * kPieceBytes : kOutOfRange;
  o.b1 = (bLive && pb >= st.np0 && pb < st.np) ? base1 + (pb - st.np0) * kPieceBytes : kOutOfRange;
  return o;
}

// ---------------------------------------------------------------------------
// sender
// ---------------------------------------------------------------------------
template <int kAux>
__device__ __forceinline__ void run_sender(const KernelArgs& a, int s, int r, int ch, int lane) {
  Stream st;
  setup_stream(st, a, r, ch);
  if (st.msgs == 0) return;
  uint8_t* senderRow = a.workspace + static_cast<uint64_t>(s) * a.rowStrideBytes;
  uint8_t* receiverRow = a.workspace + static_cast<uint64_t>(r) * a.rowStrideBytes;
  int64_t* info = reinterpret_cast<int64_t*>(senderRow + sender_info_offset(a.cpSize, a.maxChannels, r, ch));
  st.fifo = make_rsrc(receiverRow + fifo_offset(s, ch, a.maxChannels), kFifoBytes);
  st.field0 = make_rsrc(a.rank[s].send0, a.sendBytes0);
  st.field1 = make_rsrc(a.rank[s].send1, a.sendBytes1);
  st.stride0 = a.sendStride0;
  st.stride1 = a.sendStride1;

  // the counters are only needed once the first payload loads are in flight
  int64_t step = info[0];
  int64_t tail = info[1];

  for (int firstMsg = 0; firstMsg < st.msgs; firstMsg += st.msgsPerEntry) {
    const int runMsgs = min(st.msgsPerEntry, st.msgs - firstMsg);
    const uint32_t runUnits = static_cast<uint32_t>(runMsgs) * st.unitsPerMsg;
    for (uint32_t U0 = 0; U0 < runUnits; U0 += kUnitsInFlight * kWaveLanes) {
      u32x2 wa[kUnitsInFlight], wb[kUnitsInFlight];
      bool needField1 = false;
#pragma unroll
      for (int i = 0; i < kUnitsInFlight; ++i) {
        uint32_t U = U0 + i * kWaveLanes + lane;
        UnitOffsets o = unit_offsets(st, firstMsg, U, U < runUnits);
        wa[i] = __builtin_amdgcn_raw_buffer_load_b64(st.field0, o.a0, 0, kAuxNone);
        wb[i] = __builtin_amdgcn_raw_buffer_load_b64(st.field0, o.b0, 0, kAuxNone);
        needField1 |= (o.a1 != kOutOfRange) | (o.b1 != kOutOfRange);
      }
      if (__ballot(needField1) != 0ull) {
#pragma unroll
        for (int i = 0; i < kUnitsInFlight; ++i) {
          uint32_t U = U0 + i * kWaveLanes + lane;
          UnitOffsets o = unit_offsets(st, firstMsg, U, U < runUnits);
          wa[i] |= __builtin_amdgcn_raw_buffer_load_b64(st.field1, o.a1, 0, kAuxNone);
          wb[i] |= __builtin_amdgcn_raw_buffer_load_b64(st.field1, o.b1, 0, kAuxNone);
        }
      }
      if (U0 == 0) {
        // open the FIFO entry of this run (csrc/helix_alltoall.cu:377-390)
        if (firstMsg > 0) {
          step += 1;
          wait_stores_acknowledged();
          if (lane == 0) st_counter(&info[0], step);
        }
        SpinGuard guard(a.spinLimitTicks);
        while (tail + kFifoDepth <= step) {  // the entry is free once the receiver released step - 4
          tail = ld_counter(&info[1]);
          if (tail + kFifoDepth > step) break;
          if (guard.expired()) {
            raise_status(a.status, kStatusSendTimeout, lane);
            return;
          }
          __builtin_amdgcn_s_sleep(4);
        }
      }
      const uint32_t entryOffset = static_cast<uint32_t>(step & (kFifoDepth - 1)) * kFifoEntryBytes;
      const uint32_t stepLo = static_cast<uint32_t>(step);
      const uint32_t stepHi = static_cast<uint32_t>(static_cast<uint64_t>(step) >> 32);
#pragma unroll
      for (int i = 0; i < kUnitsInFlight; ++i) {
        uint32_t U = U0 + i * kWaveLanes + lane;
        bool flag = (U & 7u) == 7u;
        u32x4 v = {wa[i].x, wa[i].y, flag ? stepLo : wb[i].x, flag ? stepHi : wb[i].y};
        uint32_t off = U < runUnits ? entryOffset + U * kUnitBytes : kOutOfRange;
        __builtin_amdgcn_raw_buffer_store_b128(v, st.fifo, off, 0, kAux);
      }
    }
  }
  wait_stores_acknowledged();
  if (lane == 0) st_counter(&info[0], step + 1);  // close the last entry (csrc/helix_alltoall.cu:409-412)
}

// ---------------------------------------------------------------------------
// receiver
// ---------------------------------------------------------------------------
template <int kAux>
__device__ __forceinline__ void run_receiver(const KernelArgs& a, int r, int s, int ch, int lane) {
  Stream st;
  setup_stream(st, a, s, ch);
  if (st.msgs == 0) return;
  uint8_t* senderRow = a.workspace + static_cast<uint64_t>(s) * a.rowStrideBytes;
  uint8_t* receiverRow = a.workspace + static_cast<uint64_t>(r) * a.rowStrideBytes;
  int64_t* senderInfo = reinterpret_cast<int64_t*>(senderRow + sender_info_offset(a.cpSize, a.maxChannels, r, ch));
  int64_t* info = reinterpret_cast<int64_t*>(receiverRow + receiver_info_offset(a.cpSize, a.maxChannels, s, ch));
  st.fifo = make_rsrc(receiverRow + fifo_offset(s, ch, a.maxChannels), kFifoBytes);
  st.field0 = make_rsrc(a.rank[r].recv0, a.recvBytes0);
  st.field1 = make_rsrc(a.rank[r].recv1, a.recvBytes1);
  st.stride0 = a.recvStride0;
  st.stride1 = a.recvStride1;

  int64_t step = info[1];
  // The sender's head is the acquire token of a whole run: once it is beyond
  // `step`, every line of that step is in memory (the sender waits for its
  // stores before it moves head) and the run can be read in one pass.
  int64_t head = ld_counter(&senderInfo[0]);
  const int flagLane = lane | 7;

  for (int firstMsg = 0; firstMsg < st.msgs; firstMsg += st.msgsPerEntry) {
    const int runMsgs = min(st.msgsPerEntry, st.msgs - firstMsg);
    const uint32_t runUnits = static_cast<uint32_t>(runMsgs) * st.unitsPerMsg;
    if (firstMsg > 0) {
      // every line of the previous entry has been consumed: hand it back to
      // the sender (csrc/helix_alltoall.cu:427-449)
      step += 1;
      if (lane == 0) {
        st_counter(&info[1], step);
        st_counter(&senderInfo[1], step);
      }
      if (head <= step) head = ld_counter(&senderInfo[0]);
    }
    bool runClosed = head > step;
    const uint32_t entryOffset = static_cast<uint32_t>(step & (kFifoDepth - 1)) * kFifoEntryBytes;
    const uint32_t stepLo = static_cast<uint32_t>(step);
    const uint32_t stepHi = static_cast<uint32_t>(static_cast<uint64_t>(step) >> 32);
    for (uint32_t U0 = 0; U0 < runUnits; U0 += kUnitsInFlight * kWaveLanes) {
      bool pending[kUnitsInFlight];
#pragma unroll
      for (int i = 0; i < kUnitsInFlight; ++i) pending[i] = (U0 + i * kWaveLanes + lane) < runUnits;
      SpinGuard guard(a.spinLimitTicks);
      for (;;) {
        bool landed[kUnitsInFlight];
        if (runClosed) {
#pragma unroll
          for (int i = 0; i < kUnitsInFlight; ++i) landed[i] = pending[i];
        } else {
          // The sender may still be writing. Acquire line by line: first the flag
          // words (upper half of each line's last unit, loaded by the eight flag
          // lanes only), then -- with offsets that depend on what those loads
          // returned -- the units of the lines whose flag carries the step. A unit
          // is never read before its line's flag was seen, whatever the
          // granularity at which the memory system serves a 128-byte line.
#pragma unroll
          for (int i = 0; i < kUnitsInFlight; ++i) {
            uint32_t U = U0 + i * kWaveLanes + lane;
            bool isFlagLane = (U & 7u) == 7u;
            uint32_t off = (pending[i] && isFlagLane) ? entryOffset + U * kUnitBytes + kPieceBytes : kOutOfRange;
            u32x2 f = __builtin_amdgcn_raw_buffer_load_b64(st.fifo, off, 0, kAux);
            bool ok = !pending[i] || !isFlagLane || (f.x == stepLo && f.y == stepHi);
            unsigned long long okMask = __ballot(ok);
            landed[i] = pending[i] && ((okMask >> flagLane) & 1ull) != 0ull;
          }
        }
        u32x4 v[kUnitsInFlight];
#pragma unroll
        for (int i = 0; i < kUnitsInFlight; ++i) {
          uint32_t U = U0 + i * kWaveLanes + lane;
          uint32_t off = landed[i] ? entryOffset + U * kUnitBytes : kOutOfRange;
          v[i] = __builtin_amdgcn_raw_buffer_load_b128(st.fifo, off, 0, kAux);
        }
        // every unit that is consumed carries its line's flag in the very load that brought it
        bool anyPending = false;
        bool flagsAgree = true;
#pragma unroll
        for (int i = 0; i < kUnitsInFlight; ++i) {
          uint32_t U = U0 + i * kWaveLanes + lane;
          bool isFlagLane = (U & 7u) == 7u;
          bool ok = !landed[i] || !isFlagLane || (v[i].z == stepLo && v[i].w == stepHi);
          unsigned long long okMask = __ballot(ok);
          bool lineOk = ((okMask >> flagLane) & 1ull) != 0ull;
          flagsAgree &= !landed[i] || lineOk;
          landed[i] = landed[i] && lineOk;
          pending[i] = pending[i] && !landed[i];
          anyPending |= pending[i];
        }
        if (__ballot(!flagsAgree) != 0ull) runClosed = false;  // not what the token promised: go line by line
        bool needField1 = false;
#pragma unroll
        for (int i = 0; i < kUnitsInFlight; ++i) {
          uint32_t U = U0 + i * kWaveLanes + lane;
          UnitOffsets o = unit_offsets(st, firstMsg, U, landed[i]);
          u32x2 wa = {v[i].x, v[i].y};
          u32x2 wb = {v[i].z, v[i].w};
          __builtin_amdgcn_raw_buffer_store_b64(wa, st.field0, o.a0, 0, kAuxNone);
          __builtin_amdgcn_raw_buffer_store_b64(wb, st.field0, o.b0, 0, kAuxNone);
          needField1 |= (o.a1 != kOutOfRange) | (o.b1 != kOutOfRange);
        }
        if (__ballot(needField1) != 0ull) {
#pragma unroll
          for (int i = 0; i < kUnitsInFlight; ++i) {
            uint32_t U = U0 + i * kWaveLanes + lane;
            UnitOffsets o = unit_offsets(st, firstMsg, U, landed[i]);
            u32x2 wa = {v[i].x, v[i].y};
            u32x2 wb = {v[i].z, v[i].w};
            __builtin_amdgcn_raw_buffer_store_b64(wa, st.field1, o.a1, 0, kAuxNone);
            __builtin_amdgcn_raw_buffer_store_b64(wb, st.field1, o.b1, 0, kAuxNone);
          }
        }
        if (__ballot(anyPending) == 0ull) break;
        if (guard.expired()) {
          raise_status(a.status, kStatusRecvTimeout, lane);
          return;
        }
        __builtin_amdgcn_s_sleep(1);
        asm volatile("" ::: "memory");
      }
    }
  }
  if (lane == 0) {  // close the last entry (csrc/helix_alltoall.cu:468-472)
    st_counter(&info[1], step + 1);
    st_counter(&senderInfo[1], step + 1);
  }
}

// Wavefront w of a launch: sender wavefronts come first in dispatch order so
// that no receiver can occupy a slot a not-yet-started sender needs.
// Within a direction, w = (local rank * runChannels + channel) * cp + peer:
// neighbouring wavefronts touch neighbouring rows of the same entry.
__global__ __launch_bounds__(kBlockThreads) void helix_exchange_kernel(KernelArgs a) {
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWaveLanes);
  const int lane = static_cast<int>(threadIdx.x) % kWaveLanes;
  int w = static_cast<int>(blockIdx.x) * kWavesPerBlock + wave;
  const int perDirection = a.rankCount * a.runChannels * a.cpSize;
  const int senders = a.doSend ? perDirection : 0;
  const int total = senders + (a.doRecv ? perDirection : 0);
  if (w >= total) return;
  const bool isSender = w < senders;
  if (!isSender) w -= senders;
  const int peer = w % a.cpSize;
  const int t = w / a.cpSize;
  const int ch = t % a.runChannels;
  const int local = a.rankBegin + t / a.runChannels;
  if (isSender) {
    run_sender<kAuxSc1>(a, local, peer, ch, lane);
  } else {
    run_receiver<kAuxSc1>(a, local, peer, ch, lane);
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

template <int kDtype>
__device__ __forceinline__ uint32_t narrow1(float v);
template <>
__device__ __forceinline__ uint32_t narrow1<0>(float v) {  // fp32 -> bf16, round to nearest even, NaN stays NaN
  uint32_t b = __float_as_uint(v);
  if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (b >> 16) | 0x0040u;
  return (b + 0x7FFFu + ((b >> 16) & 1u)) >> 16;
}
template <>
__device__ __forceinline__ uint32_t narrow1<1>(float v) {
  return static_cast<uint32_t>(__half_as_ushort(__float2half_rn(v)));
}

// Receive half of the fused form. A wavefront serves one (receiver, channel)
// and all cpSize senders at once: lane L owns run unit U (the same unit of
// the same message in every sender's FIFO, since all streams of a channel
// share one layout), loads that unit from each sender's FIFO, and reduces
// over the senders in registers:
//   out[e, h, :] = sum_s w[s, h] * partial_o_s[e, h, :],  w = softmax_s(lse[s, h])
// (patches/dcp_alltoall_helix.py:142-207). The statistics of head h live in
// piece np0 + h of each message. Every distinct statistics line the lanes of
// a wavefront need is fetched once per wavefront, by lanes 0..7 in the
// pattern of a payload line (lane u takes unit u, so the line is validated by
// its own flag unit in the same load), and handed to the lanes that need it
// with lane shuffles. The softmax runs online over groups of eight senders,
// so nothing but two accumulators survives a group. The `parts` wavefronts of
// a workgroup split the units of a run between them. No LDS, one barrier.
// The kernel is bounded by instruction issue rather than by memory: exp and
// ln use the hardware's base-2 units.
struct CombineCtx {
  __amdgpu_buffer_rsrc_t fifos;  // the whole FIFO region of the receiver's row
  uint32_t channelBase;          // byte offset of sender 0's FIFO of this channel
  uint32_t senderStride;         // bytes between the FIFOs of consecutive senders
  uint32_t stepLo, stepHi;       // lane q: step counter of sender q's stream
};

__device__ __forceinline__ uint32_t lane_value(uint32_t v, int q) {
  return static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), q));
}
__device__ __forceinline__ uint32_t shuffle_from(uint32_t v, int srcLane) {
  return static_cast<uint32_t>(__shfl(static_cast<int>(v), srcLane, kWaveLanes));
}

// byte offset of sender q's open FIFO entry inside the receiver's FIFO region
__device__ __forceinline__ uint32_t entry_base(const CombineCtx& cx, int q, uint32_t stepLo) {
  return cx.channelBase + static_cast<uint32_t>(q) * cx.senderStride + (stepLo & (kFifoDepth - 1)) * kFifoEntryBytes;
}

// exp and ln on the hardware's base-2 units (v_exp_f32 / v_log_f32, about 1 ulp):
// the combine is bounded by instruction issue, and its result is rounded to
// 8 mantissa bits anyway. exp(-inf) = 0, ln(0) = -inf, ln(x < 0) = NaN hold.
__device__ __forceinline__ float fast_exp(float x) { return __builtin_amdgcn_exp2f(x * 1.4426950408889634f); }
__device__ __forceinline__ float fast_log(float x) { return __builtin_amdgcn_logf(x) * 0.6931471805599453f; }

// Running softmax-weighted sum of one 8-byte piece (4 elements) over the senders.
struct OnlineSum {
  float m, total;
  float acc[4];
  __device__ __forceinline__ void init() {
    m = -INFINITY;
    total = 0.0f;
    acc[0] = acc[1] = acc[2] = acc[3] = 0.0f;
  }
  // raise the running maximum to cover `candidate`
  __device__ __forceinline__ void rescale(float candidate) {
    float mNew = fmaxf(m, candidate);
    float scale = (mNew == -INFINITY) ? 1.0f : fast_exp(m - mNew);  // m == -inf: nothing accumulated yet, scale is 0
    m = mNew;
    total *= scale;
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] *= scale;
  }
  __device__ __forceinline__ float weight(float lse) const { return (m == -INFINITY) ? 0.0f : fast_exp(lse - m); }
  __device__ __forceinline__ void add(float e, const float (&f)[4]) {
    total += e;
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] += e * f[c];
  }
  __device__ __forceinline__ float lse_value() const { return fast_log(total) + (m == -INFINITY ? 0.0f : m); }
  __device__ __forceinline__ float inv_total() const { return 1.0f / fmaxf(total, 1e-10f); }
};

// log-sum-exp of head h from the 8-byte statistics piece {s0, s1} that holds it;
// NaN and +-inf count as "no contribution".
//   mode 0: piece h = {lse, unused}     mode 1: piece h = {running max, running sum}
//   mode 2: piece h/2 = {lse of head 2*(h/2), lse of head 2*(h/2)+1}
__device__ __forceinline__ float lse_of_stats(uint32_t s0, uint32_t s1, int statsMode, uint32_t h) {
  float x = __uint_as_float((statsMode == 2 && (h & 1u)) ? s1 : s0);
  if (statsMode == 1) x = x + fast_log(__uint_as_float(s1));  // running max + ln(running sum)
  return (isnan(x) || isinf(x)) ? -INFINITY : x;
}

template <int kDtype>
__device__ __forceinline__ u32x2 narrow_piece(const OnlineSum& o) {
  const float inv = o.inv_total();
  u32x2 r = {narrow1<kDtype>(o.acc[0] * inv) | (narrow1<kDtype>(o.acc[1] * inv) << 16),
             narrow1<kDtype>(o.acc[2] * inv) | (narrow1<kDtype>(o.acc[3] * inv) << 16)};
  return r;
}

template <int kDtype>
__device__ __forceinline__ void run_combine_receiver(const KernelArgs& a, int r, int ch, int part, int parts,
                                                     int lane) {
  constexpr int kGroup = 8;  // senders whose loads are in flight together
  Stream st;
  setup_stream(st, a, 0, ch);
  if (st.msgs == 0) return;  // uniform over the workgroup: same channel
  uint8_t* receiverRow = a.workspace + static_cast<uint64_t>(r) * a.rowStrideBytes;
  CombineCtx cx;
  cx.fifos = make_rsrc(receiverRow, static_cast<uint32_t>(fifo_region_bytes(a.cpSize, a.maxChannels)));
  cx.channelBase = static_cast<uint32_t>(fifo_offset(0, ch, a.maxChannels));
  cx.senderStride = static_cast<uint32_t>(fifo_offset(1, 0, a.maxChannels));
  __amdgpu_buffer_rsrc_t outRsrc = make_rsrc(a.rank[r].recv0, a.recvBytes0);
  __amdgpu_buffer_rsrc_t lseRsrc = make_rsrc(a.rank[r].recv1, a.rank[r].recv1 ? a.recvBytes1 : 0u);
  const uint32_t piecesPerHead = static_cast<uint32_t>(a.headDim) * 2u / kPieceBytes;
  const int flagLane = lane | 7;

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
  __syncthreads();  // every part has read the counters before part 0 moves them
  if (part == 0 && lane < a.cpSize) {
    // rounds never put more than the four entries in flight, so the entries can
    // be handed back up front; nothing reads these counters before the launch ends
    const MsgShape sh = make_msg_shape(a.field0Bytes, a.field1Bytes);
    int64_t done = myStep + entries_for_msgs(st.msgs, sh);
    st_counter(&myInfo[1], done);
    st_counter(&mySenderInfo[1], done);
  }

  for (int firstMsg = 0; firstMsg < st.msgs; firstMsg += st.msgsPerEntry, myStep += 1) {
    const int runMsgs = min(st.msgsPerEntry, st.msgs - firstMsg);
    const uint32_t runUnits = static_cast<uint32_t>(runMsgs) * st.unitsPerMsg;
    cx.stepLo = static_cast<uint32_t>(myStep);
    cx.stepHi = static_cast<uint32_t>(static_cast<uint64_t>(myStep) >> 32);
    {
      // Acquire the run from every sender: a head beyond the step says that all
      // lines of the step are in memory (the sender waits for its stores before
      // it moves head). Every unit needs all cpSize senders anyway.
      SpinGuard guard(a.spinLimitTicks);
      for (;;) {
        const bool closed = lane >= a.cpSize || ld_counter(&mySenderInfo[0]) > myStep;
        if (__ballot(!closed) == 0ull) break;
        if (guard.expired()) {
          raise_status(a.status, kStatusRecvTimeout, lane);
          return;
        }
        __builtin_amdgcn_s_sleep(8);
      }
      asm volatile("" ::: "memory");
    }
    for (uint32_t U0 = static_cast<uint32_t>(part) * kWaveLanes; U0 < runUnits;
         U0 += static_cast<uint32_t>(parts) * kWaveLanes) {
      const uint32_t U = U0 + lane;
      const RunUnit d = decode_run_unit(U, st.lines, st.magic);
      const bool live = U < runUnits;
      const bool dataA = live && d.piece0 < st.np0;
      const bool dataB = live && !d.flag && d.piece0 + 1 < st.np0;
      if (__ballot(dataA) == 0ull) continue;  // statistics, padding: nothing to reduce here
      const uint32_t hA = head_of_piece(d.piece0, a.headMagic);
      const uint32_t hB = dataB ? head_of_piece(d.piece0 + 1, a.headMagic) : hA;
      const uint32_t entry = static_cast<uint32_t>(a.entryBegin + ch) + (firstMsg + d.msg) * a.runChannels;
      // where the statistics of heads hA / hB sit: run line and word inside it
      const uint32_t psA = st.np0 + (a.statsMode == 2 ? hA >> 1 : hA), psB = st.np0 + (a.statsMode == 2 ? hB >> 1 : hB);
      const uint32_t lineA = d.msg * st.lines + psA / kPiecesPerLine, wordA = psA % kPiecesPerLine;
      const uint32_t lineB = d.msg * st.lines + psB / kPiecesPerLine, wordB = psB % kPiecesPerLine;
      // piece B shares the weights of piece A unless it starts the next head
      const bool ownB = dataB && hB != hA;
      const bool anyOwnB = __ballot(ownB) != 0ull;

      OnlineSum sumA, sumB;
      sumA.init();
      sumB.init();

      for (int g = 0; g < a.cpSize; g += kGroup) {
        u32x4 v[kGroup];
        float lseA[kGroup], lseB[kGroup];
        SpinGuard guard(a.spinLimitTicks);
        for (;;) {
          // payload unit of every sender of the group
#pragma unroll
          for (int j = 0; j < kGroup; ++j) {
            const int q = g + j;
            if (q < a.cpSize) {
              const uint32_t base = entry_base(cx, q, lane_value(cx.stepLo, q));
              v[j] = __builtin_amdgcn_raw_buffer_load_b128(cx.fifos, live ? base + U * kUnitBytes : kOutOfRange, 0, kAuxSc1);
            }
          }
          // Statistics: every distinct line some lane needs is fetched once per
          // wavefront, by lanes 0..7 in the pattern of a payload line (lane u takes
          // unit u, so the line is validated by its own flag unit in the same
          // load), and handed to the lanes that need it with lane shuffles.
          bool ok = true;
          bool pendA = dataA, pendB = ownB;
          for (;;) {
            const unsigned long long need = __ballot(pendA || pendB);
            if (need == 0ull) break;
            const int leader = __ffsll(static_cast<long long>(need)) - 1;
            const uint32_t line = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(pendA ? lineA : lineB), leader));
            const bool takeA = pendA && lineA == line, takeB = pendB && lineB == line;
            const uint32_t unitOff = line * kLineBytes + static_cast<uint32_t>(lane) * kUnitBytes;
#pragma unroll
            for (int j = 0; j < kGroup; ++j) {
              const int q = g + j;
              if (q < a.cpSize) {
                const uint32_t sLo = lane_value(cx.stepLo, q), sHi = lane_value(cx.stepHi, q);
                const uint32_t base = entry_base(cx, q, sLo);
                const u32x4 sv = __builtin_amdgcn_raw_buffer_load_b128(cx.fifos, lane < 8 ? base + unitOff : kOutOfRange, 0, kAuxSc1);
                const unsigned long long landed = __ballot(lane != 7 || (sv.z == sLo && sv.w == sHi));
                ok &= ((landed >> 7) & 1ull) != 0ull;
                // every lane takes part in every shuffle (a lane can only be read while it is active)
                const int srcA = static_cast<int>(wordA >> 1);
                const uint32_t ax = shuffle_from(sv.x, srcA), ay = shuffle_from(sv.y, srcA);
                const uint32_t az = shuffle_from(sv.z, srcA), aw = shuffle_from(sv.w, srcA);
                const float la = lse_of_stats((wordA & 1u) ? az : ax, (wordA & 1u) ? aw : ay, a.statsMode, hA);
                if (takeA) lseA[j] = la;
                if (anyOwnB) {
                  const int srcB = static_cast<int>(wordB >> 1);
                  const uint32_t bx = shuffle_from(sv.x, srcB), by = shuffle_from(sv.y, srcB);
                  const uint32_t bz = shuffle_from(sv.z, srcB), bw = shuffle_from(sv.w, srcB);
                  const float lb = lse_of_stats((wordB & 1u) ? bz : bx, (wordB & 1u) ? bw : by, a.statsMode, hB);
                  if (takeB) lseB[j] = lb;
                }
              }
            }
            pendA = pendA && !takeA;
            pendB = pendB && !takeB;
          }
          // payload lines: flag unit of each line, shared through a ballot
#pragma unroll
          for (int j = 0; j < kGroup; ++j) {
            const int q = g + j;
            if (q < a.cpSize) {
              const uint32_t sLo = lane_value(cx.stepLo, q), sHi = lane_value(cx.stepHi, q);
              const unsigned long long landed = __ballot(!(live && d.flag) || (v[j].z == sLo && v[j].w == sHi));
              ok &= ((landed >> flagLane) & 1ull) != 0ull;
            }
          }
          if (__ballot(!ok) == 0ull) break;
          if (guard.expired()) {
            raise_status(a.status, kStatusRecvTimeout, lane);
            return;
          }
          __builtin_amdgcn_s_sleep(16);
          asm volatile("" ::: "memory");
        }
        float gmaxA = -INFINITY, gmaxB = -INFINITY;
#pragma unroll
        for (int j = 0; j < kGroup; ++j) {
          if (g + j < a.cpSize) {
            if (!dataA) lseA[j] = -INFINITY;
            if (!ownB) lseB[j] = lseA[j];
            gmaxA = fmaxf(gmaxA, lseA[j]);
            gmaxB = fmaxf(gmaxB, lseB[j]);
          }
        }
        sumA.rescale(gmaxA);
        sumB.rescale(gmaxB);  // equals gmaxA for every lane whose second piece shares the head
#pragma unroll
        for (int j = 0; j < kGroup; ++j) {
          if (g + j < a.cpSize) {
            float f[4];
            u32x2 pa = {v[j].x, v[j].y};
            u32x2 pb = {v[j].z, v[j].w};
            const float ea = sumA.weight(lseA[j]);
            widen4<kDtype>(pa, f);
            sumA.add(ea, f);
            const float eb = anyOwnB ? sumB.weight(lseB[j]) : ea;
            widen4<kDtype>(pb, f);
            sumB.add(eb, f);
          }
        }
      }
      // the lane that holds the first piece of a head reports that head's log-sum-exp
      const bool reportA = dataA && d.piece0 == hA * piecesPerHead;
      const bool reportB = dataB && d.piece0 + 1 == hB * piecesPerHead;
      __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(sumA.lse_value()), lseRsrc,
                                            reportA ? (entry * a.heads + hA) * 4u : kOutOfRange, 0, kAuxNone);
      __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(sumB.lse_value()), lseRsrc,
                                            reportB ? (entry * a.heads + hB) * 4u : kOutOfRange, 0, kAuxNone);
      const uint32_t rowByte = entry * (st.np0 * kPieceBytes);
      __builtin_amdgcn_raw_buffer_store_b64(narrow_piece<kDtype>(sumA), outRsrc,
                                            dataA ? rowByte + d.piece0 * kPieceBytes : kOutOfRange, 0, kAuxNone);
      __builtin_amdgcn_raw_buffer_store_b64(narrow_piece<kDtype>(sumB), outRsrc,
                                            dataB ? rowByte + (d.piece0 + 1) * kPieceBytes : kOutOfRange, 0, kAuxNone);
    }
  }
}

// Workgroups of `parts` wavefronts (blockDim.x / 64). The first
// ceil(senderStreams / parts) workgroups send, one stream per wavefront; the
// rest receive and combine, one workgroup per (receiver, channel).
template <int kDtype>
__global__ __launch_bounds__(kMaxCombineParts * kWaveLanes) void helix_combine_kernel(KernelArgs a) {
  const int parts = static_cast<int>(blockDim.x) / kWaveLanes;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWaveLanes);
  const int lane = static_cast<int>(threadIdx.x) % kWaveLanes;
  const int senderStreams = a.doSend ? a.rankCount * a.runChannels * a.cpSize : 0;
  const int sendBlocks = (senderStreams + parts - 1) / parts;
  int b = static_cast<int>(blockIdx.x);
  if (b < sendBlocks) {
    const int w = b * parts + wave;
    if (w >= senderStreams) return;
    const int t = w / a.cpSize;
    run_sender<kAuxSc1>(a, a.rankBegin + t / a.runChannels, w % a.cpSize, t % a.runChannels, lane);
    return;
  }
  b -= sendBlocks;
  run_combine_receiver<kDtype>(a, a.rankBegin + b / a.runChannels, b % a.runChannels, wave, parts, lane);
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

hipError_t launch_exchange(const KernelArgs& a, hipStream_t stream) {
  int directions = (a.doSend ? 1 : 0) + (a.doRecv ? 1 : 0);
  int waves = directions * waves_per_direction(a);
  if (waves <= 0) return hipSuccess;
  int blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
  hipLaunchKernelGGL(helix_exchange_kernel, dim3(blocks), dim3(kBlockThreads), 0, stream, a);
  return hipGetLastError();
}

hipError_t launch_combine(const KernelArgs& a, int parts, hipStream_t stream) {
  const int senderStreams = a.doSend ? a.rankCount * a.runChannels * a.cpSize : 0;
  if (a.rankCount * a.runChannels <= 0) return hipSuccess;
  if (parts < 1) parts = 1;
  if (parts > kMaxCombineParts) parts = kMaxCombineParts;
  const int blocks = (senderStreams + parts - 1) / parts + a.rankCount * a.runChannels;
  dim3 block(static_cast<unsigned>(parts * kWaveLanes));
  if (a.dtype == 1) {
    hipLaunchKernelGGL(helix_combine_kernel<1>, dim3(blocks), block, 0, stream, a);
  } else {
    hipLaunchKernelGGL(helix_combine_kernel<0>, dim3(blocks), block, 0, stream, a);
  }
  return hipGetLastError();
}

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
