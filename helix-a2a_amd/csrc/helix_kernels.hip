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
    }
    const uint32_t entryOffset = static_cast<uint32_t>(step & (kFifoDepth - 1)) * kFifoEntryBytes;
    const uint32_t stepLo = static_cast<uint32_t>(step);
    const uint32_t stepHi = static_cast<uint32_t>(static_cast<uint64_t>(step) >> 32);
    for (uint32_t U0 = 0; U0 < runUnits; U0 += kUnitsInFlight * kWaveLanes) {
      bool pending[kUnitsInFlight];
#pragma unroll
      for (int i = 0; i < kUnitsInFlight; ++i) pending[i] = (U0 + i * kWaveLanes + lane) < runUnits;
      SpinGuard guard(a.spinLimitTicks);
      for (;;) {
        u32x4 v[kUnitsInFlight];
#pragma unroll
        for (int i = 0; i < kUnitsInFlight; ++i) {
          uint32_t U = U0 + i * kWaveLanes + lane;
          uint32_t off = pending[i] ? entryOffset + U * kUnitBytes : kOutOfRange;
          v[i] = __builtin_amdgcn_raw_buffer_load_b128(st.fifo, off, 0, kAux);
        }
        bool anyPending = false;
        bool landed[kUnitsInFlight];
        bool needField1 = false;
#pragma unroll
        for (int i = 0; i < kUnitsInFlight; ++i) {
          uint32_t U = U0 + i * kWaveLanes + lane;
          bool isFlagLane = (U & 7u) == 7u;
          bool ok = !pending[i] || !isFlagLane || (v[i].z == stepLo && v[i].w == stepHi);
          unsigned long long okMask = __ballot(ok);
          bool lineOk = (okMask >> flagLane) & 1ull;
          landed[i] = pending[i] && lineOk;
          UnitOffsets o = unit_offsets(st, firstMsg, U, landed[i]);
          u32x2 wa = {v[i].x, v[i].y};
          u32x2 wb = {v[i].z, v[i].w};
          __builtin_amdgcn_raw_buffer_store_b64(wa, st.field0, o.a0, 0, kAuxNone);
          __builtin_amdgcn_raw_buffer_store_b64(wb, st.field0, o.b0, 0, kAuxNone);
          needField1 |= (o.a1 != kOutOfRange) | (o.b1 != kOutOfRange);
          pending[i] = pending[i] && !lineOk;
          anyPending |= pending[i];
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

hipError_t launch_combine_recv(const KernelArgs&, hipStream_t) { return hipErrorNotSupported; }

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
