// helix_kernels.hip -- gfx950 kernels of the Helix all-to-all.
//
// One wavefront owns one stream = (sender rank, receiver rank, channel) in one
// direction, the role a warp has in the reference kernel
// (csrc/helix_alltoall.cu:315-474). A sender wavefront reads its messages from
// the send tensors, turns them into LL128 lines in registers and stores the
// lines into the receiver's FIFO; a receiver wavefront polls the FIFO lines
// until their flags carry the expected step, then stores the payload into the
// receive tensors. There is no staging copy and no barrier: data moves
// global -> registers -> FIFO -> registers -> global with 16 bytes per lane.
//
// FIFO lines are written and polled with the sc1 cache policy (device-scope
// coherence: every XCD has its own L2, and sender and receiver of a stream
// may run on different XCDs). FIFO accesses go through buffer descriptors
// that span exactly one FIFO, so the hardware drops anything out of range.
#include "helix_kernels.hpp"

namespace helix {
namespace {

using u32x2 = uint32_t __attribute__((ext_vector_type(2)));
using u32x4 = uint32_t __attribute__((ext_vector_type(4)));
// payload rows are only guaranteed 8-byte alignment at odd lines
struct __attribute__((packed, aligned(8))) U32x4A8 { u32x4 v; };

// gfx940+ buffer cache-policy immediates: bit 0 sc0, bit 1 nt, bit 4 sc1.
// sc1 alone is device scope. (The compiler's "volatile" bit 31 would widen
// the access to system scope; polling loops use a compiler barrier instead.)
constexpr int kAuxSc1 = 16;
constexpr uint32_t kRsrcWord3 = 0x00020000u;  // raw buffer, 32-bit data format

constexpr uint32_t kStatusRecvTimeout = 1u;
constexpr uint32_t kStatusSendTimeout = 2u;

// units a lane keeps in flight per chunk of a message
constexpr int kUnitsInFlight = 4;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_fifo_rsrc(uint8_t* base) {
  return __builtin_amdgcn_make_buffer_rsrc(base, 0, kFifoBytes, kRsrcWord3);
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

__device__ __forceinline__ u32x2 ld_piece(const uint8_t* row0, const uint8_t* row1, const MsgShape& sh, int p) {
  u32x2 z = {0u, 0u};
  if (p < sh.np0) return *reinterpret_cast<const u32x2*>(row0 + p * kPieceBytes);
  if (p < sh.np) return *reinterpret_cast<const u32x2*>(row1 + (p - sh.np0) * kPieceBytes);
  return z;
}

__device__ __forceinline__ void st_piece(uint8_t* row0, uint8_t* row1, const MsgShape& sh, int p, u32x2 v) {
  if (p < sh.np0) {
    *reinterpret_cast<u32x2*>(row0 + p * kPieceBytes) = v;
  } else if (p < sh.np) {
    *reinterpret_cast<u32x2*>(row1 + (p - sh.np0) * kPieceBytes) = v;
  }
}

// wire unit g of a message, built from the send rows
__device__ __forceinline__ u32x4 load_unit(const uint8_t* row0, const uint8_t* row1, const MsgShape& sh, int g,
                                           u32x2 step) {
  int p0 = unit_first_piece(g);
  bool flag = unit_has_flag(g);
  if (!flag && p0 + 1 < sh.np0) {
    return reinterpret_cast<const U32x4A8*>(row0 + p0 * kPieceBytes)->v;
  }
  if (!flag && p0 >= sh.np0 && p0 + 1 < sh.np) {
    return reinterpret_cast<const U32x4A8*>(row1 + (p0 - sh.np0) * kPieceBytes)->v;
  }
  u32x2 a = ld_piece(row0, row1, sh, p0);
  u32x2 b = flag ? step : ld_piece(row0, row1, sh, p0 + 1);
  u32x4 r = {a.x, a.y, b.x, b.y};
  return r;
}

// payload of wire unit g, scattered into the receive rows
__device__ __forceinline__ void store_unit(uint8_t* row0, uint8_t* row1, const MsgShape& sh, int g, u32x4 v) {
  int p0 = unit_first_piece(g);
  bool flag = unit_has_flag(g);
  if (!flag && p0 + 1 < sh.np0) {
    reinterpret_cast<U32x4A8*>(row0 + p0 * kPieceBytes)->v = v;
    return;
  }
  if (!flag && p0 >= sh.np0 && p0 + 1 < sh.np) {
    reinterpret_cast<U32x4A8*>(row1 + (p0 - sh.np0) * kPieceBytes)->v = v;
    return;
  }
  u32x2 a = {v.x, v.y};
  st_piece(row0, row1, sh, p0, a);
  if (!flag) {
    u32x2 b = {v.z, v.w};
    st_piece(row0, row1, sh, p0 + 1, b);
  }
}

__device__ __forceinline__ void send_message(const uint8_t* row0, const uint8_t* row1, const MsgShape& sh,
                                             __amdgpu_buffer_rsrc_t fifo, uint32_t msgOffset, u32x2 step,
                                             int lane) {
  for (int g0 = 0; g0 < sh.units; g0 += kUnitsInFlight * kWaveLanes) {
    u32x4 v[kUnitsInFlight];
#pragma unroll
    for (int i = 0; i < kUnitsInFlight; ++i) {
      int g = g0 + i * kWaveLanes + lane;
      u32x4 z = {0u, 0u, 0u, 0u};
      v[i] = z;
      if (g < sh.units) v[i] = load_unit(row0, row1, sh, g, step);
    }
#pragma unroll
    for (int i = 0; i < kUnitsInFlight; ++i) {
      int g = g0 + i * kWaveLanes + lane;
      if (g < sh.units) {
        __builtin_amdgcn_raw_buffer_store_b128(v[i], fifo, msgOffset + g * kUnitBytes, 0, kAuxSc1);
      }
    }
  }
}

// Returns false when the bounded wait expired.
__device__ __forceinline__ bool recv_message(uint8_t* row0, uint8_t* row1, const MsgShape& sh,
                                             __amdgpu_buffer_rsrc_t fifo, uint32_t msgOffset, u32x2 step, int lane,
                                             uint64_t spinLimitTicks) {
  const int flagLane = lane | 7;
  for (int g0 = 0; g0 < sh.units; g0 += kUnitsInFlight * kWaveLanes) {
    bool pending[kUnitsInFlight];
#pragma unroll
    for (int i = 0; i < kUnitsInFlight; ++i) pending[i] = (g0 + i * kWaveLanes + lane) < sh.units;
    SpinGuard guard(spinLimitTicks);
    for (;;) {
      u32x4 v[kUnitsInFlight];
#pragma unroll
      for (int i = 0; i < kUnitsInFlight; ++i) {
        int g = g0 + i * kWaveLanes + lane;
        u32x4 z = {0u, 0u, 0u, 0u};
        v[i] = z;
        if (pending[i]) {
          v[i] = __builtin_amdgcn_raw_buffer_load_b128(fifo, msgOffset + g * kUnitBytes, 0, kAuxSc1);
        }
      }
      bool anyPending = false;
#pragma unroll
      for (int i = 0; i < kUnitsInFlight; ++i) {
        int g = g0 + i * kWaveLanes + lane;
        bool ok = !pending[i] || !unit_has_flag(g) || (v[i].z == step.x && v[i].w == step.y);
        unsigned long long okMask = __ballot(ok);
        bool lineOk = (okMask >> flagLane) & 1ull;
        if (pending[i] && lineOk) {
          store_unit(row0, row1, sh, g, v[i]);
          pending[i] = false;
        }
        anyPending |= pending[i];
      }
      if (__ballot(anyPending) == 0ull) break;
      if (guard.expired()) return false;
      __builtin_amdgcn_s_sleep(1);
      asm volatile("" ::: "memory");
    }
  }
  return true;
}

__device__ __forceinline__ void raise_status(uint32_t* status, uint32_t bits, int lane) {
  if (lane == 0) atomicOr(status, bits);
}

__device__ void run_sender(const KernelArgs& a, int s, int r, int ch, int lane) {
  const MsgShape sh = make_msg_shape(a.field0Bytes, a.field1Bytes);
  uint8_t* senderRow = a.workspace + static_cast<uint64_t>(s) * a.rowStrideBytes;
  uint8_t* receiverRow = a.workspace + static_cast<uint64_t>(r) * a.rowStrideBytes;
  int64_t* info = reinterpret_cast<int64_t*>(senderRow + sender_info_offset(a.cpSize, a.maxChannels, r, ch));
  __amdgpu_buffer_rsrc_t fifo = make_fifo_rsrc(receiverRow + fifo_offset(s, ch, a.maxChannels));

  int64_t tail = info[1];
  FifoCursor cur = make_cursor(info[0]);
  const uint8_t* base0 = a.rank[s].send0;
  const uint8_t* base1 = a.rank[s].send1;

  for (int e = a.entryBegin + ch; e < a.entryEnd; e += a.runChannels) {
    if (cursor_needs_new_entry(cur, sh.lines)) {
      bool closedOne;
      cursor_open_entry(cur, &closedOne);
      if (closedOne) st_counter(&info[0], cur.step);
      // wait for room: the entry is free once the receiver released step - 4
      SpinGuard guard(a.spinLimitTicks);
      while (tail + kFifoDepth <= cur.step) {
        tail = ld_counter(&info[1]);
        if (tail + kFifoDepth > cur.step) break;
        if (guard.expired()) {
          raise_status(a.status, kStatusSendTimeout, lane);
          return;
        }
        __builtin_amdgcn_s_sleep(4);
      }
    }
    uint64_t rowIndex = static_cast<uint64_t>(e) * a.cpSize + r;
    const uint8_t* row0 = base0 + rowIndex * static_cast<uint64_t>(a.sendStride0);
    const uint8_t* row1 = base1 + rowIndex * static_cast<uint64_t>(a.sendStride1);
    u32x2 step = {static_cast<uint32_t>(cur.step), static_cast<uint32_t>(static_cast<uint64_t>(cur.step) >> 32)};
    send_message(row0, row1, sh, fifo, fifo_unit_offset(cursor_entry_index(cur), cur.lineBase, 0), step, lane);
    cur.lineBase += sh.lines;
  }
  if (cur.open && lane == 0) st_counter(&info[0], cur.step + 1);
}

__device__ void run_receiver(const KernelArgs& a, int r, int s, int ch, int lane) {
  const MsgShape sh = make_msg_shape(a.field0Bytes, a.field1Bytes);
  uint8_t* senderRow = a.workspace + static_cast<uint64_t>(s) * a.rowStrideBytes;
  uint8_t* receiverRow = a.workspace + static_cast<uint64_t>(r) * a.rowStrideBytes;
  int64_t* senderInfo = reinterpret_cast<int64_t*>(senderRow + sender_info_offset(a.cpSize, a.maxChannels, r, ch));
  int64_t* info = reinterpret_cast<int64_t*>(receiverRow + receiver_info_offset(a.cpSize, a.maxChannels, s, ch));
  __amdgpu_buffer_rsrc_t fifo = make_fifo_rsrc(receiverRow + fifo_offset(s, ch, a.maxChannels));

  FifoCursor cur = make_cursor(info[1]);
  uint8_t* base0 = a.rank[r].recv0;
  uint8_t* base1 = a.rank[r].recv1;

  for (int e = a.entryBegin + ch; e < a.entryEnd; e += a.runChannels) {
    if (cursor_needs_new_entry(cur, sh.lines)) {
      bool closedOne;
      cursor_open_entry(cur, &closedOne);
      if (closedOne && lane == 0) {
        // every line of the closed entry is already in registers or stored:
        // hand the entry back to the sender
        st_counter(&info[1], cur.step);
        st_counter(&senderInfo[1], cur.step);
      }
    }
    uint64_t rowIndex = static_cast<uint64_t>(e) * a.cpSize + s;
    uint8_t* row0 = base0 + rowIndex * static_cast<uint64_t>(a.recvStride0);
    uint8_t* row1 = base1 + rowIndex * static_cast<uint64_t>(a.recvStride1);
    u32x2 step = {static_cast<uint32_t>(cur.step), static_cast<uint32_t>(static_cast<uint64_t>(cur.step) >> 32)};
    bool ok = recv_message(row0, row1, sh, fifo, fifo_unit_offset(cursor_entry_index(cur), cur.lineBase, 0), step,
                           lane, a.spinLimitTicks);
    if (!ok) {
      raise_status(a.status, kStatusRecvTimeout, lane);
      return;
    }
    cur.lineBase += sh.lines;
  }
  if (cur.open && lane == 0) {
    st_counter(&info[1], cur.step + 1);
    st_counter(&senderInfo[1], cur.step + 1);
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
    run_sender(a, local, peer, ch, lane);
  } else {
    run_receiver(a, local, peer, ch, lane);
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
