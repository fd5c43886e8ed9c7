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

// Receive half of the fused form: the cpSize wavefronts of a workgroup each
// poll one sender's FIFO for the same (receiver, channel), park the payload
// pieces in LDS, and the workgroup then reduces over the senders:
//   out[e, h, :] = sum_s w[s, h] * partial_o_s[e, h, :],  w = softmax_s(lse[s, h])
// (patches/dcp_alltoall_helix.py:142-207). LDS: [cp][np] pieces, then [cp][heads] weights.
template <int kDtype>
__device__ __forceinline__ void run_combine_receiver(const KernelArgs& a, int r, int s, int ch, int lane,
                                                     uint8_t* lds, int* failed) {
  Stream st;
  setup_stream(st, a, s, ch);
  if (st.msgs == 0) return;  // uniform over the workgroup: same channel
  uint8_t* senderRow = a.workspace + static_cast<uint64_t>(s) * a.rowStrideBytes;
  uint8_t* receiverRow = a.workspace + static_cast<uint64_t>(r) * a.rowStrideBytes;
  int64_t* senderInfo = reinterpret_cast<int64_t*>(senderRow + sender_info_offset(a.cpSize, a.maxChannels, r, ch));
  int64_t* info = reinterpret_cast<int64_t*>(receiverRow + receiver_info_offset(a.cpSize, a.maxChannels, s, ch));
  st.fifo = make_rsrc(receiverRow + fifo_offset(s, ch, a.maxChannels), kFifoBytes);
  __amdgpu_buffer_rsrc_t outRsrc = make_rsrc(a.rank[r].recv0, a.recvBytes0);
  float* lseOut = reinterpret_cast<float*>(a.rank[r].recv1);

  u32x2* pieces = reinterpret_cast<u32x2*>(lds);                                    // [cp][np]
  float* weights = reinterpret_cast<float*>(lds + static_cast<size_t>(a.cpSize) * st.np * kPieceBytes);  // [cp][heads]
  u32x2* myPieces = pieces + static_cast<size_t>(s) * st.np;

  int64_t step = info[1];
  const int flagLane = lane | 7;
  const int tid = static_cast<int>(threadIdx.x);
  const int threads = static_cast<int>(blockDim.x);

  for (int k = 0; k < st.msgs; ++k) {
    const int posInRun = k % st.msgsPerEntry;
    if (k > 0 && posInRun == 0) {
      step += 1;
      if (lane == 0) {
        st_counter(&info[1], step);
        st_counter(&senderInfo[1], step);
      }
    }
    const uint32_t msgOffset = static_cast<uint32_t>(step & (kFifoDepth - 1)) * kFifoEntryBytes +
                               static_cast<uint32_t>(posInRun) * st.lines * kLineBytes;
    const uint32_t stepLo = static_cast<uint32_t>(step);
    const uint32_t stepHi = static_cast<uint32_t>(static_cast<uint64_t>(step) >> 32);
    bool timedOut = false;
    for (uint32_t U0 = 0; U0 < st.unitsPerMsg && !timedOut; U0 += kUnitsInFlight * kWaveLanes) {
      bool pending[kUnitsInFlight];
#pragma unroll
      for (int i = 0; i < kUnitsInFlight; ++i) pending[i] = (U0 + i * kWaveLanes + lane) < st.unitsPerMsg;
      SpinGuard guard(a.spinLimitTicks);
      for (;;) {
        u32x4 v[kUnitsInFlight];
#pragma unroll
        for (int i = 0; i < kUnitsInFlight; ++i) {
          uint32_t U = U0 + i * kWaveLanes + lane;
          uint32_t off = pending[i] ? msgOffset + U * kUnitBytes : kOutOfRange;
          v[i] = __builtin_amdgcn_raw_buffer_load_b128(st.fifo, off, 0, kAuxSc1);
        }
        bool anyPending = false;
#pragma unroll
        for (int i = 0; i < kUnitsInFlight; ++i) {
          uint32_t U = U0 + i * kWaveLanes + lane;
          bool isFlagLane = (U & 7u) == 7u;
          bool ok = !pending[i] || !isFlagLane || (v[i].z == stepLo && v[i].w == stepHi);
          unsigned long long okMask = __ballot(ok);
          bool lineOk = (okMask >> flagLane) & 1ull;
          if (pending[i] && lineOk) {
            uint32_t pa = static_cast<uint32_t>(unit_first_piece(static_cast<int>(U)));
            if (pa < st.np) {
              u32x2 wa = {v[i].x, v[i].y};
              myPieces[pa] = wa;
            }
            if (!isFlagLane && pa + 1 < st.np) {
              u32x2 wb = {v[i].z, v[i].w};
              myPieces[pa + 1] = wb;
            }
          }
          pending[i] = pending[i] && !lineOk;
          anyPending |= pending[i];
        }
        if (__ballot(anyPending) == 0ull) break;
        if (guard.expired()) {
          timedOut = true;
          break;
        }
        __builtin_amdgcn_s_sleep(1);
        asm volatile("" ::: "memory");
      }
    }
    if (timedOut) {
      raise_status(a.status, kStatusRecvTimeout, lane);
      if (lane == 0) atomicOr(failed, 1);
    }
    __syncthreads();
    if (*failed) return;  // every wavefront of the workgroup sees the same value here

    // weights of every (sender, head): softmax over the senders of the log-sum-exp
    const int entry = a.entryBegin + ch + k * a.runChannels;
    for (int h = tid; h < a.heads; h += threads) {
      float lse[kMaxCpSize];
      float m = -INFINITY;
#pragma unroll
      for (int q = 0; q < kMaxCpSize; ++q) {
        if (q < a.cpSize) {
          u32x2 st2 = pieces[static_cast<size_t>(q) * st.np + st.np0 + h];  // {stats[2h], stats[2h+1]}
          float x = __uint_as_float(st2.x);
          if (a.statsMode == 1) x = x + logf(__uint_as_float(st2.y));   // running max + ln(running sum)
          if (isnan(x) || isinf(x)) x = -INFINITY;
          lse[q] = x;
          m = fmaxf(m, x);
        }
      }
      if (m == -INFINITY) m = 0.0f;
      float total = 0.0f;
#pragma unroll
      for (int q = 0; q < kMaxCpSize; ++q) {
        if (q < a.cpSize) {
          float w = expf(lse[q] - m);
          if (isnan(w)) w = 0.0f;
          lse[q] = w;
          total += w;
        }
      }
      float inv = 1.0f / fmaxf(total, 1e-10f);
#pragma unroll
      for (int q = 0; q < kMaxCpSize; ++q) {
        if (q < a.cpSize) weights[q * a.heads + h] = lse[q] * inv;
      }
      if (lseOut != nullptr) lseOut[static_cast<size_t>(entry) * a.heads + h] = logf(total) + m;
    }
    __syncthreads();

    // weighted sum over the senders, 4 elements (one piece) per thread and step
    for (uint32_t j = static_cast<uint32_t>(tid); j < st.np0; j += static_cast<uint32_t>(threads)) {
      uint32_t h = head_of_piece(j, a.headMagic);
      float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
      for (int q = 0; q < a.cpSize; ++q) {
        float f[4];
        widen4<kDtype>(pieces[static_cast<size_t>(q) * st.np + j], f);
        float w = weights[q * a.heads + h];
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[c] += w * f[c];
      }
      u32x2 o = {narrow1<kDtype>(acc[0]) | (narrow1<kDtype>(acc[1]) << 16),
                 narrow1<kDtype>(acc[2]) | (narrow1<kDtype>(acc[3]) << 16)};
      uint32_t off = static_cast<uint32_t>(entry) * (st.np0 * kPieceBytes) + j * kPieceBytes;
      __builtin_amdgcn_raw_buffer_store_b64(o, outRsrc, off, 0, kAuxNone);
    }
    __syncthreads();  // LDS is reused by the next message
  }
  if (lane == 0) {
    st_counter(&info[1], step + 1);
    st_counter(&senderInfo[1], step + 1);
  }
}

// Workgroups of cpSize wavefronts. The first rankCount*runChannels workgroups
// send (workgroup = (sender, channel), wavefront = receiver), the rest receive
// and combine (workgroup = (receiver, channel), wavefront = sender).
template <int kDtype>
__global__ __launch_bounds__(kMaxCpSize * kWaveLanes) void helix_combine_kernel(KernelArgs a) {
  extern __shared__ __align__(16) uint8_t dynamicLds[];
  __shared__ int failed;
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWaveLanes);
  const int lane = static_cast<int>(threadIdx.x) % kWaveLanes;
  const int sendBlocks = a.rankCount * a.runChannels;
  int b = static_cast<int>(blockIdx.x);
  if (b < sendBlocks) {
    run_sender<kAuxSc1>(a, a.rankBegin + b / a.runChannels, wave, b % a.runChannels, lane);
    return;
  }
  b -= sendBlocks;
  if (threadIdx.x == 0) failed = 0;
  __syncthreads();
  run_combine_receiver<kDtype>(a, a.rankBegin + b / a.runChannels, wave, b % a.runChannels, lane, dynamicLds, &failed);
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

hipError_t launch_combine(const KernelArgs& a, hipStream_t stream) {
  int blocks = 2 * a.rankCount * a.runChannels;
  if (blocks <= 0) return hipSuccess;
  const MsgShape sh = make_msg_shape(a.field0Bytes, a.field1Bytes);
  uint32_t lds = combine_lds_bytes(a.cpSize, sh, a.heads);
  dim3 block(static_cast<unsigned>(a.cpSize * kWaveLanes));
  if (a.dtype == 1) {
    if (lds > 64u * 1024u) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&helix_combine_kernel<1>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(helix_combine_kernel<1>, dim3(blocks), block, lds, stream, a);
  } else {
    if (lds > 64u * 1024u) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&helix_combine_kernel<0>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds));
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(helix_combine_kernel<0>, dim3(blocks), block, lds, stream, a);
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
