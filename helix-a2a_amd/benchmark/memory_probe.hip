// memory_probe.hip -- a yardstick for the exchange kernels: chunked copies with their access pattern and none
// of their protocol.
//
// A stream's wavefront of the Helix exchange moves one run: a few KiB that are contiguous on the FIFO side
// (a slot per stream) and contiguous or in rows on the tensor side. This kernel moves
// `chunks` such chunks: chunk c is `chunk_bytes` long, read at src + c * src_stride and written at
// dst + c * dst_stride, by `waves_per_chunk` wavefronts that each take a contiguous slice of whole 1 KiB
// wave accesses and walk it in passes of up to six 16-byte units per lane, all loads of a pass before its
// first store -- what the exchange kernel's wavefronts do, without counters, tokens, flags, line format or
// index arithmetic. Same occupancy (four wavefronts per SIMD, six for teams), same buffer-descriptor accesses.
//
// What this copy reaches on a shape is what the memory system gives chunk-per-wavefront traffic of that shape;
// bench.py --probe chunk-copy puts the exchange kernels beside it. Measuring equipment: the product library
// does not contain or load it.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

using u32x4 = uint32_t __attribute__((ext_vector_type(4)));

constexpr int kLanes = 64;
constexpr int kUnit = 16;
constexpr int kMaxInFlight = 6;
constexpr uint32_t kOutOfRange = 0x80000000u;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, static_cast<int>(bytes), 0x00020000u);
}

struct ProbeArgs {
  const uint8_t* src;
  uint8_t* dst;
  uint64_t srcStride, dstStride;
  uint32_t chunkBytes, chunks;
  int wavesPerChunk;  // = wavefronts of a workgroup when > 1 (a team), else two independent wavefronts per workgroup
  int mode;           // 0 copy, 1 read only, 2 write only
  uint32_t* sink;
};

// K units per lane in flight
template <int K>
__device__ __forceinline__ void move_slice(const ProbeArgs& a, __amdgpu_buffer_rsrc_t s, __amdgpu_buffer_rsrc_t d,
                                           uint32_t begin, uint32_t end, int lane) {
  u32x4 acc = {0u, 0u, 0u, 0u};
  for (uint32_t u0 = begin; u0 < end; u0 += K * kLanes) {
    u32x4 v[K];
#pragma unroll
    for (int i = 0; i < K; ++i) {
      const uint32_t u = u0 + i * kLanes + lane;
      if (a.mode != 2) v[i] = __builtin_amdgcn_raw_buffer_load_b128(s, u < end ? u * kUnit : kOutOfRange, 0, 0);
      else v[i] = u32x4{u, 1u, 2u, 3u};
    }
#pragma unroll
    for (int i = 0; i < K; ++i) {
      const uint32_t u = u0 + i * kLanes + lane;
      if (a.mode != 1) __builtin_amdgcn_raw_buffer_store_b128(v[i], d, u < end ? u * kUnit : kOutOfRange, 0, 0);
      else acc ^= v[i];
    }
  }
  if (a.mode == 1 && (acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) a.sink[0] = 1;  // keeps the loads alive
}

// kTeam: several wavefronts per chunk, one workgroup per chunk, six wavefronts per SIMD (as the exchange kernel's teams)
template <bool kTeam>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(kTeam ? 6 : 4, kTeam ? 6 : 4))) void helix_probe_chunk_copy_kernel(ProbeArgs a) {
  const int wave = static_cast<int>(threadIdx.x) / kLanes, lane = static_cast<int>(threadIdx.x) % kLanes;
  const int wavesPerBlock = static_cast<int>(blockDim.x) / kLanes;
  uint32_t chunk;
  int part;
  if (a.wavesPerChunk > 1) {
    chunk = blockIdx.x;
    part = wave;
  } else {
    chunk = blockIdx.x * wavesPerBlock + wave;
    part = 0;
  }
  if (chunk >= a.chunks) return;
  const __amdgpu_buffer_rsrc_t s = rsrc(a.src + chunk * a.srcStride, a.chunkBytes);
  const __amdgpu_buffer_rsrc_t d = rsrc(a.dst + chunk * a.dstStride, a.chunkBytes);
  const uint32_t units = a.chunkBytes / kUnit;
  const uint32_t perLane = (units + kLanes - 1) / kLanes;
  const uint32_t slice = (perLane + a.wavesPerChunk - 1) / a.wavesPerChunk * kLanes;
  const uint32_t begin = min(units, static_cast<uint32_t>(part) * slice), end = min(units, begin + slice);
  // the fewest passes of at most six units per lane, then the smallest count that still makes that many passes
  const uint32_t slicePerLane = slice / kLanes;
  const uint32_t passes = (slicePerLane + kMaxInFlight - 1) / kMaxInFlight;
  const uint32_t k = passes ? (slicePerLane + passes - 1) / passes : 1;
  switch (k) {
    case 1: move_slice<1>(a, s, d, begin, end, lane); break;
    case 2: move_slice<2>(a, s, d, begin, end, lane); break;
    case 3: move_slice<3>(a, s, d, begin, end, lane); break;
    case 4: move_slice<4>(a, s, d, begin, end, lane); break;
    case 5: move_slice<5>(a, s, d, begin, end, lane); break;
    default: move_slice<6>(a, s, d, begin, end, lane); break;
  }
}

__device__ uint32_t g_sink[4];

}  // namespace

// One launch of the chunked copy on `stream`. Returns the hipError_t of the launch (0 = ok), or -1 for arguments
// the kernel is not written for (chunk_bytes a multiple of 16 below 2 GiB, 1..8 wavefronts per chunk).
extern "C" int helix_probe_chunk_copy(const void* src, uint64_t src_stride, void* dst, uint64_t dst_stride,
                                      uint32_t chunk_bytes, uint32_t chunks, int waves_per_chunk, int mode, void* stream) {
  if (chunk_bytes == 0 || chunk_bytes % kUnit != 0 || chunk_bytes >= 0x80000000u || chunks == 0 || waves_per_chunk < 1 ||
      waves_per_chunk > 8 || mode < 0 || mode > 2 || src == nullptr || dst == nullptr)
    return -1;
  ProbeArgs a;
  a.src = static_cast<const uint8_t*>(src);
  a.dst = static_cast<uint8_t*>(dst);
  a.srcStride = src_stride;
  a.dstStride = dst_stride;
  a.chunkBytes = chunk_bytes;
  a.chunks = chunks;
  a.wavesPerChunk = waves_per_chunk;
  a.mode = mode;
  void* sink = nullptr;
  hipError_t err = hipGetSymbolAddress(&sink, HIP_SYMBOL(g_sink));
  if (err != hipSuccess) return static_cast<int>(err);
  a.sink = static_cast<uint32_t*>(sink);
  const int wavesPerBlock = waves_per_chunk > 1 ? waves_per_chunk : 2;
  const uint32_t blocks = waves_per_chunk > 1 ? chunks : (chunks + wavesPerBlock - 1) / wavesPerBlock;
  if (waves_per_chunk > 1)
    hipLaunchKernelGGL(helix_probe_chunk_copy_kernel<true>, dim3(blocks), dim3(wavesPerBlock * kLanes), 0,
                       static_cast<hipStream_t>(stream), a);
  else
    hipLaunchKernelGGL(helix_probe_chunk_copy_kernel<false>, dim3(blocks), dim3(wavesPerBlock * kLanes), 0,
                       static_cast<hipStream_t>(stream), a);
  return static_cast<int>(hipGetLastError());
}
