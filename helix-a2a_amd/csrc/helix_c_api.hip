// helix_c_api.hip -- host side of the C ABI declared in include/helix_a2a.h.
//
// Validates launch descriptors the way the reference binding validates its
// tensors (csrc/torch_binding.cpp:40-63,65-129), picks the channel count,
// splits a call into stream-ordered rounds when one round would overflow the
// FIFOs, and launches the gfx950 kernels. Errors come back as status codes
// with a thread-local message; nothing here aborts the process.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

#include "../../include/helix_a2a.h"
#include "helix_kernels.hpp"

namespace {

using namespace helix;

thread_local char g_lastError[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_lastError, sizeof(g_lastError), fmt, ap);
  va_end(ap);
  return code;
}

#define HELIX_HIP_TRY(call)                                                                       \
  do {                                                                                            \
    hipError_t err__ = (call);                                                                    \
    if (err__ != hipSuccess)                                                                      \
      return fail(HELIX_A2A_ERR_RUNTIME, "%s failed: %s", #call, hipGetErrorString(err__));       \
  } while (0)

std::atomic<uint64_t> g_spinLimitUs{2000000};
std::atomic<int> g_singleRound{0};
std::atomic<int> g_checked{-1};  // -1: not decided yet (HELIX_A2A_CHECKED is read once)

bool checked_mode() {
  int v = g_checked.load();
  if (v < 0) {
    const char* env = std::getenv("HELIX_A2A_CHECKED");
    v = (env && *env && std::strcmp(env, "0") != 0) ? 1 : 0;
    g_checked.store(v);
  }
  return v != 0;
}
// Units per lane a wavefront takes of a run before the run is shared with another wavefront:
// -1 = kMaxUnitsInFlight, and only while the launch leaves wavefront slots of the device free;
// 0 = never share; 1..6 = always share beyond that many.
std::atomic<int> g_unitsPerWavefront{-1};
std::atomic<int> g_teamUnits{-1};

// Wavefronts per stream a launch may use at most. The automatic rule looks at the whole exchange (both
// directions of all cp ranks), not at the launch, so that the send and receive halves of one exchange
// cut their runs the same way even when they are issued as separate launches of different extent.
int max_parts_for(const KernelArgs& a, int cuCount) {
  const int mode = g_unitsPerWavefront.load();
  if (mode == 0) return 1;
  if (mode > 0) return kMaxStreamParts;
  return auto_max_parts(a.cpSize, a.runChannels, cuCount);
}
int team_units() { return g_teamUnits.load(); }

int units_per_part() {
  const int mode = g_unitsPerWavefront.load();
  return mode > 0 ? mode : kMaxUnitsInFlight;
}

constexpr int kMaxDevices = 64;
struct DeviceState {
  std::once_flag once;
  hipError_t initError = hipSuccess;
  int cuCount = 0;
  uint32_t* status = nullptr;  // device status word
  uint8_t* scratch = nullptr;  // this device's copy of the built-in workspace (helix_a2a_alltoall_loopback_static)
  std::mutex scratchMutex;
  int scratchCp = 0;           // cp_size the built-in workspace is laid out and initialised for (0 = not yet)
  bool scratchInGraphs = false;  // a call on the built-in workspace was captured: replays lay it out behind the host's back
};
DeviceState g_devices[kMaxDevices];

// status word: one per device, lives until the process ends
__device__ uint32_t g_statusWord[4];

// Built-in workspace of helix_a2a_alltoall_loopback_static: room for kStaticStreams FIFOs
// (sender, receiver, channel) with their two counter blocks, 64.06 MiB, held by every device the
// library runs on until the process ends. In host code the name is only a handle for
// hipGetSymbolAddress; kernels and fills get the per-device address kept in DeviceState::scratch.
constexpr int kStaticStreams = HELIX_A2A_STATIC_MAX_STREAMS;
constexpr size_t kStaticScratchBytes = static_cast<size_t>(kStaticStreams) * (kFifoBytes + 2 * kFifoInfoBytes);
static __device__ __align__(256) uint8_t scratch[kStaticScratchBytes];

int device_state(DeviceState** out) {
  int dev = 0;
  HELIX_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(HELIX_A2A_ERR_RUNTIME, "device index %d out of range", dev);
  DeviceState& st = g_devices[dev];
  std::call_once(st.once, [&]() {
    hipDeviceProp_t prop;
    st.initError = hipGetDeviceProperties(&prop, dev);
    if (st.initError != hipSuccess) return;
    st.cuCount = prop.multiProcessorCount;
    void* p = nullptr;
    st.initError = hipGetSymbolAddress(&p, HIP_SYMBOL(g_statusWord));
    if (st.initError != hipSuccess) return;
    st.status = static_cast<uint32_t*>(p);
    st.initError = hipMemset(st.status, 0, sizeof(uint32_t) * 4);
    if (st.initError != hipSuccess) return;
    void* sp = nullptr;
    st.initError = hipGetSymbolAddress(&sp, HIP_SYMBOL(scratch));
    if (st.initError != hipSuccess) return;
    st.scratch = static_cast<uint8_t*>(sp);
  });
  if (st.initError != hipSuccess)
    return fail(HELIX_A2A_ERR_RUNTIME, "device %d setup failed: %s", dev, hipGetErrorString(st.initError));
  *out = &st;
  return HELIX_A2A_OK;
}

int resolve_cu_count(int cuCount, int* out) {
  if (cuCount < 0) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "cu_count must be >= 0, got %d", cuCount);
  if (cuCount > 0) {
    *out = cuCount;
    return HELIX_A2A_OK;
  }
  DeviceState* st = nullptr;
  int rc = device_state(&st);
  if (rc != HELIX_A2A_OK) return rc;
  *out = st->cuCount;
  return HELIX_A2A_OK;
}

int check_cp_size(int cpSize) {
  if (cpSize < 1 || cpSize > kMaxCpSize)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "cp_size must be in [1, %d], got %d", kMaxCpSize, cpSize);
  return HELIX_A2A_OK;
}

// One wavefront per (sender, receiver, channel) and direction. A wavefront
// walks its stream's messages one chunk after the other, so the exchange gets
// faster with every channel that still has an entry to carry, on every shape
// measured on MI355X (256 CUs): as many channels as the workspace layout and
// the entry count allow. (The reference derives its count from what fits its
// shared memory, csrc/helix_alltoall.cu:502-535; nothing is staged here.)
int auto_channels(int cpSize, int entryCount, int cuCount) {
  int c = max_channel_count(cpSize, cuCount);
  if (c > entryCount) c = entryCount;
  if (c < 1) c = 1;
  return c;
}

int env_channel_count() {
  // HELIX_A2A_CHANNEL_COUNT as in csrc/torch_binding.cpp:25-32, but re-read on
  // every call so a sweep can change it without restarting the process.
  const char* env = std::getenv("HELIX_A2A_CHANNEL_COUNT");
  if (!env || !*env) return 0;
  int v = std::atoi(env);
  return v > 0 ? v : 0;
}

// A workspace the library provides itself, in place of the descriptor's.
struct BuiltinWorkspace {
  uint8_t* base;
  uint64_t rowStrideBytes;
  int maxChannels;
};

struct Plan {
  KernelArgs args;
  int entryCount;
  int roundEntries;  // entries per stream-ordered round (multiple of runChannels)
  MsgShape shape;
  int cuCount;
};

int check_field(const helix_a2a_field_t& f, const char* name, int eltSize, int entryCount, int cpSize,
                bool needData, int align = kPieceBytes) {
  if (needData && f.data == nullptr) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "%s: data pointer is null", name);
  if (f.element_size != eltSize)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "%s: element size must be %d bytes, got %d", name, eltSize,
                f.element_size);
  if (f.element_count <= 0) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "%s: element count must be positive", name);
  long bytes = static_cast<long>(f.element_count) * f.element_size;
  if (f.stride_bytes < bytes || (f.stride_bytes % align) != 0)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "%s: row stride %d must be a multiple of %d and >= row size %ld", name,
                f.stride_bytes, align, bytes);
  if ((reinterpret_cast<uintptr_t>(f.data) % align) != 0)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "%s: data pointer must be %d-byte aligned", name, align);
  double extent = static_cast<double>(entryCount) * cpSize * f.stride_bytes;
  if (extent >= 2147483648.0)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "%s: tensor extent %.0f bytes exceeds 2 GiB", name, extent);
  return HELIX_A2A_OK;
}

// Validate `count` rank descriptors that share one exchange and build the
// kernel argument block. Checks that need no device come first, so that a
// malformed descriptor is reported even where no GPU is present. `exchangeOutputs` selects whether recv_fields are
// checked (exchange) or ignored (combine).
// `packedStats`: softmax_stats holds one float per head (combine, HELIX_A2A_STATS_LSE_PACKED), any count.
int build_plan(const helix_a2a_params_t* ranks, int count, bool exchangeOutputs, Plan* plan,
               const BuiltinWorkspace* builtin = nullptr, bool packedStats = false) {
  if (ranks == nullptr || count < 1) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "no rank descriptors given");
  const helix_a2a_params_t& p0 = ranks[0];
  int rc = check_cp_size(p0.cp_size);
  if (rc) return rc;
  const int cp = p0.cp_size;
  if (count > cp) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "%d rank descriptors for cp_size %d", count, cp);
  if (p0.entry_count < 0) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "entry_count must be >= 0");
  if (builtin != nullptr) {
    if (p0.workspace != nullptr)
      return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "the workspace pointer must be null: this call uses the built-in workspace");
  } else {
    if (p0.workspace == nullptr) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "workspace pointer is null");
    if ((reinterpret_cast<uintptr_t>(p0.workspace) % kUnitBytes) != 0 || (p0.workspace_stride_u64 % 2) != 0)
      return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "workspace rows must be 16-byte aligned");
  }

  KernelArgs a;
  std::memset(&a, 0, sizeof(a));
  bool seen[kMaxCpSize] = {false};
  for (int i = 0; i < count; ++i) {
    const helix_a2a_params_t& p = ranks[i];
    if (p.cp_size != cp || p.entry_count != p0.entry_count || p.workspace != p0.workspace ||
        p.workspace_stride_u64 != p0.workspace_stride_u64 || p.max_channel_count != p0.max_channel_count ||
        p.channel_count != p0.channel_count)
      return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "rank descriptor %d disagrees with descriptor 0", i);
    if (p.cp_rank < 0 || p.cp_rank >= cp)
      return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "cp_rank must be in [0, cp_size), got %d", p.cp_rank);
    if (seen[p.cp_rank]) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "cp_rank %d given twice", p.cp_rank);
    seen[p.cp_rank] = true;
    if (p.cp_rank != p0.cp_rank + i)
      return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "rank descriptors must be consecutive ranks in ascending order");
    const bool haveData = p.entry_count > 0;
    if ((rc = check_field(p.send_fields[0], "send partial_o", 2, p.entry_count, cp, haveData))) return rc;
    if ((rc = check_field(p.send_fields[1], "send softmax_stats", 4, p.entry_count, cp, haveData, packedStats ? 4 : kPieceBytes)))
      return rc;
    for (int f = 0; f < 2; ++f) {
      if (p.send_fields[f].element_count != p0.send_fields[f].element_count ||
          p.send_fields[f].stride_bytes != p0.send_fields[f].stride_bytes)
        return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "rank descriptor %d: field %d shape differs from descriptor 0", i, f);
    }
    if (exchangeOutputs) {
      if ((rc = check_field(p.recv_fields[0], "recv partial_o", 2, p.entry_count, cp, haveData))) return rc;
      if ((rc = check_field(p.recv_fields[1], "recv softmax_stats", 4, p.entry_count, cp, haveData))) return rc;
      for (int f = 0; f < 2; ++f) {
        if (p.recv_fields[f].element_count != p0.send_fields[f].element_count ||
            p.recv_fields[f].stride_bytes != p0.recv_fields[f].stride_bytes)
          return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "rank descriptor %d: recv field %d shape differs", i, f);
      }
    }
    RankPtrs& rp = a.rank[p.cp_rank];
    rp.send0 = static_cast<const uint8_t*>(p.send_fields[0].data);
    rp.send1 = static_cast<const uint8_t*>(p.send_fields[1].data);
    rp.recv0 = static_cast<uint8_t*>(p.recv_fields[0].data);
    rp.recv1 = static_cast<uint8_t*>(p.recv_fields[1].data);
  }

  const int f0 = p0.send_fields[0].element_count * 2;
  const int f1 = p0.send_fields[1].element_count * 4;
  // csrc/torch_binding.cpp:95-97,105-106
  if (f0 % 16 != 0) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "partial_o rows must be a multiple of 16 bytes, got %d", f0);
  if (!packedStats && (p0.send_fields[1].element_count < 2 || p0.send_fields[1].element_count % 2 != 0))
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "softmax_stats last dimension must be even and >= 2, got %d",
                p0.send_fields[1].element_count);
  MsgShape sh = make_msg_shape(f0, f1);
  if (sh.lines > kFifoEntryLines)
    return fail(HELIX_A2A_ERR_CAPACITY, "a message of %d bytes needs %d lines, more than one FIFO entry (%d lines)",
                f0 + f1, sh.lines, kFifoEntryLines);

  // everything above is pure argument checking; from here on the device is consulted
  int cuCount = 0;
  rc = resolve_cu_count(0, &cuCount);
  if (rc) return rc;
  const int maxCh = builtin ? builtin->maxChannels : max_channel_count(cp, cuCount);
  if (builtin == nullptr) {
    if (p0.max_channel_count != maxCh)
      return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "max_channel_count %d does not match the device's %d (cp_size %d, %d CUs)",
                  p0.max_channel_count, maxCh, cp, cuCount);
    if (p0.workspace_stride_u64 * 8ull < workspace_bytes(cp, maxCh))
      return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "workspace row of %llu bytes is smaller than the %llu bytes cp_size %d needs",
                  static_cast<unsigned long long>(p0.workspace_stride_u64 * 8ull),
                  static_cast<unsigned long long>(workspace_bytes(cp, maxCh)), cp);
  }

  // a wavefront's descriptor of its stream's lines reaches over three quarters of the FIFO region and a slot
  if (static_cast<uint64_t>(kFifoDepth - 1) * fifo_position_bytes(cp, maxCh) + kFifoEntryBytes >= 0x80000000ull)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "a FIFO region of %d x %d streams is beyond what the kernels address", cp, maxCh);

  int channels = p0.channel_count > 0 ? p0.channel_count : env_channel_count();
  if (channels > maxCh) {
    if (p0.channel_count > 0 || builtin == nullptr)
      return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "channel_count %d exceeds max_channel_count %d", channels, maxCh);
    channels = maxCh;  // the environment's count is a wish, and the built-in workspace is smaller than a caller's
  }
  if (channels <= 0) {
    channels = auto_channels(cp, p0.entry_count, cuCount);
    if (channels > maxCh) channels = maxCh;
  }

  DeviceState* st = nullptr;
  if ((rc = device_state(&st))) return rc;

  a.workspace = builtin ? builtin->base : reinterpret_cast<uint8_t*>(p0.workspace);
  a.rowStrideBytes = builtin ? builtin->rowStrideBytes : p0.workspace_stride_u64 * 8ull;
  a.cpSize = cp;
  a.maxChannels = maxCh;
  a.runChannels = channels;
  a.entryBegin = 0;
  a.entryEnd = p0.entry_count;
  a.field0Bytes = f0;
  a.field1Bytes = f1;
  a.sendStride0 = p0.send_fields[0].stride_bytes;
  a.sendStride1 = p0.send_fields[1].stride_bytes;
  a.recvStride0 = exchangeOutputs ? p0.recv_fields[0].stride_bytes : 0;
  a.recvStride1 = exchangeOutputs ? p0.recv_fields[1].stride_bytes : 0;
  const uint64_t rows = static_cast<uint64_t>(p0.entry_count) * cp;
  a.sendBytes0 = static_cast<uint32_t>(rows * a.sendStride0);
  a.sendBytes1 = static_cast<uint32_t>(rows * a.sendStride1);
  a.recvBytes0 = static_cast<uint32_t>(rows * a.recvStride0);
  a.recvBytes1 = static_cast<uint32_t>(rows * a.recvStride1);
  a.npMagic = div_magic(static_cast<uint32_t>(sh.np));
  a.nsMagic = div_magic(static_cast<uint32_t>(sh.np - sh.np0));
  a.rankBegin = p0.cp_rank;
  a.rankCount = count;
  a.spinLimitTicks = g_spinLimitUs.load() * 100ull;
  a.status = st->status;

  plan->args = a;
  plan->entryCount = p0.entry_count;
  plan->shape = sh;
  plan->cuCount = cuCount;
  // a stream may put 4 entries worth of messages in flight before it needs the receiver
  long perStream = static_cast<long>(kFifoDepth) * msgs_per_fifo_entry(sh);
  long roundEntries = perStream * channels;
  plan->roundEntries = roundEntries > 2000000000L ? 2000000000 : static_cast<int>(roundEntries);
  return HELIX_A2A_OK;
}

int launch_rounds(Plan& plan, bool send, bool recv, bool allowRounds, hipStream_t stream) {
  KernelArgs a = plan.args;
  a.doSend = send ? 1 : 0;
  a.doRecv = recv ? 1 : 0;
  if (plan.entryCount == 0) return HELIX_A2A_OK;
  const bool fits = plan.entryCount <= plan.roundEntries;
  if (!fits && !allowRounds)
    return fail(HELIX_A2A_ERR_CAPACITY,
                "%d entries over %d channels put more than %d FIFO entries in flight per stream; "
                "raise the channel count or use the loopback call",
                plan.entryCount, a.runChannels, kFifoDepth);
  if (!fits && send && recv && g_singleRound.load()) {
    // in-kernel back-pressure needs every wavefront of the launch resident
    long waves = 2L * waves_per_direction(a);
    if (waves > static_cast<long>(plan.cuCount) * 8)
      return fail(HELIX_A2A_ERR_CAPACITY, "single-round launch of %ld wavefronts is not guaranteed co-resident", waves);
    HELIX_HIP_TRY(launch_exchange(a, kMaxUnitsInFlight, 1, 0, stream));  // senders wait on the one tail counter: one wavefront per stream
    return HELIX_A2A_OK;
  }
  for (int begin = 0; begin < plan.entryCount; begin += plan.roundEntries) {
    a.entryBegin = begin;
    long end = static_cast<long>(begin) + plan.roundEntries;
    a.entryEnd = end > plan.entryCount ? plan.entryCount : static_cast<int>(end);
    HELIX_HIP_TRY(launch_exchange(a, units_per_part(), max_parts_for(a, plan.cuCount), team_units(), stream));
  }
  return HELIX_A2A_OK;
}

// Wait for `stream`, read the device status word and clear it. Everything is ordered on `stream` itself (nothing
// goes through the legacy default stream, which may not be touched while some other stream is being captured).
int read_status(DeviceState* st, hipStream_t stream, uint32_t* out) {
  uint32_t host = 0;
  HELIX_HIP_TRY(hipMemcpyAsync(&host, st->status, sizeof(host), hipMemcpyDeviceToHost, stream));
  HELIX_HIP_TRY(hipStreamSynchronize(stream));
  if (host != 0) {
    HELIX_HIP_TRY(hipMemsetAsync(st->status, 0, sizeof(uint32_t), stream));
    HELIX_HIP_TRY(hipStreamSynchronize(stream));
  }
  *out = host;
  return HELIX_A2A_OK;
}

// End of every exchange call: nothing in the normal mode, a synchronous status check in checked mode.
int finish_call(int rc, hipStream_t stream) {
  if (rc != HELIX_A2A_OK || !checked_mode()) return rc;
  // a stream that is being captured into a graph cannot be waited for: the check is left to the replays' caller
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone) return rc;
  DeviceState* st = nullptr;
  if ((rc = device_state(&st))) return rc;
  uint32_t status = 0;
  if ((rc = read_status(st, stream, &status))) return rc;
  if (status == 0) return HELIX_A2A_OK;
  return fail(HELIX_A2A_ERR_DEVICE, "the exchange raised device status 0x%x (%s%s%s%s); re-initialise the workspace", status,
              (status & HELIX_A2A_STATUS_RECV_TIMEOUT) ? "receive wait timed out " : "",
              (status & HELIX_A2A_STATUS_SEND_TIMEOUT) ? "send wait timed out " : "",
              (status & HELIX_A2A_STATUS_INTERNAL) ? "corrupt line " : "",
              (status & HELIX_A2A_STATUS_BROKEN_WORKSPACE) ? "workspace broken by an earlier failure" : "");
}

}  // namespace

extern "C" {

int helix_a2a_max_channel_count(int cp_size, int cu_count) {
  if (check_cp_size(cp_size)) return -1;
  int cu = 0;
  if (resolve_cu_count(cu_count, &cu)) return -1;
  return max_channel_count(cp_size, cu);
}

int64_t helix_a2a_workspace_size_per_rank(int cp_size, int cu_count) {
  int maxCh = helix_a2a_max_channel_count(cp_size, cu_count);
  if (maxCh < 0) return -1;
  return static_cast<int64_t>(workspace_bytes(cp_size, maxCh));
}

int helix_a2a_auto_channel_count(int cp_size, int entry_count, int cu_count) {
  if (check_cp_size(cp_size)) return -1;
  if (entry_count < 0) {
    fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "entry_count must be >= 0");
    return -1;
  }
  int cu = 0;
  if (resolve_cu_count(cu_count, &cu)) return -1;
  return auto_channels(cp_size, entry_count, cu);
}

int helix_a2a_init_workspace(uint64_t* local_row, int cp_size, int cu_count, void* stream) {
  int rc = check_cp_size(cp_size);
  if (rc) return rc;
  if (local_row == nullptr) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "workspace row pointer is null");
  if ((reinterpret_cast<uintptr_t>(local_row) % kUnitBytes) != 0)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "workspace row must be 16-byte aligned");
  int cu = 0;
  if ((rc = resolve_cu_count(cu_count, &cu))) return rc;
  int maxCh = max_channel_count(cp_size, cu);
  HELIX_HIP_TRY(launch_init_row(reinterpret_cast<uint8_t*>(local_row), fifo_region_bytes(cp_size, maxCh),
                                2 * info_region_bytes(cp_size, maxCh), static_cast<hipStream_t>(stream)));
  return HELIX_A2A_OK;
}

int helix_a2a_alltoall(const helix_a2a_params_t* params, void* stream) {
  Plan plan;
  int rc = build_plan(params, 1, true, &plan);
  if (rc) return rc;
  // both halves in one launch: with peers on the same queue behind this call
  // the receive half can only time out, so rounds are not an option here
  return finish_call(launch_rounds(plan, true, true, plan.args.cpSize == 1, static_cast<hipStream_t>(stream)),
                     static_cast<hipStream_t>(stream));
}

int helix_a2a_alltoall_send(const helix_a2a_params_t* per_rank, int rank_count, void* stream) {
  Plan plan;
  int rc = build_plan(per_rank, rank_count, true, &plan);
  if (rc) return rc;
  return launch_rounds(plan, true, false, false, static_cast<hipStream_t>(stream));
}

int helix_a2a_alltoall_recv(const helix_a2a_params_t* per_rank, int rank_count, void* stream) {
  Plan plan;
  int rc = build_plan(per_rank, rank_count, true, &plan);
  if (rc) return rc;
  return finish_call(launch_rounds(plan, false, true, false, static_cast<hipStream_t>(stream)),
                     static_cast<hipStream_t>(stream));
}

int helix_a2a_alltoall_loopback(const helix_a2a_params_t* per_rank, int cp_size, void* stream) {
  if (per_rank == nullptr) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "no rank descriptors given");
  if (per_rank[0].cp_size != cp_size || per_rank[0].cp_rank != 0)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "loopback needs descriptors of ranks 0..cp_size-1 in order");
  Plan plan;
  int rc = build_plan(per_rank, cp_size, true, &plan);
  if (rc) return rc;
  return finish_call(launch_rounds(plan, true, true, true, static_cast<hipStream_t>(stream)), static_cast<hipStream_t>(stream));
}

int helix_a2a_alltoall_loopback_static(const helix_a2a_params_t* per_rank, int cp_size, int reset, void* stream) {
  if (per_rank == nullptr) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "no rank descriptors given");
  int rc = check_cp_size(cp_size);
  if (rc) return rc;
  if (per_rank[0].cp_size != cp_size || per_rank[0].cp_rank != 0)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "loopback needs descriptors of ranks 0..cp_size-1 in order");
  if (cp_size * cp_size > kStaticStreams)
    return fail(HELIX_A2A_ERR_CAPACITY,
                "the built-in workspace holds %d FIFOs, cp_size %d needs at least %d (cp_size <= %d); "
                "use helix_a2a_alltoall_loopback with a workspace of your own",
                kStaticStreams, cp_size, cp_size * cp_size, HELIX_A2A_STATIC_MAX_CP_SIZE);
  DeviceState* st = nullptr;
  if ((rc = device_state(&st))) return rc;
  BuiltinWorkspace ws;
  ws.maxChannels = kStaticStreams / (cp_size * cp_size);
  ws.rowStrideBytes = workspace_bytes(cp_size, ws.maxChannels);
  ws.base = st->scratch;  // the device address from hipGetSymbolAddress, never the array's name
  Plan plan;
  if ((rc = build_plan(per_rank, cp_size, true, &plan, &ws))) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  {
    // The array keeps the last call's contents. Its layout depends on cp_size, so a change of cp_size
    // (or the first call, or a caller's request) lays it out again: FIFO bytes 0xFF, counters 0, by a
    // fill kernel in stream order ahead of the exchange.
    // A captured call always records the fill kernels: whatever ran on the array between two replays of the
    // graph, every replay starts from a layout of its own. From then on the host no longer knows what layout
    // the array holds when an eager call arrives, so eager calls lay it out every time as well.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    const bool capturing = hipStreamIsCapturing(s, &capture) == hipSuccess && capture != hipStreamCaptureStatusNone;
    std::lock_guard<std::mutex> lock(st->scratchMutex);
    if (capturing) st->scratchInGraphs = true;
    if (reset || st->scratchInGraphs || st->scratchCp != cp_size) {
      for (int r = 0; r < cp_size; ++r)
        HELIX_HIP_TRY(launch_init_row(ws.base + static_cast<uint64_t>(r) * ws.rowStrideBytes,
                                      fifo_region_bytes(cp_size, ws.maxChannels),
                                      2 * info_region_bytes(cp_size, ws.maxChannels), s));
      st->scratchCp = cp_size;
    }
  }
  return finish_call(launch_rounds(plan, true, true, true, s), s);
}

int helix_a2a_alltoall_combine_loopback(const helix_a2a_params_t* per_rank, const helix_a2a_combine_out_t* out,
                                        int cp_size, int stats_mode, int dtype, void* stream) {
  if (per_rank == nullptr || out == nullptr)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "no rank descriptors or outputs given");
  if (per_rank[0].cp_size != cp_size || per_rank[0].cp_rank != 0)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "loopback needs descriptors of ranks 0..cp_size-1 in order");
  const bool base2 = (stats_mode & HELIX_A2A_STATS_BASE2) != 0;
  stats_mode &= ~HELIX_A2A_STATS_BASE2;
  if (stats_mode != HELIX_A2A_STATS_LSE && stats_mode != HELIX_A2A_STATS_MAX_SUM &&
      stats_mode != HELIX_A2A_STATS_LSE_PACKED)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "unknown stats_mode %d", stats_mode);
  if (base2 && stats_mode == HELIX_A2A_STATS_MAX_SUM)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "HELIX_A2A_STATS_BASE2 applies to log-sum-exp statistics, not to (max, sum) pairs");
  if (dtype != HELIX_A2A_DTYPE_BF16 && dtype != HELIX_A2A_DTYPE_FP16)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "unknown dtype %d", dtype);
  if (cp_size > kMaxCombineCpSize)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "the fused combine serves cp_size <= %d, got %d", kMaxCombineCpSize,
                cp_size);
  Plan plan;
  int rc = build_plan(per_rank, cp_size, false, &plan, nullptr, stats_mode == HELIX_A2A_STATS_LSE_PACKED);
  if (rc) return rc;
  KernelArgs& a = plan.args;
  const int x = per_rank[0].send_fields[0].element_count;
  const int statsWidth = per_rank[0].send_fields[1].element_count;
  const int heads = stats_mode == HELIX_A2A_STATS_LSE_PACKED ? statsWidth : statsWidth / 2;
  if (heads < 1 || x % heads != 0 || (x / heads) % 4 != 0 || x / heads < 32)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT,
                "combine needs partial_o rows of heads * head_dim elements with head_dim a multiple of 4 and >= 32 "
                "(row of %d elements, %d heads)", x, heads);
  a.heads = heads;
  a.headDim = x / heads;
  a.statsMode = stats_mode;
  a.lseBase2 = base2 ? 1 : 0;
  a.dtype = dtype;
  a.headMagic = head_div_magic(static_cast<uint32_t>(a.headDim) * 2u / kPieceBytes);
  a.np0Magic = div_magic(static_cast<uint32_t>(plan.shape.np0));
  const uint64_t outBytes = static_cast<uint64_t>(plan.entryCount) * a.field0Bytes;
  if (outBytes >= 2147483648ull) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "combined output exceeds 2 GiB");
  a.recvBytes0 = static_cast<uint32_t>(outBytes);
  a.recvBytes1 = static_cast<uint32_t>(static_cast<uint64_t>(plan.entryCount) * heads * 4u);
  for (int r = 0; r < cp_size; ++r) {
    if (plan.entryCount > 0 && out[r].combined == nullptr)
      return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "combined output of rank %d is null", r);
    if ((reinterpret_cast<uintptr_t>(out[r].combined) % kPieceBytes) != 0 ||
        (reinterpret_cast<uintptr_t>(out[r].lse_out) % 4) != 0)
      return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "combine outputs of rank %d are misaligned", r);
    a.rank[r].recv0 = static_cast<uint8_t*>(out[r].combined);
    a.rank[r].recv1 = reinterpret_cast<uint8_t*>(out[r].lse_out);
  }
  if (plan.entryCount == 0) return HELIX_A2A_OK;
  for (int begin = 0; begin < plan.entryCount; begin += plan.roundEntries) {
    a.entryBegin = begin;
    long end = static_cast<long>(begin) + plan.roundEntries;
    a.entryEnd = end > plan.entryCount ? plan.entryCount : static_cast<int>(end);
    // wavefronts per (receiver, channel): enough to cover a round's output pieces once, and to fill the device
    int msgs = stream_msg_count(a.entryBegin, a.entryEnd, 0, a.runChannels);
    int perEntry = msgs_per_fifo_entry(plan.shape);
    long runPieces = static_cast<long>(msgs < perEntry ? msgs : perEntry) * plan.shape.np0;
    long perTurn = (cp_size <= 16 ? 2 : 1) * kWaveLanes;  // pieces a wavefront takes per turn
    long cover = (runPieces + perTurn - 1) / perTurn;
    long fill = static_cast<long>(plan.cuCount) * 16 / (static_cast<long>(cp_size) * a.runChannels);
    long parts = cover < fill ? cover : fill;
    if (parts < 1) parts = 1;
    if (parts > kMaxCombineParts) parts = kMaxCombineParts;
    a.doSend = 1;
    a.doRecv = 1;
    HELIX_HIP_TRY(launch_combine(a, static_cast<int>(parts), static_cast<hipStream_t>(stream)));
  }
  return finish_call(HELIX_A2A_OK, static_cast<hipStream_t>(stream));
}

int helix_a2a_device_status(uint32_t* status, void* stream) {
  if (status == nullptr) return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "status pointer is null");
  DeviceState* st = nullptr;
  int rc = device_state(&st);
  if (rc) return rc;
  return read_status(st, static_cast<hipStream_t>(stream), status);
}

void helix_a2a_set_checked_mode(int enabled) { g_checked.store(enabled ? 1 : 0); }

void helix_a2a_set_spin_limit_us(uint64_t microseconds) { g_spinLimitUs.store(microseconds); }

void helix_a2a_set_single_round(int enabled) { g_singleRound.store(enabled ? 1 : 0); }


int helix_a2a_set_team_units(int units) {
  if (units < -1 || units > kMaxUnitsInFlight)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "units per team wavefront must be in [-1, %d], got %d", kMaxUnitsInFlight, units);
  g_teamUnits.store(units);
  return HELIX_A2A_OK;
}

int helix_a2a_set_units_per_wavefront(int units) {
  if (units < -1 || units > kMaxUnitsInFlight)
    return fail(HELIX_A2A_ERR_INVALID_ARGUMENT, "units per wavefront must be in [-1, %d], got %d", kMaxUnitsInFlight, units);
  g_unitsPerWavefront.store(units);
  return HELIX_A2A_OK;
}

const char* helix_a2a_last_error(void) { return g_lastError; }

const char* helix_a2a_version(void) { return "0.1.0"; }

}  // extern "C"
