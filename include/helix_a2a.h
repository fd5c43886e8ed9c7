/*
 * helix_a2a.h -- C ABI of the MI355X (gfx950) Helix all-to-all library.
 *
 * This is the boundary a host binding talks to. It takes the place of the
 * reference's libtorch binding (csrc/torch_binding.cpp) and of the C++ entry
 * points that binding calls (csrc/helix_alltoall.h:35-43). Everything here is
 * plain C: pointers, sizes, an opaque stream handle (a hipStream_t passed as
 * void*). The library never allocates or frees tensor memory; inputs, outputs
 * and the workspace belong to the caller and must stay alive until the stream
 * has drained.
 *
 * Every function that can fail returns 0 on success and a non-zero
 * HELIX_A2A_ERR_* code otherwise; helix_a2a_last_error() then returns a
 * thread-local, human readable message. Nothing in this library calls abort().
 *
 * Vocabulary
 *   cp_size      number of context-parallel ranks taking part in the exchange
 *   entry        one row index e of the [E, cp_size, *] send/receive tensors
 *   message      the two fields (partial_o row, softmax_stats row) of one
 *                (entry, peer) pair; it travels through one FIFO
 *   channel      entries are dealt round-robin over `channel_count` channels;
 *                every (sender, receiver, channel) triple owns one FIFO
 *   FIFO         4 entries x 128 KiB in the receiver's workspace row, written
 *                by the sender with LL128 lines (120 payload bytes + 8-byte
 *                flag), polled by the receiver
 */
#ifndef HELIX_A2A_H_
#define HELIX_A2A_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HELIX_A2A_MAX_CP_SIZE 32
#define HELIX_A2A_MAX_COMBINE_CP_SIZE 32 /* helix_a2a_alltoall_combine_loopback */

/* helix_a2a_alltoall_loopback_static: FIFOs the built-in workspace holds, and the largest cp_size that fits */
#define HELIX_A2A_STATIC_MAX_STREAMS 128
#define HELIX_A2A_STATIC_MAX_CP_SIZE 11

/* error codes */
#define HELIX_A2A_OK 0
#define HELIX_A2A_ERR_INVALID_ARGUMENT 1 /* a parameter failed validation        */
#define HELIX_A2A_ERR_RUNTIME 2          /* a HIP runtime call failed            */
#define HELIX_A2A_ERR_CAPACITY 3         /* traffic does not fit the FIFOs in the requested mode */
#define HELIX_A2A_ERR_DEVICE 4           /* checked mode: the exchange raised bits in the device status word */

/* bits of the device status word (helix_a2a_device_status) */
#define HELIX_A2A_STATUS_RECV_TIMEOUT 1u /* a receiver gave up polling for a line */
#define HELIX_A2A_STATUS_SEND_TIMEOUT 2u /* a sender gave up waiting for FIFO room */
#define HELIX_A2A_STATUS_INTERNAL 4u     /* a kernel met a state its launch checks exclude (corrupt workspace) */
#define HELIX_A2A_STATUS_BROKEN_WORKSPACE 8u /* an exchange did nothing: an earlier failure left its workspace unusable */

/*
 * One field of a message. Same members and meaning as the reference's
 * HelixFieldInfo (csrc/helix_alltoall.h:16-21): row `i` of the field starts at
 * data + i * stride_bytes and holds element_count * element_size bytes.
 */
typedef struct helix_a2a_field {
  void* data;
  int32_t element_count;
  int32_t element_size;
  int32_t stride_bytes;
} helix_a2a_field_t;

/*
 * Launch descriptor of one rank. Same members and meaning as the reference's
 * HelixAllToAllParams (csrc/helix_alltoall.h:23-33), as filled in by
 * csrc/torch_binding.cpp:131-169:
 *   send_fields[0] / recv_fields[0]  partial_o      [entry_count, cp_size, D]  2-byte elements
 *   send_fields[1] / recv_fields[1]  softmax_stats  [entry_count, cp_size, S]  4-byte elements
 *   row index of message (entry e, peer p) is e * cp_size + p in all four.
 *   workspace            base of the [cp_size, workspace_stride_u64] uint64 tensor
 *   channel_count        0 = choose automatically, otherwise 1..max_channel_count
 *   max_channel_count    must equal helix_a2a_max_channel_count(cp_size, cu_count of the device)
 */
typedef struct helix_a2a_params {
  helix_a2a_field_t send_fields[2];
  helix_a2a_field_t recv_fields[2];
  int32_t entry_count;
  uint64_t* workspace;
  uint64_t workspace_stride_u64;
  int32_t cp_rank;
  int32_t cp_size;
  int32_t channel_count;
  int32_t max_channel_count;
} helix_a2a_params_t;

/*
 * Output descriptor of the fused LSE-weighted combine (one per rank).
 *   combined   [entry_count, heads * head_dim] 2-byte elements (same type as partial_o)
 *   lse_out    [entry_count, heads] fp32 global log-sum-exp, or NULL
 * The reduction it performs is the one the reference's caller applies after
 * the exchange (patches/dcp_alltoall_helix.py:142-207).
 */
typedef struct helix_a2a_combine_out {
  void* combined;
  float* lse_out;
} helix_a2a_combine_out_t;

/* how softmax_stats encodes the per-(entry, head) weight */
#define HELIX_A2A_STATS_LSE 0     /* stats[2h] = natural-log LSE, stats[2h+1] ignored (patches/dcp_alltoall_helix.py:560-567) */
#define HELIX_A2A_STATS_MAX_SUM 1 /* stats[2h] = running max, stats[2h+1] = running sum; LSE = max + ln(sum) */
#define HELIX_A2A_STATS_LSE_PACKED 2 /* stats[h] = natural-log LSE of head h: the caller's [B, H] LSE tensor as it is, any
                                        number of heads per rank, rows 4-byte aligned (patches/dcp_alltoall_helix.py:545-571
                                        pads it to pairs only for the reference kernel) */
#define HELIX_A2A_STATS_BASE2 16     /* or-ed to one of the two LSE modes: the LSE values are base-2 logarithms, and lse_out is
                                        written as one (is_lse_base_on_e = False, patches/dcp_alltoall_helix.py:183-186,199-203) */

/* element type of partial_o for the combine arithmetic */
#define HELIX_A2A_DTYPE_BF16 0
#define HELIX_A2A_DTYPE_FP16 1

/*
 * Largest channel count the workspace is laid out for.
 * Replaces computeHelixMaxChannelCount (csrc/helix_alltoall.h:35,
 * csrc/helix_alltoall.cu:590-603). cu_count = 0 queries the current device
 * (needs a GPU); any positive value is pure arithmetic.
 * Returns the count (>= 1), or -1 on error.
 */
int helix_a2a_max_channel_count(int cp_size, int cu_count);

/*
 * Bytes of workspace one rank needs (one row of the workspace tensor).
 * Replaces computeHelixWorkspaceSizePerRank (csrc/helix_alltoall.h:37,
 * csrc/helix_alltoall.cu:605-614) behind
 * torch.ops.helix_a2a.get_helix_workspace_size_per_rank (csrc/torch_binding.cpp:34-38).
 * Returns -1 on error.
 */
int64_t helix_a2a_workspace_size_per_rank(int cp_size, int cu_count);

/*
 * Channel count an automatic launch would run with for this problem on a
 * device with cu_count compute units (0 = current device): the counterpart of
 * computeChannelAndGroupCount (csrc/helix_alltoall.cu:486-535), re-derived for
 * one wavefront per (sender, receiver, channel) on 256 CUs -- as many channels
 * as the layout provides and the entries can fill. Returns -1 on error.
 */
int helix_a2a_auto_channel_count(int cp_size, int entry_count, int cu_count);

/*
 * Reset one rank's workspace row: FIFO region to 0xFF bytes, head/tail
 * counters to zero. Asynchronous on `stream`.
 * Replaces initializeHelixWorkspace (csrc/helix_alltoall.h:39-40,
 * csrc/helix_alltoall.cu:629-644) behind
 * torch.ops.helix_a2a.initialize_helix_workspace (csrc/torch_binding.cpp:40-63).
 */
int helix_a2a_init_workspace(uint64_t* local_row, int cp_size, int cu_count, void* stream);

/*
 * One rank's full exchange (send half and receive half in one launch), the
 * call a multi-device deployment makes on every rank. Replaces
 * launchHelixAllToAll (csrc/helix_alltoall.h:42-43, csrc/helix_alltoall.cu:616-623)
 * behind torch.ops.helix_a2a.alltoall_helix_native (csrc/torch_binding.cpp:65-175).
 * The receive half polls for lines its peers write; if they never arrive the
 * bounded wait expires, the kernel exits and HELIX_A2A_STATUS_RECV_TIMEOUT is
 * raised in the device status word.
 */
int helix_a2a_alltoall(const helix_a2a_params_t* params, void* stream);

/*
 * The two halves of helix_a2a_alltoall as separate launches, for `rank_count`
 * logical ranks that share one device and one workspace tensor. All senders
 * must have been enqueued (same stream, or ordered by events) before the
 * matching receive launch. The traffic of one call must fit the FIFOs
 * (HELIX_A2A_ERR_CAPACITY otherwise), because a send launch cannot be
 * back-pressured by a receive launch queued behind it.
 * Same reference counterpart as helix_a2a_alltoall (the sender branch,
 * csrc/helix_alltoall.cu:360-412, and the receiver branch, :413-473).
 * Order: the send launch of an exchange must have completed, or be ordered
 * ahead of its receive launch on one stream or by events, and the receive
 * launch of one exchange ahead of the send launch of the next on the same
 * workspace. When a stream's runs are shared by several wavefronts (see
 * helix_a2a_set_units_per_wavefront) only the first of them keeps the counter
 * that senders wait on for FIFO room, so halves that run unordered beside each
 * other could overwrite an entry that is still being read.
 */
int helix_a2a_alltoall_send(const helix_a2a_params_t* per_rank, int rank_count, void* stream);
int helix_a2a_alltoall_recv(const helix_a2a_params_t* per_rank, int rank_count, void* stream);

/*
 * Loopback exchange: all cp_size logical ranks of one device in a single
 * fused launch. per_rank[r] must have cp_rank == r; all descriptors share
 * workspace, shapes and strides. Sender wavefronts are placed before receiver
 * wavefronts in dispatch order. channel_count is taken from per_rank[0].
 * After the stream drains, recv of rank r holds
 *   recv_r[e, s, :] = send_s[e, r, :]     for both fields.
 */
int helix_a2a_alltoall_loopback(const helix_a2a_params_t* per_rank, int cp_size, void* stream);

/*
 * helix_a2a_alltoall_loopback without a workspace argument and without any
 * allocation. No counterpart in the reference; it is for callers that cannot
 * allocate device memory at this point (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). The FIFOs live in a
 * workspace built into the library: a device array of
 * HELIX_A2A_STATIC_MAX_STREAMS x (512 KiB + 512 B) = 67 174 400 bytes that
 * every GPU the library runs on holds until the process ends. The workspace
 * members of the descriptors must be NULL / 0 (max_channel_count is ignored);
 * everything else is as for helix_a2a_alltoall_loopback, same results.
 *   limit   cp_size * cp_size <= HELIX_A2A_STATIC_MAX_STREAMS, i.e. cp_size <= 11
 *           (HELIX_A2A_ERR_CAPACITY beyond); the channel count is at most
 *           128 / cp_size^2, so large exchanges run slower than with a full workspace.
 *   state   the array keeps its contents between calls. It is laid out again
 *           (FIFO bytes 0xFF, counters 0, by a fill kernel on `stream`) on the
 *           first call on a device, when cp_size differs from the previous
 *           call's, and when `reset` is non-zero (required after a time-out
 *           reported by helix_a2a_device_status).
 *   races   all calls on one GPU share that GPU's array: they must be ordered
 *           with respect to each other (one stream, or events). Calls that
 *           overlap on one GPU race.
 *   capture a call recorded into a graph always records the fill kernels too,
 *           so that every replay lays the array out for itself whatever ran on it
 *           in between; after the first such capture on a device, eager calls on
 *           that device lay the array out on every call as well (the host cannot
 *           know what a replay left behind). Checked mode does nothing on a
 *           capturing stream.
 * The very first library call on a device performs the one-time set-up
 * (device query, symbol addresses); make any library call before starting a
 * graph capture.
 */
int helix_a2a_alltoall_loopback_static(const helix_a2a_params_t* per_rank, int cp_size, int reset, void* stream);

/*
 * Loopback exchange fused with the LSE-weighted combine: the receive half
 * reduces the cp_size partial outputs of each (entry, head) instead of storing
 * them. recv_fields of per_rank are ignored; out[r] receives rank r's result.
 * stats_mode is one of HELIX_A2A_STATS_*, optionally or-ed with HELIX_A2A_STATS_BASE2.
 * heads = send_fields[1].element_count / 2 (element_count itself for HELIX_A2A_STATS_LSE_PACKED),
 * head_dim = send_fields[0].element_count / heads; head_dim must be a multiple of 4 and at least 32.
 */
int helix_a2a_alltoall_combine_loopback(const helix_a2a_params_t* per_rank,
                                        const helix_a2a_combine_out_t* out, int cp_size,
                                        int stats_mode, int dtype, void* stream);

/*
 * Read the device status word of the current device into *status (0 = no
 * error since the last read) and clear it. Synchronises `stream`.
 * No counterpart in the reference, whose waits are unbounded.
 */
int helix_a2a_device_status(uint32_t* status, void* stream);

/*
 * What a failure inside a kernel does. The reference's waits are unbounded: a
 * peer that never sends hangs the GPU. Here a wait that exceeds the spin limit,
 * or a line whose flag disagrees with its token, ends the wavefront, raises its
 * bit in the device status word and marks the workspace broken (a word in row
 * 0's counter region). Every wavefront that runs afterwards on that workspace
 * -- the rest of the launch and every launch queued behind it -- writes nothing
 * and raises HELIX_A2A_STATUS_BROKEN_WORKSPACE, so the output tensors of
 * such an exchange keep whatever they held before; the FIFO counters are no
 * longer consistent. (The pass of at most 6 KiB in which a wavefront meets a
 * corrupt line goes out as it came; the wavefront stores nothing after it.
 * Where the wavefronts of a workgroup walk a run as a team, the others finish
 * the pass they are in, and the stream's counters stay where they were.) helix_a2a_init_workspace on row 0 (with the other rows)
 * makes the workspace usable again. The calls themselves return at launch, so
 * a caller learns of a failure from helix_a2a_device_status, or at once in
 * checked mode:
 *
 * helix_a2a_set_checked_mode(1): every exchange call waits for its stream and
 * reads the status word before it returns, and returns HELIX_A2A_ERR_DEVICE
 * (message: the bits) if it is not zero. For bring-up and tests; it makes the
 * calls synchronous. A call on a stream that is being captured into a graph
 * cannot wait and skips the check. Default 0. The environment variable
 * HELIX_A2A_CHECKED=1 switches it on from the start.
 * The status word is one per device, and reading it clears it: with exchanges
 * in flight from several host threads (or on several workspaces) a reader may
 * take the bits another exchange raised. Checked mode and
 * helix_a2a_device_status are meant for one thread of control per device; the
 * broken word, which stops the exchanges behind a failure, is per workspace.
 */
void helix_a2a_set_checked_mode(int enabled);

/*
 * Upper bound, in microseconds, of any single in-kernel wait (receiver line
 * poll, sender FIFO-room wait). Default 2 000 000. Tests of the time-out path
 * set a tiny value so that every kernel still runs to completion.
 */
void helix_a2a_set_spin_limit_us(uint64_t microseconds);

/*
 * 0 (default): a loopback call whose per-FIFO traffic exceeds the four FIFO
 * entries is split into stream-ordered rounds. 1: it is issued as one launch
 * and senders wait in-kernel for receivers to release entries; accepted only
 * when the whole grid is co-resident.
 */
void helix_a2a_set_single_round(int enabled);

/*
 * How much of a stream's run one wavefront takes (process-wide; takes effect
 * with the next call). A run can be shared by up to 16 wavefronts per
 * direction, each with a step counter of its own in the stream's counter
 * blocks.
 *   -1 (default)  share runs longer than 6 units per lane (6 KiB), but only
 *                 while the launch leaves wavefront slots of the device free:
 *                 few streams with long runs are spread over the device, a
 *                 launch that fills it anyway is left alone
 *    0            never: one wavefront per stream however long its runs (the
 *                 reference's shape, one warp per stream,
 *                 csrc/helix_alltoall.cu:315-330)
 *    1..6         always share runs longer than that many units per lane
 * The send and the receive half of one exchange must run under the same
 * setting. No counterpart in the reference. Returns 0 or
 * HELIX_A2A_ERR_INVALID_ARGUMENT.
 */
int helix_a2a_set_units_per_wavefront(int units);

/*
 * Teams (process-wide; takes effect with the next call). In a launch that
 * keeps one wavefront per stream and direction, the wavefronts of a workgroup
 * can walk one stream's run together, each a slice of it: only the first of
 * them touches the stream's counters and hands the step to the others through
 * LDS, so the same bytes move in more, shorter wavefronts without any more
 * counter traffic, and the two halves of an exchange may differ in it.
 *   -1 (default)  runs of three or more passes (more than 12 units per lane)
 *                 in a launch whose wavefronts queue for slots: one pass per
 *                 wavefront, at most 8 wavefronts
 *    0            never
 *    1..6         always, with at most that many units per lane and wavefront
 * No counterpart in the reference, which keeps one warp per stream whatever
 * its length (csrc/helix_alltoall.cu:315-334). Returns 0 or
 * HELIX_A2A_ERR_INVALID_ARGUMENT.
 */
int helix_a2a_set_team_units(int units);

/* thread-local message of the most recent failure on this thread ("" if none) */
const char* helix_a2a_last_error(void);

/* "major.minor.patch" of the library */
const char* helix_a2a_version(void);

#ifdef __cplusplus
}
#endif

#endif /* HELIX_A2A_H_ */
