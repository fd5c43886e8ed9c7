/*
 * helix_ref_model.c -- CPU restatement of the reference's Helix all-to-all.
 *
 * TEST INFRASTRUCTURE ONLY. This file is the checker the GPU path is compared
 * with (tests/, the smoke test, and the cpu_baseline leg of bench.py). Nothing
 * in the product path may call, link or load it.
 *
 * It re-states, in plain sequential C, what the reference's CUDA kernel does
 * with a message on its way from a sender rank to a receiver rank:
 *
 *   sizes          csrc/helix_alltoall.cu:292-309, csrc/ll128_proto.cuh:148-153
 *   geometry       csrc/helix_alltoall.cu:61-75,194-242
 *   workspace      csrc/helix_alltoall.cu:590-614 (size), :629-644 (init)
 *   channel count  csrc/helix_alltoall.cu:486-535
 *   LL128 pack     csrc/ll128_proto.cuh:73-106
 *   LL128 check    csrc/ll128_proto.cuh:30-71
 *   LL128 unpack   csrc/ll128_proto.cuh:108-139
 *   sender loop    csrc/helix_alltoall.cu:360-412
 *   receiver loop  csrc/helix_alltoall.cu:413-473
 *
 * The reference runs one warp per (peer, channel, direction) on every rank,
 * concurrently. Here every such warp is a small state machine that advances
 * one message at a time; a scheduler interleaves them until all are done, so
 * the FIFO back-pressure (sender waits for `tail`) and the receiver's flag
 * polling are exercised as real blocking conditions. Warp-lane parallelism is
 * written out as loops over the 128-byte blocks the lanes would own.
 *
 * The byte layout this model produces inside the FIFOs is the REFERENCE's
 * (rotating flag slot, tail blocks). The GPU build uses a different line
 * format on purpose; only the exchanged tensors are compared.
 *
 * Pinned by tests/test_oracle.py: closed form recv_r[e,s,:] == send_s[e,r,:]
 * (tests/test_alltoall.py:314-329 of the reference), the fill vectors of
 * tests/test_mnnvl.py:177-213, the size closed form of tests/test_phase2.py:13-35,
 * the init pattern of tests/test_phase2.py:48-62, hand-derived known-answer
 * blocks for pack, flag positions, pack/unpack round trips, and schedule
 * independence.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define REF_FIFO_DEPTH 4
#define REF_FIFO_ENTRY_BYTES (128 * 1024)
#define REF_BLOCK_BYTES 128
#define REF_WORDS_PER_BLOCK 16
#define REF_FIFO_ENTRY_BLOCKS (REF_FIFO_ENTRY_BYTES / REF_BLOCK_BYTES)
#define REF_FIFO_TOTAL_BYTES (REF_FIFO_ENTRY_BYTES * REF_FIFO_DEPTH)
#define REF_INFO_BYTES 256 /* sizeof(HelixFifoInfo): {int64 head; int64 tail} aligned to 256 */
#define REF_MAX_GROUPS_PER_BLOCK 8

typedef struct ref_field {
  uint8_t* data;
  int32_t element_count;
  int32_t element_size;
  int32_t stride; /* bytes */
} ref_field_t;

typedef struct ref_params {
  ref_field_t send_fields[2];
  ref_field_t recv_fields[2];
  int32_t entry_count;
  uint8_t* workspace;
  uint64_t workspace_stride_bytes;
  int32_t cp_rank;
  int32_t cp_size;
  int32_t channel_count; /* 0 = derive */
  int32_t max_channel_count;
} ref_params_t;

static int ceil_div(int a, int b) { return (a + b - 1) / b; }
static int align_up(int v, int a) { return ceil_div(v, a) * a; }

/* ---- sizes ------------------------------------------------------------- */

/* csrc/helix_alltoall.cu:292-298 */
int ref_unpacked_size(int field0_bytes, int field1_bytes) {
  return align_up(align_up(field0_bytes, 16) + align_up(field1_bytes, 16), REF_BLOCK_BYTES);
}

/* csrc/ll128_proto.cuh:148-153: one tail block per 15 data blocks */
int ref_proto_size(int packed_bytes) {
  int tail = (packed_bytes + 15 * 128 - 1) / (15 * 128) * 128;
  return packed_bytes + tail;
}

/* csrc/helix_alltoall.cu:590-603 */
int ref_max_channel_count(int cp_size, int sm_count) {
  int blocks_per_channel = 2 * ceil_div(cp_size, REF_MAX_GROUPS_PER_BLOCK);
  int c = sm_count / blocks_per_channel;
  return c > 1 ? c : 1;
}

/* csrc/helix_alltoall.cu:605-614 */
uint64_t ref_workspace_size(int cp_size, int sm_count) {
  uint64_t max_ch = (uint64_t)ref_max_channel_count(cp_size, sm_count);
  uint64_t fifo = (uint64_t)REF_FIFO_TOTAL_BYTES * cp_size * max_ch;
  uint64_t info = (uint64_t)REF_INFO_BYTES * cp_size * max_ch;
  return fifo + info + info;
}

/* csrc/helix_alltoall.cu:629-644 */
void ref_init_workspace(uint8_t* local_row, int cp_size, int sm_count) {
  uint64_t max_ch = (uint64_t)ref_max_channel_count(cp_size, sm_count);
  uint64_t fifo = (uint64_t)REF_FIFO_TOTAL_BYTES * cp_size * max_ch;
  uint64_t info = (uint64_t)REF_INFO_BYTES * cp_size * max_ch;
  memset(local_row, 0xFF, fifo);
  memset(local_row + fifo, 0, info + info);
}

/* csrc/helix_alltoall.cu:486-535. Returns the channel count; *groups_out gets
 * the warps per block. Returns -1 when even one group does not fit. */
int ref_channel_and_group_count(int cp_size, int field0_bytes, int field1_bytes, int sm_count,
                                int max_dynamic_smem, int* groups_out) {
  int unpacked = ref_unpacked_size(field0_bytes, field1_bytes);
  int proto = ref_proto_size(unpacked);
  int single = unpacked > proto ? unpacked : proto;
  int groups = cp_size < REF_MAX_GROUPS_PER_BLOCK ? cp_size : REF_MAX_GROUPS_PER_BLOCK;
  while (groups > 0 && single * groups > max_dynamic_smem) groups--;
  if (groups == 0) return -1;
  if (groups_out) *groups_out = groups;
  int blocks_per_channel = 2 * ceil_div(cp_size, groups);
  int c = sm_count / blocks_per_channel;
  return c > 1 ? c : 1;
}

/* ---- LL128, reference layout ----------------------------------------------
 * `shm` holds P packed data blocks followed by ceil(P/15) tail blocks, 16
 * words each. `base` is the index of block 0 inside its FIFO entry; the flag
 * of block b sits in word (base + b) % 16.                                   */

static int tail_slot(int j, int tail_flag_slot) { return j >= tail_flag_slot ? j + 1 : j; }

/* csrc/ll128_proto.cuh:73-106 */
void ref_proto_pack(uint64_t* shm, uint64_t step, int P, int base) {
  int groups = ceil_div(P, 15);
  for (int q = 0; q < groups; ++q) {
    int tail_block = P + q;
    int tail_flag_slot = (base + tail_block) % REF_WORDS_PER_BLOCK;
    uint64_t* tail = shm + (size_t)tail_block * REF_WORDS_PER_BLOCK;
    for (int j = 0; j < 15; ++j) { /* the 15 worker lanes of a half warp */
      int b = q * 15 + j;
      uint64_t moved = step; /* lanes past the last block fill with the step value */
      if (b < P) {
        uint64_t* flag = shm + (size_t)b * REF_WORDS_PER_BLOCK + (base + b) % REF_WORDS_PER_BLOCK;
        moved = *flag;
        *flag = step;
      }
      tail[tail_slot(j, tail_flag_slot)] = moved;
    }
    tail[tail_flag_slot] = step; /* lane 15 of the half warp */
  }
}

/* csrc/ll128_proto.cuh:108-139 */
void ref_proto_unpack(uint64_t* shm, int P, int base) {
  int groups = ceil_div(P, 15);
  for (int q = 0; q < groups; ++q) {
    int tail_block = P + q;
    int tail_flag_slot = (base + tail_block) % REF_WORDS_PER_BLOCK;
    const uint64_t* tail = shm + (size_t)tail_block * REF_WORDS_PER_BLOCK;
    for (int j = 0; j < 15; ++j) {
      int b = q * 15 + j;
      if (b < P) {
        shm[(size_t)b * REF_WORDS_PER_BLOCK + (base + b) % REF_WORDS_PER_BLOCK] = tail[tail_slot(j, tail_flag_slot)];
      }
    }
  }
}

/* csrc/ll128_proto.cuh:30-71 with USE_FINISH = false: number of blocks,
 * counted from `loaded`, whose flag already equals `step` (the warp looks at
 * 32 blocks at a time and stops at the first one that is not valid, which is
 * the length of the valid prefix). */
int ref_check_received(const uint64_t* shm, uint64_t step, int count, int base, int loaded) {
  int valid = 0;
  for (int idx = loaded; idx < count; ++idx) {
    uint64_t v = shm[(size_t)idx * REF_WORDS_PER_BLOCK + (base + idx) % REF_WORDS_PER_BLOCK];
    if (v != step) break;
    valid++;
  }
  return valid;
}

/* ---- workspace geometry (csrc/helix_alltoall.cu:194-242) ------------------- */

static uint8_t* fifo_base(const ref_params_t* p, int sender, int receiver, int channel) {
  uint8_t* row = p->workspace + (uint64_t)receiver * p->workspace_stride_bytes;
  return row + ((uint64_t)sender * p->max_channel_count + channel) * REF_FIFO_TOTAL_BYTES;
}
static int64_t* sender_info(const ref_params_t* p, int sender, int receiver, int channel) {
  uint8_t* row = p->workspace + (uint64_t)sender * p->workspace_stride_bytes;
  uint64_t off = (uint64_t)REF_FIFO_TOTAL_BYTES * p->cp_size * p->max_channel_count;
  off += ((uint64_t)receiver * p->max_channel_count + channel) * REF_INFO_BYTES;
  return (int64_t*)(row + off); /* [0] = head, [1] = tail */
}
static int64_t* receiver_info(const ref_params_t* p, int sender, int receiver, int channel) {
  uint8_t* row = p->workspace + (uint64_t)receiver * p->workspace_stride_bytes;
  uint64_t off = (uint64_t)REF_FIFO_TOTAL_BYTES * p->cp_size * p->max_channel_count;
  off += (uint64_t)REF_INFO_BYTES * p->cp_size * p->max_channel_count;
  off += ((uint64_t)sender * p->max_channel_count + channel) * REF_INFO_BYTES;
  return (int64_t*)(row + off);
}

/* ---- one warp = one state machine --------------------------------------------- */

typedef struct warp_state {
  const ref_params_t* params; /* descriptor of the rank this warp runs on */
  int is_sender;
  int sender, receiver, channel;
  int next_entry;     /* entry index the warp handles next */
  int entry_index;    /* FIFO entry in use, -1 before the first */
  int block_base;     /* next free block in that entry */
  int64_t counter;    /* head (sender) or tail (receiver) */
  int64_t seen_tail;  /* sender's cached tail */
  int waiting_room;   /* sender rolled over and waits for the receiver */
  int need_release;   /* receiver owes a tail publication */
  int loaded;         /* receiver: valid blocks of the current message so far */
  int in_message;     /* receiver: current message already located */
  int finished;
  uint64_t* shm;
} warp_state_t;

typedef struct msg_sizes {
  int f0, f1, packed_blocks, proto_blocks, shm_bytes;
} msg_sizes_t;

static msg_sizes_t sizes_of(const ref_params_t* p) {
  msg_sizes_t m;
  m.f0 = p->send_fields[0].element_count * p->send_fields[0].element_size;
  m.f1 = p->send_fields[1].element_count * p->send_fields[1].element_size;
  int unpacked = ref_unpacked_size(m.f0, m.f1);
  int proto = ref_proto_size(unpacked);
  m.packed_blocks = unpacked / REF_BLOCK_BYTES;
  m.proto_blocks = proto / REF_BLOCK_BYTES;
  m.shm_bytes = unpacked > proto ? unpacked : proto;
  return m;
}

/* Sender, one message (csrc/helix_alltoall.cu:368-408). Returns 1 on progress. */
static int sender_step(warp_state_t* w, int run_channels) {
  const ref_params_t* p = w->params;
  msg_sizes_t m = sizes_of(p);
  int64_t* info = sender_info(p, w->sender, w->receiver, w->channel);
  if (w->finished) return 0;
  if (w->next_entry >= p->entry_count) {
    /* :409-412 -- block_base starts at the entry size, so the counter moves
     * even for a warp that had no entry to send */
    if (w->block_base > 0) {
      w->counter++;
      info[0] = w->counter;
    }
    w->finished = 1;
    return 1;
  }
  if (!w->waiting_room && w->block_base + m.proto_blocks > REF_FIFO_ENTRY_BLOCKS) {
    if (w->entry_index >= 0) {
      w->counter++;
      info[0] = w->counter;
    }
    w->entry_index = (int)(w->counter % REF_FIFO_DEPTH);
    w->block_base = 0;
    w->waiting_room = 1;
  }
  if (w->waiting_room) {
    if (w->seen_tail + REF_FIFO_DEPTH <= w->counter) w->seen_tail = info[1];
    if (w->seen_tail + REF_FIFO_DEPTH <= w->counter) return 0; /* FIFO full */
    w->waiting_room = 0;
  }
  int data_index = w->next_entry * p->cp_size + w->receiver;
  uint8_t* shm8 = (uint8_t*)w->shm;
  memset(shm8, 0, (size_t)m.shm_bytes);
  memcpy(shm8, p->send_fields[0].data + (size_t)data_index * p->send_fields[0].stride, (size_t)m.f0);
  memcpy(shm8 + m.f0, p->send_fields[1].data + (size_t)data_index * p->send_fields[1].stride, (size_t)m.f1);
  ref_proto_pack(w->shm, (uint64_t)w->counter, m.packed_blocks, w->block_base);
  uint8_t* entry = fifo_base(p, w->sender, w->receiver, w->channel) + (size_t)w->entry_index * REF_FIFO_ENTRY_BYTES;
  memcpy(entry + (size_t)w->block_base * REF_BLOCK_BYTES, shm8, (size_t)m.proto_blocks * REF_BLOCK_BYTES);
  w->block_base += m.proto_blocks;
  w->next_entry += run_channels;
  return 1;
}

/* Receiver, one message (csrc/helix_alltoall.cu:417-467). Returns 1 on progress. */
static int receiver_step(warp_state_t* w, int run_channels) {
  const ref_params_t* p = w->params;
  msg_sizes_t m = sizes_of(p);
  int64_t* rinfo = receiver_info(p, w->sender, w->receiver, w->channel);
  int64_t* sinfo = sender_info(p, w->sender, w->receiver, w->channel);
  if (w->finished) return 0;
  if (w->next_entry >= p->entry_count) {
    if (w->block_base > 0) { /* :468-472 */
      w->counter++;
      rinfo[1] = w->counter;
      sinfo[1] = w->counter;
    }
    w->finished = 1;
    return 1;
  }
  if (!w->in_message) {
    if (w->block_base + m.proto_blocks > REF_FIFO_ENTRY_BLOCKS) {
      if (w->entry_index >= 0) {
        w->counter++;
        w->need_release = 1;
      }
      w->entry_index = (int)(w->counter % REF_FIFO_DEPTH);
      w->block_base = 0;
    }
    w->in_message = 1;
    w->loaded = 0;
  }
  /* one turn of the polling loop :441-456 */
  uint8_t* entry = fifo_base(p, w->sender, w->receiver, w->channel) + (size_t)w->entry_index * REF_FIFO_ENTRY_BYTES;
  uint8_t* shm8 = (uint8_t*)w->shm;
  memcpy(shm8 + (size_t)w->loaded * REF_BLOCK_BYTES,
         entry + (size_t)(w->block_base + w->loaded) * REF_BLOCK_BYTES,
         (size_t)(m.proto_blocks - w->loaded) * REF_BLOCK_BYTES);
  int progressed = 0;
  if (w->need_release) {
    rinfo[1] = w->counter;
    sinfo[1] = w->counter;
    w->need_release = 0;
    progressed = 1;
  }
  int got = ref_check_received(w->shm, (uint64_t)w->counter, m.proto_blocks, w->block_base, w->loaded);
  w->loaded += got;
  if (w->loaded < m.proto_blocks) return progressed || got > 0;
  ref_proto_unpack(w->shm, m.packed_blocks, w->block_base);
  int data_index = w->next_entry * p->cp_size + w->sender;
  memcpy(p->recv_fields[0].data + (size_t)data_index * p->recv_fields[0].stride, shm8, (size_t)m.f0);
  memcpy(p->recv_fields[1].data + (size_t)data_index * p->recv_fields[1].stride, shm8 + m.f0, (size_t)m.f1);
  w->block_base += m.proto_blocks;
  w->next_entry += run_channels;
  w->in_message = 0;
  return 1;
}

/*
 * Run one alltoall call of all `cp_size` ranks (per_rank[r].cp_rank == r) that
 * share one workspace.
 *   schedule 0: round robin, every warp advances by at most one message per pass
 *   schedule 1: senders run until they block, then receivers, and so on
 * sm_count / max_dynamic_smem stand for the device the reference would run on.
 * Returns 0, or -1 bad arguments, -2 allocation failure, -3 no warp can move
 * (a deadlock, which the protocol must never reach).
 */
int ref_alltoall_all_ranks(const ref_params_t* per_rank, int cp_size, int sm_count, int max_dynamic_smem,
                           int schedule) {
  if (!per_rank || cp_size < 1) return -1;
  msg_sizes_t m = sizes_of(&per_rank[0]);
  int channels = per_rank[0].channel_count;
  if (channels <= 0)
    channels = ref_channel_and_group_count(cp_size, m.f0, m.f1, sm_count, max_dynamic_smem, NULL);
  if (channels <= 0 || channels > per_rank[0].max_channel_count) return -1;
  if (m.proto_blocks > REF_FIFO_ENTRY_BLOCKS) return -1;
  for (int r = 0; r < cp_size; ++r)
    if (per_rank[r].cp_rank != r || per_rank[r].cp_size != cp_size) return -1;

  size_t warps = (size_t)2 * cp_size * cp_size * channels;
  warp_state_t* w = (warp_state_t*)calloc(warps, sizeof(warp_state_t));
  if (!w) return -2;
  size_t n = 0;
  for (int dir = 0; dir < 2; ++dir)
    for (int rank = 0; rank < cp_size; ++rank)
      for (int peer = 0; peer < cp_size; ++peer)
        for (int ch = 0; ch < channels; ++ch) {
          warp_state_t* s = &w[n++];
          s->params = &per_rank[rank];
          s->is_sender = dir == 0;
          s->sender = s->is_sender ? rank : peer;   /* :334-335 */
          s->receiver = s->is_sender ? peer : rank;
          s->channel = ch;
          s->next_entry = ch;
          s->entry_index = -1;
          s->block_base = REF_FIFO_ENTRY_BLOCKS;    /* :353 */
          if (s->is_sender) {
            int64_t* info = sender_info(s->params, s->sender, s->receiver, ch);
            s->counter = info[0];                   /* :365-366 */
            s->seen_tail = info[1];
          } else {
            s->counter = receiver_info(s->params, s->sender, s->receiver, ch)[1]; /* :414 */
          }
          s->shm = (uint64_t*)malloc((size_t)m.shm_bytes);
          if (!s->shm) {
            for (size_t i = 0; i < n; ++i) free(w[i].shm);
            free(w);
            return -2;
          }
        }

  int rc = 0;
  for (;;) {
    size_t done = 0;
    int progress = 0;
    for (int phase = 0; phase < 2; ++phase) {
      for (size_t i = 0; i < warps; ++i) {
        warp_state_t* s = &w[i];
        if (schedule == 1 && s->is_sender != (phase == 0)) continue;
        if (schedule == 0 && phase == 1) continue;
        if (s->finished) continue;
        do {
          int moved = s->is_sender ? sender_step(s, channels) : receiver_step(s, channels);
          progress |= moved;
          if (!moved) break;
        } while (schedule == 1 && !s->finished);
      }
    }
    for (size_t i = 0; i < warps; ++i) done += (size_t)w[i].finished;
    if (done == warps) break;
    if (!progress) {
      rc = -3;
      break;
    }
  }
  for (size_t i = 0; i < warps; ++i) free(w[i].shm);
  free(w);
  return rc;
}
