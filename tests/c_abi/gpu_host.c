/* A plain C host that drives the exchange on the GPU through include/helix_a2a.h and the HIP runtime's C
 * API alone -- no torch, no Python: what a replacement of the reference's libtorch binding
 * (csrc/torch_binding.cpp:131-172) does between its tensor checks and its return. It allocates the
 * workspace and the tensors with hipMalloc, initialises every row, runs the loopback exchange, the two
 * split halves and the entry point with the built-in workspace on integer-coded payloads, and compares
 * every element with the closed form out[r][e, s, i] = in[s][e, r, i]. Built by tests/helix_testing.py
 * (gcc, C99); run by tests/test_gpu_exchange.py. Exit status 0 when everything holds. */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "helix_a2a.h"

#define CP 4
#define ENTRIES 37
#define X 576 /* 2-byte elements per partial_o row: 1152 bytes */
#define S 12  /* 4-byte elements per softmax_stats row */

static int failures = 0;
#define CHECK(cond)                                      \
  do {                                                   \
    if (!(cond)) {                                       \
      printf("FAILED: %s (line %d)\n", #cond, __LINE__); \
      failures++;                                        \
    }                                                    \
  } while (0)
#define HIP_OK(call)                                                                   \
  do {                                                                                 \
    hipError_t e_ = (call);                                                            \
    if (e_ != hipSuccess) {                                                            \
      printf("FAILED: %s: %s (line %d)\n", #call, hipGetErrorString(e_), __LINE__);    \
      return 2;                                                                        \
    }                                                                                  \
  } while (0)
#define A2A_OK(call)                                                                   \
  do {                                                                                 \
    int rc_ = (call);                                                                  \
    if (rc_ != HELIX_A2A_OK) {                                                         \
      printf("FAILED: %s -> %d: %s (line %d)\n", #call, rc_, helix_a2a_last_error(), __LINE__); \
      return 3;                                                                        \
    }                                                                                  \
  } while (0)

static uint16_t code_o(int rank, int e, int p, int i, int salt) { return (uint16_t)(rank * 4099 + e * 523 + p * 67 + i + salt); }
static uint32_t code_s(int rank, int e, int p, int i, int salt) {
  return ((uint32_t)rank << 24) | ((uint32_t)e << 12) | ((uint32_t)p << 8) | (uint32_t)(i + salt);
}

static uint16_t* host_o[CP];
static uint32_t* host_s[CP];
static void *dev_o[CP], *dev_s[CP], *out_o[CP], *out_s[CP];
static const size_t bytes_o = (size_t)ENTRIES * CP * X * 2, bytes_s = (size_t)ENTRIES * CP * S * 4;

static int upload(int salt) {
  int r, e, p, i;
  for (r = 0; r < CP; ++r) {
    for (e = 0; e < ENTRIES; ++e)
      for (p = 0; p < CP; ++p) {
        for (i = 0; i < X; ++i) host_o[r][((size_t)e * CP + p) * X + i] = code_o(r, e, p, i, salt);
        for (i = 0; i < S; ++i) host_s[r][((size_t)e * CP + p) * S + i] = code_s(r, e, p, i, salt);
      }
    HIP_OK(hipMemcpy(dev_o[r], host_o[r], bytes_o, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dev_s[r], host_s[r], bytes_s, hipMemcpyHostToDevice));
    HIP_OK(hipMemset(out_o[r], 0xEE, bytes_o));
    HIP_OK(hipMemset(out_s[r], 0xEE, bytes_s));
  }
  return 0;
}

/* out[r][e, s, i] == in[s][e, r, i] for every element of both fields */
static int verify(int salt, const char* what) {
  int r, e, s, i;
  long bad = 0;
  for (r = 0; r < CP; ++r) {
    HIP_OK(hipMemcpy(host_o[r], out_o[r], bytes_o, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(host_s[r], out_s[r], bytes_s, hipMemcpyDeviceToHost));
    for (e = 0; e < ENTRIES; ++e)
      for (s = 0; s < CP; ++s) {
        for (i = 0; i < X; ++i) bad += host_o[r][((size_t)e * CP + s) * X + i] != code_o(s, e, r, i, salt);
        for (i = 0; i < S; ++i) bad += host_s[r][((size_t)e * CP + s) * S + i] != code_s(s, e, r, i, salt);
      }
  }
  printf("%s: %ld wrong element(s)\n", what, bad);
  if (bad) failures++;
  return 0;
}

int main(void) {
  helix_a2a_params_t params[CP];
  hipStream_t stream;
  uint64_t* workspace = NULL;
  uint32_t status = 77;
  int r, rc;
  const int max_channels = helix_a2a_max_channel_count(CP, 0); /* asks the device */
  const int64_t row_bytes = helix_a2a_workspace_size_per_rank(CP, 0);

  CHECK(max_channels >= 1 && row_bytes == (int64_t)(524288 + 512) * CP * max_channels);
  HIP_OK(hipStreamCreate(&stream));
  HIP_OK(hipMalloc((void**)&workspace, (size_t)row_bytes * CP));
  for (r = 0; r < CP; ++r) {
    host_o[r] = (uint16_t*)malloc(bytes_o);
    host_s[r] = (uint32_t*)malloc(bytes_s);
    HIP_OK(hipMalloc(&dev_o[r], bytes_o));
    HIP_OK(hipMalloc(&dev_s[r], bytes_s));
    HIP_OK(hipMalloc(&out_o[r], bytes_o));
    HIP_OK(hipMalloc(&out_s[r], bytes_s));
  }
  memset(params, 0, sizeof(params));
  for (r = 0; r < CP; ++r) {
    helix_a2a_params_t* p = &params[r];
    p->send_fields[0].data = dev_o[r];
    p->recv_fields[0].data = out_o[r];
    p->send_fields[1].data = dev_s[r];
    p->recv_fields[1].data = out_s[r];
    p->send_fields[0].element_count = p->recv_fields[0].element_count = X;
    p->send_fields[0].element_size = p->recv_fields[0].element_size = 2;
    p->send_fields[0].stride_bytes = p->recv_fields[0].stride_bytes = X * 2;
    p->send_fields[1].element_count = p->recv_fields[1].element_count = S;
    p->send_fields[1].element_size = p->recv_fields[1].element_size = 4;
    p->send_fields[1].stride_bytes = p->recv_fields[1].stride_bytes = S * 4;
    p->entry_count = ENTRIES;
    p->workspace = workspace;
    p->workspace_stride_u64 = (uint64_t)row_bytes / 8;
    p->cp_rank = r;
    p->cp_size = CP;
    p->channel_count = 0;
    p->max_channel_count = max_channels;
  }
  for (r = 0; r < CP; ++r) A2A_OK(helix_a2a_init_workspace(workspace + (size_t)r * (row_bytes / 8), CP, 0, stream));

  /* 1. all ranks in one launch, twice (the FIFO entries rotate) */
  if (upload(1)) return 2;
  A2A_OK(helix_a2a_alltoall_loopback(params, CP, stream));
  HIP_OK(hipStreamSynchronize(stream));
  if (verify(1, "loopback")) return 2;
  if (upload(2)) return 2;
  A2A_OK(helix_a2a_alltoall_loopback(params, CP, stream));
  HIP_OK(hipStreamSynchronize(stream));
  if (verify(2, "loopback again")) return 2;

  /* 2. the halves of the per-rank call: every rank's send half, then the receive half of all */
  if (upload(3)) return 2;
  for (r = 0; r < CP; ++r) A2A_OK(helix_a2a_alltoall_send(&params[r], 1, stream));
  A2A_OK(helix_a2a_alltoall_recv(params, CP, stream));
  HIP_OK(hipStreamSynchronize(stream));
  if (verify(3, "send halves + receive half")) return 2;

  /* 3. a descriptor that disagrees with the device is refused, nothing is launched */
  for (r = 0; r < CP; ++r) params[r].max_channel_count += 1;
  rc = helix_a2a_alltoall_loopback(params, CP, stream);
  CHECK(rc == HELIX_A2A_ERR_INVALID_ARGUMENT && strstr(helix_a2a_last_error(), "max_channel_count") != NULL);
  for (r = 0; r < CP; ++r) params[r].max_channel_count -= 1;

  /* 4. the entry point that allocates nothing: same exchange through the library's built-in workspace */
  if (upload(4)) return 2;
  for (r = 0; r < CP; ++r) {
    params[r].workspace = NULL;
    params[r].workspace_stride_u64 = 0;
    params[r].max_channel_count = 0;
  }
  A2A_OK(helix_a2a_alltoall_loopback_static(params, CP, 0, stream));
  HIP_OK(hipStreamSynchronize(stream));
  if (verify(4, "loopback through the built-in workspace")) return 2;

  A2A_OK(helix_a2a_device_status(&status, stream));
  CHECK(status == 0);

  for (r = 0; r < CP; ++r) {
    hipFree(dev_o[r]); hipFree(dev_s[r]); hipFree(out_o[r]); hipFree(out_s[r]);
    free(host_o[r]); free(host_s[r]);
  }
  hipFree(workspace);
  hipStreamDestroy(stream);
  printf("%s: %d failure(s)\n", failures ? "gpu_host FAILED" : "gpu_host ok", failures);
  return failures ? 1 : 0;
}
