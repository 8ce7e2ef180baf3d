/*
 * Plain-C client of libodc_hip.so: proves that include/odc_hip.h is a C header and that the
 * library is usable without Python or torch. Builds with
 *   hipcc -x c -std=c11 -I include tests/c_abi/abi_check.c -L odc_amd/csrc -lodc_hip -o tests/c_abi/abi_check
 * and exits 0 after checking, on the current GPU, W=5 virtual ranks with an odd shard size:
 *   gather            against memcmp of the shards,
 *   scatter-accumulate (bf16 -> fp32, two calls, zero-padded gradient) against a scalar loop,
 *   clear             against zero,
 *   error codes       for bad arguments.
 */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "odc_hip.h"

#define CHECK(cond)                                                        \
  do {                                                                     \
    if (!(cond)) {                                                         \
      fprintf(stderr, "FAILED %s:%d: %s (%s)\n", __FILE__, __LINE__, #cond, odc_last_error()); \
      return 1;                                                            \
    }                                                                      \
  } while (0)

static float widen(uint16_t b) {
  uint32_t u = (uint32_t)b << 16;
  float f;
  memcpy(&f, &u, 4);
  return f;
}

int main(void) {
  enum { W = 5, S = 10007 };
  CHECK(odc_abi_version() == ODC_HIP_ABI_VERSION);
  odc_arena* arena = NULL;
  CHECK(odc_arena_create(0, 1024, 0, &arena) == ODC_ERR_INVALID);
  CHECK(odc_arena_create(W, 1u << 20, 0, &arena) == ODC_OK);
  uint64_t shard_off = 0, acc_off = 0, too_big = 0;
  CHECK(odc_arena_alloc(arena, S * 2, &shard_off) == ODC_OK);
  CHECK(odc_arena_alloc(arena, S * 4, &acc_off) == ODC_OK);
  CHECK(odc_arena_alloc(arena, 1u << 21, &too_big) == ODC_ERR_NOMEM);

  /* shards: rank r, element i holds bf16 bits of a small integer-valued pattern */
  uint16_t* host_shards = (uint16_t*)malloc((size_t)W * S * 2);
  for (int r = 0; r < W; ++r)
    for (int i = 0; i < S; ++i) host_shards[(size_t)r * S + i] = (uint16_t)(0x3f80 + ((r * 131 + i * 7) & 0x7f));
  for (int r = 0; r < W; ++r) {
    void* p = odc_arena_ptr(arena, (uint32_t)r, shard_off);
    CHECK(p != NULL);
    CHECK(hipMemcpy(p, host_shards + (size_t)r * S, S * 2, hipMemcpyHostToDevice) == hipSuccess);
    uint32_t rank = 99;
    uint64_t off = 0, inner = 0;
    CHECK(odc_arena_locate(arena, (char*)p + 6, &rank, &off, &inner) == ODC_OK);
    CHECK(rank == (uint32_t)r && off == shard_off && inner == 6);
  }

  /* gather */
  void* full = NULL;
  CHECK(hipMalloc(&full, (size_t)W * S * 2) == hipSuccess);
  odc_gather_item gi = {full, shard_off, S * 2};
  CHECK(odc_gather(arena, &gi, 1, W, NULL) == ODC_ERR_INVALID); /* first_rank out of range */
  CHECK(odc_gather(arena, &gi, 1, 3, NULL) == ODC_OK);
  uint16_t* host_full = (uint16_t*)malloc((size_t)W * S * 2);
  CHECK(hipMemcpy(host_full, full, (size_t)W * S * 2, hipMemcpyDeviceToHost) == hipSuccess);
  CHECK(memcmp(host_full, host_shards, (size_t)W * S * 2) == 0);

  /* clear, then two scatter-accumulates of a gradient that is 11 elements short of W*S */
  odc_span span = {acc_off, S * 4};
  CHECK(odc_clear(arena, &span, 1, NULL) == ODC_OK);
  const uint64_t valid = (uint64_t)W * S - 11;
  odc_accum_item ai = {full, valid, acc_off, S};
  CHECK(odc_scatter_accumulate(arena, &ai, 1, ODC_DTYPE_BF16, 7, NULL) == ODC_ERR_INVALID);
  CHECK(odc_scatter_accumulate(arena, &ai, 1, ODC_DTYPE_BF16, ODC_DTYPE_F32, NULL) == ODC_OK);
  CHECK(odc_scatter_accumulate(arena, &ai, 1, ODC_DTYPE_BF16, ODC_DTYPE_F32, NULL) == ODC_OK);
  CHECK(hipDeviceSynchronize() == hipSuccess);
  float* host_acc = (float*)malloc(S * 4);
  for (int r = 0; r < W; ++r) {
    CHECK(hipMemcpy(host_acc, odc_arena_ptr(arena, (uint32_t)r, acc_off), S * 4, hipMemcpyDeviceToHost) == hipSuccess);
    for (int i = 0; i < S; ++i) {
      const uint64_t g = (uint64_t)r * S + i;
      const float x = g < valid ? widen(host_full[g]) : 0.0f;
      volatile float want = 0.0f + x;
      want = want + x;
      CHECK(memcmp(&host_acc[i], (const void*)&want, 4) == 0);
    }
  }
  /* scatter-store over the stale sums: as if cleared first, then accumulated once */
  CHECK(odc_scatter_store(arena, &ai, 1, ODC_DTYPE_BF16, ODC_DTYPE_F32, NULL) == ODC_OK);
  CHECK(hipDeviceSynchronize() == hipSuccess);
  for (int r = 0; r < W; ++r) {
    CHECK(hipMemcpy(host_acc, odc_arena_ptr(arena, (uint32_t)r, acc_off), S * 4, hipMemcpyDeviceToHost) == hipSuccess);
    for (int i = 0; i < S; ++i) {
      const uint64_t g = (uint64_t)r * S + i;
      volatile float want = 0.0f + (g < valid ? widen(host_full[g]) : 0.0f);
      CHECK(memcmp(&host_acc[i], (const void*)&want, 4) == 0);
    }
  }
  CHECK(odc_clear(arena, &span, 1, NULL) == ODC_OK);
  CHECK(hipDeviceSynchronize() == hipSuccess);
  for (int r = 0; r < W; ++r) {
    CHECK(hipMemcpy(host_acc, odc_arena_ptr(arena, (uint32_t)r, acc_off), S * 4, hipMemcpyDeviceToHost) == hipSuccess);
    for (int i = 0; i < S; ++i) CHECK(host_acc[i] == 0.0f);
  }
  odc_arena_info info;
  CHECK(odc_arena_get_info(arena, &info) == ODC_OK);
  CHECK(info.world_size == W && info.n_allocations == 2);
  CHECK(odc_arena_free(arena, shard_off) == ODC_OK);
  CHECK(odc_arena_free(arena, shard_off) == ODC_ERR_NOT_FOUND);
  CHECK(hipFree(full) == hipSuccess);
  CHECK(odc_arena_destroy(arena) == ODC_OK);
  free(host_shards);
  free(host_full);
  free(host_acc);
  printf("abi_check ok\n");
  return 0;
}
