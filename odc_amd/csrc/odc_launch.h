// odc_launch.h — what the host side of libodc_hip.so hands to its device side.
//
// The library is two translation units. odc_host.cpp is plain C++ (no HIP header): the C ABI,
// the symmetric arena, argument validation and launch planning. odc_kernels.hip holds the gfx950
// kernels and the few runtime calls (device queries, the one hipMalloc, the launches). They meet
// in this header: the per-launch descriptors, which travel BY VALUE in the kernel-argument
// segment, and the functions of namespace odc_device. A second implementation of odc_device that
// has no device (tests/cpu/no_device.cpp) lets the host side be built with g++ and run under
// AddressSanitizer / UBSan on bookkeeping-only and dry-run arenas.
#ifndef ODC_LAUNCH_H_
#define ODC_LAUNCH_H_

#include <stdint.h>

#include "odc_tiles.h"

namespace odc_launch {

using odc_tiles::kMaxItems;
using odc_tiles::TileTable;

// One record per item, read with scalar loads by the workgroup that works on the item.
struct GatherDesc {
  uint8_t* dst;
  uint64_t src_off;
  uint64_t seg_bytes;
};
struct GatherLaunch {
  TileTable tt;
  const uint8_t* base;  // arena base (rank 0 region)
  uint64_t rank_stride;
  GatherDesc item[kMaxItems];
};

struct CastGatherDesc {
  uint8_t* dst;         // where rank 0's converted segment goes
  uint64_t dst_stride;  // bytes from one rank's converted segment to the next rank's
  uint64_t src_off;
  uint64_t seg_elems;
};
struct CastGatherLaunch {
  TileTable tt;
  const uint8_t* base;
  uint64_t rank_stride;
  CastGatherDesc item[kMaxItems];
};

struct AccumDesc {
  const uint8_t* grad;
  uint64_t grad_elems;
  uint64_t acc_off;
  uint64_t seg_elems;
};
struct AccumLaunch {
  TileTable tt;
  uint8_t* base;
  uint64_t rank_stride;
  AccumDesc item[kMaxItems];
};

struct ClearDesc {
  uint64_t off;
  uint64_t seg_bytes;
};
struct ClearLaunch {
  TileTable tt;
  uint8_t* base;
  uint64_t rank_stride;
  ClearDesc item[kMaxItems];
};

struct PublishDesc {
  uint8_t* out;  // may be null: divide in place only
  uint64_t acc_off;
  uint64_t seg_elems;
};
struct PublishLaunch {  // one rank's region only: tt.world == 1
  TileTable tt;
  uint8_t* region;      // base of the publishing rank's region
  float divisor;
  float reciprocal;     // exact 1 / divisor when divide == 2
  uint32_t divide;      // 0: leave the accumulation untouched, 1: divide, 2: multiply by reciprocal
  PublishDesc item[kMaxItems];
};
static_assert(sizeof(GatherLaunch) <= 4096 && sizeof(AccumLaunch) <= 4096 && sizeof(PublishLaunch) <= 4096 &&
                  sizeof(CastGatherLaunch) <= 4096 && sizeof(ClearLaunch) <= 4096,
              "launch descriptors must fit the kernel-argument segment");

}  // namespace odc_launch

// The device side. Every function returns 0 or a runtime error code that error_string() names;
// dtype arguments are odc_dtype codes.
namespace odc_device {

struct Properties {
  int n_cu;            // compute units
  int lds_per_cu;      // bytes of LDS per compute unit
  int lds_per_wg_max;  // most LDS one workgroup may claim
};

int get_current(int* device);
int set_current(int device);
int properties(int device, Properties* out);
int allocate(void** ptr, uint64_t bytes);  // on the current device
int release(void* ptr);                    // waits for the current device, then frees
bool is_out_of_memory(int code);
const char* error_string(int code);

// Which dtype pairs have a kernel: (gradient, accumulation), (shard, output), (accumulation, output).
bool has_accum(int grad_dtype, int acc_dtype);
bool has_cast_gather(int src_dtype, int dst_dtype);
bool has_publish(int acc_dtype, int out_dtype);

// One launch of `grid` workgroups on `stream`, each claiming `lds_bytes` of LDS it never touches
// (a residency cap; 0 = none). The workgroup size belongs to the kernel.
int launch_gather(const odc_launch::GatherLaunch& launch, uint32_t grid, uint32_t lds_bytes, void* stream);
int launch_cast_gather(int src_dtype, int dst_dtype, const odc_launch::CastGatherLaunch& launch, uint32_t grid,
                       uint32_t lds_bytes, void* stream);
int launch_accum(int grad_dtype, int acc_dtype, bool store, const odc_launch::AccumLaunch& launch, uint32_t grid,
                 uint32_t lds_bytes, void* stream);
int launch_clear(const odc_launch::ClearLaunch& launch, uint32_t grid, void* stream);
int launch_publish(int acc_dtype, int out_dtype, const odc_launch::PublishLaunch& launch, uint32_t grid,
                   uint32_t lds_bytes, void* stream);

}  // namespace odc_device

#endif  // ODC_LAUNCH_H_
