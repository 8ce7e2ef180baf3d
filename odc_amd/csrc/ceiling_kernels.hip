// libodc_ceiling.so — the simplest kernels that move the same bytes as the product kernels, over
// flat arrays with no descriptors, no tile search and no edge handling: what this GPU's memory
// system sustains for each traffic mix. bench.py times them next to the product kernels and
// prints them as roofline.practical_ceiling. Measurement only; nothing in the package calls them.
//
//   read   : 16 B per lane per step, summed into a register          (read 1 B per byte)
//   write  : zeros                                                    (write 1 B per byte)
//   copy   : dst[i] = src[i]                                          (read 1 + write 1 per byte)
//   rmw    : acc[i] += widen(grad[i]), bf16 -> fp32                   (10 B per element)
//
// Same shapes as the product kernels: 256-thread workgroups with 4, or 512-thread workgroups
// with 2 (odc_ceiling_set_threads), independent 128-bit nontemporal loads per stream per lane
// before the first store, one 16 KiB tile per step, grid-stride.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr uint64_t kTileVecs = 1024;  // 16 KiB of the 16-byte stream per tile
int g_threads = 256;                  // workgroup size of the next launches: 256 (x4) or 512 (x2)

template <int kThreads, int kUnroll>
__global__ __launch_bounds__(kThreads) void read_kernel(const u32x4* src, uint64_t n_tiles, uint32_t* sink) {
  u32x4 sum = {0u, 0u, 0u, 0u};
  for (uint64_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
    const u32x4* s = src + t * kTileVecs + threadIdx.x;
    u32x4 v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) v[u] = __builtin_nontemporal_load(s + u * kThreads);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) sum ^= v[u];
  }
  if ((sum.x ^ sum.y ^ sum.z ^ sum.w) == 0x9e3779b9u) *sink = 1;  // keeps the loads alive
}

template <int kThreads, int kUnroll>
__global__ __launch_bounds__(kThreads) void write_kernel(u32x4* dst, uint64_t n_tiles) {
  const u32x4 zero = {0u, 0u, 0u, 0u};
  for (uint64_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
    u32x4* d = dst + t * kTileVecs + threadIdx.x;
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) d[u * kThreads] = zero;
  }
}

template <int kThreads, int kUnroll>
__global__ __launch_bounds__(kThreads) void copy_kernel(u32x4* dst, const u32x4* src, uint64_t n_tiles) {
  for (uint64_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
    const u32x4* s = src + t * kTileVecs + threadIdx.x;
    u32x4* d = dst + t * kTileVecs + threadIdx.x;
    u32x4 v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) v[u] = __builtin_nontemporal_load(s + u * kThreads);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) __builtin_nontemporal_store(v[u], d + u * kThreads);
  }
}

template <int kThreads, int kUnroll>
__global__ __launch_bounds__(kThreads) void rmw_kernel(f32x4* acc, const u32x2* grad, uint64_t n_tiles) {
  for (uint64_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
    f32x4* a = acc + t * kTileVecs + threadIdx.x;
    const u32x2* g = grad + t * kTileVecs + threadIdx.x;
    u32x2 gv[kUnroll];
    f32x4 av[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) gv[u] = __builtin_nontemporal_load(g + u * kThreads);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) av[u] = __builtin_nontemporal_load(a + u * kThreads);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      f32x4 x;
      x.x = __uint_as_float(gv[u].x << 16);
      x.y = __uint_as_float(gv[u].x & 0xffff0000u);
      x.z = __uint_as_float(gv[u].y << 16);
      x.w = __uint_as_float(gv[u].y & 0xffff0000u);
      av[u] += x;
      __builtin_nontemporal_store(av[u], a + u * kThreads);
    }
  }
}

// grid: workgroups_per_cu == 0 -> one workgroup per tile; else that many persistent per CU
uint32_t grid_for(uint64_t n_tiles, int workgroups_per_cu) {
  if (workgroups_per_cu <= 0) return (uint32_t)n_tiles;
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  const uint64_t g = (uint64_t)cus * (uint64_t)workgroups_per_cu;
  return (uint32_t)(g < n_tiles ? g : n_tiles);
}

int finish() { return hipGetLastError() == hipSuccess ? 0 : -1; }

}  // namespace

extern "C" {

// Workgroup size of the launches that follow: 256 threads (4 loads per lane) or 512 (2 per lane).
// Returns 0, or -1 for any other value.
int odc_ceiling_set_threads(int threads) {
  if (threads != 256 && threads != 512) return -1;
  g_threads = threads;
  return 0;
}

// Each call launches one kernel over whole tiles only: the sizes are rounded DOWN to a multiple
// of a tile (16 KiB of the 16-byte stream; 4096 elements for rmw) and the number of bytes the
// launch really moves is returned through *moved. lds_bytes is dynamic LDS the kernel never
// touches (caps the workgroups resident per CU, as the product's launches do). All pointers must
// be 16-byte aligned. Returns 0 or -1.
int odc_ceiling_read(const void* src, uint64_t nbytes, void* sink, int workgroups_per_cu, uint32_t lds_bytes,
                     void* stream, uint64_t* moved) {
  const uint64_t n_tiles = nbytes / (kTileVecs * 16);
  if (moved) *moved = n_tiles * kTileVecs * 16;
  if (!n_tiles) return 0;
  const dim3 grid(grid_for(n_tiles, workgroups_per_cu));
  hipStream_t q = static_cast<hipStream_t>(stream);
  if (g_threads == 512)
    hipLaunchKernelGGL((read_kernel<512, 2>), grid, dim3(512), lds_bytes, q, static_cast<const u32x4*>(src), n_tiles,
                       static_cast<uint32_t*>(sink));
  else
    hipLaunchKernelGGL((read_kernel<256, 4>), grid, dim3(256), lds_bytes, q, static_cast<const u32x4*>(src), n_tiles,
                       static_cast<uint32_t*>(sink));
  return finish();
}

int odc_ceiling_write(void* dst, uint64_t nbytes, int workgroups_per_cu, uint32_t lds_bytes, void* stream,
                      uint64_t* moved) {
  const uint64_t n_tiles = nbytes / (kTileVecs * 16);
  if (moved) *moved = n_tiles * kTileVecs * 16;
  if (!n_tiles) return 0;
  const dim3 grid(grid_for(n_tiles, workgroups_per_cu));
  hipStream_t q = static_cast<hipStream_t>(stream);
  if (g_threads == 512)
    hipLaunchKernelGGL((write_kernel<512, 2>), grid, dim3(512), lds_bytes, q, static_cast<u32x4*>(dst), n_tiles);
  else
    hipLaunchKernelGGL((write_kernel<256, 4>), grid, dim3(256), lds_bytes, q, static_cast<u32x4*>(dst), n_tiles);
  return finish();
}

int odc_ceiling_copy(void* dst, const void* src, uint64_t nbytes, int workgroups_per_cu, uint32_t lds_bytes,
                     void* stream, uint64_t* moved) {
  const uint64_t n_tiles = nbytes / (kTileVecs * 16);
  if (moved) *moved = 2 * n_tiles * kTileVecs * 16;
  if (!n_tiles) return 0;
  const dim3 grid(grid_for(n_tiles, workgroups_per_cu));
  hipStream_t q = static_cast<hipStream_t>(stream);
  if (g_threads == 512)
    hipLaunchKernelGGL((copy_kernel<512, 2>), grid, dim3(512), lds_bytes, q, static_cast<u32x4*>(dst),
                       static_cast<const u32x4*>(src), n_tiles);
  else
    hipLaunchKernelGGL((copy_kernel<256, 4>), grid, dim3(256), lds_bytes, q, static_cast<u32x4*>(dst),
                       static_cast<const u32x4*>(src), n_tiles);
  return finish();
}

int odc_ceiling_rmw(void* acc_f32, const void* grad_bf16, uint64_t n_elems, int workgroups_per_cu,
                    uint32_t lds_bytes, void* stream, uint64_t* moved) {
  const uint64_t n_tiles = n_elems / (kTileVecs * 4);
  if (moved) *moved = 10 * n_tiles * kTileVecs * 4;
  if (!n_tiles) return 0;
  const dim3 grid(grid_for(n_tiles, workgroups_per_cu));
  hipStream_t q = static_cast<hipStream_t>(stream);
  if (g_threads == 512)
    hipLaunchKernelGGL((rmw_kernel<512, 2>), grid, dim3(512), lds_bytes, q, static_cast<f32x4*>(acc_f32),
                       static_cast<const u32x2*>(grad_bf16), n_tiles);
  else
    hipLaunchKernelGGL((rmw_kernel<256, 4>), grid, dim3(256), lds_bytes, q, static_cast<f32x4*>(acc_f32),
                       static_cast<const u32x2*>(grad_bf16), n_tiles);
  return finish();
}

}  // extern "C"
