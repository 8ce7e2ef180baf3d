// An odc_device (odc_amd/csrc/odc_launch.h) for a machine without a GPU: every runtime call fails
// with "no device", and the dtype tables say what odc_kernels.hip implements (every pair of the
// three dtypes). Linked with odc_amd/csrc/odc_host.cpp by g++ under AddressSanitizer and UBSan,
// it gives the host side of libodc_hip.so as a library whose bookkeeping-only and dry-run arenas
// work exactly as in the real one: allocation bookkeeping, argument validation, work-list
// splitting, tile tables, launch shapes. No launch is ever issued.
#include "odc_hip.h"
#include "odc_launch.h"

namespace odc_device {

namespace {
constexpr int kNoDevice = 100;  // the value of hipErrorNoDevice
bool known(int dtype) { return dtype == ODC_DTYPE_BF16 || dtype == ODC_DTYPE_F16 || dtype == ODC_DTYPE_F32; }
}  // namespace

int get_current(int*) { return kNoDevice; }
int set_current(int) { return kNoDevice; }
int properties(int, Properties*) { return kNoDevice; }
int allocate(void**, uint64_t) { return kNoDevice; }
int release(void*) { return kNoDevice; }
bool is_out_of_memory(int) { return false; }
const char* error_string(int code) { return code == kNoDevice ? "no device (host-only build)" : "unknown error"; }

bool has_accum(int g, int a) { return known(g) && known(a); }
bool has_cast_gather(int s, int d) { return known(s) && known(d); }
bool has_publish(int a, int o) { return known(a) && known(o); }

int launch_gather(const odc_launch::GatherLaunch&, uint32_t, uint32_t, void*) { return kNoDevice; }
int launch_cast_gather(int, int, const odc_launch::CastGatherLaunch&, uint32_t, uint32_t, void*) { return kNoDevice; }
int launch_accum(int, int, bool, const odc_launch::AccumLaunch&, uint32_t, uint32_t, void*) { return kNoDevice; }
int launch_clear(const odc_launch::ClearLaunch&, uint32_t, void*) { return kNoDevice; }
int launch_publish(int, int, const odc_launch::PublishLaunch&, uint32_t, uint32_t, void*) { return kNoDevice; }

}  // namespace odc_device
