// The kernel launchers live in the HIP source; a host-only link of the library's C++ files needs
// their names.  The sanitizer driver never reaches them.
#include "mx_device.h"
namespace mx {
hipError_t launch_tiles(mx_dtype, const DeviceTiles &, const void *, void *, int, hipStream_t, const void *) { return hipErrorUnknown; }
hipError_t launch_csr(mx_dtype, const DeviceCsr &, const void *, void *, int, hipStream_t, void *) { return hipErrorUnknown; }
hipError_t launch_slices(mx_dtype, const DeviceSlices &, const void *, void *, int, hipStream_t, int, const DeviceTiles *, void *) { return hipErrorUnknown; }
hipError_t launch_fused(mx_dtype, const DeviceSlices &, const void *, void *, int, hipStream_t, void *, unsigned *, unsigned) { return hipErrorUnknown; }
hipError_t fused_placement_ok(int, int *ok) { *ok = 0; return hipErrorUnknown; }
hipError_t prepare_slice_kernels(mx_dtype) { return hipErrorUnknown; }
hipError_t static_scratch(void **p) { *p = nullptr; return hipErrorUnknown; }
int build_slices_device(mx_dtype, int, int, int, const int *, const int *, const void *, int, int, const char *, DeviceSlices &, hipStream_t,
                        std::vector<int> *, std::vector<int> *, int) { return MX_ERR_DEVICE; }
int check_csr_device(int, int, int, const int *, const int *, hipStream_t, const char *) { return MX_ERR_DEVICE; }
int lines_per_gather_device(mx_dtype, int, const int *, hipStream_t, double *) { return MX_ERR_DEVICE; }
int upload_csr_device(mx_dtype, int, int, int, const int *, const int *, const void *, const std::vector<int> &, bool, DeviceCsr &, hipStream_t) { return MX_ERR_DEVICE; }
bool strips_can_ride(mx_dtype, const DeviceTiles &, const void *) { return false; }
struct HybridDevice::Impl {};
HybridDevice::~HybridDevice() { delete impl; }
int HybridDevice::analyse(mx_dtype, int, int, int, const int *, const int *, const void *, float, float, int, bool, bool, bool, HybridCounts *,
                          hipStream_t) { return MX_ERR_DEVICE; }
int HybridDevice::adopt(const PartitionTwin &, int, bool, bool, bool, HybridCounts *, hipStream_t) { return MX_ERR_DEVICE; }
int HybridDevice::csr_part(bool, bool, bool, int **, int **, void **, int *, char **) { return MX_ERR_DEVICE; }
int HybridDevice::block_chunks(std::vector<int> &, std::vector<int> &) { return MX_ERR_DEVICE; }
int HybridDevice::block_layout(const std::vector<int> &, const std::vector<int> &, const std::vector<int> &, long long, DeviceTiles &)
{
    return MX_ERR_DEVICE;
}
int HybridDevice::tile_chunks(bool, std::vector<int> &) { return MX_ERR_DEVICE; }
int HybridDevice::tile_layout(bool, const std::vector<int> &, const std::vector<int> &, const std::vector<int> &, long long, DeviceTiles &)
{
    return MX_ERR_DEVICE;
}
int HybridDevice::strip_layout(const std::vector<int> &, const std::vector<int> &, const std::vector<int> &, long long, DeviceTiles &)
{
    return MX_ERR_DEVICE;
}
hipError_t launch_probe_f64(const double *, const double *, double *, hipStream_t) { return hipErrorUnknown; }
hipError_t launch_probe_f16(const void *, const void *, float *, hipStream_t) { return hipErrorUnknown; }
}
// The device route of the extraction lives in a HIP source as well; the tuner names it.
extern "C" int mx_partition_create_device(const mx_csr *, float, float, mx_partition **) { return MX_ERR_DEVICE; }
