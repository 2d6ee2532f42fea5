#include "kernels.hpp"
namespace ave {
bool mx_decode_supports(const MxArgs&) { return false; }
bool nv_tile_supports(const NvArgs&) { return false; }
hipError_t launch_mx_decode(const MxArgs&, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_nv_tile(const NvArgs&, hipStream_t) { return hipErrorNotSupported; }
}
