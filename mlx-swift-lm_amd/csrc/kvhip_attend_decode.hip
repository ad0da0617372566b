// placeholder until the matrix-core decode kernels land
#include "kvhip_internal.hpp"
namespace kvhip {
bool attend_decode_supported(const AttendArgs &) { return false; }
size_t attend_decode_workspace(const AttendArgs &) { return 0; }
hipError_t launch_attend_decode(const AttendArgs &, hipStream_t) { return hipErrorNotSupported; }
}
