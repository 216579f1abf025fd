#include "fa_device.h"
#include "fa_kernels.h"
namespace fa {
hipError_t launch_decode_mla_i8(const DecodeParams &, int, hipStream_t) { return hipErrorNotSupported; }
}  // namespace fa
