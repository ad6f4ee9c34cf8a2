// Status strings, ABI version and per-thread HIP error slot.
#include "qa_common.hpp"

namespace qa {
namespace {
thread_local int g_last_hip_error = 0;
}
void set_last_hip_error(int code) { g_last_hip_error = code; }

namespace {
__global__ __launch_bounds__(256) void fill_zero_kernel(uint8_t* dst, int64_t bytes) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < bytes) dst[i] = 0;
}
}  // namespace

int fill_zero(void* dst, int64_t bytes, hipStream_t stream) {
    if (!dst || bytes <= 0) return QA_OK;
    const int64_t blocks = (bytes + 255) / 256;
    if (blocks > 0x7fffffffLL) return QA_ERR_SHAPE;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, static_cast<uint8_t*>(dst), bytes);
    return check_launch();
}
}  // namespace qa

extern "C" const char* qa_status_string(int status) {
    switch (status) {
        case QA_OK: return "ok";
        case QA_ERR_NULL: return "required pointer is null";
        case QA_ERR_SHAPE: return "size out of the supported range";
        case QA_ERR_STRIDE: return "stride or alignment requirement violated";
        case QA_ERR_UNSUPPORTED: return "unsupported configuration";
        case QA_ERR_LAUNCH: return "HIP launch failed";
        case QA_ERR_SCRATCH: return "the problem needs more scratch memory than the library's fixed buffer holds";
        default: return "unknown status";
    }
}

extern "C" int qa_abi_version(void) { return 2; }

extern "C" int qa_last_hip_error(void) { return qa::g_last_hip_error; }
