// Status strings, ABI version and per-thread HIP error slot.
#include "qa_common.hpp"

namespace qa {
namespace {
thread_local int g_last_hip_error = 0;
}
void set_last_hip_error(int code) { g_last_hip_error = code; }
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
