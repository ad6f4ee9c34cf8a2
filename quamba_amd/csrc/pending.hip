// Entry points whose kernels are not written yet report QA_ERR_UNSUPPORTED.
#include "qa_common.hpp"
extern "C" int64_t qa_ssd_workspace_bytes(const QaSsdParams*) { return 0; }
extern "C" int qa_ssd_chunk_scan_fwd(const QaSsdParams*, void*) { return QA_ERR_UNSUPPORTED; }
