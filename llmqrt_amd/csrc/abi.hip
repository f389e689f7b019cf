// ABI bookkeeping for libllmq_gfx950.so: version and status strings.
#include "llmq_common.h"

extern "C" int llmq_abi_version(void) { return 1; }

extern "C" const char* llmq_status_string(int status) {
    switch (status) {
        case LLMQ_OK: return "ok";
        case LLMQ_ERR_NULL: return "a required pointer is NULL";
        case LLMQ_ERR_DTYPE: return "unsupported dtype or format selector";
        case LLMQ_ERR_SHAPE: return "invalid or unsupported shape / stride";
        case LLMQ_ERR_WORKSPACE: return "workspace missing or too small";
        case LLMQ_ERR_LAUNCH: return "HIP launch failed";
        case LLMQ_ERR_ALIGN: return "pointer is not sufficiently aligned";
        case LLMQ_ERR_SCRATCH: return "problem needs more scratch than the library's static array holds";
        default: return "unknown status";
    }
}
