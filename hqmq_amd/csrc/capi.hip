// Version and status strings of the C ABI.
#include "common.h"

extern "C" int hqmq_version(void) { return HQMQ_VERSION; }

extern "C" const char *hqmq_status_string(int status) {
    switch (status) {
        case HQMQ_OK: return "ok";
        case HQMQ_ERR_NULL: return "a required pointer is NULL";
        case HQMQ_ERR_SHAPE: return "a size is out of the supported range";
        case HQMQ_ERR_DTYPE: return "unknown or unsupported dtype";
        case HQMQ_ERR_LAYOUT: return "bit widths inconsistent with the layout rules";
        case HQMQ_ERR_WORKSPACE: return "workspace too small";
        case HQMQ_ERR_ALIGN: return "a pointer or stride is not aligned as required";
        case HQMQ_ERR_SCRATCH: return "the call does not fit the library's static scratch (8 MiB of split partials; skip_combine is not available)";
        default: return status > 0 ? hipGetErrorString((hipError_t)status) : "unknown status";
    }
}
