// Library-level entry points of libmodelopt_hip.so (version and error strings).
#include "../../include/modelopt_hip.h"

extern "C" int mo_version(void) { return 1; }

extern "C" const char* mo_error_string(int status) {
    switch (status) {
        case MO_OK: return "ok";
        case MO_ERR_ARG: return "invalid argument (null pointer, negative size or misaligned buffer)";
        case MO_ERR_DTYPE: return "unsupported element type";
        case MO_ERR_UNSUPPORTED: return "request not covered by the kernels";
        case MO_ERR_LAUNCH: return "HIP runtime rejected the kernel launch";
        case MO_ERR_TOO_LARGE: return "input exceeds the fixed workspace of this entry point";
        default: return "unknown status";
    }
}
