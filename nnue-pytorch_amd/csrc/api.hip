// Entry points that launch nothing: version, error text, constants of the ABI contract.
#include "common.h"

extern "C" int nnueft_version(void) { return NNUEFT_VERSION; }

extern "C" int nnueft_bias_tile(void) { return NNUEFT_BIAS_TILE; }
extern "C" int nnueft_row_split(void) { return NNUEFT_ROW_SPLIT; }
extern "C" int nnueft_row_window(int B) { return B > 0 ? nnueft_window_positions(B) : 0; }

extern "C" const char* nnueft_error_string(int code) {
    switch (code) {
        case 0: return "success";
        case NNUEFT_E_ARG: return "nnueft: invalid argument (null pointer, bad dimension or odd L1)";
        case NNUEFT_E_WORKSPACE: return "nnueft: workspace missing, not 256-byte aligned or too small";
        case NNUEFT_E_UNSUPPORTED: return "nnueft: dimension beyond what the kernels index";
        case NNUEFT_E_SCRATCH:
            return "nnueft: sizes beyond the library's fixed scratch memory (2 MiB: pass a workspace to "
                   "nnueft_double_fwd instead)";
        default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "nnueft: unknown error code";
}
