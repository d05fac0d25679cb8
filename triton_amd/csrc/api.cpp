// Library-level entry points that launch nothing.
#include "../../include/triton_amd.h"

extern "C" int tamd_version(void) { return TAMD_VERSION; }

extern "C" const char *tamd_error_string(int code) {
  switch (code) {
    case 0: return "ok";
    case TAMD_E_INVALID: return "invalid argument";
    case TAMD_E_UNSUPPORTED: return "combination not supported by this build";
    case TAMD_E_ALIGNMENT: return "pointer or stride misaligned";
    case TAMD_E_TOO_LARGE: return "problem exceeds the fixed capacity of this entry point";
    default: return code > 0 ? "HIP runtime error" : "unknown error";
  }
}
