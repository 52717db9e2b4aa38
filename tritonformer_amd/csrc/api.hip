// Status strings and version of the C ABI.
#include "common.h"

extern "C" const char* tf_status_string(int status) {
  switch (status) {
    case TF_OK: return "ok";
    case TF_EINVAL: return "invalid argument (size, null pointer or unsupported combination)";
    case TF_EDTYPE: return "dtype not supported by this entry point";
    case TF_EALIGN: return "pointer or stride violates an alignment requirement";
    case TF_ESHAPE: return "shape precondition violated";
    case TF_EWORKSPACE: return "workspace missing or too small";
    case TF_ELAUNCH: return "HIP kernel launch failed";
  }
  return "unknown status";
}

extern "C" int tf_version(void) { return 100; }
