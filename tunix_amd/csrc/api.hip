// Status strings and ABI version of the C interface.
#include "tmx_common.h"

extern "C" const char* tmx_status_string(int status) {
  switch (status) {
    case TMX_OK: return "ok";
    case TMX_ERR_ARG: return "invalid argument (null pointer or inconsistent optional arguments)";
    case TMX_ERR_SHAPE: return "shape violates the kernel's tiling rules";
    case TMX_ERR_LAUNCH: return "HIP launch failed";
    case TMX_ERR_UNSUPPORTED: return "unsupported configuration";
    case TMX_ERR_SCRATCH: return "the request needs more scratch memory than the library's static buffer holds";
    case TMX_ERR_DEVICE_WAIT: return "a bounded wait inside a kernel ran out: results since the last status check are invalid";
    default: return "unknown status";
  }
}

extern "C" int tmx_abi_version(void) { return 4; }
