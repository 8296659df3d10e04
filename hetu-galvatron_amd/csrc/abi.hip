// ABI version and status strings of libgalvatron_moe.so.
#include "gmoe_common.h"

extern "C" int gmoe_abi_version(void) { return GMOE_ABI_VERSION; }

extern "C" const char* gmoe_status_string(int status) {
  switch (status) {
    case GMOE_OK: return "ok";
    case GMOE_ERR_INVALID: return "invalid argument (null pointer, bad shape, misaligned buffer or bad flag)";
    case GMOE_ERR_UNSUPPORTED: return "request not supported by this build of the library";
    case GMOE_ERR_LAUNCH: return "HIP reported an error while launching a kernel";
    case GMOE_ERR_TOO_LARGE: return "sizes beyond the fixed maximum of this entry point (use the variant with a workspace)";
    default: return "unknown status";
  }
}
