// Status strings and ABI version of the lpmm HIP library.
#include "lpmm_hip.h"

extern "C" const char *lpmm_status_string(int status)
{
    switch (status) {
    case LPMM_OK: return "ok";
    case LPMM_ERR_NULL: return "a required pointer is NULL";
    case LPMM_ERR_ALIGN: return "a pointer does not meet its required alignment";
    case LPMM_ERR_SIZE: return "a size or count is out of range";
    case LPMM_ERR_LAUNCH: return "the HIP runtime reported an error at kernel launch";
    case LPMM_ERR_ARG: return "an argument has an unknown value";
    default: return "unknown status";
    }
}

extern "C" int lpmm_abi_version(void) { return LPMM_HIP_ABI_VERSION; }
