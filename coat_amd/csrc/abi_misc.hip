// Version and error strings of the C ABI.
#include "coat_host.h"

#define COAT_STR2(x) #x
#define COAT_STR(x) COAT_STR2(x)
extern "C" int coat_abi_version(void) { return COAT_ABI_VERSION; }

extern "C" const char* coat_version(void) { return "coat_amd 0.3 (gfx950, ABI " COAT_STR(COAT_ABI_VERSION) ")"; }

extern "C" const char* coat_status_string(int status) {
    switch (status) {
        case COAT_OK: return "ok";
        case COAT_EINVAL: return "invalid argument (null pointer, negative size or unknown enum)";
        case COAT_ESHAPE: return "shape contract violated (group / tile divisibility or scale length)";
        case COAT_EDTYPE: return "unsupported dtype combination";
        case COAT_EQGROUP: return "Only Support 128 per-group quantization currently";
        case COAT_EALIGN: return "tensor base address must be 16-byte aligned";
        default: return status > 0 ? hipGetErrorString((hipError_t)status) : "unknown coat status";
    }
}
