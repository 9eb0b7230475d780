// Library-level entry points of libsnnf that belong to no kernel family.
#include "snnf_common.h"

namespace snnf {

char* last_error_buffer() {
    static thread_local char buffer[512] = {0};
    return buffer;
}

}  // namespace snnf

extern "C" int snnf_abi_version(void) { return 1; }

extern "C" const char* snnf_status_string(int status) {
    switch (status) {
        case SNNF_OK: return "ok";
        case SNNF_ERR_INVALID_ARGUMENT: return "invalid argument";
        case SNNF_ERR_UNSUPPORTED: return "unsupported configuration";
        case SNNF_ERR_LAUNCH: return "kernel launch failed";
        case SNNF_ERR_WORKSPACE: return "workspace missing or too small";
        default: return "unknown status";
    }
}

extern "C" const char* snnf_last_error(void) { return snnf::last_error_buffer(); }
