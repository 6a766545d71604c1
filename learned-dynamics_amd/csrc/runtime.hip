// Status strings and the per-thread error text of the C ABI.
#include "common.hpp"

namespace mg {
char* last_error_buffer() {
    static thread_local char buf[512] = {0};
    return buf;
}
}  // namespace mg

extern "C" {

const char* mg_status_string(int status) {
    switch (status) {
        case MG_OK: return "ok";
        case MG_ERR_INVALID_ARGUMENT: return "invalid argument";
        case MG_ERR_HIP: return "HIP runtime error";
        case MG_ERR_BOX_TOO_SMALL: return "box dimension must be greater than 3*cutoff";
        case MG_ERR_WORKSPACE: return "workspace too small";
        case MG_ERR_UNSUPPORTED: return "unsupported";
    }
    return "unknown status";
}

const char* mg_last_error(void) { return mg::last_error_buffer(); }

int mg_abi_version(void) { return 1; }

}  // extern "C"
