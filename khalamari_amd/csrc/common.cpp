#include "common.h"

namespace khm {
std::string& last_error_storage() {
    static thread_local std::string message;
    return message;
}
}  // namespace khm

extern "C" const char* khm_last_error(void) { return khm::last_error_storage().c_str(); }
extern "C" const char* khm_version(void) { return "khalamari_amd gqa-sdpa 0.1 (gfx950)"; }
