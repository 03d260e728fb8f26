// Error reporting and version query of the librlk_hip C ABI.
#include "rlk_common.hpp"

#include <string.h>

namespace {
thread_local char g_last_error[256] = "";
}

int rlk_fail(int code, const char* msg)
{
    strncpy(g_last_error, msg ? msg : "", sizeof(g_last_error) - 1);
    g_last_error[sizeof(g_last_error) - 1] = '\0';
    return code;
}

extern "C" {

int rlk_version(void) { return 100; }

const char* rlk_last_error(void) { return g_last_error; }

}  // extern "C"
