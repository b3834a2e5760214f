#include "launch_status.hpp"

namespace {
thread_local int g_last_status = CAA_OK;
}

namespace caa {
void set_status(int code) { g_last_status = code; }
}  // namespace caa

extern "C" int cuda_agent_amd_last_status(void) {
    const int code = g_last_status;
    g_last_status = CAA_OK;
    return code;
}
