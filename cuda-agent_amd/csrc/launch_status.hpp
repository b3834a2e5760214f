// Per-thread status word shared by every launcher of the library.
//
// Launchers keep the workspace's C ABI (void return, asynchronous, no device query). When a
// launcher is handed a shape it has no kernel for it launches nothing and records a code
// here; cuda_agent_amd_last_status() returns the code of the calling thread's most recent
// failure since the last query and resets it to 0.
#pragma once

enum CudaAgentAmdStatus : int {
    CAA_OK = 0,
    CAA_UNSUPPORTED_SHAPE = 1,   // a dimension the kernels are not instantiated for
    CAA_BAD_ARGUMENT = 2,        // null pointer, misaligned base, negative size
    CAA_WORKSPACE_TOO_SMALL = 3, // caller-provided scratch is smaller than *_workspace_bytes()
    CAA_SCRATCH_LIMIT = 4,       // the problem needs more than the library's own static scratch holds
    CAA_RUNTIME_ERROR = 5,       // a HIP runtime call of the launcher's set-up failed
};

namespace caa {
void set_status(int code);
}

extern "C" int cuda_agent_amd_last_status(void);
