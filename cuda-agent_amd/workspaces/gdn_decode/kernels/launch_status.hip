// Shared with the C-ABI library: the per-thread status word the launchers report through.
#include "../../../csrc/launch_status.hip"
