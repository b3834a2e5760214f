// The kernels and their extern "C" launchers live in the package's csrc/ directory, from which
// the torch-free C-ABI library is also built; this translation unit compiles the same
// source into the workspace extension.
#include "../../../csrc/moe_requant_fix.hip"
