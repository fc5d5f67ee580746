// Storage for the CPU execution shim's per-launch state.  Test infrastructure only.
#define TAH_EMU_IMPL
#include <hip/hip_runtime.h>
