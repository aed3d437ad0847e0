// placeholder, replaced below
#include "common.h"
#include "launch.h"
namespace gridnet {
bool step_fast_supports(const StepArgs &, bool) { return false; }
size_t step_fast_backward_workspace(const StepArgs &) { return 0; }
int step_forward_fast(const StepArgs &, hipStream_t) { return fail(GRIDNET_ERR_ARGUMENT, "no fast path"); }
int step_backward_fast(const StepArgs &, hipStream_t) { return fail(GRIDNET_ERR_ARGUMENT, "no fast path"); }
}
