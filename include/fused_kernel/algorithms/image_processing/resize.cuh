// The include path the Fused Kernel Library's README uses for this header (its files have since been renamed to .h);
// everything is provided by the umbrella header of this library.
#include "fk/fused_kernel.h"
#include "fk/core/global_types.h"
