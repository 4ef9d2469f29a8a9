// Same include path as the Fused Kernel Library header of this name, so user code written against it compiles
// unchanged; everything is provided by the umbrella header of this library.
#include "fk/fused_kernel.h"
#include "fk/core/global_types.h"
