/* Test infrastructure: stand-in for <hip/hip_ext.h> (see hip_runtime.h beside it). */
#include <hip/hip_runtime.h>
