#pragma once
// The reference gates include this for device selection helpers; the gfx950 shims need nothing
// from it beyond the HIP runtime.
#include <hip/hip_runtime.h>
