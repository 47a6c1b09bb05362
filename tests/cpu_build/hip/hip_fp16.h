// __half lives in the stand-in's hip_runtime.h.
#include "hip_runtime.h"
