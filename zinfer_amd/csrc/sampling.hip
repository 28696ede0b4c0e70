// Sampling kernels (placeholder for the first build step; filled in below).
#include "zf_common.h"
extern "C" int zf_sampling_version() { return 1; }
