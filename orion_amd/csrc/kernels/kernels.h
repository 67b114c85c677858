// Internal header of the co-location kernel library: pulls in the public C ABI.
#pragma once
#include "orion_kernels.h"
