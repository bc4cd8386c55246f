// Forwarding header for `#include "ntsCUDA.hpp"` (core/coocsc.hpp, utils/cuda_memory.hpp).
#include "../ntsHIP.hpp"
