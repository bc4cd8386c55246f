// Forwarding header for `#include "cuda/cuda_type.h"` (VertexId_CUDA and the launch constants live
// in the HIP veneer).
#include "../../ntsHIP.hpp"
