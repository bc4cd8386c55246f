// Forwarding header: makes the NeutronBench tree's `#include "cuda/ntsCUDA.hpp"` resolve to the
// HIP veneer when this directory precedes the tree on the include path.
#include "../../ntsHIP.hpp"
