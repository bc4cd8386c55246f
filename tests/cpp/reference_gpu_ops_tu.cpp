// Translation unit for the compile check in tests/test_reference_compiles_against_veneer.py: the
// NeutronBench GPU operator and layout headers, included from the reference tree itself with its
// GPU switch on, must parse against the HIP veneer that replaces cuda/ntsCUDA.hpp.
#include "comm/logger.h"
#include "core/ntsSingleGPUFusedGraphOp.hpp"
#include "core/ntsDistGPUGraphOp.hpp"
#include "core/coocsc.hpp"
#include "core/FullyRepGraph.hpp"
#include "utils/cuda_memory.hpp"
#include "core/ntsDataloador.hpp"
int main() { return 0; }
