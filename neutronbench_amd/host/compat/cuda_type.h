// Forwarding header for `#include "cuda_type.h"`.
#include "../ntsHIP.hpp"
