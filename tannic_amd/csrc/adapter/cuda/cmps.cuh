// Found by the patched front end (frontend.patch) as "cuda/cmps.cuh"; everything lives in one header on the include path.
#pragma once
#include "tannic_hip_adapter.hpp"
