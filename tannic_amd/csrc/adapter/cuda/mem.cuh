// Found by the front end as "cuda/mem.cuh"; everything lives in one header on the include path.
#pragma once
#include "tannic_hip_adapter.hpp"
