// Found by the front end as "cuda/concat.cuh"; everything lives in one header on the include path.
#pragma once
#include "tannic_hip_adapter.hpp"
