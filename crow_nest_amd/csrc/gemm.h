// placeholder until the MFMA GEMM lands
#pragma once
#include "device_common.h"
