#pragma once
#include "tim/vx/detail/hotpath_ops.h"
