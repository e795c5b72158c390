#pragma once
#include "tim/vx/detail/core_api.h"
