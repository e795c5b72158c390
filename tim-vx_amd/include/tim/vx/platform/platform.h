#pragma once
#include "tim/vx/detail/platform_api.h"
