#pragma once
#include "gtest/gtest.h"
