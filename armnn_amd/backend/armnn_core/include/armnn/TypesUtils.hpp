// Minimal host core: the helpers of include/armnn/TypesUtils.hpp that backends call.
#pragma once
#include "Types.hpp"
