#pragma once
#include <hostcore/BackendHelpers.hpp>   // OptimizationViews
