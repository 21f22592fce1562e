#pragma once
#include <hostcore/Utility.hpp>   // IgnoreUnused
