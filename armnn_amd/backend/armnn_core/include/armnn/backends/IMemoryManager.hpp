#pragma once
#include <hostcore/MemoryInterfaces.hpp>   // IMemoryManager
