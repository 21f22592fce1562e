#pragma once
#include <hostcore/MemoryInterfaces.hpp>   // ITensorHandleFactory, Capability, EdgeStrategy
