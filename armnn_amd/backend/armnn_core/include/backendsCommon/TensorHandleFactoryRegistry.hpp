#pragma once
#include <hostcore/MemoryInterfaces.hpp>   // TensorHandleFactoryRegistry
