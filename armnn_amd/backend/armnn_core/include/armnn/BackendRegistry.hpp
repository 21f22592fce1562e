#pragma once
#include <hostcore/BackendLifecycle.hpp>   // BackendRegistry, BackendRegistryInstance
