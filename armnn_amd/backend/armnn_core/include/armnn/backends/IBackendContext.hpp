#pragma once
#include <hostcore/BackendLifecycle.hpp>   // IBackendContext, IBackendModelContext
