// Everything a client of the public API needs, in dependency order.
#pragma once
#include "Types.hpp"
#include "Exceptions.hpp"
#include "Optional.hpp"
#include "Tensor.hpp"
#include "Descriptors.hpp"
#include "BackendId.hpp"
#include "BackendOptions.hpp"
#include "INetwork.hpp"
#include "IRuntime.hpp"
#include "Utils.hpp"
#include <hostcore/BackendLifecycle.hpp>
