// The reference keeps Graph in a header of its own (src/armnn/Graph.hpp); here it lives with Layer.
#pragma once
#include "Layer.hpp"
