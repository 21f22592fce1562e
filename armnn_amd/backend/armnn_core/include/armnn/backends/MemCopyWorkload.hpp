#pragma once
#include <hostcore/BackendHelpers.hpp>   // CopyMemGenericWorkload
