// Process-wide device state of the backend: which GPU, the stream every workload launches on, and the translation
// of C-ABI status codes into Arm NN exceptions.  All GPU work goes through include/armnn_mi355x.h.
#pragma once
#include <armnn/TypesUtils.hpp>
#include <armnn/Exceptions.hpp>
#include <armnn/Tensor.hpp>

#include <armnn_mi355x.h>

#include <string>

namespace armnn
{
namespace mi355x
{
/// number of usable devices; 0 when there is none or the driver cannot be reached
int DeviceCount();
/// selects device 0 on first use; throws BackendUnavailableException when there is no device
void EnsureDevice();
/// the stream all workloads and tensor-handle copies are ordered on
mi355x_stream_t Stream();
void Synchronize();

/// throws RuntimeException carrying mi355x_last_error() when `status` is non-zero
void Check(int status, const char* what);

/// activation TensorInfo -> mi355x_quant; throws InvalidArgumentException for other data types
mi355x_quant ToQuant(const TensorInfo& info);
int32_t ToDType(DataType t);
} // namespace mi355x
} // namespace armnn
