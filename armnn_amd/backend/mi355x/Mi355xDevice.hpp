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
/// Whether layer support may answer "yes".  The runtime lists every dynamically loaded backend as usable even when its
/// backend context could not be created (src/armnn/Runtime.cpp:684-687 against :501), so on a machine without the device
/// the optimizer would still place layers here and LoadNetwork would fail; layer support therefore answers "no" for
/// every layer while this is false, and Optimize({"Mi355x", "CpuRef"}) falls back.  True when a device is visible, or
/// after AssumeDevice(true): for optimizing on a machine that lacks the device (and for host-only tests of the rules).
bool DeviceUsable();
void AssumeDevice(bool assume);
/// selects device 0 on first use; throws BackendUnavailableException when there is no device
void EnsureDevice();
/// The stream workloads and tensor-handle copies are ordered on.  If the calling thread has lanes running (see below) they
/// are joined first, so whatever is queued through this stream comes after everything queued before it.
mi355x_stream_t Stream();
/// joins the lanes and waits for the stream
void Synchronize();
/// how many times any thread has waited for the stream so far.  An inference ends with such a wait (the runtime maps the
/// network's outputs), so a value that has not changed means "still the same inference".
unsigned long long SyncEpoch();

/// Lanes.  Every image of a batch is computed independently, so a workload may run its batch as Lanes() contiguous
/// slices, slice k on LaneStream(k): one slice's launches then fill the ramp-up, tail and launch gaps of the others, and
/// the input of a later slice crosses the bus while an earlier one computes.  Lane 0 is the stream of Stream().
///   Fork()  the lanes continue, independently, after everything queued so far (no-op while forked)
///   Join()  stream 0 continues after everything queued on every lane (no-op while joined)
/// The forked/joined state belongs to the calling thread; a thread leaves EnqueueWorkload joined because reading a
/// network output goes through Stream().
constexpr unsigned int kMaxLanes = 4;
unsigned int Lanes();
/// 1 .. kMaxLanes; the initial value is 2, or what the environment variable MI355X_LANES says.  Raising it above 1 throws
/// while a network loaded for one stream is alive: its tensors share addresses, which lanes must not.
void SetLanes(unsigned int lanes);
/// memory managers that let tensors share addresses announce themselves here (+1 when created, -1 when destroyed)
void CountAddressSharingArena(int delta);
/// Device memory a tensor handle adopted announces its range here.  Two live ranges that overlap mean tensors share
/// addresses (a caller's memory plan that reuses a buffer for tensors whose lifetimes do not meet): such tensors are only
/// safe in launch order, so LanesFor() answers 1 while any overlap is alive.  NoteAdoptedRange returns true when the new
/// range overlaps a live one; pass that to ForgetAdoptedRange when the handle lets go of the memory.
bool NoteAdoptedRange(const void* begin, size_t bytes);
void ForgetAdoptedRange(const void* begin, size_t bytes, bool overlapped);
/// the smallest slice worth a lane of its own: a batch splits only into slices of at least this many images
constexpr unsigned int kMinLaneBatch = 8;
/// number of slices a workload over `batch` images should run as: Lanes() if that divides the batch into slices of at
/// least kMinLaneBatch and no adopted ranges overlap, else 1
unsigned int LanesFor(unsigned int batch);
mi355x_stream_t LaneStream(unsigned int lane);
void Fork();
void Join();
/// Host-to-device transfer from pinned memory (the staging copy of a tensor handle or an adopted buffer), queued without
/// waiting for it: `bytes` in `lanes` equal parts queued back to back on one copy queue, so part k arrives
/// at k+1 times a part's transfer time; lane k continues as soon as its part is there.  Leaves the lanes forked.
void UploadInLanes(void* dstDevice, const void* srcHost, size_t bytes, unsigned int lanes);

/// throws RuntimeException carrying mi355x_last_error() when `status` is non-zero
void Check(int status, const char* what);

/// activation TensorInfo -> mi355x_quant; throws InvalidArgumentException for other data types
mi355x_quant ToQuant(const TensorInfo& info);
int32_t ToDType(DataType t);
} // namespace mi355x
} // namespace armnn
