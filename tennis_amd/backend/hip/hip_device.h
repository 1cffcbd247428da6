// The "hip" device of the backend: what TenniS's CUDA backend keeps in CUDAContextHandle
// (include/kernels/gpu/cuda_context.h:13-43) minus the BLAS handle -- every kernel is hand-written.
#pragma once
#include "tsx_ts.h"

namespace ts {
namespace hip {

static const char *const DEVICE = "hip";   // DeviceType holds at most 7 characters

struct HipContextHandle {
    void *stream = nullptr;   // hipStream_t of this DeviceContext
    int device_id = 0;
    Tensor scratch;           // kernel scratch shared by the operators of this context (see context_scratch)
};

// Device tensor of `bytes` bytes (any size: shaped [ceil(bytes / 16), 16], so sizes of 2 GiB and more do not
// overflow an int32 extent).
Tensor byte_tensor(const MemoryDevice &device, size_t bytes);

// Scratch of at least `bytes` bytes in the memory of the DeviceContext bound to the calling thread, for kernels
// that need a workspace for the duration of one operator call (the staged activations of a quantized
// convolution).  One buffer per context, grown to the largest request and reused by every operator of the
// context: its stream orders the kernels that write and read it, the way the reference's operators share
// the stack's scratch frame.  `own` is used instead when no context is bound (an operator driven by hand).
void *context_scratch(size_t bytes, const MemoryDevice &device, Tensor &own);

// Stream of the DeviceContext bound to the calling thread (nullptr = default stream when an
// operator is driven without a Workbench).
void *current_stream();

// Throws the reference's way (TS_LOG_ERROR << eject) when a C-ABI launcher reports an error
// (include/kernels/gpu/gpu_kernel.h:13-19).
void check(int tsx_rc, const char *what);

// The host operator of the same name, created on first use with the same parameters.  TenniS falls back to
// the host only for operators a device does not register at all (src/global/operator_factory.cpp:60-81); a
// registered "hip" class that meets a data type, format or mode its kernel does not cover hands the call to
// this delegate instead of failing, so a graph that ran on the host keeps running on the device: inputs
// reach the host through Tensor::view, the result is a host tensor the next operator views back.
class HostDelegate {
public:
    int run(Operator &self, Stack &stack);

private:
    Operator::shared m_host;
};

template <typename OP>
class OperatorOnHip : public OP {
public:
    MemoryDevice running_memory_device() override { return MemoryDevice(DEVICE, current_device_id()); }
    static int current_device_id();

    int run(Stack &stack) override {
        if (!covers(stack)) return m_delegate.run(*this, stack);
        return OP::run(stack);
    }

protected:
    // false: the inputs on the stack need the host operator (see HostDelegate)
    virtual bool covers(Stack &) { return true; }

private:
    HostDelegate m_delegate;
};

int context_device_id();
template <typename OP>
int OperatorOnHip<OP>::current_device_id() { return context_device_id(); }

}  // namespace hip
}  // namespace ts
