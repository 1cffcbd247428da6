// Device plumbing a TenniS backend registers at static-init time, for device type "hip":
// allocator, the three converters, the compute->memory map and the device admin -- the pattern
// of src/kernels/gpu/memory_gpu.cpp:36-119 and src/kernels/gpu/cuda_context.cpp:12-53.
#include "hip_device.h"

#include <atomic>
#include <hip/hip_runtime_api.h>

#include "tsx_hip.h"

namespace ts {
namespace hip {

namespace {

void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) TS_LOG_ERROR << "[hip] " << what << ": " << hipGetErrorString(e) << eject;
}

hipStream_t stream_of_context() {
    auto *context = ctx::get<DeviceContext>();
    if (!context || !context->handle) return nullptr;
    return static_cast<hipStream_t>(reinterpret_cast<HipContextHandle *>(context->handle)->stream);
}

// malloc / free / realloc-with-copy in one function (include/global/hard_allocator.h:46-82)
void *hip_allocator(int id, size_t new_size, void *mem, size_t mem_size) {
    hip_check(hipSetDevice(id), "hipSetDevice");
    if (new_size == 0) {
        if (mem) hip_check(hipFree(mem), "hipFree");
        return nullptr;
    }
    void *fresh = nullptr;
    const hipError_t err = hipMalloc(&fresh, new_size);
    if (err == hipErrorOutOfMemory || (err == hipSuccess && fresh == nullptr)) {
        (void)hipGetLastError();   // the failed allocation must not show up at the next launch check
        // what the reference's allocators throw (src/kernels/gpu/memory_gpu.cpp:54), so that callers that
        // catch it (and Workbench's memory-pressure handling) see the same type from this device
        throw OutOfMemoryException(MemoryDevice(DEVICE, id), new_size);
    }
    hip_check(err, "hipMalloc");
    if (mem) {
        const size_t keep = mem_size < new_size ? mem_size : new_size;
        if (keep) hip_check(hipMemcpy(fresh, mem, keep, hipMemcpyDeviceToDevice), "hipMemcpy");
        hip_check(hipFree(mem), "hipFree");
    }
    return fresh;
}

// Copies run on the context stream.  Host buffers here are pageable, so every copy is completed
// before returning: a host source may be released right after, and a host destination is read
// right after (the device->host copy is the one barrier before results are used, as in the
// reference, src/kernels/gpu/memory_gpu.cpp:106-108).
void copy(void *dst, const void *src, size_t size, hipMemcpyKind kind, int device_id) {
    hip_check(hipSetDevice(device_id), "hipSetDevice");
    hipStream_t stream = stream_of_context();
    hip_check(hipMemcpyAsync(dst, src, size, kind, stream), "hipMemcpyAsync");
    hip_check(hipStreamSynchronize(stream), "hipStreamSynchronize");
}
void hip_from_cpu(int dst_id, void *dst, int, const void *src, size_t size) { copy(dst, src, size, hipMemcpyHostToDevice, dst_id); }
void cpu_from_hip(int, void *dst, int src_id, const void *src, size_t size) { copy(dst, src, size, hipMemcpyDeviceToHost, src_id); }
void hip_from_hip(int dst_id, void *dst, int, const void *src, size_t size) { copy(dst, src, size, hipMemcpyDeviceToDevice, dst_id); }

}  // namespace

Tensor byte_tensor(const MemoryDevice &device, size_t bytes) {
    const size_t rows = (bytes + 15) / 16;
    if (rows > size_t(0x7fffffff)) TS_LOG_ERROR << "[hip] buffer of " << bytes << " bytes exceeds a tensor's extents" << eject;
    return Tensor(device, INT8, Shape({int32_t(rows ? rows : 1), 16}));
}

void *context_scratch(size_t bytes, const MemoryDevice &device, Tensor &own) {
    auto *context = ctx::get<DeviceContext>();
    Tensor &slot = (context && context->handle && context->memory_device == device)
                       ? reinterpret_cast<HipContextHandle *>(context->handle)->scratch
                       : own;
    if (slot.empty() || size_t(slot.count()) < bytes || slot.device() != device) {
        // kernels already queued on the context's stream may still use the old buffer: drain it before the free
        hip_check(hipStreamSynchronize(stream_of_context()), "hipStreamSynchronize");
        slot = byte_tensor(device, bytes);
    }
    return slot.data();
}

namespace {
std::atomic<long> g_host_delegate_runs{0};
}  // namespace

int HostDelegate::run(Operator &self, Stack &stack) {
    g_host_delegate_runs.fetch_add(1);
    if (!m_host) {
        Operator::shared host;
        try {
            host = OperatorCreator::Create(CPU, self.op(), true);
        } catch (const Exception &) {
            host = nullptr;
        }
        if (!host)
            TS_LOG_ERROR << "[hip] " << self.op() << ": these inputs need the host operator, and no \"cpu\" operator "
                         << "of that name is registered in this build" << eject;
        // as OperatorInstruction::clone does (src/runtime/instruction.cpp:91-103): same parameters, then init()
        for (auto &param : self.params()) host->set(param.first, param.second);
        host->init();
        m_host = host;
    }
    return m_host->run(stack);
}

namespace {

void hip_admin(DeviceHandle **handle, int device_id, DeviceAdmin::Action action) {
    auto **h = reinterpret_cast<HipContextHandle **>(handle);
    switch (action) {
        case DeviceAdmin::INITIALIZATION: {
            hip_check(hipSetDevice(device_id), "hipSetDevice");
            auto *fresh = new HipContextHandle;
            fresh->device_id = device_id;
            hipStream_t stream = nullptr;
            hip_check(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking), "hipStreamCreateWithFlags");   // default priority
            fresh->stream = stream;
            *h = fresh;
            break;
        }
        case DeviceAdmin::FINALIZATION:
            if (*h) {
                (void) hipSetDevice((*h)->device_id);
                if ((*h)->stream) (void) hipStreamDestroy(static_cast<hipStream_t>((*h)->stream));
                delete *h;
                *h = nullptr;
            }
            break;
        case DeviceAdmin::ACTIVATION:
            hip_check(hipSetDevice(device_id), "hipSetDevice");
            break;
        case DeviceAdmin::SYNCHRONIZE:
            if (*h) {
                hip_check(hipSetDevice((*h)->device_id), "hipSetDevice");
                hip_check(hipStreamSynchronize(static_cast<hipStream_t>((*h)->stream)), "hipStreamSynchronize");
            }
            break;
    }
}

struct RegisterHipDevice {
    RegisterHipDevice() {
        HardAllocator::Register(DEVICE, hip_allocator);
        HardConverter::Register(DEVICE, DEVICE, hip_from_hip);
        HardConverter::Register(DEVICE, CPU, hip_from_cpu);
        HardConverter::Register(CPU, DEVICE, cpu_from_hip);
        ComputingMemory::Register(DEVICE, DEVICE);
        DeviceAdmin::Register(DEVICE, hip_admin);
    }
} register_hip_device;

}  // namespace

void *current_stream() { return stream_of_context(); }

int context_device_id() {
    auto *context = ctx::get<DeviceContext>();
    if (context && context->handle) return reinterpret_cast<HipContextHandle *>(context->handle)->device_id;
    return 0;
}

void check(int tsx_rc, const char *what) {
    if (tsx_rc != 0) TS_LOG_ERROR << "[hip] " << what << " failed (" << tsx_rc << "): " << tsx_last_error() << eject;
}

}  // namespace hip
}  // namespace ts

// How many operator runs on device "hip" were handed to the host operator so far in this process (inputs a "hip"
// class does not cover).  Tests hold it still around every case the device must compute itself.
extern "C" __attribute__((visibility("default"))) long tsx_hip_host_delegate_count() { return ts::hip::g_host_delegate_runs.load(); }
