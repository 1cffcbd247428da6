// TEST INFRASTRUCTURE ONLY.  A thin extern "C" driver over the *compiled TenniS
// reference library* (oracle/_ref/libtennis_ref.so, built by oracle/ref.mk from
// the reference sources where they lie).  It lets the Python tests and the CPU
// baseline leg of bench.py run the reference's own operators on raw buffers.
// Nothing in the shipped product path links, loads or calls this file.
//
// Operators are driven exactly as the reference's operator test runner does
// (tools/run_test/test_case.hpp:424-522): Workbench(cpu) -> offline_create(bubble,
// strict=true) -> offline_run.  Two algorithm-level entry points are exposed
// directly because no operator reaches them on x86: Winograd F(6,3)
// (src/kernels/cpu/winograd_algorithm.cpp:846-947) and the int8 GEMM primitive
// (src/kernels/cpu/math_cpu.cpp:238-244).
#include <cstdint>
#include <chrono>
#include <cstring>
#include <string>
#include <vector>
#include <memory>
#include <exception>
#include <map>
#include <stdexcept>
#include <dlfcn.h>

#include "runtime/workbench.h"
#include "module/bubble.h"
#include "module/module.h"
#include "core/tensor.h"
#include "core/tensor_builder.h"
#include "backend/common_structure.h"
#include "kernels/cpu/winograd_algorithm.h"
#include "kernels/cpu/math_cpu.h"
#include "global/setup.h"
#include "global/memory_device.h"
#include "utils/ctxmgr_lite.h"

extern "C" {

// A host tensor crossing the boundary.  dtype uses the reference's DTYPE codes
// (include/core/dtype.h:11-47): INT8=1, INT32=5, FLOAT32=10, CHAR8=13, BOOLEAN=21.
struct ref_tensor {
    const char *name;   // parameter name (ignored for inputs)
    int32_t dtype;
    int32_t ndim;
    const int32_t *shape;
    const void *data;
};

struct ref_output {
    int32_t dtype;
    int32_t ndim;
    int32_t shape[8];
    void *data;          // caller-provided buffer
    int64_t capacity;    // bytes available in data
    int64_t bytes;       // bytes written
};

static thread_local std::string g_last_error;

const char *ref_last_error() { return g_last_error.c_str(); }

}  // extern "C"

namespace {

ts::Tensor make_tensor(const ref_tensor &t) {
    ts::Shape shape;
    for (int i = 0; i < t.ndim; ++i) shape.push_back(t.shape[i]);
    ts::Tensor out(ts::DTYPE(t.dtype), shape);
    size_t bytes = size_t(out.count()) * size_t(ts::type_bytes(ts::DTYPE(t.dtype)));
    if (bytes) std::memcpy(out.data(), t.data, bytes);
    return out;
}

struct Bench {
    std::shared_ptr<ts::Workbench> bench;
    int threads = -1;
};

Bench &bench_for(int threads, const std::string &device = ts::CPU) {
    static thread_local std::map<std::string, Bench> benches;
    Bench &b = benches[device];
    if (!b.bench) {
        ts::setup();
        b.bench = std::make_shared<ts::Workbench>(ts::ComputingDevice(device, 0));
    }
    if (b.threads != threads) {
        b.bench->runtime().set_computing_thread_number(threads);
        b.threads = threads;
    }
    return b;
}

// Algorithm-level calls allocate scratch tensors "in flow", which needs the same
// thread-local contexts Workbench binds around its own entry points
// (src/runtime/workbench.cpp:32-65).
struct BindAll {
    explicit BindAll(ts::Workbench &bench)
        : rt(bench.runtime()), wb(bench), prev(ts::DeviceContext::Switch(&bench.device())) {}
    ~BindAll() { ts::DeviceContext::Switch(prev); }
    ts::ctx::bind<ts::RuntimeContext> rt;
    ts::ctx::bind<ts::Workbench> wb;
    ts::DeviceContext *prev;
};

template <typename F>
int guarded(F f) {
    try {
        f();
        return 0;
    } catch (const std::exception &e) {
        g_last_error = e.what();
        return 1;
    } catch (...) {
        g_last_error = "unknown exception";
        return 1;
    }
}

}  // namespace

extern "C" {

// Load a device plugin (a shared library whose static initialisers register operators and
// device plumbing with this process's TenniS registries, e.g. the "hip" backend compiled
// against the real TenniS headers).
int ref_load_plugin(const char *path) {
    return guarded([&] {
        if (!dlopen(path, RTLD_NOW | RTLD_GLOBAL)) throw std::runtime_error(dlerror());
    });
}

int ref_run_op_on(const char *device, int strict, const char *op, int nparams, const ref_tensor *params, int ninputs,
                  const ref_tensor *inputs, int threads, ref_output *out);

// Run one reference operator on the CPU device.  Returns 0 on success.
int ref_run_op(const char *op, int nparams, const ref_tensor *params, int ninputs,
               const ref_tensor *inputs, int threads, ref_output *out) {
    return ref_run_op_on(ts::CPU, 1, op, nparams, params, ninputs, inputs, threads, out);
}

// Same, on a Workbench of the named computing device: the operator is looked up the way the
// runtime does it: strict = this device only; otherwise device -> its memory device -> cpu, the
// order a compiled graph uses (src/global/operator_factory.cpp:60-81).
int ref_run_op_on(const char *device, int strict, const char *op, int nparams, const ref_tensor *params, int ninputs,
                  const ref_tensor *inputs, int threads, ref_output *out) {
    return guarded([&] {
        Bench &b = bench_for(threads, device);
        ts::ctx::bind<ts::RuntimeContext> bind_rt(b.bench->runtime());
        ts::Bubble bubble(op, op, 1);
        for (int i = 0; i < nparams; ++i) bubble.set(params[i].name, make_tensor(params[i]));
        auto oper = b.bench->offline_create(bubble, strict != 0);
        if (!oper) throw std::runtime_error(std::string("no operator ") + op);
        std::vector<ts::Tensor> in, res;
        for (int i = 0; i < ninputs; ++i) in.push_back(make_tensor(inputs[i]));
        b.bench->offline_run(oper, in, res);
        if (res.size() != 1) throw std::runtime_error("operator returned != 1 outputs");
        ts::Tensor y = res[0].view(ts::MemoryDevice(ts::CPU));
        out->dtype = int32_t(y.dtype());
        out->ndim = int32_t(y.dims());
        for (int i = 0; i < out->ndim && i < 8; ++i) out->shape[i] = y.size(i);
        out->bytes = int64_t(y.count()) * ts::type_bytes(y.dtype());
        if (out->bytes > out->capacity) throw std::runtime_error("output buffer too small");
        std::memcpy(out->data, y.data(), size_t(out->bytes));
    });
}

// The reference's own tensor file format (`.t`: Tensor::serialize / externalize, src/core/tensor.cpp:314-389,
// through tensor::save / tensor::load, include/core/tensor_builder.h:153-159): written and read by the compiled
// library itself, to make fixtures for and cross-check an independent reader / writer of the format.
int ref_save_tensor(const char *path, const ref_tensor *t) {
    return guarded([&] { ts::tensor::save(path, make_tensor(*t)); });
}

int ref_load_tensor(const char *path, ref_output *out) {
    return guarded([&] {
        ts::Tensor y = ts::tensor::load(path);
        if (y.fields_count() != 1) throw std::runtime_error("packed tensors are not supported by this driver");
        out->dtype = int32_t(y.dtype());
        out->ndim = int32_t(y.dims());
        for (int i = 0; i < out->ndim && i < 8; ++i) out->shape[i] = y.size(i);
        out->bytes = int64_t(y.count()) * ts::type_bytes(y.dtype());
        if (out->bytes > out->capacity) throw std::runtime_error("output buffer too small");
        std::memcpy(out->data, y.data(), size_t(out->bytes));
    });
}

// A module file (`.tsm`, Module::Load, src/module/module.cpp:295-330) loaded into a Workbench of the named
// computing device and run once: the reference's own reader, graph compiler and runtime, to cross-check an
// independent reader / writer / runner of the format.  Copies output slot 0 back.
int ref_run_module(const char *path, const char *device, int ninputs, const ref_tensor *inputs, int threads, ref_output *out) {
    return guarded([&] {
        auto module = ts::Module::Load(path);
        auto bench = ts::Workbench::Load(module, ts::ComputingDevice(device, 0));
        bench->runtime().set_computing_thread_number(threads);
        for (int i = 0; i < ninputs; ++i) bench->input(i, make_tensor(inputs[i]));
        bench->run();
        ts::Tensor y = bench->output(0).view(ts::MemoryDevice(ts::CPU));
        out->dtype = int32_t(y.dtype());
        out->ndim = int32_t(y.dims());
        for (int i = 0; i < out->ndim && i < 8; ++i) out->shape[i] = y.size(i);
        out->bytes = int64_t(y.count()) * ts::type_bytes(y.dtype());
        if (out->bytes > out->capacity) throw std::runtime_error("output buffer too small");
        std::memcpy(out->data, y.data(), size_t(out->bytes));
    });
}

// The same, timed: the module is loaded and compiled once, run `warmup` times, then `reps` times against the wall
// clock; every run ends with output 0 read back to the host (the one synchronisation a caller of the runtime
// sees).  Inputs are bound once.  A host tensor bound to a Workbench is copied to the device by the first operator
// that reads it, on EVERY run (new data each run is the normal case); with resident != 0 the inputs are moved to
// the device's memory before the loop and bound from there, the case of a caller whose data is already on the
// device.
int ref_time_module(const char *path, const char *device, int ninputs, const ref_tensor *inputs, int threads, int warmup,
                    int reps, int resident, double *ms_per_run, ref_output *out) {
    return guarded([&] {
        auto module = ts::Module::Load(path);
        const ts::ComputingDevice computing(device, 0);
        auto bench = ts::Workbench::Load(module, computing);
        bench->runtime().set_computing_thread_number(threads);
        for (int i = 0; i < ninputs; ++i) {
            ts::Tensor t = make_tensor(inputs[i]);
            if (resident) {
                BindAll bind(*bench);   // the converters need the device context
                t = t.view(ts::ComputingMemory::Query(computing));
            }
            bench->input(i, t);
        }
        ts::Tensor y;
        for (int r = 0; r < warmup; ++r) {
            bench->run();
            y = bench->output(0).view(ts::MemoryDevice(ts::CPU));
        }
        const auto t0 = std::chrono::steady_clock::now();
        for (int r = 0; r < reps; ++r) {
            bench->run();
            y = bench->output(0).view(ts::MemoryDevice(ts::CPU));
        }
        const auto t1 = std::chrono::steady_clock::now();
        *ms_per_run = std::chrono::duration<double, std::milli>(t1 - t0).count() / (reps > 0 ? reps : 1);
        out->dtype = int32_t(y.dtype());
        out->ndim = int32_t(y.dims());
        for (int i = 0; i < out->ndim && i < 8; ++i) out->shape[i] = y.size(i);
        out->bytes = int64_t(y.count()) * ts::type_bytes(y.dtype());
        if (out->bytes > out->capacity) throw std::runtime_error("output buffer too small");
        std::memcpy(out->data, y.data(), size_t(out->bytes));
    });
}

// Conv2dWinogradAlgorithm<float>::winograd_f63 / winograd_f23 on raw weights
// (kernel_transformed=false).  pad = {top, bottom, left, right}.
int ref_winograd(int f63, const float *x, int n, int c, int h, int w, const float *k, int cout,
                 const int *pad, float padding_value, float *out, int ho, int wo, int threads) {
    return guarded([&] {
        Bench &b = bench_for(threads);
        BindAll bind(*b.bench);
        ts::Tensor tx(ts::FLOAT32, {n, c, h, w});
        ts::Tensor tk(ts::FLOAT32, {cout, c, 3, 3});
        ts::Tensor ty(ts::FLOAT32, {n, cout, ho, wo});
        std::memcpy(tx.data(), x, sizeof(float) * size_t(tx.count()));
        std::memcpy(tk.data(), k, sizeof(float) * size_t(tk.count()));
        ts::Padding2D padding(pad[0], pad[1], pad[2], pad[3]);
        if (f63)
            ts::cpu::Conv2dWinogradAlgorithm<float>::winograd_f63(tx, padding, padding_value, tk, ty, false);
        else
            ts::cpu::Conv2dWinogradAlgorithm<float>::winograd_f23(tx, padding, padding_value, tk, ty, false);
        std::memcpy(out, ty.data(), sizeof(float) * size_t(ty.count()));
    });
}

// cpu::math<int8,int32>::gemm(NoTrans, NoTrans, M, N, K, 1, A, B, 0, C), row-major.
int ref_gemm_i8(int m, int n, int k, const int8_t *a, const int8_t *bm, int32_t *c) {
    return guarded([&] {
        ts::cpu::math<int8_t, int32_t>::gemm(ts::blas::NoTrans, ts::blas::NoTrans, m, n, k, 1, a, bm, 0, c);
    });
}

// cpu::math<float,float>::gemm(M,N,K,1,A,B,0,C, pack A, pack B): the pack8 + kernel_8x8 path.
int ref_gemm_f32(int m, int n, int k, const float *a, const float *bm, float *c, int threads) {
    return guarded([&] {
        Bench &b = bench_for(threads);
        BindAll bind(*b.bench);
        ts::cpu::math<float, float>::gemm(m, n, k, 1.f, a, bm, 0.f, c, true, true);
    });
}

}  // extern "C"
