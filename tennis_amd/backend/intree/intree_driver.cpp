// extern "C" access to TenniS's own runtime with this repository's "hip" device backend built into it
// (libtennis_hip.so, intree.mk): what an application linking that library does in C++ -- load a module into a
// Workbench on ComputingDevice("hip"), bind inputs, run, read outputs -- reachable from Python for the in-tree tests
// and the network-through-the-runtime figure.  The operator entry follows the reference's operator test runner
// (tools/run_test/test_case.hpp:424-522): Workbench(device) -> offline_create(bubble, strict) -> offline_run.
#include <atomic>
#include <chrono>
#include <cstdint>
#include <cstring>
#include <exception>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include "core/tensor.h"
#include "global/memory_device.h"
#include "global/setup.h"
#include "module/bubble.h"
#include "module/module.h"
#include "runtime/workbench.h"
#include "utils/ctxmgr_lite.h"

extern "C" long tsx_hip_fused_chain_count();
extern "C" long tsx_hip_handover_count();
extern "C" long tsx_hip_dual_output_count();
extern "C" long tsx_hip_host_delegate_count();

extern "C" {

// A host tensor crossing the boundary; dtype in TenniS's DTYPE codes (include/core/dtype.h:11-47)
struct intree_tensor {
    const char *name;   // parameter name (ignored for inputs)
    int32_t dtype;
    int32_t ndim;
    const int32_t *shape;
    const void *data;
};

struct intree_output {
    int32_t dtype;
    int32_t ndim;
    int32_t shape[8];
    void *data;          // caller-provided buffer
    int64_t capacity;    // bytes available in data
    int64_t bytes;       // bytes written
};

static thread_local std::string g_last_error;

const char *intree_last_error() { return g_last_error.c_str(); }

}  // extern "C"

namespace {

ts::Tensor make_tensor(const intree_tensor &t) {
    ts::Shape shape;
    for (int i = 0; i < t.ndim; ++i) shape.push_back(t.shape[i]);
    ts::Tensor out(ts::DTYPE(t.dtype), shape);
    const size_t bytes = size_t(out.count()) * size_t(ts::type_bytes(ts::DTYPE(t.dtype)));
    if (bytes) std::memcpy(out.data(), t.data, bytes);
    return out;
}

void copy_out(const ts::Tensor &device_tensor, intree_output *out) {
    ts::Tensor y = device_tensor.view(ts::MemoryDevice(ts::CPU));
    out->dtype = int32_t(y.dtype());
    out->ndim = int32_t(y.dims());
    for (int i = 0; i < out->ndim && i < 8; ++i) out->shape[i] = y.size(i);
    out->bytes = int64_t(y.count()) * ts::type_bytes(y.dtype());
    if (out->bytes > out->capacity) throw std::runtime_error("output buffer too small");
    std::memcpy(out->data, y.data(), size_t(out->bytes));
}

struct Bench {
    std::shared_ptr<ts::Workbench> bench;
    int threads = -1;
};

Bench &bench_for(int threads, const std::string &device) {
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

// the thread-local contexts Workbench binds around its own entry points (src/runtime/workbench.cpp:32-65), for
// tensor conversions made outside them
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

// One operator in a Workbench of the named computing device ("cpu" or "hip").  strict: the operator registered
// for this device only; otherwise device -> its memory device -> cpu, the order a compiled graph uses
// (src/global/operator_factory.cpp:60-81).
int intree_run_op(const char *device, int strict, const char *op, int nparams, const intree_tensor *params, int ninputs,
                  const intree_tensor *inputs, int threads, intree_output *out) {
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
        copy_out(res[0], out);
    });
}

// A module file (`.tsm`, Module::Load, src/module/module.cpp:295-330) loaded into a Workbench of the named device
// and run once: TenniS's reader, graph compiler and runtime.  Copies output slot 0 back.
int intree_run_module(const char *path, const char *device, int ninputs, const intree_tensor *inputs, int threads,
                      intree_output *out) {
    return guarded([&] {
        auto module = ts::Module::Load(path);
        auto bench = ts::Workbench::Load(module, ts::ComputingDevice(device, 0));
        bench->runtime().set_computing_thread_number(threads);
        for (int i = 0; i < ninputs; ++i) bench->input(i, make_tensor(inputs[i]));
        bench->run();
        copy_out(bench->output(0), out);
    });
}

// The same, timed: loaded and compiled once, run `warmup` times, then `reps` times against the wall clock; every
// run ends with output 0 read back to the host (the one synchronisation a caller of the runtime sees).  A host
// tensor bound to a Workbench is copied to the device by the first operator that reads it, on every run; with
// resident != 0 the inputs are moved to the device's memory before the loop and bound from there.
int intree_time_module(const char *path, const char *device, int ninputs, const intree_tensor *inputs, int threads,
                       int warmup, int reps, int resident, double *ms_per_run, intree_output *out) {
    return guarded([&] {
        auto module = ts::Module::Load(path);
        const ts::ComputingDevice computing(device, 0);
        auto bench = ts::Workbench::Load(module, computing);
        bench->runtime().set_computing_thread_number(threads);
        for (int i = 0; i < ninputs; ++i) {
            ts::Tensor t = make_tensor(inputs[i]);
            if (resident) {
                BindAll bind(*bench);
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
        copy_out(y, out);
    });
}

// TenniS's threading contract (include/utils/ctxmgr_lite_support.h:13,47-95; Workbench::clone,
// src/runtime/workbench.cpp; OperatorInstruction::clone, src/runtime/instruction.cpp:91-103): one Workbench per
// thread, further ones cloned from the first.  The module is loaded once on `device`; the Workbench is cloned
// `nthreads - 1` times; thread t then runs its own Workbench `runs` times on input set t (ninputs tensors each,
// inputs[t * ninputs + i]) and keeps output 0 of its last run in outs[t].  All threads start together.
int intree_run_module_cloned(const char *path, const char *device, int nthreads, int runs, int ninputs,
                             const intree_tensor *inputs, intree_output *outs) {
    return guarded([&] {
        if (nthreads < 1 || runs < 1) throw std::runtime_error("nthreads and runs must be positive");
        auto module = ts::Module::Load(path);
        std::vector<std::shared_ptr<ts::Workbench>> benches;
        benches.push_back(ts::Workbench::Load(module, ts::ComputingDevice(device, 0)));
        benches[0]->runtime().set_computing_thread_number(1);
        for (int t = 1; t < nthreads; ++t) benches.push_back(benches[0]->clone());
        std::vector<std::string> errors;
        errors.resize(size_t(nthreads));
        std::atomic<int> ready{0};
        std::vector<std::thread> pool;
        for (int t = 0; t < nthreads; ++t) {
            pool.emplace_back([&, t] {
                try {
                    auto &bench = *benches[size_t(t)];
                    for (int i = 0; i < ninputs; ++i) bench.input(i, make_tensor(inputs[t * ninputs + i]));
                    ready.fetch_add(1);
                    while (ready.load() < nthreads) std::this_thread::yield();
                    for (int r = 0; r < runs; ++r) {
                        bench.run();
                        copy_out(bench.output(0), &outs[t]);
                    }
                } catch (const std::exception &e) {
                    ready.fetch_add(nthreads);   // never leave the others spinning
                    errors[size_t(t)] = e.what();
                } catch (...) {
                    ready.fetch_add(nthreads);
                    errors[size_t(t)] = "unknown exception";
                }
            });
        }
        for (auto &th : pool) th.join();
        for (int t = 0; t < nthreads; ++t)
            if (!errors[size_t(t)].empty()) throw std::runtime_error("thread " + std::to_string(t) + ": " + errors[size_t(t)]);
    });
}

// Chains replaced by the "hip" device's zipper option so far; of which write a staged int8 output for the
// convolutions behind them / return the fp32 form as well; operator runs handed to the host operator.
long intree_fused_chain_count() { return tsx_hip_fused_chain_count(); }
long intree_handover_count() { return tsx_hip_handover_count(); }
long intree_dual_output_count() { return tsx_hip_dual_output_count(); }
long intree_host_delegate_count() { return tsx_hip_host_delegate_count(); }

}  // extern "C"
