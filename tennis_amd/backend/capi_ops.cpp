// extern "C" driver over the operator layer, used by the tests and by non-C++ hosts: create an
// operator by (device, name) through OperatorCreator, set its parameters, init(), and run it on
// host tensors the way TenniS's operator test runner does (tools/run_test/test_case.hpp:424-522:
// bench(device) -> offline_create(bubble, strict) -> offline_run).
#include <cstring>
#include <string>

#include "hip/tsx_ts.h"

extern "C" {

// dtype uses TenniS's DTYPE codes (include/core/dtype.h:11-47)
struct tsxop_tensor {
    const char *name;   // parameter name (ignored for inputs)
    int32_t dtype;
    int32_t ndim;
    const int32_t *shape;
    const void *data;
};

struct tsxop_output {
    int32_t dtype;
    int32_t ndim;
    int32_t shape[8];
    void *data;         // caller buffer
    int64_t capacity;   // bytes available
    int64_t bytes;      // bytes written
};

}  // extern "C"

namespace {

thread_local std::string g_error;

ts::Tensor host_tensor(const tsxop_tensor &t) {
    ts::Shape shape;
    for (int i = 0; i < t.ndim; ++i) shape.push_back(t.shape[i]);
    return ts::tensor::build(ts::DTYPE(t.dtype), shape, t.data);
}

template <typename F>
int guarded(F f) {
    try {
        f();
        return 0;
    } catch (const ts::OperatorNotFoundException &e) {
        g_error = e.what();
        return 2;
    } catch (const std::exception &e) {
        g_error = e.what();
        return 1;
    }
}

}  // namespace

extern "C" {

const char *tsxop_last_error() { return g_error.c_str(); }

// 1 when (device, op) has its own registration (no fallback), else 0.
int tsxop_is_registered(const char *device, const char *op) {
    return ts::OperatorCreator::Query(device, op, true) ? 1 : 0;
}

// Host-only half of the above: create, set parameters, init().  Touches no device, so it also
// runs where there is no GPU; returns like tsxop_run_op.
int tsxop_check_params(const char *device, const char *op, int strict, int nparams, const tsxop_tensor *params) {
    return guarded([&] {
        auto oper = ts::OperatorCreator::Create(device, op, strict != 0);
        oper->set("#op", ts::tensor::from(std::string(op)));
        oper->set("#name", ts::tensor::from(std::string(op)));
        for (int i = 0; i < nparams; ++i) oper->set(params[i].name, host_tensor(params[i]));
        oper->init();
    });
}

// Creates `op` for `device` (strict != 0: no fallback to the host operator), sets the parameters,
// runs init() and one run() on the inputs (host tensors; the operator views them on its own memory
// device), and copies the single output back.  `infer_only` != 0 stops after infer() and returns
// only dtype/shape.  Returns 0, 1 (operator raised: tsxop_last_error) or 2 (operator not found).
int tsxop_run_op(const char *device, int device_id, const char *op, int strict, int nparams, const tsxop_tensor *params,
                 int ninputs, const tsxop_tensor *inputs, int infer_only, tsxop_output *out) {
    return guarded([&] {
        ts::ComputingDevice computing(device, device_id);
        ts::DeviceContext context(computing);
        ts::DeviceContext *previous = ts::DeviceContext::Switch(&context);
        struct Restore {
            ts::DeviceContext *previous;
            ~Restore() { ts::DeviceContext::Switch(previous); }
        } restore{previous};

        auto oper = ts::OperatorCreator::Create(device, op, strict != 0);
        oper->set("#op", ts::tensor::from(std::string(op)));
        oper->set("#name", ts::tensor::from(std::string(op)));
        for (int i = 0; i < nparams; ++i) oper->set(params[i].name, host_tensor(params[i]));
        oper->init();

        ts::Stack stack(context.memory_device);
        for (int i = 0; i < ninputs; ++i) stack.push(host_tensor(inputs[i]));
        if (infer_only) {
            std::vector<ts::Tensor::Prototype> protos;
            if (oper->infer(stack, protos) != 1 || protos.size() != 1) throw ts::Exception("infer returned != 1 outputs");
            out->dtype = protos[0].dtype();
            out->ndim = int32_t(protos[0].dims());
            for (int i = 0; i < out->ndim; ++i) out->shape[i] = protos[0].size(size_t(i));
            out->bytes = 0;
            return;
        }
        const int returned = oper->run(stack);
        if (returned != 1 || int(stack.size()) != ninputs + 1) throw ts::Exception("operator returned != 1 outputs");
        ts::Tensor y = stack[ninputs].view(ts::MemoryDevice(ts::CPU));   // device -> host: synchronises the stream
        out->dtype = y.dtype();
        out->ndim = int32_t(y.dims());
        for (int i = 0; i < out->ndim; ++i) out->shape[i] = y.size(size_t(i));
        out->bytes = int64_t(y.count()) * ts::type_bytes(y.dtype());
        if (out->bytes > out->capacity) throw ts::Exception("output buffer too small");
        std::memcpy(out->data, y.data(), size_t(out->bytes));
    });
}

}  // extern "C"
