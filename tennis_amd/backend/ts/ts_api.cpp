// Implementation of the API slice declared in ts_api.h (see that header for the reference
// interfaces each part restates).
#include "ts_api.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <mutex>

namespace ts {

// ---------------------------------------------------------------- dtype
int type_bytes(DTYPE dtype) {
    switch (dtype) {
        case VOID: return 0;
        case INT8: case UINT8: case CHAR8: case UNKNOWN8: case BOOLEAN: return 1;
        case INT16: case UINT16: case FLOAT16: case CHAR16: case UNKNOWN16: return 2;
        case INT32: case UINT32: case FLOAT32: case CHAR32: case UNKNOWN32: return 4;
        case INT64: case UINT64: case FLOAT64: case UNKNOWN64: return 8;
        case PTR: return int(sizeof(void *));
        case UNKNOWN128: return 16;
    }
    return 0;
}

const char *type_str(DTYPE dtype) {
    switch (dtype) {
        case INT8: return "int8";
        case UINT8: return "uint8";
        case INT32: return "int32";
        case INT64: return "int64";
        case FLOAT32: return "float32";
        case FLOAT64: return "float64";
        case CHAR8: return "char8";
        case BOOLEAN: return "bool";
        default: return "unknown";
    }
}

// ---------------------------------------------------------------- registries
namespace {
template <typename K, typename V>
struct Registry {
    std::mutex mutex;
    std::map<K, V> map;
    void put(const K &k, const V &v) {
        std::lock_guard<std::mutex> lock(mutex);
        map[k] = v;
    }
    bool find(const K &k, V *v) {
        std::lock_guard<std::mutex> lock(mutex);
        auto it = map.find(k);
        if (it == map.end()) return false;
        *v = it->second;
        return true;
    }
};
Registry<DeviceType, HardAllocator::function> &allocators() { static Registry<DeviceType, HardAllocator::function> r; return r; }
Registry<std::pair<DeviceType, DeviceType>, HardConverter::function> &converters() {
    static Registry<std::pair<DeviceType, DeviceType>, HardConverter::function> r;
    return r;
}
Registry<DeviceType, DeviceType> &computing_memory() { static Registry<DeviceType, DeviceType> r; return r; }
Registry<DeviceType, DeviceAdmin::function> &admins() { static Registry<DeviceType, DeviceAdmin::function> r; return r; }
Registry<std::pair<DeviceType, std::string>, OperatorCreator::function> &creators() {
    static Registry<std::pair<DeviceType, std::string>, OperatorCreator::function> r;
    return r;
}

// The host itself: plain malloc/free and memcpy, registered like any other device.
void *cpu_allocator(int, size_t new_size, void *mem, size_t mem_size) {
    if (new_size == 0) {
        std::free(mem);
        return nullptr;
    }
    if (mem == nullptr) return std::malloc(new_size);
    void *fresh = std::malloc(new_size);
    if (fresh && mem_size) std::memcpy(fresh, mem, std::min(new_size, mem_size));
    std::free(mem);
    return fresh;
}
void cpu_converter(int, void *dst, int, const void *src, size_t size) { std::memcpy(dst, src, size); }
struct RegisterCpu {
    RegisterCpu() {
        HardAllocator::Register(CPU, cpu_allocator);
        HardConverter::Register(CPU, CPU, cpu_converter);
        ComputingMemory::Register(CPU, CPU);
    }
} register_cpu;
}  // namespace

void HardAllocator::Register(const DeviceType &device_type, const function &allocator) { allocators().put(device_type, allocator); }
HardAllocator::function HardAllocator::Query(const DeviceType &device_type) {
    function f;
    if (!allocators().find(device_type, &f)) TS_LOG_ERROR << "No allocator registered for device: " << device_type << eject;
    return f;
}
void HardConverter::Register(const DeviceType &dst, const DeviceType &src, const function &converter) {
    converters().put(std::make_pair(dst, src), converter);
}
HardConverter::function HardConverter::Query(const DeviceType &dst, const DeviceType &src) {
    function f;   // exact pair only, no fallback (src/core/memory.cpp:99-122)
    if (!converters().find(std::make_pair(dst, src), &f))
        TS_LOG_ERROR << "Can not access memory copy from " << src << " to " << dst << eject;
    return f;
}
void ComputingMemory::Register(const DeviceType &compute, const DeviceType &memory) { computing_memory().put(compute, memory); }
MemoryDevice ComputingMemory::Query(const ComputingDevice &compute_device) {
    DeviceType memory;
    if (!computing_memory().find(compute_device.type(), &memory))
        TS_LOG_ERROR << "No memory device registered for computing device: " << compute_device.type() << eject;
    return MemoryDevice(memory, compute_device.id());
}
void DeviceAdmin::Register(const DeviceType &device_type, const function &admin) { admins().put(device_type, admin); }
DeviceAdmin::function DeviceAdmin::Query(const DeviceType &device_type) {
    function f;
    admins().find(device_type, &f);   // devices without an admin (the host) return an empty function
    return f;
}

// ---------------------------------------------------------------- device context
namespace {
thread_local DeviceContext *g_context = nullptr;
}
void DeviceContext::initialize(const ComputingDevice &device) {
    finalize();
    computing_device = device;
    memory_device = ComputingMemory::Query(device);
    auto admin = DeviceAdmin::Query(device.type());
    if (admin) admin(&handle, device.id(), DeviceAdmin::INITIALIZATION);
}
void DeviceContext::finalize() {
    if (handle) {
        auto admin = DeviceAdmin::Query(computing_device.type());
        if (admin) admin(&handle, computing_device.id(), DeviceAdmin::FINALIZATION);
        handle = nullptr;
    }
}
void DeviceContext::active() const {
    auto admin = DeviceAdmin::Query(computing_device.type());
    if (admin) admin(const_cast<DeviceHandle **>(&handle), computing_device.id(), DeviceAdmin::ACTIVATION);
}
void DeviceContext::synchronize() const {
    auto admin = DeviceAdmin::Query(computing_device.type());
    if (admin) admin(const_cast<DeviceHandle **>(&handle), computing_device.id(), DeviceAdmin::SYNCHRONIZE);
}
DeviceContext *DeviceContext::Switch(DeviceContext *context) {
    // the outgoing context is synchronised before the switch (src/core/device_context.cpp:61-71)
    DeviceContext *previous = g_context;
    if (previous && previous != context) previous->synchronize();
    g_context = context;
    if (context) context->active();
    return previous;
}
namespace ctx {
template <> DeviceContext *get<DeviceContext>() { return g_context; }
template <> DeviceContext &ref<DeviceContext>() {
    if (!g_context) TS_LOG_ERROR << "Empty context:<ts::DeviceContext>" << eject;
    return *g_context;
}
}  // namespace ctx

// ---------------------------------------------------------------- memory and tensor
Memory::Hard::~Hard() {
    if (ptr) HardAllocator::Query(device.type())(device.id(), 0, ptr, capacity);
}
Memory::Memory(const MemoryDevice &device, size_t size) : m_device(device), m_size(size) {
    m_hard = std::make_shared<Hard>();
    m_hard->device = device;
    m_hard->capacity = size;
    if (size) {
        m_hard->ptr = HardAllocator::Query(device.type())(device.id(), size, nullptr, 0);
        if (!m_hard->ptr) TS_LOG_ERROR << "Out of memory: " << size << " bytes on " << device.type() << ":" << device.id() << eject;
    }
}
void memcpy(const Memory &dst, const Memory &src, size_t size) {
    if (!size) return;
    HardConverter::Query(dst.device().type(), src.device().type())(dst.device().id(), dst.data(), src.device().id(), src.data(), size);
}

std::string to_string(const Shape &shape) {
    std::ostringstream out;
    out << "[";
    for (size_t i = 0; i < shape.size(); ++i) out << (i ? ", " : "") << shape[i];
    out << "]";
    return out.str();
}

int Tensor::Prototype::count() const {
    int n = 1;
    for (auto d : m_sizes) n *= d;
    return n;
}

Tensor::Tensor(const MemoryDevice &device, DTYPE dtype, const Shape &sizes) : m_device(device), m_proto(dtype, sizes) {
    m_sync = std::make_shared<Sync>();
    m_sync->home = device;
    m_sync->copies[device] = Memory(device, size_t(m_proto.count()) * size_t(type_bytes(dtype)));
}
const MemoryDevice &Tensor::device() const { return m_device; }
void *Tensor::data() const {
    if (!m_sync) return nullptr;
    return m_sync->copies.at(m_device).data();
}
Tensor Tensor::view(const MemoryDevice &device) const {
    if (!m_sync) return *this;
    Tensor out = *this;
    out.m_device = device;
    if (m_sync->copies.count(device)) return out;
    const Memory &src = m_sync->copies.at(m_device);
    Memory dst(device, src.size());
    memcpy(dst, src, src.size());
    m_sync->copies[device] = dst;
    return out;
}
Tensor Tensor::Pack(const std::vector<Tensor> &fields) {
    if (fields.empty()) return Tensor();
    Tensor packed = fields[0];
    packed.m_fields.assign(fields.begin() + 1, fields.end());
    return packed;
}

Tensor Tensor::field(size_t offset) const {
    if (offset >= fields_count()) TS_LOG_ERROR << "Tensor offset output range error. Access index " << offset << " in range(" << fields_count() << ")" << eject;
    if (offset == 0) {
        Tensor first = *this;
        first.m_fields.clear();
        return first;
    }
    return m_fields[offset - 1];
}

Tensor Tensor::clone() const {
    if (!m_sync) return Tensor();
    Tensor out(m_device, m_proto);
    const Memory &src = m_sync->copies.at(m_device);
    memcpy(out.m_sync->copies.at(m_device), src, src.size());
    return out;
}
Tensor Tensor::reshape(const Shape &shape) const {
    Shape fixed = shape;
    int64_t known = 1;
    int infer = -1;
    for (size_t i = 0; i < fixed.size(); ++i) {
        if (fixed[i] < 0) {
            if (infer >= 0) TS_LOG_ERROR << "Can not reshape " << to_string(sizes()) << " to " << to_string(shape) << eject;
            infer = int(i);
        } else {
            known *= fixed[i];
        }
    }
    if (infer >= 0) {
        if (known == 0 || count() % known) TS_LOG_ERROR << "Can not reshape " << to_string(sizes()) << " to " << to_string(shape) << eject;
        fixed[size_t(infer)] = int32_t(count() / known);
        known *= fixed[size_t(infer)];
    }
    if (known != count()) TS_LOG_ERROR << "Can not reshape " << to_string(sizes()) << " to " << to_string(shape) << eject;
    Tensor out = *this;
    out.m_proto = Prototype(dtype(), fixed);
    return out;
}
void Tensor::broadcast() const {
    if (!m_sync) return;
    for (auto it = m_sync->copies.begin(); it != m_sync->copies.end();)
        it = (it->first == m_device) ? std::next(it) : m_sync->copies.erase(it);
    m_sync->home = m_device;
}

// ---------------------------------------------------------------- parameter helpers
namespace tensor {
Tensor build(DTYPE dtype, const Shape &shape, const void *data) {
    Tensor t(dtype, shape);
    const size_t bytes = size_t(t.count()) * size_t(type_bytes(dtype));
    if (bytes) std::memcpy(t.data(), data, bytes);
    return t;
}
Tensor from(const std::string &value) { return build(CHAR8, Shape({int32_t(value.size())}), value.data()); }
Tensor from(float value) { return build(FLOAT32, Shape(), &value); }
Tensor from(int value) { int32_t v = value; return build(INT32, Shape(), &v); }
Tensor from(bool value) { uint8_t v = value ? 1 : 0; return build(BOOLEAN, Shape(), &v); }

namespace {
double element_as_double(const Tensor &host, int i) {
    switch (host.dtype()) {
        case INT8: return host.data<int8_t>()[i];
        case UINT8: case BOOLEAN: case CHAR8: return host.data<uint8_t>()[i];
        case INT16: return host.data<int16_t>()[i];
        case UINT16: return host.data<uint16_t>()[i];
        case INT32: return host.data<int32_t>()[i];
        case UINT32: return host.data<uint32_t>()[i];
        case INT64: return double(host.data<int64_t>()[i]);
        case UINT64: return double(host.data<uint64_t>()[i]);
        case FLOAT32: return host.data<float>()[i];
        case FLOAT64: return host.data<double>()[i];
        default: TS_LOG_ERROR << "Can not convert dtype " << type_str(host.dtype()) << eject;
    }
}
}  // namespace

Tensor cast(DTYPE dtype, const Tensor &value) {
    Tensor host = value.view(MemoryDevice(CPU));
    if (host.dtype() == dtype) return host;
    Tensor out(dtype, host.sizes());
    const int n = host.count();
    for (int i = 0; i < n; ++i) {
        const double v = element_as_double(host, i);
        switch (dtype) {
            case INT8: out.data<int8_t>()[i] = int8_t(v); break;
            case UINT8: out.data<uint8_t>()[i] = uint8_t(v); break;
            case BOOLEAN: out.data<uint8_t>()[i] = v != 0; break;
            case INT32: out.data<int32_t>()[i] = int32_t(v); break;
            case INT64: out.data<int64_t>()[i] = int64_t(v); break;
            case FLOAT32: out.data<float>()[i] = float(v); break;
            case FLOAT64: out.data<double>()[i] = v; break;
            default: TS_LOG_ERROR << "Can not cast to dtype " << type_str(dtype) << eject;
        }
    }
    return out;
}
std::string to_string(const Tensor &value) {
    Tensor host = value.view(MemoryDevice(CPU));
    if (host.dtype() != CHAR8) TS_LOG_ERROR << "Can not convert dtype " << type_str(host.dtype()) << " to string" << eject;
    return std::string(host.data<char>(), size_t(host.count()));
}
int to_int(const Tensor &value) {
    if (value.count() != 1) TS_LOG_ERROR << "Can not convert count=" << value.count() << " tensor to int" << eject;
    return int(element_as_double(value.view(MemoryDevice(CPU)), 0));
}
float to_float(const Tensor &value) {
    if (value.count() != 1) TS_LOG_ERROR << "Can not convert count=" << value.count() << " tensor to float" << eject;
    return float(element_as_double(value.view(MemoryDevice(CPU)), 0));
}
bool to_bool(const Tensor &value) { return to_int(value) != 0; }
namespace array {
std::vector<float> to_float(const Tensor &value) {
    Tensor f = cast(FLOAT32, value);
    return std::vector<float>(f.data<float>(), f.data<float>() + f.count());
}
std::vector<int32_t> to_int(const Tensor &value) {
    Tensor f = cast(INT32, value);
    return std::vector<int32_t>(f.data<int32_t>(), f.data<int32_t>() + f.count());
}
}  // namespace array
}  // namespace tensor

// ---------------------------------------------------------------- stack
size_t Stack::relative2absolute(int i) const {
    return i >= 0 ? m_base + size_t(i) : m_stack.size() - size_t(-i);
}
Tensor *Stack::push(const Tensor &tensor) {
    m_stack.push_back(tensor);
    return &m_stack.back();
}
Tensor *Stack::index(int i) {
    const size_t at = relative2absolute(i);
    if (at < m_base || at >= m_stack.size()) TS_LOG_ERROR << "Access index " << i << " out of range of stack" << eject;
    return &m_stack[at];
}
const Tensor *Stack::index(int i) const { return const_cast<Stack *>(this)->index(i); }
void Stack::pop(size_t pop_size) {
    while (pop_size-- && m_stack.size() > m_base) m_stack.pop_back();
}
void Stack::erase(int i) { m_stack.erase(m_stack.begin() + std::ptrdiff_t(relative2absolute(i))); }
void Stack::erase(int beg, int end) {
    const size_t b = relative2absolute(beg), e = relative2absolute(end);
    if (b > e || e > m_stack.size()) TS_LOG_ERROR << "Erase range out of stack" << eject;
    m_stack.erase(m_stack.begin() + std::ptrdiff_t(b), m_stack.begin() + std::ptrdiff_t(e));
}
void Stack::push_base(int i) {
    m_base_stack.push_back(m_base);
    m_base = relative2absolute(i);
}
void Stack::pop_base() {
    if (m_base_stack.empty()) {
        m_base = 0;
        return;
    }
    m_base = m_base_stack.back();
    m_base_stack.pop_back();
}

// ---------------------------------------------------------------- operator
void Operator::init() {
    const auto missing = unsatisfied_fields();
    if (!missing.empty()) {
        std::ostringstream oss;
        oss << "Operator " << op() << "(" << name() << ") has unsatisfied fields: ";
        for (size_t i = 0; i < missing.size(); ++i) oss << (i ? ", " : "") << "\"" << missing[i] << "\"";
        TS_LOG_ERROR << oss.str() << eject;
    }
}
bool Operator::has(const std::string &param) const { return m_params.count(param) != 0; }
void Operator::set(const std::string &param, const Tensor &value) {
    const bool retention = !param.empty() && param[0] == retention_param_sign;
    if (!retention && !m_optional_fields.count(param) && !m_required_fields.count(param))
        TS_LOG_ERROR << "Unidentified param \"" << param << "\" for operator " << op() << eject;
    m_params[param] = value;
}
Tensor &Operator::get(const std::string &param) {
    auto it = m_params.find(param);
    if (it == m_params.end()) TS_LOG_ERROR << "Unidentified param \"" << param << "\"" << eject;
    return it->second;
}
const Tensor &Operator::get(const std::string &param) const { return const_cast<Operator *>(this)->get(param); }
void Operator::clear(const std::string &param) { m_params.erase(param); }
std::vector<std::string> Operator::unsatisfied_fields() const {
    std::vector<std::string> missing;
    for (auto &f : m_required_fields)
        if (!m_params.count(f)) missing.push_back(f);
    std::sort(missing.begin(), missing.end());
    return missing;
}
void Operator::field(const std::string &param, FieldAttr attr, const Tensor &default_value) {
    field(param, attr);
    m_params[param] = default_value;
}
void Operator::field(const std::string &param, FieldAttr attr) {
    if (attr == REQUIRED) {
        m_required_fields.insert(param);
        m_optional_fields.erase(param);
    } else {
        m_optional_fields.insert(param);
        m_required_fields.erase(param);
    }
}
std::string Operator::op() const {
    auto it = m_params.find("#op");
    return it == m_params.end() ? std::string() : tensor::to_string(it->second);
}
std::string Operator::name() const {
    auto it = m_params.find("#name");
    return it == m_params.end() ? std::string() : tensor::to_string(it->second);
}

void OperatorCreator::Register(const DeviceType &device_type, const std::string &operator_name, const function &creator) {
    creators().put(std::make_pair(device_type, operator_name), creator);
}
OperatorCreator::function OperatorCreator::Query(const DeviceType &device_type, const std::string &operator_name, bool strict) {
    function f;
    if (creators().find(std::make_pair(device_type, operator_name), &f)) return f;
    if (strict) return nullptr;
    DeviceType memory;   // the device's memory device, then the host (src/global/operator_factory.cpp:60-81)
    if (computing_memory().find(device_type, &memory) && memory != device_type &&
        creators().find(std::make_pair(memory, operator_name), &f))
        return f;
    if (device_type != DeviceType(CPU) && creators().find(std::make_pair(DeviceType(CPU), operator_name), &f)) return f;
    return nullptr;
}
Operator::shared OperatorCreator::Create(const DeviceType &device_type, const std::string &operator_name, bool strict) {
    auto creator = Query(device_type, operator_name, strict);
    if (!creator) throw OperatorNotFoundException("No operator \"" + operator_name + "\" registered on " + device_type.std());
    return creator();
}
void OperatorCreator::Clear() {
    std::lock_guard<std::mutex> lock(creators().mutex);
    creators().map.clear();
}

// ---------------------------------------------------------------- conv helpers and names
Size2D conv2d_forward(const Size2D &x, const Padding2D &padding, const KSize2D &ksize, const Stride2D &stride,
                      const Dilation2D &dilation) {
    Size2D y;   // integer division, as in the reference
    y.height = (x.height + padding.top + padding.bottom - (dilation.height * (ksize.height - 1) + 1)) / stride.height + 1;
    y.width = (x.width + padding.left + padding.right - (dilation.width * (ksize.width - 1) + 1)) / stride.width + 1;
    return y;
}

Size2D pooling2d_forward(const Size2D &x, const Padding2D &padding, const KSize2D &ksize, const Stride2D &stride) {
    Size2D y;
    y.height = int(std::ceil((x.height + padding.top + padding.bottom - ksize.height) / float(stride.height) + 1));
    y.width = int(std::ceil((x.width + padding.left + padding.right - ksize.width) / float(stride.width) + 1));
    return y;
}

namespace name {
const char *const type = "type";
const char *const padding_type = "padding_type";
const char *const ksize = "ksize";
const char *const NCHW = "NCHW";
const char *const NHWC = "NHWC";
const char *const format = "format";
const char *const padding = "padding";
const char *const padding_value = "padding_value";
const char *const stride = "stride";
const char *const dilation = "dilation";
const char *const kernel_packed = "kernel_packed";
const char *const dim = "dim";
const char *const epsilon = "epsilon";
const char *const scale = "scale";
const char *const quantize_scale = "quantize_scale";
const char *const dequantize_scales = "dequantize_scales";
const char *const winograd_mode = "winograd_mode";
const char *const kernel_winograd_transformed = "kernel_winograd_transformed";
namespace typo { const char *const dialations = "dialations"; }
}  // namespace name

}  // namespace ts
