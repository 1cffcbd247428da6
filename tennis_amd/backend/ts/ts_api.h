// Self-contained restatement of the slice of the TenniS C++ API that a device backend is
// written against (names, signatures and error behaviour as in the reference), so that the
// "hip" operator classes in ../hip build and run without the TenniS tree.  With the real
// TenniS headers on the include path (-DTSX_WITH_TENNIS) the same operator sources compile
// against TenniS itself and this header is not used.
//
// Reference interfaces restated (paths relative to the TenniS tree):
//   DTYPE, type_bytes                       include/core/dtype.h:11-90
//   DeviceType/Device/MemoryDevice/...      include/core/device.h:23-241
//   Shape, Tensor, Tensor::Prototype        include/core/tensor.h:23-350
//   HardAllocator / HardConverter           include/global/hard_allocator.h:46-118, hard_converter.h:16-62
//   ComputingMemory / DeviceAdmin           include/global/memory_device.h:35-66, device_admin.h:16-69
//   DeviceContext (ctx handle)              include/core/device_context.h:20-60
//   Stack                                   include/runtime/stack.h:22-373
//   Operator, field/set/get/init            include/runtime/operator.h:16-140, src/runtime/operator.cpp:26-193
//   OperatorCreator, TS_REGISTER_OPERATOR   include/global/operator_factory.h:20-97, src/global/operator_factory.cpp:34-100
//   TS_LOG_ERROR << eject, TS_AUTO_CHECK    include/utils/log.h:162-187, include/utils/assert.h
//   Padding2D/Stride2D/..., conv2d_forward  include/backend/common_structure.h:10-78, common_function.h:30-40
//   tensor::from/cast/to_* helpers          include/core/tensor_builder.h:55-150
#pragma once
#include <cstdint>
#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace ts {

// ---------------------------------------------------------------- errors and logging
class Exception : public std::exception {
public:
    Exception() = default;
    explicit Exception(const std::string &message) : m_message(message) {}
    const char *what() const noexcept override { return m_message.c_str(); }

private:
    std::string m_message;
};

class EjectionException : public Exception {
public:
    using Exception::Exception;
};

class OperatorNotFoundException : public Exception {
public:
    using Exception::Exception;
};

struct Eject {};
static const Eject eject{};

// `TS_LOG_ERROR << "msg" << eject;` throws EjectionException carrying the message.
class LogStream {
public:
    template <typename T>
    LogStream &operator<<(const T &value) {
        m_buffer << value;
        return *this;
    }
    [[noreturn]] void operator<<(const Eject &) { throw EjectionException(m_buffer.str()); }

private:
    std::ostringstream m_buffer;
};

#define TS_LOG_ERROR ::ts::LogStream()
#define TS_AUTO_CHECK(condition)                                                              \
    do {                                                                                      \
        if (!(condition)) TS_LOG_ERROR << "Check failed: (" #condition ")" << ::ts::eject;   \
    } while (0)

// ---------------------------------------------------------------- dtype
enum DTYPE {
    VOID = 0, INT8 = 1, UINT8 = 2, INT16 = 3, UINT16 = 4, INT32 = 5, UINT32 = 6, INT64 = 7, UINT64 = 8,
    FLOAT16 = 9, FLOAT32 = 10, FLOAT64 = 11, PTR = 12, CHAR8 = 13, CHAR16 = 14, CHAR32 = 15,
    UNKNOWN8 = 16, UNKNOWN16 = 17, UNKNOWN32 = 18, UNKNOWN64 = 19, UNKNOWN128 = 20, BOOLEAN = 21,
};
int type_bytes(DTYPE dtype);
const char *type_str(DTYPE dtype);

template <typename T> struct dtypeid;
template <> struct dtypeid<int8_t> { static const DTYPE id = INT8; };
template <> struct dtypeid<uint8_t> { static const DTYPE id = UINT8; };
template <> struct dtypeid<int32_t> { static const DTYPE id = INT32; };
template <> struct dtypeid<int64_t> { static const DTYPE id = INT64; };
template <> struct dtypeid<float> { static const DTYPE id = FLOAT32; };
template <> struct dtypeid<double> { static const DTYPE id = FLOAT64; };
template <> struct dtypeid<char> { static const DTYPE id = CHAR8; };
template <> struct dtypeid<bool> { static const DTYPE id = BOOLEAN; };

// ---------------------------------------------------------------- devices
// DeviceType is a fixed 8-byte string in the reference (names are at most 7 characters).
class DeviceType {
public:
    DeviceType() { m_name[0] = 0; }
    DeviceType(const char *name) { assign(name); }
    DeviceType(const std::string &name) { assign(name.c_str()); }
    std::string std() const { return m_name; }
    const char *c_str() const { return m_name; }
    bool operator==(const DeviceType &rhs) const { return std::strcmp(m_name, rhs.m_name) == 0; }
    bool operator!=(const DeviceType &rhs) const { return !(*this == rhs); }
    bool operator<(const DeviceType &rhs) const { return std::strcmp(m_name, rhs.m_name) < 0; }

private:
    void assign(const char *name) {
        if (std::strlen(name) > 7) TS_LOG_ERROR << "Device name too long (max 7): " << name << eject;
        std::strncpy(m_name, name, 8);
    }
    char m_name[8];
};
inline std::ostream &operator<<(std::ostream &out, const DeviceType &t) { return out << t.c_str(); }

static const char *const CPU = "cpu";
static const char *const HIP = "hip";   // this backend's device type

class Device {
public:
    Device() : m_type(CPU), m_id(0) {}
    Device(const DeviceType &type, int id = 0) : m_type(type), m_id(id) {}
    const DeviceType &type() const { return m_type; }
    int id() const { return m_id; }
    bool operator==(const Device &rhs) const { return m_type == rhs.m_type && m_id == rhs.m_id; }
    bool operator!=(const Device &rhs) const { return !(*this == rhs); }
    bool operator<(const Device &rhs) const { return m_type < rhs.m_type || (m_type == rhs.m_type && m_id < rhs.m_id); }

private:
    DeviceType m_type;
    int m_id;
};
class MemoryDevice : public Device { public: using Device::Device; MemoryDevice() = default; };
class ComputingDevice : public Device { public: using Device::Device; ComputingDevice() = default; };

// Memory management hooks a device backend registers at static-init time.
class HardAllocator {
public:
    // new_size == 0: free; mem == nullptr: malloc; else realloc keeping the first mem_size bytes
    using function = std::function<void *(int id, size_t new_size, void *mem, size_t mem_size)>;
    static void Register(const DeviceType &device_type, const function &allocator);
    static function Query(const DeviceType &device_type);
};
class HardConverter {
public:
    using function = std::function<void(int dst_id, void *dst, int src_id, const void *src, size_t size)>;
    static void Register(const DeviceType &dst_device_type, const DeviceType &src_device_type, const function &converter);
    static function Query(const DeviceType &dst_device_type, const DeviceType &src_device_type);
};
class ComputingMemory {
public:
    static void Register(const DeviceType &compute_device_type, const DeviceType &memory_device_type);
    static MemoryDevice Query(const ComputingDevice &compute_device);   // throws when unregistered
};
class DeviceHandle;
class DeviceAdmin {
public:
    enum Action { INITIALIZATION, FINALIZATION, ACTIVATION, SYNCHRONIZE };
    using function = std::function<void(DeviceHandle **handle, int device_id, Action action)>;
    static void Register(const DeviceType &device_type, const function &admin);
    static function Query(const DeviceType &device_type);
};

// The per-thread device context an operator finds while it runs (ctx::ref<DeviceContext>()).
class DeviceContext {
public:
    DeviceContext() = default;
    explicit DeviceContext(const ComputingDevice &device) { initialize(device); }
    ~DeviceContext() { finalize(); }
    DeviceContext(const DeviceContext &) = delete;
    DeviceContext &operator=(const DeviceContext &) = delete;
    void initialize(const ComputingDevice &device);
    void finalize();
    void active() const;
    void synchronize() const;
    DeviceHandle *handle = nullptr;
    ComputingDevice computing_device;
    MemoryDevice memory_device;
    // binds this context to the calling thread; returns the previous one
    static DeviceContext *Switch(DeviceContext *context);
};
namespace ctx {
template <typename T> T &ref();
template <> DeviceContext &ref<DeviceContext>();
template <typename T> T *get();
template <> DeviceContext *get<DeviceContext>();
}  // namespace ctx

// ---------------------------------------------------------------- tensor
class Shape {   // at most 7 extents, like otl::vector<int32_t, 7>
public:
    Shape() = default;
    Shape(std::initializer_list<int32_t> dims) { for (auto d : dims) push_back(d); }
    explicit Shape(const std::vector<int32_t> &dims) { for (auto d : dims) push_back(d); }
    void push_back(int32_t d) {
        if (m_size >= 7) TS_LOG_ERROR << "Shape holds at most 7 dims" << eject;
        m_dims[m_size++] = d;
    }
    void resize(size_t n) { if (n > 7) TS_LOG_ERROR << "Shape holds at most 7 dims" << eject; m_size = n; }
    size_t size() const { return m_size; }
    int32_t &operator[](size_t i) { return m_dims[i]; }
    const int32_t &operator[](size_t i) const { return m_dims[i]; }
    const int32_t *begin() const { return m_dims; }
    const int32_t *end() const { return m_dims + m_size; }
    void erase(const int32_t *first, const int32_t *last) {
        const size_t b = size_t(first - m_dims), e = size_t(last - m_dims);
        for (size_t i = e; i < m_size; ++i) m_dims[b + i - e] = m_dims[i];
        m_size -= e - b;
    }
    void insert(const int32_t *pos, int32_t d) {
        const size_t at = size_t(pos - m_dims);
        if (m_size >= 7) TS_LOG_ERROR << "Shape holds at most 7 dims" << eject;
        for (size_t i = m_size; i > at; --i) m_dims[i] = m_dims[i - 1];
        m_dims[at] = d;
        ++m_size;
    }
    bool operator==(const Shape &rhs) const { return m_size == rhs.m_size && std::equal(begin(), end(), rhs.begin()); }
    bool operator!=(const Shape &rhs) const { return !(*this == rhs); }
    std::vector<int32_t> std() const { return std::vector<int32_t>(begin(), end()); }

private:
    int32_t m_dims[7] = {0};
    size_t m_size = 0;
};
std::string to_string(const Shape &shape);

// Thrown by a HardAllocator that cannot serve a request (include/global/hard_allocator.h:20-44).
class OutOfMemoryException : public Exception {
public:
    explicit OutOfMemoryException(const MemoryDevice &device, size_t failed_size)
        : Exception(OutOfMemoryMessage(device, failed_size)), m_device(device), m_failed_size(failed_size) {}
    static std::string OutOfMemoryMessage(const MemoryDevice &device, size_t failed_size) {
        return "No enough memory on " + std::string(device.type().c_str()) + ":" + std::to_string(device.id()) + ", " +
               std::to_string(failed_size) + "B needed.";
    }
    const Device &device() const { return m_device; }
    size_t failed_size() const { return m_failed_size; }

private:
    MemoryDevice m_device;
    size_t m_failed_size;
};

// One allocation on one device, released through the device's HardAllocator.
class Memory {
public:
    Memory() = default;
    Memory(const MemoryDevice &device, size_t size);
    void *data() const { return m_hard ? m_hard->ptr : nullptr; }
    size_t size() const { return m_size; }
    const MemoryDevice &device() const { return m_device; }
    bool empty() const { return !m_hard; }

private:
    struct Hard {
        ~Hard();
        MemoryDevice device;
        void *ptr = nullptr;
        size_t capacity = 0;
    };
    std::shared_ptr<Hard> m_hard;
    MemoryDevice m_device;
    size_t m_size = 0;
};
void memcpy(const Memory &dst, const Memory &src, size_t size);

class Tensor {
public:
    class Prototype {
    public:
        Prototype() = default;
        Prototype(DTYPE dtype, const Shape &sizes) : m_dtype(dtype), m_sizes(sizes) {}
        DTYPE dtype() const { return m_dtype; }
        const Shape &sizes() const { return m_sizes; }
        size_t dims() const { return m_sizes.size(); }
        int32_t size(size_t i) const { return m_sizes[i]; }
        int count() const;
        int type_bytes() const { return ::ts::type_bytes(m_dtype); }
        bool operator==(const Prototype &rhs) const { return m_dtype == rhs.m_dtype && m_sizes == rhs.m_sizes; }

    private:
        DTYPE m_dtype = VOID;
        Shape m_sizes;
    };

    Tensor() = default;
    Tensor(const MemoryDevice &device, DTYPE dtype, const Shape &sizes);
    Tensor(DTYPE dtype, const Shape &sizes) : Tensor(MemoryDevice(CPU), dtype, sizes) {}
    Tensor(const MemoryDevice &device, const Prototype &proto) : Tensor(device, proto.dtype(), proto.sizes()) {}
    explicit Tensor(const Prototype &proto) : Tensor(MemoryDevice(CPU), proto) {}

    bool empty() const { return !m_sync; }
    const MemoryDevice &device() const;
    DTYPE dtype() const { return m_proto.dtype(); }
    const Shape &sizes() const { return m_proto.sizes(); }
    size_t dims() const { return m_proto.dims(); }
    int32_t size(size_t i) const { return m_proto.size(i); }
    int count() const { return m_proto.count(); }
    const Prototype &proto() const { return m_proto; }
    bool has_shape(const Shape &shape) const { return m_proto.sizes() == shape; }
    bool has_shape(std::initializer_list<int32_t> shape) const { return has_shape(Shape(shape)); }
    bool has_shape(int32_t d0) const { return has_shape(Shape({d0})); }

    void *data() const;
    template <typename T> T *data() const { return reinterpret_cast<T *>(data()); }
    template <typename T> T &data(size_t i) const { return data<T>()[i]; }

    // A tensor whose memory is valid on `device`: this one if it already lives there, else a copy
    // made through the registered HardConverter and cached next to the original (SyncMemory).
    Tensor view(const MemoryDevice &device) const;
    Tensor clone() const;                       // deep copy on the same device
    Tensor reshape(const Shape &shape) const;   // -1 infers one extent
    // marks this device's copy as the current one: cached copies on other devices are dropped
    void broadcast() const;

    // Packed tensors (include/core/tensor.h:230-242): an operator with several results pushes ONE tensor whose
    // fields are the results; field 0 is the tensor itself, `_field` nodes pick the others.
    static Tensor Pack(const std::vector<Tensor> &fields);
    Tensor field(size_t offset) const;
    size_t fields_count() const { return empty() ? 0 : 1 + m_fields.size(); }

private:
    struct Sync {
        MemoryDevice home;
        std::map<Device, Memory> copies;
    };
    std::shared_ptr<Sync> m_sync;
    MemoryDevice m_device;   // the copy this handle reads
    Prototype m_proto;
    std::vector<Tensor> m_fields;   // fields 1.. of a packed tensor
};

// ---------------------------------------------------------------- small parameter helpers
namespace tensor {
Tensor from(const std::string &value);
inline Tensor from(const char *value) { return from(std::string(value)); }
Tensor from(float value);
Tensor from(int value);
Tensor from(bool value);
template <typename T> Tensor from(T value);
template <> inline Tensor from<bool>(bool value) { return from(value); }
template <> inline Tensor from<float>(float value) { return from(value); }
template <> inline Tensor from<int>(int value) { return from(value); }
Tensor build(DTYPE dtype, const Shape &shape, const void *data);   // copies count*type_bytes from host
Tensor cast(DTYPE dtype, const Tensor &value);                     // host tensors, numeric dtypes
std::string to_string(const Tensor &value);
int to_int(const Tensor &value);
float to_float(const Tensor &value);
bool to_bool(const Tensor &value);
namespace array {
std::vector<float> to_float(const Tensor &value);
std::vector<int32_t> to_int(const Tensor &value);
}  // namespace array
}  // namespace tensor

// ---------------------------------------------------------------- stack
class Stack {
public:
    explicit Stack(const MemoryDevice &device) : m_device(device) {}
    Tensor make(DTYPE dtype, const Shape &shape) { return Tensor(m_device, dtype, shape); }
    Tensor make(DTYPE dtype, const Shape &shape, const MemoryDevice &device) { return Tensor(device, dtype, shape); }
    Tensor make(const Tensor::Prototype &proto) { return Tensor(m_device, proto); }
    Tensor make(const Tensor::Prototype &proto, const MemoryDevice &device) { return Tensor(device, proto); }
    Tensor *push(DTYPE dtype, const Shape &shape) { return push(make(dtype, shape)); }
    Tensor *push(DTYPE dtype, const Shape &shape, const MemoryDevice &device) { return push(make(dtype, shape, device)); }
    Tensor *push(const Tensor::Prototype &proto) { return push(make(proto)); }
    Tensor *push(const Tensor::Prototype &proto, const MemoryDevice &device) { return push(make(proto, device)); }
    Tensor *push(const Tensor &tensor);
    Tensor *index(int i);
    const Tensor *index(int i) const;
    Tensor &operator[](int i) { return *index(i); }
    const Tensor &operator[](int i) const { return *index(i); }
    Tensor &operator[](size_t i) { return *index(int(i)); }
    Tensor *top() { return index(-1); }
    void pop(size_t pop_size);
    void pop() { pop(1); }
    size_t size() const { return m_stack.size() - m_base; }
    void erase(int i);
    void erase(int beg, int end);
    void clear() { erase(0, int(size())); }
    size_t base() const { return m_base; }
    size_t rebase(size_t new_base) { std::swap(m_base, new_base); return new_base; }
    void push_base(int i);   // the frame starting at relative index i becomes the visible stack
    void pop_base();

private:
    size_t relative2absolute(int i) const;
    MemoryDevice m_device;
    std::vector<Tensor> m_stack;
    std::vector<size_t> m_base_stack;
    size_t m_base = 0;
};

// ---------------------------------------------------------------- operator
class Operator {
public:
    using self = Operator;
    using shared = std::shared_ptr<self>;
    enum FieldAttr { OPTIONAL, REQUIRED };
    const static char retention_param_sign = '#';

    virtual ~Operator() = default;
    // checks that every REQUIRED field was set; device operators call supper::init() first
    virtual void init();
    // inputs are stack[0..n-1]; pushes exactly one output and returns 1
    virtual int run(Stack &stack) = 0;
    virtual int infer(Stack &stack, std::vector<Tensor::Prototype> &output) = 0;

    bool has(const std::string &param) const;
    void set(const std::string &param, const Tensor &value);   // unknown names throw (STRICT checking)
    Tensor &get(const std::string &param);
    const Tensor &get(const std::string &param) const;
    void clear(const std::string &param);
    bool check_params() const { return unsatisfied_fields().empty(); }
    std::vector<std::string> unsatisfied_fields() const;
    void field(const std::string &param, FieldAttr attr, const Tensor &default_value);
    void field(const std::string &param, FieldAttr attr);
    std::string op() const;
    std::string name() const;
    const std::unordered_map<std::string, Tensor> &params() const { return m_params; }

private:
    std::unordered_map<std::string, Tensor> m_params;
    std::unordered_set<std::string> m_optional_fields;
    std::unordered_set<std::string> m_required_fields;
};

class OperatorCreator {
public:
    using function = std::function<Operator::shared(void)>;
    static void Register(const DeviceType &device_type, const std::string &operator_name, const function &creator);
    // exact (device, name), then the device's memory device, then -- unless strict -- "cpu"
    static function Query(const DeviceType &device_type, const std::string &operator_name, bool strict = false);
    static Operator::shared Create(const DeviceType &device_type, const std::string &operator_name, bool strict = false);
    static void Clear();
};

struct StaticAction {
    template <typename FUNC, typename... Args>
    explicit StaticAction(FUNC func, Args &&... args) { func(std::forward<Args>(args)...); }
};
#define TSX_CAT_(a, b) a##b
#define TSX_CAT(a, b) TSX_CAT_(a, b)
#define TS_STATIC_ACTION(func, ...) \
    namespace { ::ts::StaticAction TSX_CAT(_ts_static_action_, __LINE__)(func, ##__VA_ARGS__); }
#define TS_REGISTER_OPERATOR(CLASS_NAME, DEVICE_TYPE, OP_NAME)                                    \
    namespace {                                                                                   \
    static ::ts::Operator::shared TSX_CAT(_ts_creator_, __LINE__)() { return std::make_shared<CLASS_NAME>(); } \
    ::ts::StaticAction TSX_CAT(_ts_register_, __LINE__)(::ts::OperatorCreator::Register, DEVICE_TYPE, OP_NAME, \
                                                        TSX_CAT(_ts_creator_, __LINE__));         \
    }

// ---------------------------------------------------------------- conv structures
template <typename T> struct Aspect2D {
    Aspect2D() = default;
    Aspect2D(T top, T bottom, T left, T right) : top(top), bottom(bottom), left(left), right(right) {}
    T top = 0, bottom = 0, left = 0, right = 0;
};
template <typename T> struct Form2D {
    Form2D() = default;
    Form2D(T height, T width) : height(height), width(width) {}
    T height = 0, width = 0;
};
using Padding2D = Aspect2D<int32_t>;
using Stride2D = Form2D<int32_t>;
using KSize2D = Form2D<int32_t>;
using Dilation2D = Form2D<int32_t>;
using Size2D = Form2D<int32_t>;
enum Conv2DFormat { FORMAT_NCHW = 0, FORMAT_NHWC = 1 };
enum WinogradConv2DMode { F6X6_3X3 = 0, F2X2_3X3 = 1 };
// include/backend/common_structure.h:84-94
enum class Pooling2DType : int { MAX = 0, AVG = 1 };
enum class Padding2DType : int { BLACK = 0, COPY = 1, LOOP = 2, WHITE = 3 };
enum class Resize2DType : int { LINEAR = 0, CUBIC = 1, NEAREST = 2, HARD = 3 };   // include/backend/common_structure.h:96-101
// include/backend/common_function.h:14-20 (ceil of an fp32 quotient)
Size2D pooling2d_forward(const Size2D &x, const Padding2D &padding, const KSize2D &ksize, const Stride2D &stride);
Size2D conv2d_forward(const Size2D &x, const Padding2D &padding, const KSize2D &ksize, const Stride2D &stride,
                      const Dilation2D &dilation);

namespace name {
extern const char *const NCHW;
extern const char *const NHWC;
extern const char *const format;
extern const char *const padding;
extern const char *const padding_value;
extern const char *const stride;
extern const char *const dilation;
extern const char *const kernel_packed;
extern const char *const dim;
extern const char *const epsilon;
extern const char *const scale;
extern const char *const quantize_scale;
extern const char *const dequantize_scales;
extern const char *const winograd_mode;
extern const char *const kernel_winograd_transformed;
extern const char *const type;
extern const char *const padding_type;
extern const char *const ksize;
namespace typo { extern const char *const dialations; }
namespace layer {
inline const char *conv2d() { return "conv2d"; }
inline const char *conv2d_quantized() { return "conv2d_quantized"; }
inline const char *quantize() { return "quantize"; }
inline const char *inner_prod() { return "inner_prod"; }
inline const char *conv2d_winograd() { return "conv2d_winograd"; }
inline const char *winograd_transform_kernel() { return "winograd_transform_kernel"; }
inline const char *add_bias() { return "add_bias"; }
inline const char *relu() { return "relu"; }
inline const char *leaky_relu() { return "leaky_relu"; }
inline const char *add() { return "add"; }
inline const char *pooling2d() { return "pooling2d"; }
inline const char *global_pooling2d() { return "global_pooling2d"; }
inline const char *depthwise_conv2d() { return "depthwise_conv2d"; }
inline const char *concat() { return "concat"; }
inline const char *mul() { return "mul"; }
inline const char *softplus() { return "softplus"; }
inline const char *tanh() { return "tanh"; }
inline const char *resize2d() { return "_resize2d"; }
}  // namespace layer
}  // namespace name

}  // namespace ts
