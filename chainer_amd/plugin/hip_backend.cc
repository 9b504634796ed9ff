// ChainerX backend plugin `hip`: the Backend/Device pair and the kernel classes that forward to
// the C ABI of libhipcx.so (include/hipcx.h).
//
// Build inside a ChainerX checkout (it needs libchainerx's headers and its abseil/gsl-lite), e.g.
//   hipcc -std=c++14 -fPIC -shared -I<chainerx_cc> -I<abseil> -I<gsl-lite>/include -I<repo>/include \
//         hip_backend.cc -L<repo>/chainer_amd -lhipcx -lchainerx -o $CHAINERX_PATH/backends/hip.so
// The file name is the backend name: chainerx.get_device('hip:0') loads it through
// Context::GetBackend (chainerx/context.cc:84-111), which looks up the two extern "C" functions at
// the bottom of this file.
//
// Every kernel below follows the conventions of the reference's own backends
// (chainerx/native/kernel_regist.h:15-70, chainerx/cuda/kernel_regist.h:15-17): check devices, make
// the device current, cast inputs to out's dtype with AsType, honour strides/offset, launch
// asynchronously on the default stream.  Nothing is registered from the native backend's registry:
// its kernels would dereference device pointers on the host.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <limits>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include <absl/types/optional.h>

#include "chainerx/array.h"
#include "chainerx/axes.h"
#include "chainerx/backend.h"
#include "chainerx/backend_util.h"
#include "chainerx/context.h"
#include "chainerx/device.h"
#include "chainerx/dims.h"
#include "chainerx/dtype.h"
#include "chainerx/error.h"
#include "chainerx/kernel_registry.h"
#include "chainerx/kernels/arithmetic.h"
#include "chainerx/kernels/binary.h"
#include "chainerx/kernels/connection.h"
#include "chainerx/kernels/creation.h"
#include "chainerx/kernels/explog.h"
#include "chainerx/kernels/hyperbolic.h"
#include "chainerx/kernels/indexing.h"
#include "chainerx/kernels/linalg.h"
#include "chainerx/kernels/logic.h"
#include "chainerx/kernels/misc.h"
#include "chainerx/kernels/normalization.h"
#include "chainerx/kernels/pooling.h"
#include "chainerx/kernels/reduction.h"
#include "chainerx/kernels/rnn.h"
#include "chainerx/kernels/rounding.h"
#include "chainerx/kernels/sorting.h"
#include "chainerx/kernels/statistics.h"
#include "chainerx/kernels/trigonometric.h"
#include "chainerx/native/native_backend.h"
#include "chainerx/routines/connection.h"
#include "chainerx/routines/creation.h"
#include "chainerx/routines/indexing.h"
#include "chainerx/routines/logic.h"
#include "chainerx/routines/manipulation.h"
#include "chainerx/native/tensor_dot.h"
#include "chainerx/array_index.h"
#include "chainerx/slice.h"
#include "chainerx/scalar.h"
#include "chainerx/shape.h"

#include "hipcx.h"

namespace chainerx {
namespace hip {
namespace {

void CheckHip(hipError_t e, const char* what) {
    if (e != hipSuccess) throw BackendError{what, ": ", hipGetErrorString(e)};
}

// The error of a device allocation that fails even after the pool has released its cache (the CUDA backend's class of the
// same name, chainerx/cuda/memory_pool.h:34-37, lives in that backend's namespace and is not visible to a plugin).
class OutOfMemoryError : public ChainerxError {
public:
    using ChainerxError::ChainerxError;
};

// hipcx_status -> the ChainerX exception class named by it (chainerx/error.h:48-95).
void Check(int status) {
    if (status == HIPCX_OK) return;
    std::string msg = hipcx_last_error();
    switch (status) {
        case HIPCX_OUT_OF_MEMORY_ERROR: throw OutOfMemoryError{msg};
        case HIPCX_DIMENSION_ERROR: throw DimensionError{msg};
        case HIPCX_DTYPE_ERROR: throw DtypeError{msg};
        case HIPCX_NOT_IMPLEMENTED_ERROR: throw NotImplementedError{msg};
        case HIPCX_INDEX_ERROR: throw IndexError{msg};
        case HIPCX_BACKEND_ERROR: throw BackendError{msg};
        case HIPCX_DEVICE_ERROR: throw DeviceError{msg};
        default: throw ChainerxError{msg};
    }
}

class SetDeviceScope {
public:
    explicit SetDeviceScope(int index) {
        CheckHip(hipGetDevice(&prev_), "hipGetDevice");
        if (prev_ != index) CheckHip(hipSetDevice(index), "hipSetDevice");
        index_ = index;
    }
    ~SetDeviceScope() {
        if (prev_ != index_) (void)hipSetDevice(prev_);
    }
    SetDeviceScope(const SetDeviceScope&) = delete;
    SetDeviceScope& operator=(const SetDeviceScope&) = delete;

private:
    int prev_{0};
    int index_{0};
};

// Array -> hipcx_array: data = raw_data + offset (chainerx/backend_util.h:10-13), byte strides as they are.
hipcx_array ToC(const Array& a) {
    hipcx_array c{};
    c.data = internal::GetRawOffsetData(a);
    c.dtype = static_cast<int32_t>(a.dtype());  // same numeric codes (chainerx/dtype.h:19-29)
    c.ndim = a.ndim();
    for (int8_t i = 0; i < a.ndim(); ++i) {
        c.shape[i] = a.shape()[i];
        c.strides[i] = a.strides()[i];
    }
    return c;
}

hipcx_scalar ToC(Scalar s) {
    hipcx_scalar c{};
    switch (s.kind()) {
        case DtypeKind::kBool:
            c.kind = HIPCX_KIND_BOOL;
            c.i = static_cast<bool>(s) ? 1 : 0;
            break;
        case DtypeKind::kInt:
        case DtypeKind::kUInt:
            c.kind = HIPCX_KIND_INT;
            c.i = static_cast<int64_t>(s);
            break;
        default:
            c.kind = HIPCX_KIND_FLOAT;
            c.f = static_cast<double>(s);
            break;
    }
    return c;
}

std::vector<int8_t> ToC(const Axes& axes) { return std::vector<int8_t>(axes.begin(), axes.end()); }

// A device int32 that a kernel raises (index out of range, LAPACK-style info): zeroed with a fill kernel, read back with the
// library's blocking device-to-host copy.
std::shared_ptr<void> NewDeviceFlag(Device& device) {
    std::shared_ptr<void> flag = device.Allocate(sizeof(int32_t));
    hipcx_array d{};
    d.data = flag.get();
    d.dtype = HIPCX_INT32;
    d.ndim = 1;
    d.shape[0] = 1;
    d.strides[0] = sizeof(int32_t);
    hipcx_scalar zero{};
    zero.kind = HIPCX_KIND_INT;
    Check(hipcx_fill(&d, zero, nullptr));
    return flag;
}
int32_t ReadDeviceFlag(Device& device, const std::shared_ptr<void>& flag) {
    int32_t host = 0;
    Check(hipcx_memcpy_to_host(device.index(), &host, flag.get(), sizeof(int32_t), nullptr));
    return host;
}

class HipBackend;

// The Device interface (chainerx/device.h:24-71) over the library's device layer: every allocation comes from the pool behind
// hipcx_malloc and goes back through hipcx_free (the deleter never throws and outlives the pool: the library remembers the blocks
// that were in use when hipcx_pool_destroy took their pool away and swallows their frees, also when a new pool exists on the
// device by then), copies are the library's.
class HipDevice : public Device {
public:
    HipDevice(Backend& backend, int index) : Device{backend, index} {}

    std::shared_ptr<void> Allocate(size_t bytesize) override {
        void* ptr = nullptr;
        Check(hipcx_malloc(index(), bytesize, &ptr));  // 0 bytes -> nullptr; HIPCX_OUT_OF_MEMORY_ERROR -> OutOfMemoryError
        return Wrap(ptr);
    }

    std::shared_ptr<void> MakeDataFromForeignPointer(const std::shared_ptr<void>& data) override {
        if (data == nullptr) return data;
        Check(hipcx_check_device_pointer(index(), data.get()));
        return data;
    }

    void MemoryCopyFrom(void* dst, const void* src, size_t bytesize, Device& src_device) override {
        if (bytesize == 0) return;
        if (auto* other = dynamic_cast<HipDevice*>(&src_device)) {
            Check(hipcx_memcpy_device(index(), dst, other->index(), src, bytesize, nullptr));
        } else {  // native (host) source
            Check(hipcx_memcpy_from_host(index(), dst, src, bytesize, nullptr));
        }
    }

    void MemoryCopyTo(void* dst, const void* src, size_t bytesize, Device& dst_device) override {
        if (bytesize == 0) return;
        if (auto* other = dynamic_cast<HipDevice*>(&dst_device)) {
            Check(hipcx_memcpy_device(other->index(), dst, index(), src, bytesize, nullptr));
        } else {
            Check(hipcx_memcpy_to_host(index(), dst, src, bytesize, nullptr));
        }
    }

    std::shared_ptr<void> TransferDataFrom(Device& src_device, const std::shared_ptr<void>& src_ptr, size_t offset, size_t bytesize) override {
        std::shared_ptr<void> dst = Allocate(bytesize);
        MemoryCopyFrom(dst.get(), static_cast<const uint8_t*>(src_ptr.get()) + offset, bytesize, src_device);
        return dst;
    }

    std::shared_ptr<void> TransferDataTo(Device& dst_device, const std::shared_ptr<void>& src_ptr, size_t offset, size_t bytesize) override {
        std::shared_ptr<void> dst = dst_device.Allocate(bytesize);
        MemoryCopyTo(dst.get(), static_cast<const uint8_t*>(src_ptr.get()) + offset, bytesize, dst_device);
        return dst;
    }

    std::shared_ptr<void> FromHostMemory(const std::shared_ptr<void>& src_ptr, size_t bytesize) override {
        void* ptr = nullptr;
        Check(hipcx_from_host_memory(index(), src_ptr.get(), bytesize, &ptr, nullptr));
        return Wrap(ptr);
    }

    void Synchronize() override { Check(hipcx_synchronize(index())); }

private:
    std::shared_ptr<void> Wrap(void* ptr) {
        if (ptr == nullptr) return nullptr;
        const int device = index();
        return std::shared_ptr<void>{ptr, [device](void* p) noexcept { (void)hipcx_free(device, p); }};
    }
};

}  // namespace

class HipBackend : public Backend {
public:
    using Backend::Backend;

    std::string GetName() const override { return "hip"; }

    int GetDeviceCount() const override {
        int n = 0;
        Check(hipcx_device_count(&n));
        return n;
    }

    // Transfers inside the backend and to/from the native (host) backend, like cuda/cuda_backend.cc:49-59.
    bool SupportsTransfer(Device& src_device, Device& dst_device) override {
        Backend& src = src_device.backend();
        Backend& dst = dst_device.backend();
        if (&src == this) return &dst == this || nullptr != dynamic_cast<native::NativeBackend*>(&dst);
        if (&dst == this) return nullptr != dynamic_cast<native::NativeBackend*>(&src);
        return false;
    }

    static KernelRegistry& GetGlobalKernelRegistry() {
        static KernelRegistry* global_kernel_registry = new KernelRegistry{};
        return *global_kernel_registry;
    }

protected:
    KernelRegistry& GetParentKernelRegistry() override { return GetGlobalKernelRegistry(); }

private:
    std::unique_ptr<Device> CreateDevice(int index) override {
        int n = GetDeviceCount();
        if (index < 0 || index >= n) throw std::out_of_range{"The index number (= " + std::to_string(index) + ") is out of range"};
        return std::make_unique<HipDevice>(*this, index);
    }
};

namespace {

#define HIPCX_REGISTER_KERNEL(key_kernel_cls, kernel_cls) \
    static chainerx::internal::KernelRegistrar<chainerx::hip::HipBackend, key_kernel_cls, kernel_cls> s_hip_backend_kernel_##kernel_cls{};

Array Cast(const Array& a, Dtype dtype) { return a.dtype() == dtype ? a : a.AsType(dtype); }

// ---- elementwise: (x1, x2, out), (x1, Scalar, out), (Scalar, x2, out), (x, out) ----
#define HIPCX_BINARY_KERNEL(Name, entry)                                                  \
    class Hip##Name##Kernel : public Name##Kernel {                                       \
    public:                                                                               \
        void Call(const Array& x1, const Array& x2, const Array& out) override {          \
            Device& device = x1.device();                                                 \
            device.CheckDevicesCompatible(x1, x2, out);                                   \
            SetDeviceScope scope{device.index()};                                         \
            hipcx_array a = ToC(Cast(x1, out.dtype())), b = ToC(Cast(x2, out.dtype())), o = ToC(out); \
            Check(entry(&a, &b, &o, nullptr));                                            \
        }                                                                                 \
    };                                                                                    \
    HIPCX_REGISTER_KERNEL(Name##Kernel, Hip##Name##Kernel)

#define HIPCX_BINARY_AS_KERNEL(Name, entry)                                               \
    class Hip##Name##Kernel : public Name##Kernel {                                       \
    public:                                                                               \
        void Call(const Array& x1, Scalar x2, const Array& out) override {                \
            Device& device = x1.device();                                                 \
            device.CheckDevicesCompatible(x1, out);                                       \
            SetDeviceScope scope{device.index()};                                         \
            hipcx_array a = ToC(Cast(x1, out.dtype())), o = ToC(out);                     \
            Check(entry(&a, ToC(x2), &o, nullptr));                                       \
        }                                                                                 \
    };                                                                                    \
    HIPCX_REGISTER_KERNEL(Name##Kernel, Hip##Name##Kernel)

#define HIPCX_UNARY_KERNEL(Name, entry)                                                   \
    class Hip##Name##Kernel : public Name##Kernel {                                       \
    public:                                                                               \
        void Call(const Array& x, const Array& out) override {                            \
            Device& device = x.device();                                                  \
            device.CheckDevicesCompatible(x, out);                                        \
            SetDeviceScope scope{device.index()};                                         \
            hipcx_array a = ToC(Cast(x, out.dtype())), o = ToC(out);                      \
            Check(entry(&a, &o, nullptr));                                                \
        }                                                                                 \
    };                                                                                    \
    HIPCX_REGISTER_KERNEL(Name##Kernel, Hip##Name##Kernel)

HIPCX_BINARY_KERNEL(Add, hipcx_add)
HIPCX_BINARY_KERNEL(Subtract, hipcx_subtract)
HIPCX_BINARY_KERNEL(Multiply, hipcx_multiply)
HIPCX_BINARY_KERNEL(Divide, hipcx_divide)
HIPCX_BINARY_AS_KERNEL(AddAS, hipcx_add_as)
HIPCX_BINARY_AS_KERNEL(SubtractAS, hipcx_subtract_as)
HIPCX_BINARY_AS_KERNEL(MultiplyAS, hipcx_multiply_as)
HIPCX_BINARY_AS_KERNEL(DivideAS, hipcx_divide_as)
HIPCX_UNARY_KERNEL(Exp, hipcx_exp)
HIPCX_UNARY_KERNEL(Log, hipcx_log)
HIPCX_UNARY_KERNEL(Tanh, hipcx_tanh)
HIPCX_UNARY_KERNEL(Sqrt, hipcx_sqrt)

class HipDivideSAKernel : public DivideSAKernel {
public:
    void Call(Scalar x1, const Array& x2, const Array& out) override {
        Device& device = x2.device();
        device.CheckDevicesCompatible(x2, out);
        SetDeviceScope scope{device.index()};
        hipcx_array b = ToC(Cast(x2, out.dtype())), o = ToC(out);
        Check(hipcx_divide_sa(ToC(x1), &b, &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(DivideSAKernel, HipDivideSAKernel)

// Comparisons: the operands share one dtype (promoted here as native/native_device/logic.cc does), out is bool.
#define HIPCX_COMPARE_KERNEL(Name, entry)                                                 \
    class Hip##Name##Kernel : public Name##Kernel {                                       \
    public:                                                                               \
        void Call(const Array& x1, const Array& x2, const Array& out) override {          \
            Device& device = x1.device();                                                 \
            device.CheckDevicesCompatible(x1, x2, out);                                   \
            SetDeviceScope scope{device.index()};                                         \
            Dtype dtype = PromoteTypes(x1.dtype(), x2.dtype());                           \
            hipcx_array a = ToC(Cast(x1, dtype)), b = ToC(Cast(x2, dtype)), o = ToC(out); \
            Check(entry(&a, &b, &o, nullptr));                                            \
        }                                                                                 \
    };                                                                                    \
    HIPCX_REGISTER_KERNEL(Name##Kernel, Hip##Name##Kernel)

HIPCX_COMPARE_KERNEL(Equal, hipcx_equal)
HIPCX_COMPARE_KERNEL(NotEqual, hipcx_not_equal)
HIPCX_COMPARE_KERNEL(Greater, hipcx_greater)
HIPCX_COMPARE_KERNEL(GreaterEqual, hipcx_greater_equal)

#define HIPCX_SELECT_ASSA_KERNEL(Name, entry)                                                          \
    class Hip##Name##Kernel : public Name##Kernel {                                                    \
    public:                                                                                            \
        void Call(const Array& x1, Scalar x2, Scalar pos, const Array& neg, const Array& out) override { \
            Device& device = x1.device();                                                              \
            device.CheckDevicesCompatible(x1, neg, out);                                               \
            SetDeviceScope scope{device.index()};                                                      \
            hipcx_array a = ToC(Cast(x1, out.dtype())), n = ToC(Cast(neg, out.dtype())), o = ToC(out); \
            Check(entry(&a, ToC(x2), ToC(pos), &n, &o, nullptr));                                      \
        }                                                                                              \
    };                                                                                                 \
    HIPCX_REGISTER_KERNEL(Name##Kernel, Hip##Name##Kernel)

HIPCX_SELECT_ASSA_KERNEL(IfLessElseASSA, hipcx_if_less_else_assa)        // ReLU = Maximum(x, 0), routines/misc.cc:210-216
HIPCX_SELECT_ASSA_KERNEL(IfGreaterElseASSA, hipcx_if_greater_else_assa)  // Minimum(x, scalar)

class HipIfGreaterElseAAAAKernel : public IfGreaterElseAAAAKernel {
public:
    void Call(const Array& x1, const Array& x2, const Array& pos, const Array& neg, const Array& out) override {
        Device& device = x1.device();
        device.CheckDevicesCompatible(x1, x2, pos, neg, out);
        SetDeviceScope scope{device.index()};
        Dtype dt = out.dtype();
        hipcx_array a = ToC(Cast(x1, dt)), b = ToC(Cast(x2, dt)), p = ToC(Cast(pos, dt)), n = ToC(Cast(neg, dt)), o = ToC(out);
        Check(hipcx_if_greater_else_aaaa(&a, &b, &p, &n, &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(IfGreaterElseAAAAKernel, HipIfGreaterElseAAAAKernel)

// ---- further elementwise kernels: one C entry per family, selected by an op code ----
#define HIPCX_UNARY_CODE_KERNEL(Name, code)                                               \
    class Hip##Name##Kernel : public Name##Kernel {                                       \
    public:                                                                               \
        void Call(const Array& x, const Array& out) override {                            \
            Device& device = x.device();                                                  \
            device.CheckDevicesCompatible(x, out);                                        \
            SetDeviceScope scope{device.index()};                                         \
            hipcx_array a = ToC(Cast(x, out.dtype())), o = ToC(out);                      \
            Check(hipcx_unary(code, &a, &o, nullptr));                                    \
        }                                                                                 \
    };                                                                                    \
    HIPCX_REGISTER_KERNEL(Name##Kernel, Hip##Name##Kernel)

HIPCX_UNARY_CODE_KERNEL(Erf, HIPCX_UNARY_ERF)
HIPCX_UNARY_CODE_KERNEL(Expm1, HIPCX_UNARY_EXPM1)
HIPCX_UNARY_CODE_KERNEL(Exp2, HIPCX_UNARY_EXP2)
HIPCX_UNARY_CODE_KERNEL(Log10, HIPCX_UNARY_LOG10)
HIPCX_UNARY_CODE_KERNEL(Log2, HIPCX_UNARY_LOG2)
HIPCX_UNARY_CODE_KERNEL(Log1p, HIPCX_UNARY_LOG1P)
HIPCX_UNARY_CODE_KERNEL(Sinh, HIPCX_UNARY_SINH)
HIPCX_UNARY_CODE_KERNEL(Cosh, HIPCX_UNARY_COSH)
HIPCX_UNARY_CODE_KERNEL(Arcsinh, HIPCX_UNARY_ARCSINH)
HIPCX_UNARY_CODE_KERNEL(Arccosh, HIPCX_UNARY_ARCCOSH)
HIPCX_UNARY_CODE_KERNEL(Sin, HIPCX_UNARY_SIN)
HIPCX_UNARY_CODE_KERNEL(Cos, HIPCX_UNARY_COS)
HIPCX_UNARY_CODE_KERNEL(Tan, HIPCX_UNARY_TAN)
HIPCX_UNARY_CODE_KERNEL(Arcsin, HIPCX_UNARY_ARCSIN)
HIPCX_UNARY_CODE_KERNEL(Arccos, HIPCX_UNARY_ARCCOS)
HIPCX_UNARY_CODE_KERNEL(Arctan, HIPCX_UNARY_ARCTAN)
HIPCX_UNARY_CODE_KERNEL(Ceil, HIPCX_UNARY_CEIL)
HIPCX_UNARY_CODE_KERNEL(Floor, HIPCX_UNARY_FLOOR)
HIPCX_UNARY_CODE_KERNEL(Square, HIPCX_UNARY_SQUARE)
HIPCX_UNARY_CODE_KERNEL(Abs, HIPCX_UNARY_ABS)
HIPCX_UNARY_CODE_KERNEL(Sign, HIPCX_UNARY_SIGN)

// bool out = p(x): the input keeps its dtype
#define HIPCX_PREDICATE_KERNEL(Name, code)                                                \
    class Hip##Name##Kernel : public Name##Kernel {                                       \
    public:                                                                               \
        void Call(const Array& x, const Array& out) override {                            \
            Device& device = x.device();                                                  \
            device.CheckDevicesCompatible(x, out);                                        \
            SetDeviceScope scope{device.index()};                                         \
            hipcx_array a = ToC(x), o = ToC(out);                                         \
            Check(hipcx_predicate(code, &a, &o, nullptr));                                \
        }                                                                                 \
    };                                                                                    \
    HIPCX_REGISTER_KERNEL(Name##Kernel, Hip##Name##Kernel)

HIPCX_PREDICATE_KERNEL(LogicalNot, HIPCX_PRED_LOGICAL_NOT)
HIPCX_PREDICATE_KERNEL(IsNan, HIPCX_PRED_ISNAN)
HIPCX_PREDICATE_KERNEL(IsInf, HIPCX_PRED_ISINF)
HIPCX_PREDICATE_KERNEL(IsFinite, HIPCX_PRED_ISFINITE)

#define HIPCX_LOGICAL_KERNEL(Name, code)                                                  \
    class Hip##Name##Kernel : public Name##Kernel {                                       \
    public:                                                                               \
        void Call(const Array& x1, const Array& x2, const Array& out) override {          \
            Device& device = x1.device();                                                 \
            device.CheckDevicesCompatible(x1, x2, out);                                   \
            SetDeviceScope scope{device.index()};                                         \
            Dtype dtype = PromoteTypes(x1.dtype(), x2.dtype());                           \
            hipcx_array a = ToC(Cast(x1, dtype)), b = ToC(Cast(x2, dtype)), o = ToC(out); \
            Check(hipcx_logical(code, &a, &b, &o, nullptr));                              \
        }                                                                                 \
    };                                                                                    \
    HIPCX_REGISTER_KERNEL(Name##Kernel, Hip##Name##Kernel)

HIPCX_LOGICAL_KERNEL(LogicalAnd, HIPCX_LOGICAL_AND)
HIPCX_LOGICAL_KERNEL(LogicalOr, HIPCX_LOGICAL_OR)
HIPCX_LOGICAL_KERNEL(LogicalXor, HIPCX_LOGICAL_XOR)

HIPCX_BINARY_KERNEL(Power, hipcx_power)
HIPCX_BINARY_AS_KERNEL(PowerAS, hipcx_power_as)
HIPCX_BINARY_KERNEL(Fmod, hipcx_fmod)
HIPCX_BINARY_KERNEL(Arctan2, hipcx_arctan2)

class HipPowerSAKernel : public PowerSAKernel {
public:
    void Call(Scalar x1, const Array& x2, const Array& out) override {
        Device& device = x2.device();
        device.CheckDevicesCompatible(x2, out);
        SetDeviceScope scope{device.index()};
        hipcx_array b = ToC(Cast(x2, out.dtype())), o = ToC(out);
        Check(hipcx_power_sa(ToC(x1), &b, &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(PowerSAKernel, HipPowerSAKernel)

// FloorDivide / Mod / bitwise / shift families: (x1, x2, out), (x1, Scalar, out), (Scalar, x2, out) with an op code
#define HIPCX_BINARY_CODE_KERNEL(Name, code)                                              \
    class Hip##Name##Kernel : public Name##Kernel {                                       \
    public:                                                                               \
        void Call(const Array& x1, const Array& x2, const Array& out) override {          \
            Device& device = x1.device();                                                 \
            device.CheckDevicesCompatible(x1, x2, out);                                   \
            SetDeviceScope scope{device.index()};                                         \
            hipcx_array a = ToC(Cast(x1, out.dtype())), b = ToC(Cast(x2, out.dtype())), o = ToC(out); \
            Check(hipcx_binary(code, &a, &b, &o, nullptr));                               \
        }                                                                                 \
    };                                                                                    \
    HIPCX_REGISTER_KERNEL(Name##Kernel, Hip##Name##Kernel)

#define HIPCX_BINARY_CODE_AS_KERNEL(Name, code)                                           \
    class Hip##Name##Kernel : public Name##Kernel {                                       \
    public:                                                                               \
        void Call(const Array& x1, Scalar x2, const Array& out) override {                \
            Device& device = x1.device();                                                 \
            device.CheckDevicesCompatible(x1, out);                                       \
            SetDeviceScope scope{device.index()};                                         \
            hipcx_array a = ToC(Cast(x1, out.dtype())), o = ToC(out);                     \
            Check(hipcx_binary_as(code, &a, ToC(x2), &o, nullptr));                       \
        }                                                                                 \
    };                                                                                    \
    HIPCX_REGISTER_KERNEL(Name##Kernel, Hip##Name##Kernel)

#define HIPCX_BINARY_CODE_SA_KERNEL(Name, code)                                           \
    class Hip##Name##Kernel : public Name##Kernel {                                       \
    public:                                                                               \
        void Call(Scalar x1, const Array& x2, const Array& out) override {                \
            Device& device = x2.device();                                                 \
            device.CheckDevicesCompatible(x2, out);                                       \
            SetDeviceScope scope{device.index()};                                         \
            hipcx_array b = ToC(Cast(x2, out.dtype())), o = ToC(out);                     \
            Check(hipcx_binary_sa(code, ToC(x1), &b, &o, nullptr));                       \
        }                                                                                 \
    };                                                                                    \
    HIPCX_REGISTER_KERNEL(Name##Kernel, Hip##Name##Kernel)

HIPCX_BINARY_CODE_KERNEL(FloorDivide, HIPCX_BINARY_FLOOR_DIVIDE)
HIPCX_BINARY_CODE_AS_KERNEL(FloorDivideAS, HIPCX_BINARY_FLOOR_DIVIDE)
HIPCX_BINARY_CODE_SA_KERNEL(FloorDivideSA, HIPCX_BINARY_FLOOR_DIVIDE)
HIPCX_BINARY_CODE_KERNEL(ModAA, HIPCX_BINARY_MOD)
HIPCX_BINARY_CODE_AS_KERNEL(ModAS, HIPCX_BINARY_MOD)
HIPCX_BINARY_CODE_SA_KERNEL(ModSA, HIPCX_BINARY_MOD)
HIPCX_BINARY_CODE_KERNEL(BitwiseAnd, HIPCX_BINARY_BITWISE_AND)
HIPCX_BINARY_CODE_AS_KERNEL(BitwiseAndAS, HIPCX_BINARY_BITWISE_AND)
HIPCX_BINARY_CODE_KERNEL(BitwiseOr, HIPCX_BINARY_BITWISE_OR)
HIPCX_BINARY_CODE_AS_KERNEL(BitwiseOrAS, HIPCX_BINARY_BITWISE_OR)
HIPCX_BINARY_CODE_KERNEL(BitwiseXor, HIPCX_BINARY_BITWISE_XOR)
HIPCX_BINARY_CODE_AS_KERNEL(BitwiseXorAS, HIPCX_BINARY_BITWISE_XOR)
HIPCX_BINARY_CODE_KERNEL(LeftShiftAA, HIPCX_BINARY_LEFT_SHIFT)
HIPCX_BINARY_CODE_AS_KERNEL(LeftShiftAS, HIPCX_BINARY_LEFT_SHIFT)
HIPCX_BINARY_CODE_SA_KERNEL(LeftShiftSA, HIPCX_BINARY_LEFT_SHIFT)
HIPCX_BINARY_CODE_KERNEL(RightShiftAA, HIPCX_BINARY_RIGHT_SHIFT)
HIPCX_BINARY_CODE_AS_KERNEL(RightShiftAS, HIPCX_BINARY_RIGHT_SHIFT)
HIPCX_BINARY_CODE_SA_KERNEL(RightShiftSA, HIPCX_BINARY_RIGHT_SHIFT)

// Where: the condition is cast to bool, x / y to out's dtype (native/native_device/indexing.cc:194-283)
class HipWhereKernel : public WhereKernel {
public:
    void Call(const Array& condition, const Array& x, const Array& y, const Array& out) override {
        Device& device = condition.device();
        device.CheckDevicesCompatible(condition, x, y, out);
        SetDeviceScope scope{device.index()};
        hipcx_array c = ToC(Cast(condition, Dtype::kBool)), a = ToC(Cast(x, out.dtype())), b = ToC(Cast(y, out.dtype())), o = ToC(out);
        Check(hipcx_where(&c, &a, &b, &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(WhereKernel, HipWhereKernel)

class HipWhereAASKernel : public WhereAASKernel {
public:
    void Call(const Array& condition, const Array& x, Scalar y, const Array& out) override {
        Device& device = condition.device();
        device.CheckDevicesCompatible(condition, x, out);
        SetDeviceScope scope{device.index()};
        hipcx_array c = ToC(Cast(condition, Dtype::kBool)), a = ToC(Cast(x, out.dtype())), o = ToC(out);
        Check(hipcx_where_aas(&c, &a, ToC(y), &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(WhereAASKernel, HipWhereAASKernel)

class HipWhereASAKernel : public WhereASAKernel {
public:
    void Call(const Array& condition, Scalar x, const Array& y, const Array& out) override {
        Device& device = condition.device();
        device.CheckDevicesCompatible(condition, y, out);
        SetDeviceScope scope{device.index()};
        hipcx_array c = ToC(Cast(condition, Dtype::kBool)), b = ToC(Cast(y, out.dtype())), o = ToC(out);
        Check(hipcx_where_asa(&c, ToC(x), &b, &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(WhereASAKernel, HipWhereASAKernel)

class HipWhereASSKernel : public WhereASSKernel {
public:
    void Call(const Array& condition, Scalar x, Scalar y, const Array& out) override {
        Device& device = condition.device();
        device.CheckDevicesCompatible(condition, out);
        SetDeviceScope scope{device.index()};
        hipcx_array c = ToC(Cast(condition, Dtype::kBool)), o = ToC(out);
        Check(hipcx_where_ass(&c, ToC(x), ToC(y), &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(WhereASSKernel, HipWhereASSKernel)

// ---- creation ----
class HipCopyKernel : public CopyKernel {
public:
    void Call(const Array& a, const Array& out) override {
        Device& device = a.device();
        device.CheckDevicesCompatible(a, out);
        SetDeviceScope scope{device.index()};
        hipcx_array ca = ToC(a), o = ToC(out);  // the kernel casts: every (In, Out) dtype pair
        Check(hipcx_copy(&ca, &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(CopyKernel, HipCopyKernel)

class HipFillKernel : public FillKernel {
public:
    void Call(const Array& out, Scalar value) override {
        SetDeviceScope scope{out.device().index()};
        hipcx_array o = ToC(out);
        Check(hipcx_fill(&o, ToC(value), nullptr));
    }
};
HIPCX_REGISTER_KERNEL(FillKernel, HipFillKernel)

class HipArangeKernel : public ArangeKernel {
public:
    void Call(Scalar start, Scalar step, const Array& out) override {
        SetDeviceScope scope{out.device().index()};
        hipcx_array o = ToC(out);
        Check(hipcx_arange(ToC(start), ToC(step), &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(ArangeKernel, HipArangeKernel)

// ---- reductions ----
using ReduceEntry = int (*)(const hipcx_array*, const int8_t*, int, const hipcx_array*, void*, size_t, void*);

void CallReduce(ReduceEntry entry, const Array& a, const Axes& axis, const Array& out) {
    Device& device = a.device();
    device.CheckDevicesCompatible(a, out);
    SetDeviceScope scope{device.index()};
    hipcx_array ca = ToC(a), o = ToC(out);
    std::vector<int8_t> ax = ToC(axis);
    size_t ws_bytes = hipcx_reduce_workspace_size(&ca, ax.data(), static_cast<int>(ax.size()), &o);
    std::shared_ptr<void> ws = device.Allocate(ws_bytes);  // returned to the pool after the launch: stream order keeps it safe
    Check(entry(&ca, ax.data(), static_cast<int>(ax.size()), &o, ws.get(), ws_bytes, nullptr));
}

class HipSumKernel : public SumKernel {
public:
    void Call(const Array& a, const Axes& axis, const Array& out) override { CallReduce(hipcx_sum, a, axis, out); }
};
HIPCX_REGISTER_KERNEL(SumKernel, HipSumKernel)

class HipAMaxKernel : public AMaxKernel {
public:
    void Call(const Array& a, const Axes& axis, const Array& out) override { CallReduce(hipcx_amax, a, axis, out); }
};
HIPCX_REGISTER_KERNEL(AMaxKernel, HipAMaxKernel)

class HipArgMaxKernel : public ArgMaxKernel {
public:
    void Call(const Array& a, const Axes& axis, const Array& out) override { CallReduce(hipcx_argmax, a, axis, out); }
};
HIPCX_REGISTER_KERNEL(ArgMaxKernel, HipArgMaxKernel)

class HipAMinKernel : public AMinKernel {
public:
    void Call(const Array& a, const Axes& axis, const Array& out) override { CallReduce(hipcx_amin, a, axis, out); }
};
HIPCX_REGISTER_KERNEL(AMinKernel, HipAMinKernel)

class HipArgMinKernel : public ArgMinKernel {
public:
    void Call(const Array& a, const Axes& axis, const Array& out) override { CallReduce(hipcx_argmin, a, axis, out); }
};
HIPCX_REGISTER_KERNEL(ArgMinKernel, HipArgMinKernel)

// the routines have already replaced NaNs by -inf / +inf (CX/routines/sorting.cc:96); the native NanArgMax / NanArgMin functors
// are those of ArgMax / ArgMin (native/native_device/reduction.cc:171-226)
class HipNanArgMaxKernel : public NanArgMaxKernel {
public:
    void Call(const Array& a, const Axes& axis, const Array& out) override { CallReduce(hipcx_argmax, a, axis, out); }
};
HIPCX_REGISTER_KERNEL(NanArgMaxKernel, HipNanArgMaxKernel)

class HipNanArgMinKernel : public NanArgMinKernel {
public:
    void Call(const Array& a, const Axes& axis, const Array& out) override { CallReduce(hipcx_argmin, a, axis, out); }
};
HIPCX_REGISTER_KERNEL(NanArgMinKernel, HipNanArgMinKernel)

// All / Any reduce truth values: other dtypes are cast to bool first (native/native_device/logic.cc)
class HipAllKernel : public AllKernel {
public:
    void Call(const Array& a, const Axes& axis, const Array& out) override { CallReduce(hipcx_all, Cast(a, Dtype::kBool), axis, out); }
};
HIPCX_REGISTER_KERNEL(AllKernel, HipAllKernel)

class HipAnyKernel : public AnyKernel {
public:
    void Call(const Array& a, const Axes& axis, const Array& out) override { CallReduce(hipcx_any, Cast(a, Dtype::kBool), axis, out); }
};
HIPCX_REGISTER_KERNEL(AnyKernel, HipAnyKernel)

// ---- dot / conv ----
class HipDotKernel : public DotKernel {
public:
    void Call(const Array& a, const Array& b, const Array& out) override {
        Device& device = a.device();
        device.CheckDevicesCompatible(a, b, out);
        SetDeviceScope scope{device.index()};
        hipcx_array ca = ToC(Cast(a, out.dtype())), cb = ToC(Cast(b, out.dtype())), o = ToC(out);
        size_t ws_bytes = hipcx_dot_workspace_size(&ca, &cb, &o);
        std::shared_ptr<void> ws = device.Allocate(ws_bytes);
        Check(hipcx_dot(&ca, &cb, &o, ws.get(), ws_bytes, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(DotKernel, HipDotKernel)

int64_t OutDim(int64_t in, int64_t k, int64_t s, int64_t p, bool cover_all) {
    int64_t n = hipcx_conv_out_dim(in, k, s, p, cover_all ? 1 : 0);
    if (n <= 0) throw DimensionError{"Output size should be positive."};
    return n;
}

class HipConvKernel : public ConvKernel {
public:
    Array Call(const Array& x, const Array& w, const absl::optional<Array>& b, const Dims& stride, const Dims& pad, bool cover_all,
               Dtype out_dtype, const absl::optional<Array>& out) override {
        if (out.has_value()) throw NotImplementedError{"Passing out as an argument is not yet supported."};  // like native conv.cc:52-55
        // any number of spatial axes, like the native kernel (native_device/conv.cc:57-61); the library's dedicated kernels are 2-D
        if (x.ndim() < 2 || w.ndim() != x.ndim()) throw DimensionError{"Mismatched number of dimensions in input and weights."};
        Device& device = x.device();
        device.CheckDevicesCompatible(x, w);
        if (b.has_value()) device.CheckDevicesCompatible(*b);
        SetDeviceScope scope{device.index()};
        const int8_t n = x.ndim() - 2;
        Shape out_shape{x.shape()[0], w.shape()[0]};
        std::vector<int64_t> st, pd;
        for (int8_t d = 0; d < n; ++d) {
            out_shape.emplace_back(OutDim(x.shape()[2 + d], w.shape()[2 + d], stride[d], pad[d], cover_all));
            st.push_back(stride[d]);
            pd.push_back(pad[d]);
        }
        Array y = Empty(out_shape, out_dtype, device);  // C-contiguous NCHW, like cuda/cuda_conv.cc:311
        Array xc = Cast(x, out_dtype), wc = Cast(w, out_dtype);
        hipcx_array cx = ToC(xc), cw = ToC(wc), cy = ToC(y), cb{};
        if (b.has_value()) cb = ToC(Cast(*b, out_dtype));
        size_t ws_bytes = hipcx_conv_workspace_size(&cx, &cw, &cy);
        std::shared_ptr<void> ws = device.Allocate(ws_bytes);
        Check(hipcx_conv(&cx, &cw, b.has_value() ? &cb : nullptr, st.data(), pd.data(), cover_all ? 1 : 0, &cy, ws.get(), ws_bytes, nullptr));
        return y;
    }
};
HIPCX_REGISTER_KERNEL(ConvKernel, HipConvKernel)

// ---- fixed batch norm ----
class HipFixedBatchNormKernel : public FixedBatchNormKernel {
public:
    Array Call(const Array& x, const Array& gamma, const Array& beta, const Array& mean, const Array& var, Scalar eps, const Axes& axis,
               const absl::optional<Array>& out) override {
        if (out.has_value()) throw NotImplementedError{"Passing out as an argument is not yet supported."};
        Device& device = x.device();
        device.CheckDevicesCompatible(x, gamma, beta, mean, var);
        SetDeviceScope scope{device.index()};
        Array y = EmptyLike(x, device);
        hipcx_array cx = ToC(x), cg = ToC(gamma), cb = ToC(beta), cm = ToC(mean), cv = ToC(var), cy = ToC(y);
        std::vector<int8_t> ax = ToC(axis);
        Check(hipcx_fixed_batch_norm(&cx, &cg, &cb, &cm, &cv, ToC(eps), ax.data(), static_cast<int>(ax.size()), &cy, nullptr));
        return y;
    }
};
HIPCX_REGISTER_KERNEL(FixedBatchNormKernel, HipFixedBatchNormKernel)

// ---- pooling: the states keep what the gradient kernels recompute from ----
class HipMaxPoolGradState : public MaxPoolGradState {
public:
    HipMaxPoolGradState(Array x, bool cover_all) : x_{std::move(x)}, cover_all_{cover_all} {}
    const Array& x() const { return x_; }
    bool cover_all() const { return cover_all_; }

private:
    Array x_;
    bool cover_all_;
};
class HipMaxPoolGradGradState : public MaxPoolGradGradState {
public:
    explicit HipMaxPoolGradGradState(Array x) : x_{std::move(x)} {}
    const Array& x() const { return x_; }

private:
    Array x_;
};
class HipAveragePoolGradState : public AveragePoolGradState {
public:
    explicit HipAveragePoolGradState(Array x) : x_{std::move(x)} {}
    const Array& x() const { return x_; }

private:
    Array x_;
};

Shape PoolOutShape(const Array& x, const Dims& k, const Dims& s, const Dims& p, bool cover_all) {
    if (x.ndim() < 3) throw DimensionError{"pooling needs at least one spatial axis."};
    Shape out_shape{x.shape()[0], x.shape()[1]};
    for (int8_t d = 0; d < x.ndim() - 2; ++d) out_shape.emplace_back(OutDim(x.shape()[2 + d], k[d], s[d], p[d], cover_all));
    return out_shape;
}

std::vector<int64_t> ToVector(const Dims& dims) { return std::vector<int64_t>(dims.begin(), dims.end()); }

class HipMaxPoolKernel : public MaxPoolKernel {
public:
    std::tuple<Array, std::unique_ptr<MaxPoolGradState>> Call(const Array& x, Dims kernel_size, Dims stride, Dims pad, bool cover_all,
                                                             bool return_state, const absl::optional<Array>& out) override {
        if (out.has_value()) throw NotImplementedError{"Passing out as an argument is not yet supported."};
        Device& device = x.device();
        SetDeviceScope scope{device.index()};
        Array y = Empty(PoolOutShape(x, kernel_size, stride, pad, cover_all), x.dtype(), device);
        hipcx_array cx = ToC(x), cy = ToC(y);
        std::vector<int64_t> k = ToVector(kernel_size), s = ToVector(stride), p = ToVector(pad);
        Check(hipcx_max_pool(&cx, k.data(), s.data(), p.data(), cover_all ? 1 : 0, &cy, nullptr));
        std::unique_ptr<MaxPoolGradState> state = return_state ? std::make_unique<HipMaxPoolGradState>(x, cover_all) : nullptr;
        return std::make_tuple(std::move(y), std::move(state));
    }
};
HIPCX_REGISTER_KERNEL(MaxPoolKernel, HipMaxPoolKernel)

class HipAveragePoolKernel : public AveragePoolKernel {
public:
    std::tuple<Array, std::unique_ptr<AveragePoolGradState>> Call(const Array& x, const Dims& kernel_size, const Dims& stride, const Dims& pad,
                                                                 AveragePoolPadMode pad_mode, bool return_state,
                                                                 const absl::optional<Array>& out) override {
        if (out.has_value()) throw NotImplementedError{"Passing out as an argument is not yet supported."};
        Device& device = x.device();
        SetDeviceScope scope{device.index()};
        Array y = Empty(PoolOutShape(x, kernel_size, stride, pad, false), x.dtype(), device);
        hipcx_array cx = ToC(x), cy = ToC(y);
        std::vector<int64_t> k = ToVector(kernel_size), s = ToVector(stride), p = ToVector(pad);
        int mode = pad_mode == AveragePoolPadMode::kZero ? HIPCX_PAD_ZERO : HIPCX_PAD_IGNORE;
        Check(hipcx_average_pool(&cx, k.data(), s.data(), p.data(), mode, &cy, nullptr));
        std::unique_ptr<AveragePoolGradState> state = return_state ? std::make_unique<HipAveragePoolGradState>(x) : nullptr;
        return std::make_tuple(std::move(y), std::move(state));
    }
};
HIPCX_REGISTER_KERNEL(AveragePoolKernel, HipAveragePoolKernel)

// ---- backward / training kernels ----
// Im2Col (CX/native/im2col.cc:82-149) and Col2Im (CX/native/col2im.cc:76-122): one library call each.
Array HipIm2Col(const Array& x, const Dims& k, const Dims& s, const Dims& p, bool cover_all, Scalar pad_value) {
    if (x.ndim() != 4) throw NotImplementedError{"hip backward kernels support 2 spatial dimensions."};
    Device& device = x.device();
    SetDeviceScope scope{device.index()};
    int64_t oh = OutDim(x.shape()[2], k[0], s[0], p[0], cover_all), ow = OutDim(x.shape()[3], k[1], s[1], p[1], cover_all);
    Array col = Empty(Shape{x.shape()[0], x.shape()[1], k[0], k[1], oh, ow}, x.dtype(), device);
    hipcx_array cx = ToC(x), cc = ToC(col);
    int64_t st[2] = {s[0], s[1]}, pd[2] = {p[0], p[1]};
    Check(hipcx_im2col(&cx, st, pd, cover_all ? 1 : 0, ToC(pad_value), &cc, nullptr));
    return col;
}

Array HipCol2Im(const Array& col, const Dims& s, const Dims& p, const Dims& out_size) {
    Device& device = col.device();
    SetDeviceScope scope{device.index()};
    Array out = Empty(Shape{col.shape()[0], col.shape()[1], out_size[0], out_size[1]}, col.dtype(), device);
    hipcx_array cc = ToC(col), co = ToC(out);
    int64_t st[2] = {s[0], s[1]}, pd[2] = {p[0], p[1]};
    Check(hipcx_col2im(&cc, st, pd, &co, nullptr));
    return out;
}

class HipConvGradWeightKernel : public ConvGradWeightKernel {
public:
    Array Call(Dtype w_dtype, const Shape& w_shape, const Array& x, const Array& gy, const Dims& stride, const Dims& pad, bool cover_all,
               const absl::optional<Array>& out) override {
        if (out.has_value()) throw NotImplementedError{"Passing out as an argument is not yet supported."};
        Device& device = x.device();
        device.CheckDevicesCompatible(x, gy);
        SetDeviceScope scope{device.index()};
        if (GetKind(w_dtype) == DtypeKind::kFloat) {
            // one entry, any number of spatial axes (native_device/conv.cc:91-124).  Two axes: Im2Col and the gy transpose as one
            // kernel each, then the matrix product (split over the reduction); otherwise a plain kernel with the native arithmetic
            Array xc = AsContiguous(x.dtype() == w_dtype ? x : x.AsType(w_dtype));
            Array gc = AsContiguous(gy.dtype() == w_dtype ? gy : gy.AsType(w_dtype));
            Array gw = Empty(w_shape, w_dtype, device);
            hipcx_array cx = ToC(xc), cg = ToC(gc), cw = ToC(gw);
            std::vector<int64_t> st(stride.begin(), stride.end()), pd(pad.begin(), pad.end());
            size_t ws_bytes = hipcx_conv_grad_weight_workspace_size(&cx, &cg, &cw, st.data(), pd.data(), cover_all ? 1 : 0);
            std::shared_ptr<void> ws = device.Allocate(ws_bytes);
            Check(hipcx_conv_grad_weight(&cx, &cg, st.data(), pd.data(), cover_all ? 1 : 0, &cw, ws.get(), ws_bytes, nullptr));
            return gw;
        }
        if (x.ndim() != 4) throw NotImplementedError{"hip convolution of non-floating dtypes supports 2 spatial dimensions."};
        Array col = HipIm2Col(x, Dims{w_shape[2], w_shape[3]}, stride, pad, cover_all, 0);
        return native::TensorDot(gy, col, Axes{0, 2, 3}, Axes{0, 4, 5}, w_dtype);  // dispatches DotKernel on this backend
    }
};
HIPCX_REGISTER_KERNEL(ConvGradWeightKernel, HipConvGradWeightKernel)

class HipConvTransposeKernel : public ConvTransposeKernel {
public:
    Array Call(const Array& x, const Array& w, const absl::optional<Array>& b, const Dims& stride, const Dims& pad, const Dims& out_size,
               Dtype out_dtype, const absl::optional<Array>& out) override {
        if (out.has_value()) throw NotImplementedError{"Passing out as an argument is not yet supported."};
        Device& device = x.device();
        device.CheckDevicesCompatible(x, w);
        if (b.has_value()) device.CheckDevicesCompatible(x, *b);
        SetDeviceScope scope{device.index()};
        if (GetKind(out_dtype) == DtypeKind::kFloat) {
            // one entry, any number of spatial axes (native_device/conv.cc:126-160).  Two axes: it picks the flipped forward
            // convolution (stride 1), the scattered 1x1 convolution or the native composition (matrix product over the input
            // channels, col2im, bias) by itself; otherwise a plain kernel with the native arithmetic
            Array xc = x.dtype() == out_dtype ? x : x.AsType(out_dtype);
            Array wc = w.dtype() == out_dtype ? w : w.AsType(out_dtype);
            absl::optional<Array> bc = b.has_value() ? absl::optional<Array>{b->dtype() == out_dtype ? *b : b->AsType(out_dtype)} : absl::nullopt;
            Shape out_shape{x.shape()[0], w.shape()[1]};
            std::copy(out_size.begin(), out_size.end(), std::back_inserter(out_shape));
            Array actual_out = Empty(out_shape, out_dtype, device);
            hipcx_array cx = ToC(xc), cw = ToC(wc), co = ToC(actual_out), cb{};
            if (bc.has_value()) cb = ToC(*bc);
            std::vector<int64_t> st(stride.begin(), stride.end()), pd(pad.begin(), pad.end());
            size_t ws_bytes = hipcx_conv_transpose_workspace_size(&cx, &cw, st.data(), pd.data(), &co);
            std::shared_ptr<void> ws = device.Allocate(ws_bytes);
            Check(hipcx_conv_transpose(&cx, &cw, bc.has_value() ? &cb : nullptr, st.data(), pd.data(), &co, ws.get(), ws_bytes, nullptr));
            return actual_out;
        }
        if (x.ndim() != 4) throw NotImplementedError{"hip convolution of non-floating dtypes supports 2 spatial dimensions."};
        // other dtypes: the native composition on this backend's kernels (TensorDot dispatches DotKernel here)
        Array col = native::TensorDot(w, x, Axes{0}, Axes{1}, out_dtype);  // [C_out, kh, kw, N, H, W]
        Array actual_out = HipCol2Im(col.Transpose(Axes{3, 0, 1, 2, 4, 5}), stride, pad, out_size);
        if (b.has_value()) {
            actual_out += b->AsType(out_dtype, false).Reshape(Shape{1, b->shape()[0], 1, 1});
        }
        return actual_out;
    }
};
HIPCX_REGISTER_KERNEL(ConvTransposeKernel, HipConvTransposeKernel)

// Batch normalisation in training mode and its gradient.  The reference's generic kernels are routine compositions
// (CX/routines/normalization.cc:155-250); they run on this backend's kernels as they are and remain the path for everything the
// dedicated kernels do not take (a non-contiguous x, mixed dtypes, other axis sets).  The state handed to the gradient is the
// generic one (batch mean, 1 / sqrt(var + eps), dtype of beta), so either gradient kernel can consume either forward's state.
namespace {
// Whether hipcx_batch_norm / hipcx_batch_norm_grad take this case: the library decides (hipcx_batch_norm_supported).
bool HipBatchNormApplies(const Array& x, const Axes& axis, std::initializer_list<const Array*> others) {
    hipcx_array cx = ToC(x);
    std::vector<int8_t> ax = ToC(axis);
    std::vector<hipcx_array> descs;
    for (const Array* a : others) descs.push_back(ToC(*a));
    std::vector<const hipcx_array*> ptrs;
    for (const hipcx_array& d : descs) ptrs.push_back(&d);
    return hipcx_batch_norm_supported(&cx, ax.data(), static_cast<int>(ax.size()), ptrs.data(), static_cast<int>(ptrs.size())) == 1;
}
}  // namespace

class HipBatchNormKernel : public GenericBatchNormKernel {
public:
    std::tuple<Array, std::unique_ptr<BatchNormGradState>> Call(const Array& x, const Array& gamma, const Array& beta, const Array& running_mean,
                                                               const Array& running_var, Scalar eps, Scalar decay, const Axes& axis,
                                                               bool return_state, const absl::optional<Array>& out) override {
        if (out.has_value() || !HipBatchNormApplies(x, axis, {&gamma, &beta, &running_mean, &running_var})) {
            return GenericBatchNormKernel::Call(x, gamma, beta, running_mean, running_var, eps, decay, axis, return_state, out);
        }
        Device& device = x.device();
        device.CheckDevicesCompatible(x, gamma, beta, running_mean, running_var);
        SetDeviceScope scope{device.index()};
        Array y = Empty(x.shape(), x.dtype(), device);
        Array x_mean = Empty(gamma.shape(), x.dtype(), device);
        Array x_inv_std = Empty(gamma.shape(), x.dtype(), device);
        hipcx_array cx = ToC(x), cg = ToC(gamma), cb = ToC(beta), crm = ToC(running_mean), crv = ToC(running_var), cy = ToC(y),
                    cm = ToC(x_mean), ci = ToC(x_inv_std);
        std::vector<int8_t> ax = ToC(axis);
        size_t ws_bytes = hipcx_batch_norm_workspace_size(&cx, ax.data(), static_cast<int>(ax.size()));
        std::shared_ptr<void> ws = device.Allocate(ws_bytes);
        Check(hipcx_batch_norm(&cx, &cg, &cb, &crm, &crv, ToC(eps), ToC(decay), ax.data(), static_cast<int>(ax.size()), &cy, &cm, &ci,
                               ws.get(), ws_bytes, nullptr));
        std::unique_ptr<BatchNormGradState> state =
                return_state ? std::make_unique<GenericBatchNormGradState>(std::move(x_mean), std::move(x_inv_std), beta.dtype()) : nullptr;
        return std::make_tuple(std::move(y), std::move(state));
    }
};
HIPCX_REGISTER_KERNEL(BatchNormKernel, HipBatchNormKernel)

class HipBatchNormGradKernel : public GenericBatchNormGradKernel {
public:
    std::tuple<Array, Array, Array> Call(const Array& x, const Array& gamma, const Array& gout, Scalar eps, const Axes& axis,
                                         const std::shared_ptr<BatchNormGradState>& state, const absl::optional<Array>& gx,
                                         const absl::optional<Array>& ggamma, const absl::optional<Array>& gbeta) override {
        auto* st = dynamic_cast<GenericBatchNormGradState*>(state.get());
        if (st == nullptr || gx.has_value() || ggamma.has_value() || gbeta.has_value() || !gout.IsContiguous() ||
            st->beta_dtype() != x.dtype() || !HipBatchNormApplies(x, axis, {&gamma, &gout, &st->x_mean(), &st->x_inv_std()})) {
            return GenericBatchNormGradKernel::Call(x, gamma, gout, eps, axis, state, gx, ggamma, gbeta);
        }
        Device& device = x.device();
        device.CheckDevicesCompatible(x, gamma, gout);
        SetDeviceScope scope{device.index()};
        Array actual_gx = Empty(x.shape(), x.dtype(), device);
        Array actual_ggamma = Empty(gamma.shape(), x.dtype(), device);
        Array actual_gbeta = Empty(gamma.shape(), x.dtype(), device);
        hipcx_array cx = ToC(x), cg = ToC(gamma), cgo = ToC(gout), cm = ToC(st->x_mean()), ci = ToC(st->x_inv_std()), cgx = ToC(actual_gx),
                    cgg = ToC(actual_ggamma), cgb = ToC(actual_gbeta);
        std::vector<int8_t> ax = ToC(axis);
        size_t ws_bytes = hipcx_batch_norm_workspace_size(&cx, ax.data(), static_cast<int>(ax.size()));
        std::shared_ptr<void> ws = device.Allocate(ws_bytes);
        Check(hipcx_batch_norm_grad(&cx, &cg, &cgo, &cm, &ci, ax.data(), static_cast<int>(ax.size()), &cgx, &cgg, &cgb, ws.get(), ws_bytes,
                                    nullptr));
        return std::make_tuple(std::move(actual_gx), std::move(actual_ggamma), std::move(actual_gbeta));
    }
};
HIPCX_REGISTER_KERNEL(BatchNormGradKernel, HipBatchNormGradKernel)

class HipMaxPoolGradKernel : public MaxPoolGradKernel {
public:
    std::tuple<Array, std::unique_ptr<MaxPoolGradGradState>> Call(const Array& gout, const Dims& kernel_size, const Dims& stride, const Dims& pad,
                                                                 const std::shared_ptr<MaxPoolGradState>& state, bool return_state,
                                                                 const absl::optional<Array>& gx) override {
        if (gx.has_value()) throw NotImplementedError{"Passing gx as an argument is not yet supported."};
        auto& st = dynamic_cast<HipMaxPoolGradState&>(*state);
        const Array& x = st.x();
        Device& device = x.device();
        device.CheckDevicesCompatible(x, gout);
        SetDeviceScope scope{device.index()};
        // one kernel with the bits of the native Im2Col / ArgMax / AddAt / Col2Im sequence (native/native_device/pool.cc:97-143)
        Array actual_gx = Empty(x.shape(), x.dtype(), device);
        const Array& g = gout.dtype() == x.dtype() ? gout : gout.AsType(x.dtype());
        hipcx_array cx = ToC(x), cg = ToC(g), cgx = ToC(actual_gx);
        std::vector<int64_t> k(kernel_size.begin(), kernel_size.end()), s(stride.begin(), stride.end()), p(pad.begin(), pad.end());  // any rank
        size_t ws_bytes = hipcx_max_pool_grad_workspace_size(&cg);
        std::shared_ptr<void> ws = device.Allocate(ws_bytes);
        Check(hipcx_max_pool_grad(&cx, &cg, k.data(), s.data(), p.data(), st.cover_all() ? 1 : 0, &cgx, ws.get(), ws_bytes, nullptr));
        std::unique_ptr<MaxPoolGradGradState> grad_grad_state = return_state ? std::make_unique<HipMaxPoolGradGradState>(x) : nullptr;
        return std::make_tuple(std::move(actual_gx), std::move(grad_grad_state));
    }
};
HIPCX_REGISTER_KERNEL(MaxPoolGradKernel, HipMaxPoolGradKernel)

class HipMaxPoolGradGradKernel : public MaxPoolGradGradKernel {
public:
    Array Call(const Array& ggx, const Dims& kernel_size, const Dims& stride, const Dims& pad, bool cover_all,
               const std::shared_ptr<MaxPoolGradGradState>& state, const absl::optional<Array>& ggout) override {
        if (ggout.has_value()) throw NotImplementedError{"Passing ggout as an argument is not yet supported."};
        auto& st = dynamic_cast<HipMaxPoolGradGradState&>(*state);
        const Array& x = st.x();
        Device& device = x.device();
        device.CheckDevicesCompatible(x, ggx);
        SetDeviceScope scope{device.index()};
        Array actual_ggout = Empty(PoolOutShape(x, kernel_size, stride, pad, cover_all), x.dtype(), device);
        const Array& g = ggx.dtype() == x.dtype() ? ggx : ggx.AsType(x.dtype());
        hipcx_array cx = ToC(x), cg = ToC(g), co = ToC(actual_ggout);
        std::vector<int64_t> k(kernel_size.begin(), kernel_size.end()), s(stride.begin(), stride.end()), p(pad.begin(), pad.end());  // any rank
        Check(hipcx_max_pool_grad_grad(&cx, &cg, k.data(), s.data(), p.data(), cover_all ? 1 : 0, &co, nullptr));
        return actual_ggout;
    }
};
HIPCX_REGISTER_KERNEL(MaxPoolGradGradKernel, HipMaxPoolGradGradKernel)

class HipAveragePoolGradKernel : public AveragePoolGradKernel {
public:
    Array Call(const Array& gout, const Dims& kernel_size, const Dims& stride, const Dims& pad, AveragePoolPadMode pad_mode,
               const std::shared_ptr<AveragePoolGradState>& state, const absl::optional<Array>& gx) override {
        if (gx.has_value()) throw NotImplementedError{"Passing gx as an argument is not yet supported."};
        auto& st = dynamic_cast<HipAveragePoolGradState&>(*state);
        const Array& x = st.x();
        Device& device = x.device();
        device.CheckDevicesCompatible(x, gout);
        SetDeviceScope scope{device.index()};
        // one kernel with the bits of the native broadcast / Col2Im / Divide sequence (native/native_device/pool.cc:304-346)
        Array actual_gx = Empty(x.shape(), x.dtype(), device);
        const Array& g = gout.dtype() == x.dtype() ? gout : gout.AsType(x.dtype());
        hipcx_array cg = ToC(g), cgx = ToC(actual_gx);
        std::vector<int64_t> k(kernel_size.begin(), kernel_size.end()), s(stride.begin(), stride.end()), p(pad.begin(), pad.end());  // any rank
        int mode = pad_mode == AveragePoolPadMode::kZero ? HIPCX_PAD_ZERO : HIPCX_PAD_IGNORE;
        Check(hipcx_average_pool_grad(&cg, k.data(), s.data(), p.data(), mode, &cgx, nullptr));
        return actual_gx;
    }
};
HIPCX_REGISTER_KERNEL(AveragePoolGradKernel, HipAveragePoolGradKernel)

// ---- RnnKernel / RnnBackwardKernel (chainerx/kernels/rnn.h:34-66): float32 LSTM, GRU and tanh / relu RNN, one or both directions,
// through hipcx_n_step_rnn / hipcx_n_step_rnn_backward.  The reference's NStepRnnImpl hands these kernels to the backend named "cuda"
// only (chainerx/routines/n_step_rnn.cc:210,330) and composes the routine for every other backend, so the registrations take effect
// once that test also admits "hip".  Other dtypes raise NotImplementedError.
namespace {
// What the forward pass leaves for the backward pass: the library's reserve (gate activations, states before each step, outputs of
// the lower layers) and the call's mode.
class HipRnnGradState : public RnnGradState {
public:
    std::shared_ptr<void> reserve;
    size_t reserve_bytes = 0;
    int8_t mode = 0;
    int activation = 0;
};

struct RnnOperands {
    std::vector<Array> keep;  // contiguous float32 copies where the caller's arrays are something else
    std::vector<hipcx_array> w, b, x;
    std::vector<const hipcx_array*> pw, pb, px;
};

hipcx_array PrepareRnnOperand(RnnOperands& ops, Device& device, const Array& reference, const Array& a) {
    device.CheckDevicesCompatible(reference, a);
    ops.keep.emplace_back(a.dtype() == Dtype::kFloat32 && a.IsContiguous() ? a : AsContiguous(a.AsType(Dtype::kFloat32)));
    return ToC(ops.keep.back());
}

std::vector<const hipcx_array*> PointersTo(const std::vector<hipcx_array>& v) {
    std::vector<const hipcx_array*> p;
    p.reserve(v.size());
    for (const hipcx_array& d : v) p.push_back(&d);
    return p;
}

void PrepareRnnOperands(RnnOperands& ops, Device& device, const Array& hx, const std::vector<std::vector<Array>>& ws,
                        const std::vector<std::vector<Array>>& bs, const std::vector<Array>& xs) {
    size_t n = 0;
    for (const std::vector<Array>& group : ws) n += 2 * group.size();
    ops.keep.reserve(n + xs.size() + 8);
    for (size_t i = 0; i < ws.size(); ++i) {
        for (size_t j = 0; j < ws[i].size(); ++j) {
            ops.w.push_back(PrepareRnnOperand(ops, device, hx, ws[i][j]));
            ops.b.push_back(PrepareRnnOperand(ops, device, hx, bs.at(i).at(j)));
        }
    }
    for (const Array& x : xs) ops.x.push_back(PrepareRnnOperand(ops, device, hx, x));
    ops.pw = PointersTo(ops.w), ops.pb = PointersTo(ops.b), ops.px = PointersTo(ops.x);
}

int RnnActivation(const absl::optional<std::string>& activation) { return activation.has_value() && *activation == "relu" ? 1 : 0; }
}  // namespace

class HipRnnKernel : public RnnKernel {
public:
    std::tuple<std::vector<std::vector<Array>>, std::unique_ptr<RnnGradState>> Call(
            int64_t n_layers, Array hx, absl::optional<Array> cx, const std::vector<std::vector<Array>>& ws, const std::vector<std::vector<Array>>& bs,
            const std::vector<Array>& xs, int8_t bidirectional, int8_t mode, absl::optional<std::string> activation) override {
        if (hx.dtype() != Dtype::kFloat32) throw NotImplementedError{"hip RnnKernel: float32 only."};
        if (mode == 1 && !cx.has_value()) throw ChainerxError{"hip RnnKernel: the LSTM mode needs cx."};
        Device& device = hx.device();
        SetDeviceScope scope{device.index()};
        RnnOperands ops;
        PrepareRnnOperands(ops, device, hx, ws, bs, xs);
        hipcx_array chx_ = PrepareRnnOperand(ops, device, hx, hx);
        hipcx_array ccx{};
        if (mode == 1) ccx = PrepareRnnOperand(ops, device, hx, *cx);
        const int64_t directions = bidirectional ? 2 : 1;
        Array hy = Empty(hx.shape(), Dtype::kFloat32, device);
        Array cy = mode == 1 ? Empty(hx.shape(), Dtype::kFloat32, device) : Array{};
        std::vector<Array> ys;
        std::vector<hipcx_array> dy;
        for (const Array& x : xs) {
            ys.emplace_back(Empty(Shape{x.shape()[0], directions * hx.shape()[2]}, Dtype::kFloat32, device));
            dy.push_back(ToC(ys.back()));
        }
        std::vector<const hipcx_array*> py = PointersTo(dy);
        hipcx_array chy = ToC(hy), ccy{};
        if (mode == 1) ccy = ToC(cy);
        const int n_steps = static_cast<int>(xs.size());
        // A gradient may be asked for later if any input belongs to a graph; then the forward pass keeps its reserve.
        bool training = !internal::GetArrayBody(hx)->nodes().empty() || (cx.has_value() && !internal::GetArrayBody(*cx)->nodes().empty());
        for (const Array& x : xs) training = training || !internal::GetArrayBody(x)->nodes().empty();
        for (const std::vector<Array>& group : ws) {
            for (const Array& w : group) training = training || !internal::GetArrayBody(w)->nodes().empty();
        }
        for (const std::vector<Array>& group : bs) {
            for (const Array& b : group) training = training || !internal::GetArrayBody(b)->nodes().empty();
        }
        std::unique_ptr<HipRnnGradState> state;
        void* reserve = nullptr;
        size_t reserve_bytes = 0;
        if (training) {
            state = std::make_unique<HipRnnGradState>();
            reserve_bytes = hipcx_n_step_rnn_reserve_size(static_cast<int>(n_layers), bidirectional, mode, &chx_, ops.px.data(), n_steps);
            state->reserve = device.Allocate(reserve_bytes);
            state->reserve_bytes = reserve_bytes;
            state->mode = mode;
            state->activation = RnnActivation(activation);
            reserve = state->reserve.get();
        }
        size_t ws_bytes = hipcx_n_step_rnn_workspace_size(static_cast<int>(n_layers), bidirectional, mode, 0, &chx_, ops.px.data(), n_steps);
        if (training) ws_bytes = hipcx_n_step_rnn_workspace_size(static_cast<int>(n_layers), bidirectional, mode, 1, &chx_, ops.px.data(), n_steps);
        std::shared_ptr<void> wsp = device.Allocate(ws_bytes);
        Check(hipcx_n_step_rnn(static_cast<int>(n_layers), bidirectional, mode, RnnActivation(activation), &chx_, mode == 1 ? &ccx : nullptr,
                               ops.pw.data(), ops.pb.data(), ops.px.data(), n_steps, &chy, mode == 1 ? &ccy : nullptr, py.data(), reserve,
                               reserve_bytes, wsp.get(), ws_bytes, nullptr));
        std::vector<std::vector<Array>> ret;
        std::vector<Array> states{std::move(hy)};
        if (mode == 1) states.emplace_back(std::move(cy));
        ret.emplace_back(std::move(states));
        ret.emplace_back(std::move(ys));
        return std::make_tuple(std::move(ret), std::unique_ptr<RnnGradState>{std::move(state)});
    }
};
HIPCX_REGISTER_KERNEL(RnnKernel, HipRnnKernel)

class HipRnnBackwardKernel : public RnnBackwardKernel {
public:
    // Returns {{dhx[, dcx]}, {dw, db for every matrix in ws' order}, {dxs}} as NStepRnnImpl's backward reads it
    // (chainerx/routines/n_step_rnn.cc:330-354).
    std::vector<std::vector<Array>> Call(
            int64_t n_layers, Array hx, absl::optional<Array> cx, const std::vector<std::vector<Array>>& ws, const std::vector<std::vector<Array>>& bs,
            const std::vector<Array>& xs, Array dhy, absl::optional<Array> dcy, std::vector<Array> /*ys*/, std::vector<Array> dys,
            int8_t bidirectional, const std::shared_ptr<chainerx::RnnGradState>& state) override {
        auto* st = dynamic_cast<HipRnnGradState*>(state.get());
        if (st == nullptr) throw ChainerxError{"hip RnnBackwardKernel: the forward pass kept no state (no input required a gradient)."};
        Device& device = hx.device();
        SetDeviceScope scope{device.index()};
        const int8_t mode = st->mode;
        RnnOperands ops;
        PrepareRnnOperands(ops, device, hx, ws, bs, xs);
        hipcx_array chx_ = PrepareRnnOperand(ops, device, hx, hx);
        hipcx_array cdhy = PrepareRnnOperand(ops, device, hx, dhy);
        hipcx_array cdcy{};
        const bool has_dcy = mode == 1 && dcy.has_value();
        if (has_dcy) cdcy = PrepareRnnOperand(ops, device, hx, *dcy);
        std::vector<hipcx_array> cdys;
        for (const Array& g : dys) cdys.push_back(PrepareRnnOperand(ops, device, hx, g));
        std::vector<const hipcx_array*> pdys = PointersTo(cdys);
        Array dhx = Empty(hx.shape(), Dtype::kFloat32, device);
        Array dcx = mode == 1 ? Empty(hx.shape(), Dtype::kFloat32, device) : Array{};
        std::vector<Array> dws, dbs, dxs, params;
        std::vector<hipcx_array> cdw, cdb, cdx;
        for (size_t i = 0; i < ws.size(); ++i) {
            for (size_t j = 0; j < ws[i].size(); ++j) {
                dws.emplace_back(Empty(ws[i][j].shape(), Dtype::kFloat32, device));
                dbs.emplace_back(Empty(bs.at(i).at(j).shape(), Dtype::kFloat32, device));
            }
        }
        for (const Array& x : xs) dxs.emplace_back(Empty(x.shape(), Dtype::kFloat32, device));
        for (const Array& a : dws) cdw.push_back(ToC(a));
        for (const Array& a : dbs) cdb.push_back(ToC(a));
        for (const Array& a : dxs) cdx.push_back(ToC(a));
        std::vector<const hipcx_array*> pdw = PointersTo(cdw), pdb = PointersTo(cdb), pdx = PointersTo(cdx);
        hipcx_array cdhx = ToC(dhx), cdcx{};
        if (mode == 1) cdcx = ToC(dcx);
        const int n_steps = static_cast<int>(xs.size());
        size_t ws_bytes = hipcx_n_step_rnn_workspace_size(static_cast<int>(n_layers), bidirectional, mode, 1, &chx_, ops.px.data(), n_steps);
        std::shared_ptr<void> wsp = device.Allocate(ws_bytes);
        Check(hipcx_n_step_rnn_backward(static_cast<int>(n_layers), bidirectional, mode, st->activation, &chx_, ops.pw.data(), ops.pb.data(),
                                        ops.px.data(), n_steps, &cdhy, has_dcy ? &cdcy : nullptr, pdys.data(), st->reserve.get(), st->reserve_bytes,
                                        &cdhx, mode == 1 ? &cdcx : nullptr, pdw.data(), pdb.data(), pdx.data(), wsp.get(), ws_bytes, nullptr));
        std::vector<Array> states{std::move(dhx)};
        if (mode == 1) states.emplace_back(std::move(dcx));
        for (size_t i = 0; i < dws.size(); ++i) {  // interleaved: w0, b0, w1, b1, ...
            params.emplace_back(std::move(dws[i]));
            params.emplace_back(std::move(dbs[i]));
        }
        std::vector<std::vector<Array>> ret;
        ret.emplace_back(std::move(states));
        ret.emplace_back(std::move(params));
        ret.emplace_back(std::move(dxs));
        return ret;
    }
};
HIPCX_REGISTER_KERNEL(RnnBackwardKernel, HipRnnBackwardKernel)

// ---- linear algebra: Solve, Inverse, Cholesky, Syevd, Qr, Svd (the LAPACK-backed kernels of the native backend, native_device/linalg.cc) ----
namespace {
// A zeroed device int32 for LAPACK's `info`, and the check that turns a non-zero value into the reference's ChainerxError.
std::shared_ptr<void> NewInfoFlag(Device& device) { return NewDeviceFlag(device); }
void ThrowIfInfo(Device& device, const std::shared_ptr<void>& flag, const char* what) {
    const int32_t host = ReadDeviceFlag(device, flag);
    if (host != 0) throw ChainerxError{"Unsuccessful ", what, " execution. Info = ", host};
}
}  // namespace

class HipSolveKernel : public SolveKernel {
public:
    void Call(const Array& a, const Array& b, const Array& out) override {
        Device& device = a.device();
        device.CheckDevicesCompatible(a, b, out);
        SetDeviceScope scope{device.index()};
        if (out.dtype() == Dtype::kFloat16) throw DtypeError{"Half-precision (float16) is not supported by solve"};
        hipcx_array ca = ToC(a), cb = ToC(b), co = ToC(out);
        size_t ws_bytes = hipcx_solve_workspace_size(&ca);
        std::shared_ptr<void> ws = device.Allocate(ws_bytes);
        std::shared_ptr<void> flag = NewInfoFlag(device);
        Check(hipcx_solve(&ca, &cb, &co, ws.get(), ws_bytes, static_cast<int32_t*>(flag.get()), nullptr));
        ThrowIfInfo(device, flag, "gesv (Solve)");
    }
};
HIPCX_REGISTER_KERNEL(SolveKernel, HipSolveKernel)

class HipInverseKernel : public InverseKernel {
public:
    void Call(const Array& a, const Array& out) override {
        Device& device = a.device();
        device.CheckDevicesCompatible(a, out);
        SetDeviceScope scope{device.index()};
        if (out.dtype() == Dtype::kFloat16) throw DtypeError{"Half-precision (float16) is not supported by inverse"};
        hipcx_array ca = ToC(a), co = ToC(out);
        size_t ws_bytes = hipcx_solve_workspace_size(&ca);
        std::shared_ptr<void> ws = device.Allocate(ws_bytes);
        std::shared_ptr<void> flag = NewInfoFlag(device);
        Check(hipcx_inverse(&ca, &co, ws.get(), ws_bytes, static_cast<int32_t*>(flag.get()), nullptr));
        ThrowIfInfo(device, flag, "getrf (LU)");
    }
};
HIPCX_REGISTER_KERNEL(InverseKernel, HipInverseKernel)

class HipCholeskyKernel : public CholeskyKernel {
public:
    void Call(const Array& a, const Array& out) override {
        Device& device = a.device();
        device.CheckDevicesCompatible(a, out);
        SetDeviceScope scope{device.index()};
        if (out.dtype() == Dtype::kFloat16) throw DtypeError{"Half-precision (float16) is not supported by cholesky"};
        hipcx_array ca = ToC(a), co = ToC(out);
        std::shared_ptr<void> flag = NewInfoFlag(device);
        Check(hipcx_cholesky(&ca, &co, static_cast<int32_t*>(flag.get()), nullptr));
        ThrowIfInfo(device, flag, "potrf (Cholesky)");
    }
};
HIPCX_REGISTER_KERNEL(CholeskyKernel, HipCholeskyKernel)

class HipSyevdKernel : public SyevdKernel {
public:
    void Call(const Array& a, const Array& w, const Array& v, char uplo, bool compute_v) override {
        Device& device = a.device();
        device.CheckDevicesCompatible(a, w, v);
        SetDeviceScope scope{device.index()};
        if (a.dtype() == Dtype::kFloat16) throw DtypeError{"Half-precision (float16) is not supported by eigen decomposition"};
        hipcx_array ca = ToC(a), cw = ToC(w), cv = ToC(v);
        size_t ws_bytes = hipcx_syevd_workspace_size(&ca);
        std::shared_ptr<void> ws = device.Allocate(ws_bytes);
        Check(hipcx_syevd(&ca, &cw, &cv, uplo, compute_v ? 1 : 0, ws.get(), ws_bytes, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(SyevdKernel, HipSyevdKernel)

class HipQrKernel : public QrKernel {
public:
    void Call(const Array& a, const Array& q, const Array& r, const Array& tau, QrMode mode) override {
        Device& device = a.device();
        device.CheckDevicesCompatible(a, q, r, tau);
        SetDeviceScope scope{device.index()};
        if (a.dtype() == Dtype::kFloat16) throw DtypeError{"Half-precision (float16) is not supported by QR decomposition"};
        int code = HIPCX_QR_REDUCED;
        switch (mode) {
            case QrMode::kReduced: code = HIPCX_QR_REDUCED; break;
            case QrMode::kComplete: code = HIPCX_QR_COMPLETE; break;
            case QrMode::kR: code = HIPCX_QR_R; break;
            case QrMode::kRaw: code = HIPCX_QR_RAW; break;
            default: throw ChainerxError{"Invalid QR mode"};
        }
        hipcx_array ca = ToC(a), cq = ToC(q), cr = ToC(r), ct = ToC(tau);
        size_t ws_bytes = hipcx_qr_workspace_size(&ca);
        std::shared_ptr<void> ws = device.Allocate(ws_bytes);
        const bool want_q = mode == QrMode::kReduced || mode == QrMode::kComplete;
        Check(hipcx_qr(&ca, want_q ? &cq : nullptr, &cr, &ct, code, ws.get(), ws_bytes, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(QrKernel, HipQrKernel)

class HipSvdKernel : public SvdKernel {
public:
    void Call(const Array& a, const Array& u, const Array& s, const Array& vt, bool full_matrices, bool compute_uv) override {
        Device& device = a.device();
        device.CheckDevicesCompatible(a, u, s, vt);
        SetDeviceScope scope{device.index()};
        if (a.dtype() == Dtype::kFloat16) throw DtypeError{"Half-precision (float16) is not supported by SVD"};
        hipcx_array ca = ToC(a), cu = ToC(u), cs = ToC(s), cvt = ToC(vt);
        size_t ws_bytes = hipcx_svd_workspace_size(&ca);
        std::shared_ptr<void> ws = device.Allocate(ws_bytes);
        // without compute_uv the routine hands over placeholders of shape (0,) (routines/linalg.cc:216-218): the entry ignores them
        Check(hipcx_svd(&ca, compute_uv ? &cu : nullptr, &cs, compute_uv ? &cvt : nullptr, full_matrices ? 1 : 0, compute_uv ? 1 : 0, ws.get(),
                        ws_bytes, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(SvdKernel, HipSvdKernel)

// ---- take ----
class HipTakeKernel : public TakeKernel {
public:
    void Call(const Array& a, const Array& indices, int8_t axis, const Array& out, IndexBoundsMode mode) override {
        Device& device = a.device();
        device.CheckDevicesCompatible(a, indices, out);
        SetDeviceScope scope{device.index()};
        hipcx_array ca = ToC(a), ci = ToC(indices), co = ToC(out);
        int m = HIPCX_BOUNDS_DEFAULT;
        switch (mode) {
            case IndexBoundsMode::kRaise: m = HIPCX_BOUNDS_RAISE; break;
            case IndexBoundsMode::kWrap: m = HIPCX_BOUNDS_WRAP; break;
            case IndexBoundsMode::kClip: m = HIPCX_BOUNDS_CLIP; break;
            default: break;
        }
        // kRaise: checked here, at the cost of a read-back (native_device/indexing.cc:68-74).  kDefault, what the routine passes
        // for mode=None: no flag -- the library records an out-of-range index on the device and HipDevice::Synchronize /
        // MemoryCopyTo, the calls that wait for the device, throw the IndexError before any result can be read.
        bool checks = m == HIPCX_BOUNDS_RAISE;
        std::shared_ptr<void> flag = checks ? NewDeviceFlag(device) : nullptr;
        Check(hipcx_take(&ca, &ci, axis, &co, m, static_cast<int32_t*>(flag.get()), nullptr));
        if (checks) {
            const int32_t host = ReadDeviceFlag(device, flag);
            if (host != 0) throw IndexError{"Index is out of bounds for axis ", static_cast<int>(axis), " with size ", a.shape()[axis]};
        }
    }
};
HIPCX_REGISTER_KERNEL(TakeKernel, HipTakeKernel)

int ToC(IndexBoundsMode mode) {
    switch (mode) {
        case IndexBoundsMode::kRaise: return HIPCX_BOUNDS_RAISE;
        case IndexBoundsMode::kWrap: return HIPCX_BOUNDS_WRAP;
        case IndexBoundsMode::kClip: return HIPCX_BOUNDS_CLIP;
        default: return HIPCX_BOUNDS_DEFAULT;
    }
}

class HipAddAtKernel : public AddAtKernel {
public:
    void Call(const Array& a, const Array& indices, int8_t axis, const Array& b, const Array& out, IndexBoundsMode mode) override {
        Device& device = a.device();
        device.CheckDevicesCompatible(a, indices, b, out);
        SetDeviceScope scope{device.index()};
        hipcx_array ca = ToC(a), ci = ToC(indices), cb = ToC(Cast(b, a.dtype())), co = ToC(out);
        int m = ToC(mode);
        bool checks = m == HIPCX_BOUNDS_RAISE;  // kDefault: deferred, as in HipTakeKernel
        std::shared_ptr<void> flag = checks ? NewDeviceFlag(device) : nullptr;
        Check(hipcx_add_at(&ca, &ci, axis, &cb, &co, m, static_cast<int32_t*>(flag.get()), nullptr));
        if (checks) {
            const int32_t host = ReadDeviceFlag(device, flag);
            if (host != 0) throw IndexError{"Index is out of bounds for axis ", static_cast<int>(axis), " with size ", a.shape()[axis]};
        }
    }
};
HIPCX_REGISTER_KERNEL(AddAtKernel, HipAddAtKernel)

// ---- creation patterns, Cumsum, Nansum ----
class HipIdentityKernel : public IdentityKernel {
public:
    void Call(const Array& out) override {
        SetDeviceScope scope{out.device().index()};
        hipcx_array o = ToC(out);
        Check(hipcx_identity(&o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(IdentityKernel, HipIdentityKernel)

class HipEyeKernel : public EyeKernel {
public:
    void Call(int64_t k, const Array& out) override {
        SetDeviceScope scope{out.device().index()};
        hipcx_array o = ToC(out);
        Check(hipcx_eye(k, &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(EyeKernel, HipEyeKernel)

class HipTriKernel : public TriKernel {
public:
    void Call(int64_t k, const Array& out) override {
        SetDeviceScope scope{out.device().index()};
        hipcx_array o = ToC(out);
        Check(hipcx_tri(k, &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(TriKernel, HipTriKernel)

class HipLinspaceKernel : public LinspaceKernel {
public:
    void Call(double start, double stop, const Array& out) override {
        SetDeviceScope scope{out.device().index()};
        hipcx_array o = ToC(out);
        Check(hipcx_linspace(start, stop, &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(LinspaceKernel, HipLinspaceKernel)

class HipDiagflatKernel : public DiagflatKernel {
public:
    void Call(const Array& v, int64_t k, const Array& out) override {
        Device& device = v.device();
        device.CheckDevicesCompatible(v, out);
        SetDeviceScope scope{device.index()};
        hipcx_array cv = ToC(v), o = ToC(out);
        Check(hipcx_diagflat(&cv, k, &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(DiagflatKernel, HipDiagflatKernel)

class HipCumsumKernel : public CumsumKernel {
public:
    void Call(const Array& a, int8_t axis, const Array& out) override {
        Device& device = a.device();
        device.CheckDevicesCompatible(a, out);
        SetDeviceScope scope{device.index()};
        hipcx_array ca = ToC(a), o = ToC(out);
        Check(hipcx_cumsum(&ca, axis, &o, nullptr));
    }
};
HIPCX_REGISTER_KERNEL(CumsumKernel, HipCumsumKernel)

// the routine has already replaced NaNs by zeros (CX/routines/reduction.cc:151); the native NansumKernel is its SumKernel
class HipNansumKernel : public NansumKernel {
public:
    void Call(const Array& a, const Axes& axis, const Array& out) override { CallReduce(hipcx_sum, a, axis, out); }
};
HIPCX_REGISTER_KERNEL(NansumKernel, HipNansumKernel)

}  // namespace
}  // namespace hip
}  // namespace chainerx

// NOLINTNEXTLINE(cppcoreguidelines-owning-memory)
extern "C" chainerx::Backend* CreateBackend(chainerx::Context& ctx) { return new chainerx::hip::HipBackend{ctx}; }

// NOLINTNEXTLINE(cppcoreguidelines-owning-memory)
extern "C" void DestroyBackend(chainerx::Backend* backend) { delete backend; }
