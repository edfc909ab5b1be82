// Enumerations shared by the host front-end.  Same names and numeric values as the reference's
// include/Ctools.h:150-209 (DeviceType, DType, op) and :81-120 (ErrorLevel, ErrorPlatform,
// ErrorType), plus one new device: kAMD = 7.  The reference casts DeviceType <-> ErrorPlatform by
// value (include/Ctools.h:249-251, src/Ctools.cpp:17-19) and ErrorPlatform 6 is taken by
// kAutoDiff, so the new enumerator takes 7 in both enums.
#ifndef CTORCH_AMD_HOST_CTOOLS_H
#define CTORCH_AMD_HOST_CTOOLS_H
#include <cstddef>
#include <cstdint>
#include <stdexcept>

enum class DeviceType { kCPU = 0, kCUDA = 1, kMPS = 2, kAMX = 3, kUNKNOWN = 4, kGENERAL = 5, kAMD = 7 };

enum class DType { kFloat, kDouble, kInt, kLong, kBool };

enum class op {
    Add, Sub, Neg, Mul, Div, MatMul, Dot, Cos, Sin,
    Conv, Pool,
    ReLU, Tanh, Sigmoid, Softmax,
    LReLU, PReLU,
    MSE, MAE, CE, BCE,
    Sum,
    Linear,   // not in the reference: matmul + bias row (+ ReLU) as one taped operator, Tensor::linear
    Fused,    // not in the reference: an elementwise expression evaluated in one pass, Expr::eval
    LinearCE, // not in the reference: the last layer and its class-index cross entropy, Tensor::linear_cross_entropy
    // methods the reference declares on Tensor without defining them (include/Tensor.h:824-1072); they
    // have no enumerator there because nothing tapes them
    Abs, Exp, Log, Sqrt, Square, Tan, LogSoftmax,
    Reduce,   // sum / mean / max / min / var / std along dimensions; which one is in the node's payload
};

enum class ErrorLevel { TRACE = 0, DEBUG = 1, INFO = 2, WARN = 3, ERROR = 4, FATAL = 5 };
enum class ErrorPlatform { kCPU = 0, kCUDA = 1, kMPS = 2, kAMX = 3, kUNKNOWN = 4, kGENERAL = 5, kAutoDiff = 6, kAMD = 7 };
enum class ErrorType {
    UNKNOWN = 0, MEMORY = 1, DIMENSION = 2, DEVICE_COMPAT = 3, DATATYPE = 4, KERNEL_LAUNCH = 5, TENSOR_STATE = 6,
    PLATFORM_API = 7
};
enum class PrintLevel { MINIUM = 0, MEDIUM = 1, FULL = 2 };

inline ErrorPlatform DeviceTypeToErrorPlatform(DeviceType d) { return static_cast<ErrorPlatform>(static_cast<uint32_t>(d)); }

constexpr const char* dtypeToString(DType dtype) {
    switch (dtype) {
        case DType::kFloat: return "float32";
        case DType::kDouble: return "float64";
        case DType::kInt: return "int32";
        case DType::kLong: return "int64";
        case DType::kBool: return "bool";
    }
    return "unknown";
}

constexpr size_t dtypeSize(DType dtype) {
    switch (dtype) {
        case DType::kFloat: return sizeof(float);
        case DType::kDouble: return sizeof(double);
        case DType::kInt: return sizeof(int32_t);
        case DType::kLong: return sizeof(int64_t);
        case DType::kBool: return sizeof(bool);
    }
    throw std::invalid_argument("unknown dtype");
}

#endif
