// Ctorch_Scheduler: op x DeviceType -> kernel function pointer, the reference's dispatch table
// (include/Ctorch_Scheduler.h:15-168) with the AMD column populated.  Same interface:
// getInstance(), dispatch(a, b, op), dispatch(a, op), isDeviceAvailable(); same pre-checks
// (:88-94, log only) and lazy registration under the mutex (:97-105).  One deliberate difference:
// where the reference logs "no kernel" and then calls through a null pointer (:124-128), this
// throws.
#ifndef CTORCH_AMD_HOST_SCHEDULER_H
#define CTORCH_AMD_HOST_SCHEDULER_H
#include <mutex>
#include <unordered_map>

#include "Ctorch_Error.h"
#include "Tensor.h"
#include "kernels.h"

class Ctorch_Scheduler {
   private:
    Ctorch_Scheduler() = default;
    Ctorch_Scheduler(const Ctorch_Scheduler&) = delete;
    Ctorch_Scheduler& operator=(const Ctorch_Scheduler&) = delete;
    std::mutex mutex_;
    bool inited_ = false;
    std::unordered_map<op, std::unordered_map<DeviceType, BinaryKernelFunc>> binary_kernel_map_;
    std::unordered_map<op, std::unordered_map<DeviceType, UnaryKernelFunc>> unary_kernel_map_;

    void initKernelMap() {
        binary_kernel_map_[op::Add][DeviceType::kAMD] = Add_AMD_kernel;
        binary_kernel_map_[op::Sub][DeviceType::kAMD] = Sub_AMD_kernel;
        binary_kernel_map_[op::Mul][DeviceType::kAMD] = Mul_AMD_kernel;
        binary_kernel_map_[op::Div][DeviceType::kAMD] = Div_AMD_kernel;
        binary_kernel_map_[op::MatMul][DeviceType::kAMD] = MatMul_AMD_kernel;
        binary_kernel_map_[op::Dot][DeviceType::kAMD] = Dot_AMD_kernel;
        binary_kernel_map_[op::MSE][DeviceType::kAMD] = MSE_AMD_kernel;
        binary_kernel_map_[op::CE][DeviceType::kAMD] = CrossEntropy_AMD_kernel;
        binary_kernel_map_[op::MAE][DeviceType::kAMD] = MAE_AMD_kernel;
        unary_kernel_map_[op::Neg][DeviceType::kAMD] = Neg_AMD_kernel;
        unary_kernel_map_[op::ReLU][DeviceType::kAMD] = ReLU_AMD_kernel;
        unary_kernel_map_[op::Cos][DeviceType::kAMD] = Cos_AMD_kernel;
        unary_kernel_map_[op::Sin][DeviceType::kAMD] = Sin_AMD_kernel;
        unary_kernel_map_[op::Tanh][DeviceType::kAMD] = Tanh_AMD_kernel;
        unary_kernel_map_[op::Sigmoid][DeviceType::kAMD] = Sigmoid_AMD_kernel;
        unary_kernel_map_[op::Softmax][DeviceType::kAMD] = Softmax_AMD_kernel;
        // the reference registers LReLU without a function (:51-52) and defines no LReLU kernel anywhere;
        // here the column has one
        unary_kernel_map_[op::LReLU][DeviceType::kAMD] = LReLU_AMD_kernel;
    }
    void ensureInit() {
        std::lock_guard<std::mutex> lock(mutex_);
        if (!inited_) {
            initKernelMap();
            inited_ = true;
        }
    }

   public:
    static Ctorch_Scheduler& getInstance() {
        static Ctorch_Scheduler instance_;
        return instance_;
    }

    // kAMD is available when a gfx950 device can be initialised; kCPU has no kernels in this
    // library (the reference's CPU-BASIC kernels are not part of it).
    static bool isDeviceAvailable(DeviceType dev_type);

    static DeviceType getTargetDevice(const Tensor& a, const Tensor& b) {
        if (a.device() != b.device())
            Ctorch_Error::log(ErrorLevel::ERROR, ErrorPlatform::kGENERAL, ErrorType::DEVICE_COMPAT,
                              "Ctorch_Scheduler: tensors are on different devices");
        return a.device();
    }

    // The kernel registered for (operator, device).  The reference calls whatever its lookup left in the
    // pointer, a null pointer included (include/Ctorch_Scheduler.h:128, :165); here a missing entry or a
    // device that is not there throws.
    template <class Table>
    typename Table::mapped_type::mapped_type find_kernel(Table& table, op which, DeviceType where) {
        ensureInit();
        typename Table::mapped_type::mapped_type found = nullptr;
        {
            std::lock_guard<std::mutex> lock(mutex_);
            auto row = table.find(which);
            if (row != table.end() && isDeviceAvailable(where)) {
                auto cell = row->second.find(where);
                if (cell != row->second.end()) found = cell->second;
            }
        }
        if (found == nullptr)
            Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::PLATFORM_API,
                                         "Ctorch_Scheduler: no kernel available for this op on this device");
        return found;
    }

    Tensor dispatch(const Tensor& a, const Tensor& b, op op_type) {
        if (a.dtype() != b.dtype())
            Ctorch_Error::log(ErrorLevel::ERROR, ErrorPlatform::kGENERAL, ErrorType::DATATYPE,
                              "Ctorch_Scheduler: tensor dtypes differ");
        if (op_type != op::Add && op_type != op::Mul && op_type != op::Sub && op_type != op::Div &&
            op_type != op::CE && op_type != op::MatMul && a.sizes() != b.sizes())
            Ctorch_Error::log(ErrorLevel::ERROR, ErrorPlatform::kGENERAL, ErrorType::DIMENSION,
                              "Ctorch_Scheduler: tensor shapes differ");
        BinaryKernelFunc run = find_kernel(binary_kernel_map_, op_type, getTargetDevice(a, b));
        return run(a, b);
    }

    Tensor dispatch(const Tensor& a, op op_type) {
        UnaryKernelFunc run = find_kernel(unary_kernel_map_, op_type, a.device());
        return run(a);
    }

    // Registration point for further device columns (and for tests that register a stand-in).
    void registerKernel(op o, DeviceType d, BinaryKernelFunc f) {
        ensureInit();
        std::lock_guard<std::mutex> lock(mutex_);
        binary_kernel_map_[o][d] = f;
    }
    void registerKernel(op o, DeviceType d, UnaryKernelFunc f) {
        ensureInit();
        std::lock_guard<std::mutex> lock(mutex_);
        unary_kernel_map_[o][d] = f;
    }
};
#endif
