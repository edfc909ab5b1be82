// Storage: the bytes behind a Tensor.  Same interface as the reference's include/Storage.h
// (ctor :77, data<T>() :131-151, clone() :175-181, shallow copies :98-103), with the `device` tag
// made real: a kAMD storage lives in HBM (allocated through the C ABI's ctamd_malloc, recycled by
// a size-bucketed pool so that an op's result does not pay a hipMalloc / hipFree), clone() is a
// device-to-device copy, to(device) is the explicit host <-> device transfer, and data<T>() on a
// device storage throws instead of handing a host pointer to HBM.
#ifndef CTORCH_AMD_HOST_STORAGE_H
#define CTORCH_AMD_HOST_STORAGE_H
#include <cmath>
#include <cstring>
#include <memory>
#include <type_traits>

#include "Ctools.h"
#include "Ctorch_Error.h"

namespace ctorch_amd_host {
// Device memory pool (src/DeviceMemory.cpp).  acquire() returns HBM of at least `bytes` bytes,
// release() returns it to the pool; trim() frees everything cached.
// Blocks acquired between reservation_begin() and reservation_stop() (on this thread) belong to
// the reservation: when released they are parked with it, not handed to anyone else, until
// reservation_destroy().  This is what keeps the memory of a recorded graph its own.
struct BlockReservation;
BlockReservation* reservation_begin();
void reservation_stop();
void reservation_destroy(BlockReservation* r);
void* device_acquire(size_t bytes);
void device_release(void* p, size_t bytes);
void device_trim();
void device_copy_h2d(void* dst, const void* src, size_t bytes);
void device_copy_d2h(void* dst, const void* src, size_t bytes);
void device_copy_d2d(void* dst, const void* src, size_t bytes);
void device_sync();
}  // namespace ctorch_amd_host

class Storage {
   private:
    size_t _size{};
    DType _dtype;
    DeviceType _device;
    std::shared_ptr<char[]> _data;

    template <typename T>
    void checkDType() const {
        if ((std::is_same<T, float>::value && _dtype != DType::kFloat) ||
            (std::is_same<T, double>::value && _dtype != DType::kDouble) ||
            (std::is_same<T, int32_t>::value && _dtype != DType::kInt) ||
            (std::is_same<T, int64_t>::value && _dtype != DType::kLong) ||
            (std::is_same<T, bool>::value && _dtype != DType::kBool)) {
            Ctorch_Error::throwException(ErrorPlatform::kGENERAL, ErrorType::DATATYPE, "Storage data type mismatch");
        }
    }
    // Returns a device block to the pool; it also carries what the host knows of a one-element
    // block's value, so that every tensor sharing the block sees one state (std::get_deleter).
    struct DeviceBlock {
        size_t bytes;
        bool known = false;
        float value = 0.0f;
        bool frozen = false;    // handed out as a gradient that shares the tape's bytes: read-only while shared
        // what the host saw when it uploaded the block's floats, read as class indices (converted to int
        // the way the reference converts them): the least and the greatest, or seen_bad for one that no
        // class count admits (NaN, an infinity, beyond int)
        bool seen = false, seen_bad = false;
        int lo = 0, hi = 0;
        void operator()(char* q) const { ctorch_amd_host::device_release(q, bytes); }
    };
    DeviceBlock* block() const { return _data ? std::get_deleter<DeviceBlock>(_data) : nullptr; }
    static std::shared_ptr<char[]> allocate(size_t bytes, DeviceType device) {
        if (bytes == 0) return nullptr;
        if (device == DeviceType::kAMD) {
            char* p = static_cast<char*>(ctorch_amd_host::device_acquire(bytes));
            return std::shared_ptr<char[]>(p, DeviceBlock{bytes});
        }
        return std::shared_ptr<char[]>(new char[bytes], std::default_delete<char[]>());
    }

   public:
    Storage(size_t size, DType dtype, DeviceType device = DeviceType::kCPU)
        : _size(size), _dtype(dtype), _device(device), _data(allocate(size * dtypeSize(dtype), device)) {}

    // copies `size` elements from HOST memory into the new storage (an upload for kAMD)
    template <typename T>
    Storage(const T* data, size_t size, DType dtype, DeviceType device = DeviceType::kCPU) : Storage(size, dtype, device) {
        if (size > 0 && _data.get()) {
            if (device == DeviceType::kAMD) {
                ctorch_amd_host::device_copy_h2d(_data.get(), data, size * dtypeSize(dtype));
                if (dtype == DType::kFloat && sizeof(T) == sizeof(float)) note_uploaded_floats(reinterpret_cast<const float*>(data), size);
            } else {
                std::memcpy(_data.get(), data, size * dtypeSize(dtype));
            }
        }
    }

    Storage(const Storage&) = default;
    Storage& operator=(const Storage&) = default;
    Storage(Storage&&) = default;
    Storage& operator=(Storage&&) = default;
    Storage() : _size(0), _dtype(DType::kFloat), _device(DeviceType::kCPU) {}
    ~Storage() = default;

    // host pointer; throws for a device storage (use raw() / to(kCPU))
    template <typename T>
    T* data() {
        if (_size == 0 || !_data) return nullptr;
        checkDType<T>();
        requireHost();
        return reinterpret_cast<T*>(_data.get());
    }
    template <typename T>
    const T* data() const {
        if (_size == 0 || !_data) return nullptr;
        checkDType<T>();
        requireHost();
        return reinterpret_cast<const T*>(_data.get());
    }
    // untyped pointer in the storage's own address space (HBM for kAMD); for the launch layer
    void* raw() { return _data.get(); }
    const void* raw() const { return _data.get(); }
    // true while another Storage object (a view, an alias) refers to the same bytes
    bool shared() const { return _data.use_count() > 1; }

    // The value of a one-element device storage when the host knows it without reading the device
    // (it chose it, or a kernel's result came back with another read).  One state per block: an
    // in-place writer that forgets it does so for every tensor that shares the block.
    const float* known_value() const {
        const DeviceBlock* b = block();
        return (b && b->known) ? &b->value : nullptr;
    }
    void set_known_value(float v) {
        DeviceBlock* b = block();
        if (b && _size == 1) { b->known = true; b->value = v; }
    }
    void forget_known_value() {
        if (DeviceBlock* b = block()) { b->known = false; b->seen = false; }
    }
    // Class indices uploaded from the host: the upload looked at them (a short vector of floats), so a
    // loss over them need not wait for the device to say whether they are in range.  1: every element,
    // converted to int as the reference converts it, lies in [0, classes); 0: some element does not;
    // -1: the host does not know (the block was computed on the device, written in place since, or is long).
    int class_indices_below(size_t classes) const {
        const DeviceBlock* b = block();
        if (!b || !b->seen) return -1;
        if (b->seen_bad) return 0;
        return (b->lo >= 0 && size_t(b->hi) < classes) ? 1 : 0;
    }
    static constexpr size_t kLooksAtUploadsUpTo = size_t(1) << 16;
    void note_uploaded_floats(const float* host, size_t n) {
        DeviceBlock* b = block();
        if (!b || n == 0 || n > kLooksAtUploadsUpTo) return;
        bool bad = false;
        int lo = 0, hi = 0;
        for (size_t i = 0; i < n; ++i) {
            const float v = host[i];
            if (!(std::fabs(v) < 2147483648.0f)) { bad = true; break; }     // NaN too
            const int c = static_cast<int>(v);
            if (i == 0 || c < lo) lo = c;
            if (i == 0 || c > hi) hi = c;
        }
        b->seen = true;
        b->seen_bad = bad;
        b->lo = lo;
        b->hi = hi;
    }
    // A gradient read from the tape shares the tape's bytes.  While more than one tensor holds the
    // block it must not be written in place; the front-end's in-place writers ask here first.
    void freeze() {
        if (DeviceBlock* b = block()) b->frozen = true;
    }
    bool writable() {
        DeviceBlock* b = block();
        if (!b || !b->frozen) return true;
        if (_data.use_count() > 1) return false;
        b->frozen = false;      // the last holder may do what it likes
        return true;
    }

    size_t size() const { return _size; }
    DType dtype() const { return _dtype; }
    DeviceType device() const { return _device; }
    size_t nbytes() const { return _size * dtypeSize(_dtype); }

    Storage clone() const {
        Storage s(_size, _dtype, _device);
        if (_size > 0 && _data) {
            if (_device == DeviceType::kAMD) ctorch_amd_host::device_copy_d2d(s._data.get(), _data.get(), nbytes());
            else std::memcpy(s._data.get(), _data.get(), nbytes());
            if (const float* v = known_value()) s.set_known_value(*v);
        }
        return s;
    }

    // explicit transfer: a new storage on `device` holding the same bytes
    Storage to(DeviceType device) const {
        if (device == _device) return clone();
        if (device != DeviceType::kCPU && device != DeviceType::kAMD)
            Ctorch_Error::throwException(DeviceTypeToErrorPlatform(device), ErrorType::DEVICE_COMPAT, "Storage::to: unsupported device");
        Storage s(_size, _dtype, device);
        if (_size > 0 && _data) {
            if (device == DeviceType::kAMD) {
                ctorch_amd_host::device_copy_h2d(s._data.get(), _data.get(), nbytes());
                if (_dtype == DType::kFloat) s.note_uploaded_floats(reinterpret_cast<const float*>(_data.get()), _size);
            } else {
                ctorch_amd_host::device_copy_d2h(s._data.get(), _data.get(), nbytes());
            }
        }
        return s;
    }

    void clear() {
        _data.reset();
        _size = 0;
    }
    bool empty() const { return _size == 0 || !_data; }

   private:
    void requireHost() const {
        if (_device == DeviceType::kAMD)
            Ctorch_Error::throwException(ErrorPlatform::kAMD, ErrorType::MEMORY,
                                         "Storage::data<T>(): storage is in device memory; transfer it with to(kCPU)");
    }
};
#endif
