// Implementation classes behind the public de:: objects.  Host C++ only: the GPU is
// reached exclusively through the C ABI of decx_hip.h.
#pragma once
#include "DECX.h"
#include "decx_hip.h"

#include <cstddef>
#include <memory>
#include <mutex>

namespace decx {

// Status helpers (the library-side view of de::DH).
namespace err {
void set(de::DH* h, int code, const char* text);
void success(de::DH* h);
// Translates a decx_hip return code into the handle; returns true when rc signals failure.
bool from_hip(de::DH* h, int rc, const char* what);
}  // namespace err

bool gpu_ready();
uint32_t element_size(de::_DATA_TYPES_FLAGS_ type);

// Reference-counted storage shared by SoftCopy aliases.
struct HostBlock {
    void* ptr = nullptr;
    size_t bytes = 0;
    bool pinned = false;
    ~HostBlock();
};
struct DeviceBlock {
    void* ptr = nullptr;
    size_t bytes = 0;
    ~DeviceBlock();
};

// Host matrix.  Layout rule of the original (srcs/modules/core/classes/Matrix.cxx:35-64):
// pitch = width rounded up to 32 bytes of elements, storage zero-filled.
class _Matrix : public de::Matrix {
    de::MatrixLayout _layout;
    de::_DATA_TYPES_FLAGS_ _type;
    de::_DATA_FORMATS_ _format;
    std::shared_ptr<HostBlock> _block;
    void* _data;                       // what _exp_data_ptr points at
    void assign(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height);
    bool allocate();

public:
    _Matrix();
    _Matrix(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, de::_DATA_FORMATS_ format);
    virtual uint32_t Width() const;
    virtual uint32_t Height() const;
    virtual void release();
    virtual de::Matrix& SoftCopy(de::Matrix& src);
    virtual de::_DATA_TYPES_FLAGS_ Type() const;
    virtual void Reinterpret(const de::_DATA_TYPES_FLAGS_ new_type);
    virtual de::_DATA_FORMATS_ Format() const;
    virtual ~_Matrix();

    uint32_t Pitch() const { return _layout.pitch; }
    const de::MatrixLayout& get_layout() const { return _layout; }
    bool is_init() const { return _data != nullptr; }
    void* data() const { return _data; }
    size_t total_bytes() const { return (size_t)_layout.pitch * _layout.height * _layout._single_element_size; }
    void re_construct(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height);
    bool is_pinned() const { return _block && _block->pinned; }
    int move_storage(bool pinned);     // 0 or a decx_hip error code
};

// Device matrix.  Layout rule of the original (srcs/modules/core/classes/GPU_Matrix.cu:35-61):
// pitch = width rounded up to 128 bytes of elements, storage zero-filled.
class _GPU_Matrix : public de::GPU_Matrix {
    de::MatrixLayout _layout;
    de::_DATA_TYPES_FLAGS_ _type;
    de::_DATA_FORMATS_ _format;
    std::shared_ptr<DeviceBlock> _block;
    void assign(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height);
    bool allocate();

public:
    _GPU_Matrix();
    _GPU_Matrix(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, de::_DATA_FORMATS_ format);
    virtual uint Width() const;
    virtual uint Height() const;
    virtual void release();
    virtual de::_DATA_TYPES_FLAGS_ Type() const;
    virtual void Reinterpret(const de::_DATA_TYPES_FLAGS_ new_type);
    virtual de::GPU_Matrix& SoftCopy(de::GPU_Matrix& src);
    virtual de::_DATA_FORMATS_ Format() const;
    virtual ~_GPU_Matrix();

    uint32_t Pitch() const { return _layout.pitch; }
    const de::MatrixLayout& get_layout() const { return _layout; }
    bool is_init() const { return _block && _block->ptr; }
    void* data() const { return _block ? _block->ptr : nullptr; }
    size_t total_bytes() const { return (size_t)_layout.pitch * _layout.height * _layout._single_element_size; }
    // Reshapes; storage is reallocated (and zero-filled) only when it has to grow
    // (srcs/modules/core/classes/GPU_Matrix.cu:120-134).  Returns false on allocation failure.
    bool re_construct(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height);
};

// Host vector.  Storage rule of the original (srcs/modules/core/classes/Vector.cxx): the
// allocation is the length rounded up to 32 bytes of elements, zero-filled.
class _Vector : public de::Vector {
    size_t _length, _capacity;          // elements asked for / elements allocated
    de::_DATA_TYPES_FLAGS_ _type;
    uint32_t _element_size;
    std::shared_ptr<HostBlock> _block;
    void* _data;
    void assign(de::_DATA_TYPES_FLAGS_ type, size_t length);
    bool allocate();

public:
    _Vector();
    _Vector(de::_DATA_TYPES_FLAGS_ type, size_t length);
    virtual size_t Len() const;
    virtual void release();
    virtual de::Vector& SoftCopy(de::Vector& src);
    virtual de::_DATA_TYPES_FLAGS_ Type() const;
    virtual void Reinterpret(const de::_DATA_TYPES_FLAGS_ new_type);
    virtual ~_Vector();

    bool is_init() const { return _data != nullptr; }
    void* data() const { return _data; }
    uint32_t element_bytes() const { return _element_size; }
    size_t capacity_bytes() const { return _block ? _block->bytes : 0; }
    bool re_construct(de::_DATA_TYPES_FLAGS_ type, size_t length);      // grows only
    bool is_pinned() const { return _block && _block->pinned; }
    int move_storage(bool pinned);
};

// Device vector: same length rule, storage in HBM.
class _GPU_Vector : public de::GPU_Vector {
    size_t _length, _capacity;
    de::_DATA_TYPES_FLAGS_ _type;
    uint32_t _element_size;
    std::shared_ptr<DeviceBlock> _block;
    void assign(de::_DATA_TYPES_FLAGS_ type, size_t length);
    bool allocate();

public:
    _GPU_Vector();
    _GPU_Vector(de::_DATA_TYPES_FLAGS_ type, size_t length);
    virtual size_t Len() const;
    virtual void release();
    virtual de::GPU_Vector& SoftCopy(de::GPU_Vector& src);
    virtual de::_DATA_TYPES_FLAGS_ Type() const;
    virtual void Reinterpret(const de::_DATA_TYPES_FLAGS_ new_type);
    virtual ~_GPU_Vector();

    bool is_init() const { return _block && _block->ptr; }
    void* data() const { return _block ? _block->ptr : nullptr; }
    uint32_t element_bytes() const { return _element_size; }
    bool re_construct(de::_DATA_TYPES_FLAGS_ type, size_t length);
};

// Tensor layouts of the original (srcs/modules/core/classes/Tensor.cxx:35-69, GPU_Tensor.cu:35-86): depth padded
// to 16 bytes of elements, width padded to 4 columns on the host and 8 on the device.
void assign_tensor_layout(de::TensorLayout& L, de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height,
                          uint32_t depth, bool device);

class _Tensor : public de::Tensor {
    de::TensorLayout _layout;
    de::_DATA_TYPES_FLAGS_ _type;
    std::shared_ptr<HostBlock> _block;
    void* _data;

public:
    _Tensor();
    _Tensor(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, uint32_t depth);
    virtual uint32_t Width() const;
    virtual uint32_t Height() const;
    virtual uint32_t Depth() const;
    virtual de::Tensor& SoftCopy(de::Tensor& src);
    virtual void release();
    virtual de::_DATA_TYPES_FLAGS_ Type() const;
    virtual void Reinterpret(const de::_DATA_TYPES_FLAGS_ new_type);
    virtual ~_Tensor();

    const de::TensorLayout& get_layout() const { return _layout; }
    bool is_init() const { return _data != nullptr; }
    void* data() const { return _data; }
    // makes this tensor a view of `bytes_offset` into `block` with the given shape
    void alias(const std::shared_ptr<HostBlock>& block, size_t bytes_offset, de::_DATA_TYPES_FLAGS_ type,
               uint32_t width, uint32_t height, uint32_t depth);
};

class _GPU_Tensor : public de::GPU_Tensor {
    de::TensorLayout _layout;
    de::_DATA_TYPES_FLAGS_ _type;
    std::shared_ptr<DeviceBlock> _block;
    void* _data;

public:
    _GPU_Tensor();
    _GPU_Tensor(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, uint32_t depth);
    virtual uint Width() const;
    virtual uint Height() const;
    virtual uint Depth() const;
    virtual de::GPU_Tensor& SoftCopy(de::GPU_Tensor& src);
    virtual void release();
    virtual de::_DATA_TYPES_FLAGS_ Type() const;
    virtual void Reinterpret(const de::_DATA_TYPES_FLAGS_ new_type);
    virtual de::DH Extract_SoftCopy(const uint32_t index, de::GPU_Tensor& dst) const;
    virtual ~_GPU_Tensor();

    const de::TensorLayout& get_layout() const { return _layout; }
    bool is_init() const { return _data != nullptr; }
    void* data() const { return _data; }
    size_t total_bytes() const { return (size_t)_layout.dp_x_wp * _layout.height * _layout._single_element_size; }
    bool re_construct(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, uint32_t depth);   // grows only
    void alias(const std::shared_ptr<DeviceBlock>& block, size_t bytes_offset, de::_DATA_TYPES_FLAGS_ type,
               uint32_t width, uint32_t height, uint32_t depth);
};

class _TensorArray : public de::TensorArray {
    de::TensorLayout _layout;
    de::_DATA_TYPES_FLAGS_ _type;
    uint32_t _count;
    std::shared_ptr<HostBlock> _block;
    std::shared_ptr<void*> _table;      // per-tensor pointers
    void** _table_ptr;

public:
    _TensorArray();
    _TensorArray(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, uint32_t depth, uint32_t count);
    virtual uint Width() const;
    virtual uint Height() const;
    virtual uint Depth() const;
    virtual uint TensorNum() const;
    virtual de::TensorArray& SoftCopy(de::TensorArray& src);
    virtual de::_DATA_TYPES_FLAGS_ Type() const;
    virtual void Reinterpret(const de::_DATA_TYPES_FLAGS_ new_type);
    virtual de::DH Extract_SoftCopy(const uint32_t index, de::Tensor& dst) const;
    virtual void release();
    virtual ~_TensorArray();

    size_t gap_bytes() const { return (size_t)_layout.dp_x_wp * _layout.height * _layout._single_element_size; }
    bool is_init() const { return _block && _block->ptr; }
};

class _GPU_TensorArray : public de::GPU_TensorArray {
    de::TensorLayout _layout;
    de::_DATA_TYPES_FLAGS_ _type;
    uint32_t _count;
    std::shared_ptr<DeviceBlock> _block;

public:
    _GPU_TensorArray();
    _GPU_TensorArray(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, uint32_t depth, uint32_t count);
    virtual uint Width() const;
    virtual uint Height() const;
    virtual uint Depth() const;
    virtual uint TensorNum() const;
    virtual de::_DATA_TYPES_FLAGS_ Type() const;
    virtual void Reinterpret(const de::_DATA_TYPES_FLAGS_ new_type);
    virtual de::GPU_TensorArray& SoftCopy(const de::GPU_TensorArray& src);
    virtual de::DH Extract_SoftCopy(const uint32_t index, de::GPU_Tensor& dst) const;
    virtual void release();
    virtual ~_GPU_TensorArray();

    const de::TensorLayout& get_layout() const { return _layout; }
    size_t gap_bytes() const { return (size_t)_layout.dp_x_wp * _layout.height * _layout._single_element_size; }
    bool is_init() const { return _block && _block->ptr; }
    void* data() const { return _block ? _block->ptr : nullptr; }
};

// One stream for the module, created on first use; one mutex around every GEMM call
// (the original guards its cached planner with a plain flag).
void* module_stream();
std::mutex& module_mutex();
// Host <-> device copies of pitched blocks (sizes in bytes) for callers that hold module_mutex().  Page-locked
// host memory is copied directly; pageable memory goes through page-locked bounce buffers filled by host threads.
// The copies are complete, and device -> host data in place, once stage_finish() has returned.
int stage_h2d(void* dev, size_t dpitch, const void* host, size_t hpitch, size_t width, size_t rows, bool host_pinned);
int stage_d2h(void* host, size_t hpitch, const void* dev, size_t dpitch, size_t width, size_t rows, bool host_pinned);
int stage_finish();

}  // namespace decx
