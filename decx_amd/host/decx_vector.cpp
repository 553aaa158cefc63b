// de::Vector / de::GPU_Vector, their transfers, and the two vector forms of the product
// (row vector x matrix, matrix x column vector) on host objects.
#include "decx_internal.hpp"

#include <cstdlib>
#include <cstring>

namespace {

const char* const kCudaNotInit  = "error: CUDA should be initialized first";
const char* const kTypeNotMatch = "error: The types of the two objects are not equal";
const char* const kOverranged   = "error: Failed to transfer data since it is out of range";
const char* const kDevAllocFail = "error: Fail to allocate memory on device";
const char* const kHostAllocFail = "error: Fail to allocate memory on RAM";
const char* const kClassNotInit = "error: The class is not initialized";
const char* const kUnsupportedType = "error: The data type of the input onject is not supported";
const char* const kInvalidParam = "error: The parameter(s) is(are) invalid";

size_t aligned_length(size_t length, uint32_t element_size)
{
    const size_t per32 = element_size ? 32u / element_size : 1u;
    return per32 ? (length + per32 - 1) / per32 * per32 : length;
}

}  // namespace

// ---------------------------------------------------------------- host vector

void decx::_Vector::assign(de::_DATA_TYPES_FLAGS_ type, size_t length)
{
    _type = type;
    _element_size = element_size(type);
    _length = length;
    _capacity = aligned_length(length, _element_size);
}

bool decx::_Vector::allocate()
{
    auto block = std::make_shared<HostBlock>();
    const size_t bytes = _capacity * _element_size;
    block->bytes = bytes ? (bytes + 63) / 64 * 64 : 64;
    block->ptr = std::aligned_alloc(64, block->bytes);
    if (!block->ptr) { err::set(de::GetLastError(), DECX_FAIL_ALLOCATION, kHostAllocFail); return false; }
    std::memset(block->ptr, 0, block->bytes);
    _block = block;
    _data = block->ptr;
    return true;
}

decx::_Vector::_Vector() : _data(nullptr) { _exp_data_ptr = &_data; assign(de::_VOID_, 0); }
decx::_Vector::_Vector(de::_DATA_TYPES_FLAGS_ type, size_t length) : _data(nullptr)
{
    _exp_data_ptr = &_data;
    assign(type, length);
    allocate();
}
decx::_Vector::~_Vector() {}
size_t decx::_Vector::Len() const { return _length; }
void decx::_Vector::release() { _block.reset(); _data = nullptr; }
de::_DATA_TYPES_FLAGS_ decx::_Vector::Type() const { return _type; }
void decx::_Vector::Reinterpret(const de::_DATA_TYPES_FLAGS_ t) { _type = t; }

de::Vector& decx::_Vector::SoftCopy(de::Vector& src)
{
    const _Vector& s = dynamic_cast<_Vector&>(src);
    assign(s._type, s._length);
    _block = s._block;
    _data = s._data;
    return *this;
}

bool decx::_Vector::re_construct(de::_DATA_TYPES_FLAGS_ type, size_t length)
{
    if (_type == type && _length == length && _data) return true;
    const size_t before = _block ? _block->bytes : 0;
    assign(type, length);
    if (_capacity * _element_size > before || !_data) return allocate();
    return true;
}

int decx::_Vector::move_storage(bool pinned)
{
    if (!_block || !_block->ptr) return DECX_HIP_E_INVALID_ARG;
    auto block = std::make_shared<HostBlock>();
    block->bytes = _block->bytes;
    block->pinned = pinned;
    if (pinned) {
        const int rc = decx_hip_host_malloc(&block->ptr, block->bytes);
        if (rc != DECX_HIP_OK) { block->ptr = nullptr; return rc; }
    } else {
        block->ptr = std::aligned_alloc(64, block->bytes);
        if (!block->ptr) return 2;
    }
    std::memcpy(block->ptr, _block->ptr, block->bytes);
    _block = block;
    _data = block->ptr;
    return DECX_HIP_OK;
}

_DECX_API_ de::Vector& de::CreateVectorRef() { return *(new decx::_Vector()); }
_DECX_API_ de::Vector* de::CreateVectorPtr() { return new decx::_Vector(); }
_DECX_API_ de::Vector& de::CreateVectorRef(const de::_DATA_TYPES_FLAGS_ type, size_t len)
{
    return *(new decx::_Vector(type, len));
}
_DECX_API_ de::Vector* de::CreateVectorPtr(const de::_DATA_TYPES_FLAGS_ type, size_t len)
{
    return new decx::_Vector(type, len);
}

_DECX_API_ de::DH de::cuda::PinMemory(de::Vector& src)
{
    de::DH handle; decx::err::success(&handle);
    decx::_Vector* v = dynamic_cast<decx::_Vector*>(&src);
    if (!decx::gpu_ready()) { decx::err::set(&handle, decx::DECX_FAIL_CUDA_not_init, kCudaNotInit); return handle; }
    if (!v || !v->is_init()) { decx::err::set(&handle, decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return handle; }
    if (v->is_pinned()) {
        decx::err::set(&handle, decx::DECX_FAIL_HOST_MEM_REGISTERED, "error: The host memory is already page-locked");
        return handle;
    }
    decx::err::from_hip(&handle, v->move_storage(true), "PinMemory");
    return handle;
}
_DECX_API_ de::DH de::cuda::UnpinMemory(de::Vector& src)
{
    de::DH handle; decx::err::success(&handle);
    decx::_Vector* v = dynamic_cast<decx::_Vector*>(&src);
    if (!v || !v->is_init()) { decx::err::set(&handle, decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return handle; }
    if (!v->is_pinned()) {
        decx::err::set(&handle, decx::DECX_FAIL_HOST_MEM_UNREGISTERED, "error: The host memory is not page-locked");
        return handle;
    }
    decx::err::from_hip(&handle, v->move_storage(false), "UnpinMemory");
    return handle;
}

// ---------------------------------------------------------------- device vector

void decx::_GPU_Vector::assign(de::_DATA_TYPES_FLAGS_ type, size_t length)
{
    _type = type;
    _element_size = element_size(type);
    _length = length;
    _capacity = aligned_length(length, _element_size);
}

bool decx::_GPU_Vector::allocate()
{
    auto block = std::make_shared<DeviceBlock>();
    block->bytes = _capacity * _element_size;
    int rc = decx_hip_malloc(&block->ptr, block->bytes);
    if (rc == DECX_HIP_OK && block->bytes) {
        rc = decx_hip_memset_async(block->ptr, 0, block->bytes, module_stream());
        if (rc == DECX_HIP_OK) rc = decx_hip_stream_sync(module_stream());
    }
    if (rc != DECX_HIP_OK) {
        if (rc == DECX_HIP_E_NOT_INIT) { block->ptr = nullptr; err::set(de::GetLastError(), DECX_FAIL_CUDA_not_init, kCudaNotInit); }
        else err::set(de::GetLastError(), DECX_FAIL_CUDA_ALLOCATION, kDevAllocFail);
        return false;
    }
    _block = block;
    return true;
}

decx::_GPU_Vector::_GPU_Vector() { assign(de::_VOID_, 0); }
decx::_GPU_Vector::_GPU_Vector(de::_DATA_TYPES_FLAGS_ type, size_t length) { assign(type, length); allocate(); }
decx::_GPU_Vector::~_GPU_Vector() {}
size_t decx::_GPU_Vector::Len() const { return _length; }
void decx::_GPU_Vector::release() { _block.reset(); }
de::_DATA_TYPES_FLAGS_ decx::_GPU_Vector::Type() const { return _type; }
void decx::_GPU_Vector::Reinterpret(const de::_DATA_TYPES_FLAGS_ t) { _type = t; }

de::GPU_Vector& decx::_GPU_Vector::SoftCopy(de::GPU_Vector& src)
{
    const _GPU_Vector& s = dynamic_cast<_GPU_Vector&>(src);
    assign(s._type, s._length);
    _block = s._block;
    return *this;
}

bool decx::_GPU_Vector::re_construct(de::_DATA_TYPES_FLAGS_ type, size_t length)
{
    if (_type == type && _length == length && is_init()) return true;
    const size_t before = _block ? _block->bytes : 0;
    assign(type, length);
    if (_capacity * _element_size > before || !is_init()) return allocate();
    return true;
}

_DECX_API_ de::GPU_Vector& de::CreateGPUVectorRef() { return *(new decx::_GPU_Vector()); }
_DECX_API_ de::GPU_Vector* de::CreateGPUVectorPtr() { return new decx::_GPU_Vector(); }
_DECX_API_ de::GPU_Vector& de::CreateGPUVectorRef(const de::_DATA_TYPES_FLAGS_ type, const size_t len)
{
    return *(new decx::_GPU_Vector(type, len));
}
_DECX_API_ de::GPU_Vector* de::CreateGPUVectorPtr(const de::_DATA_TYPES_FLAGS_ type, const size_t len)
{
    return new decx::_GPU_Vector(type, len);
}

// ---------------------------------------------------------------- transfers

// Checks in the order of the original (srcs/modules/core/data transmission/data_transmission.cu:37-98):
// initialised, same type, both ranges inside.  The offsets are applied as documented
// (start_src to the source, start_dst to the destination); the original swaps them in its
// pointer arithmetic, which only agrees when the two are equal.
_DECX_API_ de::DH de::Memcpy(de::Vector& host, de::GPU_Vector& device, const uint64_t start_src,
                             const uint64_t start_dst, const uint64_t len, const int flag)
{
    de::DH handle; decx::err::success(&handle);
    if (!decx::gpu_ready()) { decx::err::set(&handle, decx::DECX_FAIL_CUDA_not_init, kCudaNotInit); return handle; }
    decx::_Vector* h = dynamic_cast<decx::_Vector*>(&host);
    decx::_GPU_Vector* d = dynamic_cast<decx::_GPU_Vector*>(&device);
    if (!h || !d || !h->is_init() || !d->is_init()) {
        decx::err::set(&handle, decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return handle;
    }
    if (h->Type() != d->Type()) { decx::err::set(&handle, decx::DECX_FAIL_TYPE_MOT_MATCH, kTypeNotMatch); return handle; }
    if (flag != de::DECX_MEMCPY_H2D && flag != de::DECX_MEMCPY_D2H) {
        decx::err::set(&handle, decx::DECX_FAIL_INVALID_PARAM, kInvalidParam); return handle;
    }
    const bool h2d = flag == de::DECX_MEMCPY_H2D;
    const uint64_t src_len = h2d ? h->Len() : d->Len(), dst_len = h2d ? d->Len() : h->Len();
    if (start_src > src_len || len > src_len - start_src || start_dst > dst_len || len > dst_len - start_dst) {
        decx::err::set(&handle, decx::DECX_FAIL_MEMCPY_OVERRANGED, kOverranged); return handle;
    }
    const size_t es = h->element_bytes();
    char* hptr = (char*)h->data() + (h2d ? start_src : start_dst) * es;
    char* dptr = (char*)d->data() + (h2d ? start_dst : start_src) * es;
    int rc = DECX_HIP_OK;
    if (len) {
        std::lock_guard<std::mutex> guard(decx::module_mutex());
        rc = h2d ? decx::stage_h2d(dptr, len * es, hptr, len * es, len * es, 1, h->is_pinned())
                 : decx::stage_d2h(hptr, len * es, dptr, len * es, len * es, 1, h->is_pinned());
        const int rf = decx::stage_finish();
        if (rc == DECX_HIP_OK) rc = rf;
    }
    decx::err::from_hip(&handle, rc, "Memcpy");
    return handle;
}

// ---------------------------------------------------------------- vector x matrix, matrix x vector

namespace {

// The original (srcs/modules/BLAS/GEMM/CUDA/VMM.cu:56-185) stages the host operands into
// device buffers, runs its kernel pair and copies the result into dst's existing storage,
// with no check at all.  Here: the same staging around one kernel, preceded by the checks the
// matrix forms make (initialised, types, the shared dimension), and dst is re-created when
// its storage cannot hold the result instead of being overrun.
void vmm(decx::_Vector* vec, decx::_Matrix* mat, decx::_Vector* dst, bool mat_times_vec, uint32_t accu)
{
    de::DH* h = de::GetLastError();
    if (!decx::gpu_ready()) { decx::err::set(h, decx::DECX_FAIL_CUDA_not_init, kCudaNotInit); return; }
    if (!vec || !mat || !dst || !vec->is_init() || !mat->is_init()) {
        decx::err::set(h, decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return;
    }
    if (vec->Type() != mat->Type()) {
        decx::err::set(h, decx::DECX_FAIL_TYPE_MOT_MATCH, "Types of the input vector and matrix must be matched"); return;
    }
    const de::_DATA_TYPES_FLAGS_ type = mat->Type();
    if (type != de::_FP32_ && type != de::_FP16_) {
        decx::err::set(h, decx::DECX_FAIL_UNSUPPORTED_TYPE, kUnsupportedType); return;
    }
    if (accu > de::Fp16_Accurate_L3) { decx::err::set(h, decx::DECX_FAIL_INVALID_PARAM, kInvalidParam); return; }
    const size_t reduced = mat_times_vec ? mat->Width() : mat->Height();
    const size_t out_len = mat_times_vec ? mat->Height() : mat->Width();
    if (vec->Len() != reduced) {
        decx::err::set(h, decx::DECX_FAIL_DimsNotMatching,
                       mat_times_vec ? "The length of vector B and the width of matrix A must be identical"
                                     : "The length of vector A and the height of matrix B must be identical");
        return;
    }
    const bool f16 = type == de::_FP16_;
    const bool out_f32 = !f16 || accu == de::Fp16_Accurate_L1;
    const de::_DATA_TYPES_FLAGS_ out_type = out_f32 ? de::_FP32_ : de::_FP16_;
    const size_t out_bytes = out_len * (out_f32 ? 4u : 2u);
    if (!dst->is_init() || dst->capacity_bytes() < out_bytes || dst->Len() * dst->element_bytes() < out_bytes) {
        if (!dst->re_construct(out_type, out_len)) return;
    }

    std::lock_guard<std::mutex> guard(decx::module_mutex());
    decx::_GPU_Matrix dM(type, mat->Width(), mat->Height(), de::_NA_);
    decx::_GPU_Vector dV(type, vec->Len()), dOut(out_type, out_len);
    if (!dM.is_init() || !dV.is_init() || !dOut.is_init()) return;                 // status already set
    void* S = decx::module_stream();
    const size_t es = f16 ? 2 : 4;
    int rc = DECX_HIP_OK;
    if (mat->Width() && mat->Height()) {                   // the matrix is what takes the time: 256 MiB at 8192 x 8192
        rc = decx::stage_h2d(dM.data(), (size_t)dM.Pitch() * es, mat->data(), (size_t)mat->Pitch() * es,
                             (size_t)mat->Width() * es, mat->Height(), mat->is_pinned());
        const int rf = decx::stage_finish();
        if (rc == DECX_HIP_OK) rc = rf;
    }
    if (rc == DECX_HIP_OK && vec->Len())
        rc = decx_hip_memcpy2d_async(dV.data(), vec->Len() * es, vec->data(), vec->Len() * es, vec->Len() * es, 1, 0, S);
    if (rc == DECX_HIP_OK) {
        if (mat_times_vec) {
            rc = f16 ? decx_hip_gemv_f16((const uint16_t*)dM.data(), (const uint16_t*)dV.data(), nullptr, dOut.data(),
                                         mat->Height(), mat->Width(), dM.Pitch(), 1, 0, 1, 1.f, 1.f, out_f32, S)
                     : decx_hip_gemv_f32((const float*)dM.data(), (const float*)dV.data(), nullptr, (float*)dOut.data(),
                                         mat->Height(), mat->Width(), dM.Pitch(), 1, 0, 1, 1.f, 1.f, S);
        } else {
            rc = f16 ? decx_hip_gevm_f16((const uint16_t*)dV.data(), (const uint16_t*)dM.data(), nullptr, dOut.data(),
                                         mat->Height(), mat->Width(), dM.Pitch(), 1, 0, 1, 1.f, 1.f, out_f32, S)
                     : decx_hip_gevm_f32((const float*)dV.data(), (const float*)dM.data(), nullptr, (float*)dOut.data(),
                                         mat->Height(), mat->Width(), dM.Pitch(), 1, 0, 1, 1.f, 1.f, S);
        }
    }
    if (rc == DECX_HIP_OK && out_bytes)
        rc = decx_hip_memcpy2d_async(dst->data(), out_bytes, dOut.data(), out_bytes, out_bytes, 1, 1, S);
    if (rc == DECX_HIP_OK) rc = decx_hip_stream_sync(S);
    decx::err::from_hip(h, rc, "GEMM");
}

}  // namespace

_DECX_API_ void de::blas::cuda::GEMM(de::Vector& A, de::Matrix& B, de::Vector& dst, const uint32_t accu)
{
    de::ResetLastError();
    vmm(dynamic_cast<decx::_Vector*>(&A), dynamic_cast<decx::_Matrix*>(&B), dynamic_cast<decx::_Vector*>(&dst), false, accu);
}

_DECX_API_ void de::blas::cuda::GEMM(de::Matrix& A, de::Vector& B, de::Vector& dst, const uint32_t accu)
{
    de::ResetLastError();
    vmm(dynamic_cast<decx::_Vector*>(&B), dynamic_cast<decx::_Matrix*>(&A), dynamic_cast<decx::_Vector*>(&dst), true, accu);
}
