// de::Tensor / de::GPU_Tensor / de::TensorArray / de::GPU_TensorArray, their transfers, and
// de::nn::cuda::Conv2D on top of the implicit-GEMM convolution of the C ABI.
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

uint32_t round_up(uint32_t v, uint32_t to) { return to ? (v + to - 1) / to * to : v; }

std::shared_ptr<decx::HostBlock> host_block(size_t bytes)
{
    auto block = std::make_shared<decx::HostBlock>();
    block->bytes = bytes ? (bytes + 63) / 64 * 64 : 64;
    block->ptr = std::aligned_alloc(64, block->bytes);
    if (!block->ptr) { decx::err::set(de::GetLastError(), decx::DECX_FAIL_ALLOCATION, kHostAllocFail); return nullptr; }
    std::memset(block->ptr, 0, block->bytes);
    return block;
}

std::shared_ptr<decx::DeviceBlock> device_block(size_t bytes)
{
    auto block = std::make_shared<decx::DeviceBlock>();
    block->bytes = bytes ? bytes : 64;
    int rc = decx_hip_malloc(&block->ptr, block->bytes);
    if (rc == DECX_HIP_OK) {
        rc = decx_hip_memset_async(block->ptr, 0, block->bytes, decx::module_stream());
        if (rc == DECX_HIP_OK) rc = decx_hip_stream_sync(decx::module_stream());
    }
    if (rc != DECX_HIP_OK) {
        if (rc == DECX_HIP_E_NOT_INIT) { block->ptr = nullptr; decx::err::set(de::GetLastError(), decx::DECX_FAIL_CUDA_not_init, kCudaNotInit); }
        else decx::err::set(de::GetLastError(), decx::DECX_FAIL_CUDA_ALLOCATION, kDevAllocFail);
        return nullptr;
    }
    return block;
}

}  // namespace

void decx::assign_tensor_layout(de::TensorLayout& L, de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height,
                                uint32_t depth, bool device)
{
    L._single_element_size = (uint8_t)element_size(type);
    L.width = width; L.height = height; L.depth = depth;
    L.wpitch = round_up(width, device ? 8u : 4u);
    L.dpitch = round_up(depth, L._single_element_size ? (16u / L._single_element_size ? 16u / L._single_element_size : 1u) : 1u);
    L.dp_x_wp = (uint64_t)L.dpitch * L.wpitch;
    L.plane[0] = (uint64_t)height * width;
    L.plane[1] = (uint64_t)depth * width;
    L.plane[2] = (uint64_t)height * depth;
}

// ---------------------------------------------------------------- host tensor

decx::_Tensor::_Tensor() : _type(de::_VOID_), _data(nullptr)
{
    _exp_data_ptr = &_data; _exp_tensor_dscr = &_layout;
    assign_tensor_layout(_layout, de::_VOID_, 0, 0, 0, false);
}
decx::_Tensor::_Tensor(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, uint32_t depth) : _type(type), _data(nullptr)
{
    _exp_data_ptr = &_data; _exp_tensor_dscr = &_layout;
    assign_tensor_layout(_layout, type, width, height, depth, false);
    _block = host_block((size_t)_layout.dp_x_wp * height * _layout._single_element_size);
    _data = _block ? _block->ptr : nullptr;
}
decx::_Tensor::~_Tensor() {}
uint32_t decx::_Tensor::Width() const { return _layout.width; }
uint32_t decx::_Tensor::Height() const { return _layout.height; }
uint32_t decx::_Tensor::Depth() const { return _layout.depth; }
void decx::_Tensor::release() { _block.reset(); _data = nullptr; }
de::_DATA_TYPES_FLAGS_ decx::_Tensor::Type() const { return _type; }
void decx::_Tensor::Reinterpret(const de::_DATA_TYPES_FLAGS_ t) { _type = t; }
de::Tensor& decx::_Tensor::SoftCopy(de::Tensor& src)
{
    const _Tensor& s = dynamic_cast<_Tensor&>(src);
    _layout = s._layout; _type = s._type; _block = s._block; _data = s._data;
    return *this;
}
void decx::_Tensor::alias(const std::shared_ptr<HostBlock>& block, size_t off, de::_DATA_TYPES_FLAGS_ type,
                          uint32_t width, uint32_t height, uint32_t depth)
{
    _type = type;
    assign_tensor_layout(_layout, type, width, height, depth, false);
    _block = block;
    _data = block ? (char*)block->ptr + off : nullptr;
}

_DECX_API_ de::Tensor* de::CreateTensorPtr() { return new decx::_Tensor(); }
_DECX_API_ de::Tensor& de::CreateTensorRef() { return *(new decx::_Tensor()); }
_DECX_API_ de::Tensor* de::CreateTensorPtr(const de::_DATA_TYPES_FLAGS_ t, const uint w, const uint h, const uint d) { return new decx::_Tensor(t, w, h, d); }
_DECX_API_ de::Tensor& de::CreateTensorRef(const de::_DATA_TYPES_FLAGS_ t, const uint w, const uint h, const uint d) { return *(new decx::_Tensor(t, w, h, d)); }

// ---------------------------------------------------------------- device tensor

decx::_GPU_Tensor::_GPU_Tensor() : _type(de::_VOID_), _data(nullptr) { assign_tensor_layout(_layout, de::_VOID_, 0, 0, 0, true); }
decx::_GPU_Tensor::_GPU_Tensor(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, uint32_t depth) : _type(type), _data(nullptr)
{
    assign_tensor_layout(_layout, type, width, height, depth, true);
    _block = device_block(total_bytes());
    _data = _block ? _block->ptr : nullptr;
}
decx::_GPU_Tensor::~_GPU_Tensor() {}
uint decx::_GPU_Tensor::Width() const { return _layout.width; }
uint decx::_GPU_Tensor::Height() const { return _layout.height; }
uint decx::_GPU_Tensor::Depth() const { return _layout.depth; }
void decx::_GPU_Tensor::release() { _block.reset(); _data = nullptr; }
de::_DATA_TYPES_FLAGS_ decx::_GPU_Tensor::Type() const { return _type; }
void decx::_GPU_Tensor::Reinterpret(const de::_DATA_TYPES_FLAGS_ t) { _type = t; }
de::GPU_Tensor& decx::_GPU_Tensor::SoftCopy(de::GPU_Tensor& src)
{
    const _GPU_Tensor& s = dynamic_cast<_GPU_Tensor&>(src);
    _layout = s._layout; _type = s._type; _block = s._block; _data = s._data;
    return *this;
}
de::DH decx::_GPU_Tensor::Extract_SoftCopy(const uint32_t, de::GPU_Tensor&) const
{
    de::DH h; err::set(&h, DECX_FAIL_INVALID_PARAM, "error: extracting a channel plane of a device tensor is not provided");
    return h;
}
bool decx::_GPU_Tensor::re_construct(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, uint32_t depth)
{
    if (_type == type && _layout.width == width && _layout.height == height && _layout.depth == depth && _data) return true;
    // a view into someone else's storage (Extract_SoftCopy) is never reshaped in place
    const bool own = _block && _data == _block->ptr;
    const size_t before = own ? _block->bytes : 0;
    _type = type;
    assign_tensor_layout(_layout, type, width, height, depth, true);
    if (total_bytes() > before || !_data || !own) {
        _block = device_block(total_bytes());
        _data = _block ? _block->ptr : nullptr;
        return _data != nullptr;
    }
    return true;
}
void decx::_GPU_Tensor::alias(const std::shared_ptr<DeviceBlock>& block, size_t off, de::_DATA_TYPES_FLAGS_ type,
                              uint32_t width, uint32_t height, uint32_t depth)
{
    _type = type;
    assign_tensor_layout(_layout, type, width, height, depth, true);
    _block = block;
    _data = block ? (char*)block->ptr + off : nullptr;
}

_DECX_API_ de::GPU_Tensor* de::CreateGPUTensorPtr() { return new decx::_GPU_Tensor(); }
_DECX_API_ de::GPU_Tensor& de::CreateGPUTensorRef() { return *(new decx::_GPU_Tensor()); }
_DECX_API_ de::GPU_Tensor* de::CreateGPUTensorPtr(const de::_DATA_TYPES_FLAGS_ t, const uint w, const uint h, const uint32_t d) { return new decx::_GPU_Tensor(t, w, h, d); }
_DECX_API_ de::GPU_Tensor& de::CreateGPUTensorRef(const de::_DATA_TYPES_FLAGS_ t, const uint w, const uint h, const uint32_t d) { return *(new decx::_GPU_Tensor(t, w, h, d)); }

// ---------------------------------------------------------------- host tensor array

decx::_TensorArray::_TensorArray() : _type(de::_VOID_), _count(0), _table_ptr(nullptr)
{
    _exp_data_ptr = &_table_ptr; _exp_tensor_dscr = &_layout;
    assign_tensor_layout(_layout, de::_VOID_, 0, 0, 0, false);
}
decx::_TensorArray::_TensorArray(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, uint32_t depth, uint32_t count)
    : _type(type), _count(count), _table_ptr(nullptr)
{
    _exp_data_ptr = &_table_ptr; _exp_tensor_dscr = &_layout;
    assign_tensor_layout(_layout, type, width, height, depth, false);
    _block = host_block(gap_bytes() * count);
    if (_block) {
        _table = std::shared_ptr<void*>(new void*[count ? count : 1], std::default_delete<void*[]>());
        for (uint32_t i = 0; i < count; ++i) _table.get()[i] = (char*)_block->ptr + gap_bytes() * i;
        _table_ptr = _table.get();
    }
}
decx::_TensorArray::~_TensorArray() {}
uint decx::_TensorArray::Width() const { return _layout.width; }
uint decx::_TensorArray::Height() const { return _layout.height; }
uint decx::_TensorArray::Depth() const { return _layout.depth; }
uint decx::_TensorArray::TensorNum() const { return _count; }
de::_DATA_TYPES_FLAGS_ decx::_TensorArray::Type() const { return _type; }
void decx::_TensorArray::Reinterpret(const de::_DATA_TYPES_FLAGS_ t) { _type = t; }
void decx::_TensorArray::release() { _block.reset(); _table.reset(); _table_ptr = nullptr; }
de::TensorArray& decx::_TensorArray::SoftCopy(de::TensorArray& src)
{
    const _TensorArray& s = dynamic_cast<_TensorArray&>(src);
    _layout = s._layout; _type = s._type; _count = s._count; _block = s._block; _table = s._table; _table_ptr = s._table_ptr;
    return *this;
}
de::DH decx::_TensorArray::Extract_SoftCopy(const uint32_t index, de::Tensor& dst) const
{
    de::DH h; err::success(&h);
    _Tensor* d = dynamic_cast<_Tensor*>(&dst);
    if (!d || !is_init()) { err::set(&h, DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return h; }
    if (index >= _count) { err::set(&h, DECX_FAIL_INVALID_PARAM, kInvalidParam); return h; }
    d->alias(_block, gap_bytes() * index, _type, _layout.width, _layout.height, _layout.depth);
    return h;
}

_DECX_API_ de::TensorArray& de::CreateTensorArrayRef() { return *(new decx::_TensorArray()); }
_DECX_API_ de::TensorArray* de::CreateTensorArrayPtr() { return new decx::_TensorArray(); }
_DECX_API_ de::TensorArray& de::CreateTensorArrayRef(const de::_DATA_TYPES_FLAGS_ t, const uint w, const uint h, const uint d, const uint n) { return *(new decx::_TensorArray(t, w, h, d, n)); }
_DECX_API_ de::TensorArray* de::CreateTensorArrayPtr(const de::_DATA_TYPES_FLAGS_ t, const uint w, const uint h, const uint d, const uint n) { return new decx::_TensorArray(t, w, h, d, n); }

// ---------------------------------------------------------------- device tensor array

decx::_GPU_TensorArray::_GPU_TensorArray() : _type(de::_VOID_), _count(0) { assign_tensor_layout(_layout, de::_VOID_, 0, 0, 0, true); }
decx::_GPU_TensorArray::_GPU_TensorArray(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, uint32_t depth, uint32_t count)
    : _type(type), _count(count)
{
    assign_tensor_layout(_layout, type, width, height, depth, true);
    _block = device_block(gap_bytes() * count);
}
decx::_GPU_TensorArray::~_GPU_TensorArray() {}
uint decx::_GPU_TensorArray::Width() const { return _layout.width; }
uint decx::_GPU_TensorArray::Height() const { return _layout.height; }
uint decx::_GPU_TensorArray::Depth() const { return _layout.depth; }
uint decx::_GPU_TensorArray::TensorNum() const { return _count; }
de::_DATA_TYPES_FLAGS_ decx::_GPU_TensorArray::Type() const { return _type; }
void decx::_GPU_TensorArray::Reinterpret(const de::_DATA_TYPES_FLAGS_ t) { _type = t; }
void decx::_GPU_TensorArray::release() { _block.reset(); }
de::GPU_TensorArray& decx::_GPU_TensorArray::SoftCopy(const de::GPU_TensorArray& src)
{
    const _GPU_TensorArray& s = dynamic_cast<const _GPU_TensorArray&>(src);
    _layout = s._layout; _type = s._type; _count = s._count; _block = s._block;
    return *this;
}
de::DH decx::_GPU_TensorArray::Extract_SoftCopy(const uint32_t index, de::GPU_Tensor& dst) const
{
    de::DH h; err::success(&h);
    _GPU_Tensor* d = dynamic_cast<_GPU_Tensor*>(&dst);
    if (!d || !is_init()) { err::set(&h, DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return h; }
    if (index >= _count) { err::set(&h, DECX_FAIL_INVALID_PARAM, kInvalidParam); return h; }
    d->alias(_block, gap_bytes() * index, _type, _layout.width, _layout.height, _layout.depth);
    return h;
}

_DECX_API_ de::GPU_TensorArray& de::CreateGPUTensorArrayRef() { return *(new decx::_GPU_TensorArray()); }
_DECX_API_ de::GPU_TensorArray* de::CreateGPUTensorArrayPtr() { return new decx::_GPU_TensorArray(); }
_DECX_API_ de::GPU_TensorArray& de::CreateGPUTensorArrayRef(const de::_DATA_TYPES_FLAGS_ t, const uint w, const uint h, const uint d, const uint32_t n) { return *(new decx::_GPU_TensorArray(t, w, h, d, n)); }
_DECX_API_ de::GPU_TensorArray* de::CreateGPUTensorArrayPtr(const de::_DATA_TYPES_FLAGS_ t, const uint w, const uint h, const uint d, const uint32_t n) { return new decx::_GPU_TensorArray(t, w, h, d, n); }

// ---------------------------------------------------------------- transfers

// A box [D, W, H] between a host and a device tensor (srcs/modules/core/data transmission/
// data_transmission.cu:185-280): checks as there (initialised, both boxes inside), plus the type check the
// matrix form makes.  Rows of the box are contiguous runs of W x dpitch elements only when the whole depth is
// copied at equal channel pitches; in general one 2-D copy per image row moves W runs of D elements.
_DECX_API_ de::DH de::Memcpy(de::Tensor& host, de::GPU_Tensor& device, const de::Point3D start_src, const de::Point3D start_dst,
                             const de::Point3D size, const int flag)
{
    de::DH handle; decx::err::success(&handle);
    if (!decx::gpu_ready()) { decx::err::set(&handle, decx::DECX_FAIL_CUDA_not_init, kCudaNotInit); return handle; }
    decx::_Tensor* h = dynamic_cast<decx::_Tensor*>(&host);
    decx::_GPU_Tensor* d = dynamic_cast<decx::_GPU_Tensor*>(&device);
    if (!h || !d || !h->is_init() || !d->is_init()) { decx::err::set(&handle, decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return handle; }
    if (h->Type() != d->Type()) { decx::err::set(&handle, decx::DECX_FAIL_TYPE_MOT_MATCH, kTypeNotMatch); return handle; }
    if (flag != de::DECX_MEMCPY_H2D && flag != de::DECX_MEMCPY_D2H) { decx::err::set(&handle, decx::DECX_FAIL_INVALID_PARAM, kInvalidParam); return handle; }
    const bool h2d = flag == de::DECX_MEMCPY_H2D;
    const de::TensorLayout& SL = h2d ? h->get_layout() : d->get_layout();
    const de::TensorLayout& DL = h2d ? d->get_layout() : h->get_layout();
    auto inside = [](const de::Point3D& s, const de::Point3D& n, const de::TensorLayout& L) {
        return s.x >= 0 && s.y >= 0 && s.z >= 0 && n.x >= 0 && n.y >= 0 && n.z >= 0 &&
               (int64_t)s.x + n.x <= (int64_t)L.depth && (int64_t)s.y + n.y <= (int64_t)L.width && (int64_t)s.z + n.z <= (int64_t)L.height;
    };
    if (!inside(start_src, size, SL) || !inside(start_dst, size, DL)) {
        decx::err::set(&handle, decx::DECX_FAIL_MEMCPY_OVERRANGED, kOverranged); return handle;
    }
    const size_t es = SL._single_element_size;
    const char* sp = (const char*)(h2d ? h->data() : d->data());
    char* dp = (char*)(h2d ? d->data() : h->data());
    std::lock_guard<std::mutex> guard(decx::module_mutex());
    int rc = DECX_HIP_OK;
    for (int32_t r = 0; r < size.z && rc == DECX_HIP_OK; ++r) {
        const char* s_row = sp + (((size_t)(start_src.z + r) * SL.wpitch + start_src.y) * SL.dpitch + start_src.x) * es;
        char* d_row = dp + (((size_t)(start_dst.z + r) * DL.wpitch + start_dst.y) * DL.dpitch + start_dst.x) * es;
        rc = h2d ? decx::stage_h2d(d_row, (size_t)DL.dpitch * es, s_row, (size_t)SL.dpitch * es, (size_t)size.x * es, (size_t)size.y, false)
                 : decx::stage_d2h(d_row, (size_t)DL.dpitch * es, s_row, (size_t)SL.dpitch * es, (size_t)size.x * es, (size_t)size.y, false);
    }
    const int rs = decx::stage_finish();
    decx::err::from_hip(&handle, rc != DECX_HIP_OK ? rc : rs, "Memcpy");
    return handle;
}

// ---------------------------------------------------------------- convolution

namespace {

// Scratch kept between calls (the original keeps its planner's buffers the same way): the packed kernel
// matrix and, for extended borders, the zero-extended image.  Guarded by the module mutex.
struct ConvScratch {
    std::shared_ptr<decx::DeviceBlock> kmat, padded;
    bool ensure(std::shared_ptr<decx::DeviceBlock>& b, size_t bytes)
    {
        if (b && b->bytes >= bytes) return true;
        b = device_block(bytes);
        return b != nullptr;
    }
};
ConvScratch& conv_scratch() { static ConvScratch s; return s; }

}  // namespace

_DECX_API_ de::DH de::nn::cuda::Conv2D(de::GPU_Tensor& src, de::GPU_TensorArray& kernel, de::GPU_Tensor& dst,
                                       const de::Point2D strides, const de::extend_label extend)
{
    de::DH handle; decx::err::success(&handle);
    decx::_GPU_Tensor* s = dynamic_cast<decx::_GPU_Tensor*>(&src);
    decx::_GPU_TensorArray* k = dynamic_cast<decx::_GPU_TensorArray*>(&kernel);
    decx::_GPU_Tensor* d = dynamic_cast<decx::_GPU_Tensor*>(&dst);
    if (!decx::gpu_ready()) { decx::err::set(&handle, decx::DECX_FAIL_CUDA_not_init, kCudaNotInit); return handle; }
    if (!s || !k || !d || !s->is_init() || !k->is_init()) { decx::err::set(&handle, decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return handle; }
    if (s->Type() != k->Type()) { decx::err::set(&handle, decx::DECX_FAIL_TYPE_MOT_MATCH, kTypeNotMatch); return handle; }
    if (s->Type() != de::_FP32_) { decx::err::set(&handle, decx::DECX_FAIL_UNSUPPORTED_TYPE, kUnsupportedType); return handle; }
    if (extend != de::_EXTEND_NONE_ && extend != de::_EXTEND_CONSTANT_) {
        decx::err::set(&handle, decx::DECX_FAIL_ErrorFlag, "error: This flag is meaningless in current context"); return handle;
    }
    if (strides.x < 1 || strides.y < 1) { decx::err::set(&handle, decx::DECX_FAIL_INVALID_PARAM, kInvalidParam); return handle; }
    const uint32_t W = s->Width(), H = s->Height(), C = s->Depth(), KW = k->Width(), KH = k->Height(), OC = k->TensorNum();
    const uint32_t sx = (uint32_t)strides.x, sy = (uint32_t)strides.y;
    if (C != k->Depth()) {
        decx::err::set(&handle, decx::DECX_FAIL_DimsNotMatching, "The depth of the kernels and of the source tensor must be identical");
        return handle;
    }
    if (!KW || !KH || !OC || (extend == de::_EXTEND_NONE_ && (KW > W || KH > H))) {
        decx::err::set(&handle, decx::DECX_FAIL_ConvBadKernel, "error: The kernel does not fit the source tensor"); return handle;
    }
    const bool ext = extend == de::_EXTEND_CONSTANT_;
    const uint32_t OW = ext ? W / sx : (W - KW + 1) / sx, OH = ext ? H / sy : (H - KH + 1) / sy;
    if (!d->re_construct(de::_FP32_, OW, OH, OC)) { handle = *de::GetLastError(); return handle; }
    if (!OW || !OH) return handle;

    std::lock_guard<std::mutex> guard(decx::module_mutex());
    ConvScratch& scratch = conv_scratch();
    void* S = decx::module_stream();
    const de::TensorLayout& SL = s->get_layout();
    const de::TensorLayout& KL = k->get_layout();
    const de::TensorLayout& DL = d->get_layout();
    const uint32_t kmat_pitch = (OC + 3) / 4 * 4;
    const size_t kmat_bytes = (size_t)KH * KW * SL.dpitch * kmat_pitch * 4;
    if (!scratch.ensure(scratch.kmat, kmat_bytes)) { handle = *de::GetLastError(); return handle; }
    int rc = decx_hip_conv2d_pack_kernels_f32((const float*)k->data(), (float*)scratch.kmat->ptr, KW, KH, C, KL.dpitch, KL.wpitch,
                                              (uint64_t)KL.dp_x_wp * KH, OC, kmat_pitch, SL.dpitch, S);
    const float* image = (const float*)s->data();
    uint32_t img_wpitch = SL.wpitch;
    if (rc == DECX_HIP_OK && ext) {
        // zero-extended copy: KW / 2 columns on the left, KH / 2 rows on top, and as far right / down as the
        // last window reaches (srcs/modules/NN/convolution/CUDA/fp32/cuda_conv2D_fp32_im2col_planner.cu:270-322)
        const uint32_t left = KW / 2, top = KH / 2;
        uint32_t PW = (OW - 1) * sx + KW, PH = (OH - 1) * sy + KH;
        if (PW < W + left) PW = W + left;
        if (PH < H + top) PH = H + top;
        img_wpitch = (PW + 7) / 8 * 8;
        const size_t row_bytes = (size_t)img_wpitch * SL.dpitch * 4, bytes = row_bytes * PH;
        if (!scratch.ensure(scratch.padded, bytes)) { handle = *de::GetLastError(); return handle; }
        rc = decx_hip_memset_async(scratch.padded->ptr, 0, bytes, S);
        if (rc == DECX_HIP_OK)
            rc = decx_hip_memcpy2d_async((char*)scratch.padded->ptr + top * row_bytes + (size_t)left * SL.dpitch * 4, row_bytes,
                                         s->data(), (size_t)SL.dp_x_wp * 4, (size_t)W * SL.dpitch * 4, H, 2, S);
        image = (const float*)scratch.padded->ptr;
    }
    if (rc == DECX_HIP_OK)
        rc = decx_hip_conv2d_f32_depth(image, (const float*)scratch.kmat->ptr, (float*)d->data(), OW, OH, OC, KW, KH, SL.depth,
                                       SL.dpitch, img_wpitch, sx, sy, kmat_pitch, DL.dpitch, DL.wpitch, S);
    const int rs = decx_hip_stream_sync(S);
    decx::err::from_hip(&handle, rc != DECX_HIP_OK ? rc : rs, "Conv2D");
    return handle;
}
