// Host side of the DECX matrix-product API on MI355X: the de:: objects, transfers, the
// status handle and the GEMM entry points.  Everything that touches the GPU goes through
// the C ABI in decx_hip.h.
#include "decx_internal.hpp"

#include <cstdlib>
#include <cstring>
#include <new>
#include <thread>
#include <vector>

namespace {

de::DH g_last_error = {0, "success: No error"};
bool g_gpu_ready = false;
uint64_t g_threads = 1;
void* g_stream = nullptr;
std::mutex g_mutex;

const char* const kSuccess         = "success: No error";
const char* const kCudaNotInit     = "error: CUDA should be initialized first";
const char* const kTypeNotMatch    = "error: The types of the two objects are not equal";
const char* const kOverranged      = "error: Failed to transfer data since it is out of range";
const char* const kDevAllocFail    = "error: Fail to allocate memory on device";
const char* const kHostAllocFail   = "error: Fail to allocate memory on RAM";
const char* const kClassNotInit    = "error: The class is not initialized";
const char* const kUnsupportedType = "error: The data type of the input onject is not supported";
const char* const kInvalidParam    = "error: The parameter(s) is(are) invalid";

uint32_t round_up(uint32_t v, uint32_t to) { return (v + to - 1) / to * to; }

}  // namespace

// ---------------------------------------------------------------- status

void decx::err::set(de::DH* h, int code, const char* text)
{
    h->error_type = code;
    std::strncpy(h->error_string, text, sizeof h->error_string - 1);
    h->error_string[sizeof h->error_string - 1] = '\0';
}
void decx::err::success(de::DH* h) { set(h, decx::DECX_SUCCESS, kSuccess); }

bool decx::err::from_hip(de::DH* h, int rc, const char* what)
{
    if (rc == DECX_HIP_OK) return false;
    char text[100];
    std::snprintf(text, sizeof text, "error: %s: %s", what, decx_hip_error_string(rc));
    int code = decx::DECX_FAIL_CUDA_STREAM;
    if (rc == DECX_HIP_E_NOT_INIT || rc == DECX_HIP_E_NO_DEVICE) code = decx::DECX_FAIL_CUDA_not_init;
    else if (rc == DECX_HIP_E_INVALID_ARG) code = decx::DECX_FAIL_INVALID_PARAM;
    else if (rc == 2 /* hipErrorOutOfMemory */) code = decx::DECX_FAIL_CUDA_ALLOCATION;
    set(h, code, text);
    return true;
}

bool decx::gpu_ready() { return g_gpu_ready; }
std::mutex& decx::module_mutex() { return g_mutex; }

void* decx::module_stream()
{
    if (!g_stream && g_gpu_ready) {
        if (decx_hip_stream_create(&g_stream) != DECX_HIP_OK) g_stream = nullptr;   // null stream still works
    }
    return g_stream;
}

uint32_t decx::element_size(de::_DATA_TYPES_FLAGS_ type)
{
    switch (type) {
    case de::_FP32_: case de::_INT32_: case de::_UCHAR4_: return 4;
    case de::_FP16_: return 2;
    case de::_FP64_: case de::_COMPLEX_F32_: case de::_UINT64_: return 8;
    case de::_COMPLEX_F64_: case de::_VECTOR3F_: case de::_VECTOR4F_: return 16;
    case de::_UINT8_: return 1;
    default: return 0;
    }
}

decx::HostBlock::~HostBlock()
{
    if (!ptr) return;
    if (pinned) decx_hip_host_free(ptr); else std::free(ptr);
}
decx::DeviceBlock::~DeviceBlock() { if (ptr) decx_hip_free(ptr); }

_DECX_API_ void de::InitCuda()
{
    const int rc = decx_hip_init(0);
    g_gpu_ready = (rc == DECX_HIP_OK);
    if (!g_gpu_ready) decx::err::from_hip(&g_last_error, rc, "InitCuda");
}
_DECX_API_ void de::InitCPUInfo()
{
    const unsigned n = std::thread::hardware_concurrency();
    g_threads = n ? n : 1;
}
_DECX_API_ void de::cuda::DECX_CUDA_exit()
{
    if (g_stream) { decx_hip_stream_destroy(g_stream); g_stream = nullptr; }
}
_DECX_API_ void de::cpu::DecxSetThreadingNum(const uint64_t n) { g_threads = n ? n : 1; }
_DECX_API_ de::DH* de::GetLastError() { return &g_last_error; }
_DECX_API_ void de::ResetLastError() { decx::err::success(&g_last_error); }

_DECX_API_ de::Half de::Float2Half(const float& x) { de::Half h; h.val = decx_hip_float_to_half(x); return h; }
_DECX_API_ float de::Half2Float(const de::Half& x) { return decx_hip_half_to_float(x.val); }

// ---------------------------------------------------------------- host matrix

void decx::_Matrix::assign(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height)
{
    _type = type;
    _layout._single_element_size = (int32_t)element_size(type);
    _layout.width = width;
    _layout.height = height;
    const uint32_t per32 = _layout._single_element_size ? 32u / (uint32_t)_layout._single_element_size : 1u;
    _layout.pitch = round_up(width, per32 ? per32 : 1u);
}

bool decx::_Matrix::allocate()
{
    auto block = std::make_shared<HostBlock>();
    const size_t bytes = total_bytes();
    block->bytes = bytes ? (bytes + 63) / 64 * 64 : 64;
    block->ptr = std::aligned_alloc(64, block->bytes);
    if (!block->ptr) { err::set(de::GetLastError(), DECX_FAIL_ALLOCATION, kHostAllocFail); return false; }
    std::memset(block->ptr, 0, block->bytes);
    _block = block;
    _data = block->ptr;
    return true;
}

decx::_Matrix::_Matrix() : _format(de::_NA_), _data(nullptr)
{
    _exp_data_ptr = &_data;
    _exp_matrix_dscr = &_layout;
    assign(de::_VOID_, 0, 0);
}
decx::_Matrix::_Matrix(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, de::_DATA_FORMATS_ format)
    : _format(format), _data(nullptr)
{
    _exp_data_ptr = &_data;
    _exp_matrix_dscr = &_layout;
    assign(type, width, height);
    allocate();
}
decx::_Matrix::~_Matrix() {}
uint32_t decx::_Matrix::Width() const { return _layout.width; }
uint32_t decx::_Matrix::Height() const { return _layout.height; }
void decx::_Matrix::release() { _block.reset(); _data = nullptr; }
de::_DATA_TYPES_FLAGS_ decx::_Matrix::Type() const { return _type; }
void decx::_Matrix::Reinterpret(const de::_DATA_TYPES_FLAGS_ t) { _type = t; }   // tag only, as the original
de::_DATA_FORMATS_ decx::_Matrix::Format() const { return _format; }

de::Matrix& decx::_Matrix::SoftCopy(de::Matrix& src)
{
    const _Matrix& s = dynamic_cast<_Matrix&>(src);
    assign(s._type, s._layout.width, s._layout.height);
    _format = s._format;
    _block = s._block;                 // shared, reference counted
    _data = s._data;
    return *this;
}

void decx::_Matrix::re_construct(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height)
{
    if (_type == type && _layout.width == width && _layout.height == height && _data) return;
    const size_t before = _block ? _block->bytes : 0;
    assign(type, width, height);
    if (total_bytes() > before || !_data) allocate();
}

int decx::_Matrix::move_storage(bool pinned)
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

_DECX_API_ de::Matrix* de::CreateMatrixPtr() { return new decx::_Matrix(); }
_DECX_API_ de::Matrix& de::CreateMatrixRef() { return *(new decx::_Matrix()); }
_DECX_API_ de::Matrix* de::CreateMatrixPtr(const de::_DATA_TYPES_FLAGS_ type, const uint32_t w, const uint32_t h,
                                           const de::_DATA_FORMATS_ format)
{
    return new decx::_Matrix(type, w, h, format);
}
_DECX_API_ de::Matrix& de::CreateMatrixRef(const de::_DATA_TYPES_FLAGS_ type, const uint32_t w, const uint32_t h,
                                           const de::_DATA_FORMATS_ format)
{
    return *(new decx::_Matrix(type, w, h, format));
}

_DECX_API_ de::DH de::cuda::PinMemory(de::Matrix& src)
{
    de::DH handle; decx::err::success(&handle);
    decx::_Matrix* m = dynamic_cast<decx::_Matrix*>(&src);
    if (!decx::gpu_ready()) { decx::err::set(&handle, decx::DECX_FAIL_CUDA_not_init, kCudaNotInit); return handle; }
    if (!m || !m->is_init()) { decx::err::set(&handle, decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return handle; }
    if (m->is_pinned()) {
        decx::err::set(&handle, decx::DECX_FAIL_HOST_MEM_REGISTERED, "error: The host memory is already page-locked");
        return handle;
    }
    decx::err::from_hip(&handle, m->move_storage(true), "PinMemory");
    return handle;
}
_DECX_API_ de::DH de::cuda::UnpinMemory(de::Matrix& src)
{
    de::DH handle; decx::err::success(&handle);
    decx::_Matrix* m = dynamic_cast<decx::_Matrix*>(&src);
    if (!m || !m->is_init()) { decx::err::set(&handle, decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return handle; }
    if (!m->is_pinned()) {
        decx::err::set(&handle, decx::DECX_FAIL_HOST_MEM_UNREGISTERED, "error: The host memory is not page-locked");
        return handle;
    }
    decx::err::from_hip(&handle, m->move_storage(false), "UnpinMemory");
    return handle;
}

// ---------------------------------------------------------------- device matrix

void decx::_GPU_Matrix::assign(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height)
{
    _type = type;
    _layout._single_element_size = (int32_t)element_size(type);
    _layout.width = width;
    _layout.height = height;
    const uint32_t per128 = _layout._single_element_size ? 128u / (uint32_t)_layout._single_element_size : 1u;
    _layout.pitch = round_up(width, per128 ? per128 : 1u);
    // A single column is stored dense.  Under the 128-byte rule every element of it would sit in a cache line of its
    // own, and a product with it (N = 1: the column is the vector of a matrix-vector product, and so is the result)
    // would move a line per element, or copy the column together first on every call.  Neither the pitch nor the
    // device pointer is visible through de::GPU_Matrix, so no caller can tell; de::Memcpy converts between this
    // and the host's 32-byte rows.
    if (width == 1) _layout.pitch = 1;
}

bool decx::_GPU_Matrix::allocate()
{
    auto block = std::make_shared<DeviceBlock>();
    block->bytes = total_bytes();
    int rc = decx_hip_malloc(&block->ptr, block->bytes);
    if (rc == DECX_HIP_OK && block->bytes) {
        rc = decx_hip_memset_async(block->ptr, 0, block->bytes, module_stream());
        if (rc == DECX_HIP_OK) rc = decx_hip_stream_sync(module_stream());
    }
    if (rc != DECX_HIP_OK) {
        block->ptr = (rc == DECX_HIP_E_NOT_INIT) ? nullptr : block->ptr;
        if (rc == DECX_HIP_E_NOT_INIT) err::set(de::GetLastError(), DECX_FAIL_CUDA_not_init, kCudaNotInit);
        else err::set(de::GetLastError(), DECX_FAIL_CUDA_ALLOCATION, kDevAllocFail);
        return false;
    }
    _block = block;
    return true;
}

decx::_GPU_Matrix::_GPU_Matrix() : _format(de::_NA_) { assign(de::_VOID_, 0, 0); }
decx::_GPU_Matrix::_GPU_Matrix(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height, de::_DATA_FORMATS_ format)
    : _format(format)
{
    assign(type, width, height);
    allocate();
}
decx::_GPU_Matrix::~_GPU_Matrix() {}
uint decx::_GPU_Matrix::Width() const { return _layout.width; }
uint decx::_GPU_Matrix::Height() const { return _layout.height; }
void decx::_GPU_Matrix::release() { _block.reset(); }
de::_DATA_TYPES_FLAGS_ decx::_GPU_Matrix::Type() const { return _type; }
void decx::_GPU_Matrix::Reinterpret(const de::_DATA_TYPES_FLAGS_ t) { _type = t; }
de::_DATA_FORMATS_ decx::_GPU_Matrix::Format() const { return _format; }

de::GPU_Matrix& decx::_GPU_Matrix::SoftCopy(de::GPU_Matrix& src)
{
    const _GPU_Matrix& s = dynamic_cast<_GPU_Matrix&>(src);
    assign(s._type, s._layout.width, s._layout.height);
    _format = s._format;
    _block = s._block;
    return *this;
}

bool decx::_GPU_Matrix::re_construct(de::_DATA_TYPES_FLAGS_ type, uint32_t width, uint32_t height)
{
    if (_type == type && _layout.width == width && _layout.height == height && is_init()) return true;
    const size_t before = _block ? _block->bytes : 0;
    assign(type, width, height);
    if (total_bytes() > before || !is_init()) return allocate();
    return true;
}

_DECX_API_ de::GPU_Matrix& de::CreateGPUMatrixRef() { return *(new decx::_GPU_Matrix()); }
_DECX_API_ de::GPU_Matrix* de::CreateGPUMatrixPtr() { return new decx::_GPU_Matrix(); }
_DECX_API_ de::GPU_Matrix* de::CreateGPUMatrixPtr(const de::_DATA_TYPES_FLAGS_ type, const uint32_t w, const uint32_t h,
                                                  const de::_DATA_FORMATS_ format)
{
    return new decx::_GPU_Matrix(type, w, h, format);
}
_DECX_API_ de::GPU_Matrix& de::CreateGPUMatrixRef(const de::_DATA_TYPES_FLAGS_ type, const uint32_t w, const uint32_t h,
                                                  const de::_DATA_FORMATS_ format)
{
    return *(new decx::_GPU_Matrix(type, w, h, format));
}

// ---------------------------------------------------------------- transfers

namespace {

// rows x width bytes from one pitched host buffer to another, on several host threads for large blocks
void copy_rows_parallel(char* dst, size_t dpitch, const char* src, size_t spitch, size_t width, size_t rows)
{
    const size_t bytes = width * rows;
    size_t workers = bytes / (512u << 10);                 // one thread per 512 KiB, at most 8 and what the host has
    const size_t hw = std::thread::hardware_concurrency();
    if (workers > 8) workers = 8;
    if (hw && workers > hw) workers = hw;
    auto part = [=](size_t r0, size_t r1) {
        if (dpitch == width && spitch == width) std::memcpy(dst + r0 * width, src + r0 * width, (r1 - r0) * width);
        else for (size_t r = r0; r < r1; ++r) std::memcpy(dst + r * dpitch, src + r * spitch, width);
    };
    if (workers <= 1 || rows < workers) { part(0, rows); return; }
    std::vector<std::thread> team;
    for (size_t w = 1; w < workers; ++w) team.emplace_back(part, rows * w / workers, rows * (w + 1) / workers);
    part(0, rows / workers);
    for (auto& t : team) t.join();
}

// Streams of the host-matrix pipeline, and the page-locked bounce buffers that pageable host memory travels
// through: the runtime's own staging of pageable copies is synchronous and several times slower than filling a
// page-locked buffer with host threads and copying that asynchronously.
struct HostPipe {
    static constexpr size_t kBuf = 16u << 20;              // bytes per bounce buffer
    static constexpr int kRing = 3;                        // buffers per direction
    void* in = nullptr;        // host -> device copies
    void* out = nullptr;       // device -> host copies
    bool ok = false;
    struct Slot { void* buf = nullptr; void* done = nullptr; bool busy = false; char* host = nullptr; size_t hpitch = 0, width = 0, rows = 0; };
    Slot up[kRing], down[kRing];
    int up_next = 0, down_next = 0;

    // pageable host -> device on stream `in`
    // bytes per piece: a quarter of the block, so that filling one buffer overlaps the copy of the previous one,
    // between 1 MiB and the buffer size
    static size_t piece_bytes(size_t total)
    {
        const size_t quarter = total / 4;
        return quarter < (1u << 20) ? (1u << 20) : (quarter > kBuf ? kBuf : quarter);
    }
    // `whole`: the caller overlaps its own blocks (the panel pipeline), so pieces are as large as the buffers
    int upload(void* dev, size_t dpitch, const char* host, size_t hpitch, size_t width, size_t rows, bool whole = false)
    {
        const size_t budget = whole ? (size_t)kBuf : piece_bytes(width * rows);
        const size_t wpiece = width < budget ? width : budget;
        const size_t rpiece = budget / wpiece ? budget / wpiece : 1;
        for (size_t c0 = 0; c0 < width; c0 += wpiece) {
            const size_t w = width - c0 < wpiece ? width - c0 : wpiece;
            for (size_t r0 = 0; r0 < rows; r0 += rpiece) {
                const size_t r = rows - r0 < rpiece ? rows - r0 : rpiece;
                Slot& s = up[up_next]; up_next = (up_next + 1) % kRing;
                int rc = s.busy ? decx_hip_event_sync(s.done) : DECX_HIP_OK;     // its previous copy has left the buffer
                if (rc != DECX_HIP_OK) return rc;
                copy_rows_parallel((char*)s.buf, w, host + r0 * hpitch + c0, hpitch, w, r);
                rc = decx_hip_memcpy2d_async((char*)dev + r0 * dpitch + c0, dpitch, s.buf, w, w, r, 0, in);
                if (rc == DECX_HIP_OK) rc = decx_hip_event_record(s.done, in);
                if (rc != DECX_HIP_OK) return rc;
                s.busy = true;
            }
        }
        return DECX_HIP_OK;
    }
    int drain(Slot& s)                                     // a finished device -> host piece goes to its pageable home
    {
        if (!s.busy || !s.host) return DECX_HIP_OK;
        const int rc = decx_hip_event_sync(s.done);
        if (rc == DECX_HIP_OK) copy_rows_parallel(s.host, s.hpitch, (const char*)s.buf, s.width, s.width, s.rows);
        s.busy = false; s.host = nullptr;
        return rc;
    }
    // device -> pageable host on stream `out`; pieces land in their home when their buffer is needed again, or in flush()
    int download(char* host, size_t hpitch, const void* dev, size_t dpitch, size_t width, size_t rows, bool whole = false)
    {
        const size_t budget = whole ? (size_t)kBuf : piece_bytes(width * rows);
        const size_t wpiece = width < budget ? width : budget;
        const size_t rpiece = budget / wpiece ? budget / wpiece : 1;
        for (size_t c0 = 0; c0 < width; c0 += wpiece) {
            const size_t w = width - c0 < wpiece ? width - c0 : wpiece;
            for (size_t r0 = 0; r0 < rows; r0 += rpiece) {
                const size_t r = rows - r0 < rpiece ? rows - r0 : rpiece;
                Slot& s = down[down_next]; down_next = (down_next + 1) % kRing;
                int rc = drain(s);
                if (rc == DECX_HIP_OK) rc = decx_hip_memcpy2d_async(s.buf, w, (const char*)dev + r0 * dpitch + c0, dpitch, w, r, 1, out);
                if (rc == DECX_HIP_OK) rc = decx_hip_event_record(s.done, out);
                if (rc != DECX_HIP_OK) return rc;
                s.busy = true; s.host = host + r0 * hpitch + c0; s.hpitch = hpitch; s.width = w; s.rows = r;
            }
        }
        return DECX_HIP_OK;
    }
    int flush()
    {
        int rc = DECX_HIP_OK;
        for (int i = 0; i < kRing; ++i) {                  // oldest first
            const int r = drain(down[(down_next + i) % kRing]);
            if (rc == DECX_HIP_OK) rc = r;
        }
        return rc;
    }
};
HostPipe& host_pipe()
{
    static HostPipe p;
    if (!p.ok && decx::gpu_ready()) {
        p.ok = decx_hip_stream_create(&p.in) == DECX_HIP_OK && decx_hip_stream_create(&p.out) == DECX_HIP_OK;
        for (int i = 0; i < HostPipe::kRing && p.ok; ++i)
            p.ok = decx_hip_host_malloc(&p.up[i].buf, HostPipe::kBuf) == DECX_HIP_OK && decx_hip_event_create(&p.up[i].done) == DECX_HIP_OK &&
                   decx_hip_host_malloc(&p.down[i].buf, HostPipe::kBuf) == DECX_HIP_OK && decx_hip_event_create(&p.down[i].done) == DECX_HIP_OK;
    }
    return p;
}

}  // namespace

int decx::stage_h2d(void* dev, size_t dpitch, const void* host, size_t hpitch, size_t width, size_t rows, bool host_pinned)
{
    if (!width || !rows) return DECX_HIP_OK;
    if (!host_pinned && width * rows >= (32u << 10) && host_pipe().ok)
        return host_pipe().upload(dev, dpitch, (const char*)host, hpitch, width, rows);
    return decx_hip_memcpy2d_async(dev, dpitch, host, hpitch, width, rows, 0, decx::module_stream());
}

int decx::stage_d2h(void* host, size_t hpitch, const void* dev, size_t dpitch, size_t width, size_t rows, bool host_pinned)
{
    if (!width || !rows) return DECX_HIP_OK;
    // device data written on the module stream has to be there before the copy stream reads it
    if (!host_pinned && width * rows >= (32u << 10) && host_pipe().ok) {
        const int rs = decx_hip_stream_sync(decx::module_stream());
        return rs != DECX_HIP_OK ? rs : host_pipe().download((char*)host, hpitch, dev, dpitch, width, rows);
    }
    return decx_hip_memcpy2d_async(host, hpitch, dev, dpitch, width, rows, 1, decx::module_stream());
}

int decx::stage_finish()
{
    int rc = decx_hip_stream_sync(decx::module_stream());
    if (host_pipe().ok) {
        const int r1 = decx_hip_stream_sync(host_pipe().in), r2 = host_pipe().flush();
        if (rc == DECX_HIP_OK) rc = r1 != DECX_HIP_OK ? r1 : r2;
    }
    return rc;
}

_DECX_API_ de::DH de::Memcpy(de::Matrix& host, de::GPU_Matrix& device, const de::Point2D start_src,
                             de::Point2D start_dst, const de::Point2D size, const int flag)
{
    de::DH handle; decx::err::success(&handle);
    if (!decx::gpu_ready()) { decx::err::set(&handle, decx::DECX_FAIL_CUDA_not_init, kCudaNotInit); return handle; }
    decx::_Matrix* h = dynamic_cast<decx::_Matrix*>(&host);
    decx::_GPU_Matrix* d = dynamic_cast<decx::_GPU_Matrix*>(&device);
    if (!h || !d || !h->is_init() || !d->is_init()) {
        decx::err::set(&handle, decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return handle;
    }
    if (h->Type() != d->Type()) { decx::err::set(&handle, decx::DECX_FAIL_TYPE_MOT_MATCH, kTypeNotMatch); return handle; }
    if (flag != de::DECX_MEMCPY_H2D && flag != de::DECX_MEMCPY_D2H) {
        decx::err::set(&handle, decx::DECX_FAIL_INVALID_PARAM, kInvalidParam); return handle;
    }
    const bool h2d = flag == de::DECX_MEMCPY_H2D;
    const int64_t src_w = h2d ? h->Width() : d->Width(), src_h = h2d ? h->Height() : d->Height();
    const int64_t dst_w = h2d ? d->Width() : h->Width(), dst_h = h2d ? d->Height() : h->Height();
    if (start_src.x < 0 || start_src.y < 0 || start_dst.x < 0 || start_dst.y < 0 || size.x < 0 || size.y < 0 ||
        (int64_t)start_src.x + size.x > src_w || (int64_t)start_src.y + size.y > src_h ||
        (int64_t)start_dst.x + size.x > dst_w || (int64_t)start_dst.y + size.y > dst_h) {
        decx::err::set(&handle, decx::DECX_FAIL_MEMCPY_OVERRANGED, kOverranged); return handle;
    }
    const size_t es = (size_t)h->get_layout()._single_element_size;
    const size_t hp = (size_t)h->Pitch() * es, dp = (size_t)d->Pitch() * es;
    const de::Point2D hs = h2d ? start_src : start_dst, ds = h2d ? start_dst : start_src;
    char* hptr = (char*)h->data() + (size_t)hs.y * hp + (size_t)hs.x * es;
    char* dptr = (char*)d->data() + (size_t)ds.y * dp + (size_t)ds.x * es;
    const size_t width = (size_t)size.x * es, rows = (size_t)size.y;
    std::lock_guard<std::mutex> guard(decx::module_mutex());
    // (the runtime copies a pitched pageable block row by row: 6 MB took 7 ms that way, 0.5 ms through the bounce
    // buffers; 256 MiB run at 52 GB/s)
    int rc = h2d ? decx::stage_h2d(dptr, dp, hptr, hp, width, rows, h->is_pinned())
                 : decx::stage_d2h(hptr, hp, dptr, dp, width, rows, h->is_pinned());
    const int rf = decx::stage_finish();
    if (rc == DECX_HIP_OK) rc = rf;
    decx::err::from_hip(&handle, rc, "Memcpy");
    return handle;
}

// ---------------------------------------------------------------- the product

namespace {

// Checks shared by both GPU entry points (cuda_GEMM_LS_planner::validate in the original,
// srcs/modules/BLAS/GEMM/CUDA/large_squares/common/cuda_GEMM_LS_planner.cu:227-258, plus the
// C-shape check its CPU twin makes, srcs/modules/BLAS/GEMM/CPU/cpu_GEMM_config.cxx:208-225).
// Unlike the original, a failed check returns before anything is launched.
bool validate(const decx::_GPU_Matrix* A, const decx::_GPU_Matrix* B, const decx::_GPU_Matrix* C,
              const decx::_GPU_Matrix* dst, const de::Number* alpha, const de::Number* beta, de::DH* h)
{
    if (!decx::gpu_ready()) { decx::err::set(h, decx::DECX_FAIL_CUDA_not_init, kCudaNotInit); return false; }
    if (!A || !B || !dst || !A->is_init() || !B->is_init() || (C && !C->is_init())) {
        decx::err::set(h, decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return false;
    }
    if (A->Width() != B->Height()) {
        decx::err::set(h, decx::DECX_FAIL_DimsNotMatching,
                       "The width of matrix A and height of matrix B must be identical");
        return false;
    }
    if (A->Type() != B->Type() || (C && C->Type() != A->Type())) {
        decx::err::set(h, decx::DECX_FAIL_TYPE_MOT_MATCH, "Types of the input matrices must be matched");
        return false;
    }
    if (C && (C->Height() != A->Height() || C->Width() != B->Width())) {
        decx::err::set(h, decx::DECX_FAIL_DimsNotMatching,
                       "The height and width of the matrix C should be identical to that of matrix A and matrix B");
        return false;
    }
    if (alpha && beta && (alpha->Type() != A->Type() || beta->Type() != A->Type())) {
        decx::err::set(h, decx::DECX_FAIL_TYPE_MOT_MATCH,
                       "The input scalar alpha and beta must match the type of input matrices");
        return false;
    }
    if (A->Type() != de::_FP32_ && A->Type() != de::_FP16_ && A->Type() != de::_FP64_ &&
        A->Type() != de::_COMPLEX_F32_ && A->Type() != de::_COMPLEX_F64_) {
        decx::err::set(h, decx::DECX_FAIL_UNSUPPORTED_TYPE, kUnsupportedType); return false;
    }
    return true;
}

// device workspace kept between calls (the real expansion of B of the complex forms, the partial products of
// a split K); grow-only, guarded by the module mutex
std::shared_ptr<decx::DeviceBlock>& complex_workspace() { static std::shared_ptr<decx::DeviceBlock> w; return w; }
bool ensure_workspace(size_t need, de::DH* h)
{
    std::shared_ptr<decx::DeviceBlock>& ws = complex_workspace();
    if (ws && ws->bytes >= need) return true;
    auto block = std::make_shared<decx::DeviceBlock>();
    block->bytes = need ? need : 64;
    if (decx_hip_malloc(&block->ptr, block->bytes) != DECX_HIP_OK) {
        block->ptr = nullptr;
        decx::err::set(h, decx::DECX_FAIL_CUDA_ALLOCATION, kDevAllocFail); return false;
    }
    ws = block;
    return true;
}

struct Scalar { double re, im; };

bool gemm_device(decx::_GPU_Matrix* A, decx::_GPU_Matrix* B, decx::_GPU_Matrix* C, decx::_GPU_Matrix* dst,
                 Scalar alpha_c, Scalar beta_c, de::DH* h)
{
    const double alpha = alpha_c.re, beta = beta_c.re;
    std::lock_guard<std::mutex> guard(decx::module_mutex());
    // C may be the same object as dst: keep its storage alive and its pitch in hand across the reshape
    const uint32_t ldc = C ? C->Pitch() : 0;
    const void* c_ptr = C ? C->data() : nullptr;
    if (!dst->re_construct(A->Type(), B->Width(), A->Height())) return false;   // status already set
    void* S = decx::module_stream();
    int rc;
    if (A->Type() == de::_COMPLEX_F32_ || A->Type() == de::_COMPLEX_F64_) {
        const bool single = A->Type() == de::_COMPLEX_F32_;
        const size_t need = decx_hip_gemm_complex_workspace(single ? 4 : 8, B->Width(), A->Width());
        if (!ensure_workspace(need, h)) return false;
        std::shared_ptr<decx::DeviceBlock>& ws = complex_workspace();
        rc = single ? decx_hip_gemm_c32((const float*)A->data(), (const float*)B->data(), (const float*)c_ptr, (float*)dst->data(),
                                        A->Height(), B->Width(), A->Width(), A->Pitch(), B->Pitch(), ldc, dst->Pitch(),
                                        (float)alpha_c.re, (float)alpha_c.im, (float)beta_c.re, (float)beta_c.im, ws->ptr, ws->bytes, S)
                    : decx_hip_gemm_c64((const double*)A->data(), (const double*)B->data(), (const double*)c_ptr, (double*)dst->data(),
                                        A->Height(), B->Width(), A->Width(), A->Pitch(), B->Pitch(), ldc, dst->Pitch(),
                                        alpha_c.re, alpha_c.im, beta_c.re, beta_c.im, ws->ptr, ws->bytes, S);
    }
    else {
        // few output tiles and a long K: the product may split K through the module's workspace
        const int eb = A->Type() == de::_FP32_ ? 4 : (A->Type() == de::_FP64_ ? 8 : 2);
        const size_t need = decx_hip_gemm_workspace(eb, A->Height(), B->Width(), A->Width());
        if (need && !ensure_workspace(need, h)) return false;
        void* ws = need ? complex_workspace()->ptr : nullptr;
        const size_t ws_bytes = need ? complex_workspace()->bytes : 0;
        if (eb == 4)
            rc = decx_hip_gemm_f32_ws((const float*)A->data(), (const float*)B->data(), (const float*)c_ptr,
                                      (float*)dst->data(), A->Height(), B->Width(), A->Width(),
                                      A->Pitch(), B->Pitch(), ldc, dst->Pitch(), (float)alpha, (float)beta, ws, ws_bytes, S);
        else if (eb == 8)
            rc = decx_hip_gemm_f64_ws((const double*)A->data(), (const double*)B->data(), (const double*)c_ptr,
                                      (double*)dst->data(), A->Height(), B->Width(), A->Width(),
                                      A->Pitch(), B->Pitch(), ldc, dst->Pitch(), alpha, beta, ws, ws_bytes, S);
        else
            rc = decx_hip_gemm_f16_ws((const uint16_t*)A->data(), (const uint16_t*)B->data(), (const uint16_t*)c_ptr,
                                      (uint16_t*)dst->data(), A->Height(), B->Width(), A->Width(),
                                      A->Pitch(), B->Pitch(), ldc, dst->Pitch(), (float)alpha, (float)beta, ws, ws_bytes, S);
    }
    if (rc == DECX_HIP_OK) rc = decx_hip_stream_sync(S);                     // result complete on return
    return !decx::err::from_hip(h, rc, "GEMM");
}

Scalar scalar_of(const de::Number& n)
{
    if (n.Type() == de::_FP16_) return {de::Half2Float(n.get_data_ref<de::Half>()), 0.0};
    if (n.Type() == de::_FP64_) return {n.get_data_ref<double>(), 0.0};
    if (n.Type() == de::_COMPLEX_F32_) return {n.get_data_ref<de::CPf>().real, n.get_data_ref<de::CPf>().image};
    if (n.Type() == de::_COMPLEX_F64_) return {n.get_data_ref<de::CPd>().real, n.get_data_ref<de::CPd>().image};
    return {n.get_data_ref<float>(), 0.0};
}

}  // namespace

_DECX_API_ void de::blas::cuda::GEMM(de::GPU_Matrix& A, de::GPU_Matrix& B, de::GPU_Matrix& dst)
{
    decx::_GPU_Matrix* a = dynamic_cast<decx::_GPU_Matrix*>(&A);
    decx::_GPU_Matrix* b = dynamic_cast<decx::_GPU_Matrix*>(&B);
    decx::_GPU_Matrix* d = dynamic_cast<decx::_GPU_Matrix*>(&dst);
    if (!validate(a, b, nullptr, d, nullptr, nullptr, de::GetLastError())) return;
    gemm_device(a, b, nullptr, d, Scalar{1.0, 0.0}, Scalar{1.0, 0.0}, de::GetLastError());
}

_DECX_API_ void de::blas::cuda::GEMM(de::GPU_Matrix& A, de::GPU_Matrix& B, de::GPU_Matrix& C, de::GPU_Matrix& dst,
                                     const de::Number alpha, const de::Number beta)
{
    decx::_GPU_Matrix* a = dynamic_cast<decx::_GPU_Matrix*>(&A);
    decx::_GPU_Matrix* b = dynamic_cast<decx::_GPU_Matrix*>(&B);
    decx::_GPU_Matrix* c = dynamic_cast<decx::_GPU_Matrix*>(&C);
    decx::_GPU_Matrix* d = dynamic_cast<decx::_GPU_Matrix*>(&dst);
    if (!c) { decx::err::set(de::GetLastError(), decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return; }
    if (!validate(a, b, c, d, &alpha, &beta, de::GetLastError())) return;
    gemm_device(a, b, c, d, scalar_of(alpha), scalar_of(beta), de::GetLastError());
}

namespace {

// Streams and events of the host-matrix form, created on first use and kept.
struct EventList {
    void* ev[64];
    int n = 0;
    void* make() { void* e = nullptr; if (n < 64 && decx_hip_event_create(&e) == DECX_HIP_OK) ev[n++] = e; return e; }
    ~EventList() { for (int i = 0; i < n; ++i) decx_hip_event_destroy(ev[i]); }
};

// Host-matrix form.  The original declares these overloads (srcs/includes/DECX/BLAS/BLAS.h:69-70) and defines
// them nowhere.  Here the operands are staged through device memory in row panels of A (and C): panel p + 1
// travels host -> device while panel p is multiplied and panel p - 1 of the result travels back, on three
// streams chained by events.  Page-locked host matrices (de::cuda::PinMemory) are copied directly; pageable ones
// travel through the pipeline's page-locked bounce buffers, which several host threads fill and empty.
void gemm_host(de::Matrix& A, de::Matrix& B, de::Matrix* C, de::Matrix& dst)
{
    de::DH* h = de::GetLastError();
    decx::_Matrix* a = dynamic_cast<decx::_Matrix*>(&A);
    decx::_Matrix* b = dynamic_cast<decx::_Matrix*>(&B);
    decx::_Matrix* c = C ? dynamic_cast<decx::_Matrix*>(C) : nullptr;
    decx::_Matrix* d = dynamic_cast<decx::_Matrix*>(&dst);
    if (!decx::gpu_ready()) { decx::err::set(h, decx::DECX_FAIL_CUDA_not_init, kCudaNotInit); return; }
    if (!a || !b || !d || !a->is_init() || !b->is_init() || (C && (!c || !c->is_init()))) {
        decx::err::set(h, decx::DECX_FAIL_CLASS_NOT_INIT, kClassNotInit); return;
    }
    // device twins: they carry the shapes through the same checks as the device form
    decx::_GPU_Matrix dA(a->Type(), a->Width(), a->Height(), de::_NA_);
    decx::_GPU_Matrix dB(b->Type(), b->Width(), b->Height(), de::_NA_);
    decx::_GPU_Matrix dC, dD;
    if (!dA.is_init() || !dB.is_init()) return;
    if (c) { dC.re_construct(c->Type(), c->Width(), c->Height()); if (!dC.is_init()) return; }
    if (!validate(&dA, &dB, c ? &dC : nullptr, &dD, nullptr, nullptr, h)) return;
    if (a->Type() == de::_COMPLEX_F32_ || a->Type() == de::_COMPLEX_F64_) {   // complex: device-matrix forms only
        decx::err::set(h, decx::DECX_FAIL_UNSUPPORTED_TYPE, kUnsupportedType); return;
    }
    const uint32_t M = a->Height(), N = b->Width(), K = a->Width();
    // C may be dst: take what is needed of it before dst is reshaped
    const char* c_host = c ? (const char*)c->data() : nullptr;
    const size_t c_host_pitch = c ? (size_t)c->Pitch() : 0;
    // (when C is dst the reshape below changes nothing: C already has the result's shape)
    d->re_construct(a->Type(), N, M);
    if (!dD.re_construct(a->Type(), N, M)) return;
    if (M == 0 || N == 0) return;

    std::lock_guard<std::mutex> guard(decx::module_mutex());
    HostPipe& pipe = host_pipe();
    void* S = decx::module_stream();
    if (!pipe.ok || !S) { decx::err::set(h, decx::DECX_FAIL_CUDA_STREAM, "error: Fail to create the staging streams"); return; }
    const size_t es = (size_t)a->get_layout()._single_element_size;
    const bool f16 = a->Type() == de::_FP16_;
    // panels of at least 256 rows, at most 16 of them
    uint32_t rows_per = (M + 15) / 16;
    rows_per = (rows_per + 255) / 256 * 256;
    const uint32_t panels = (M + rows_per - 1) / rows_per;

    EventList events;
    int rc = DECX_HIP_OK;
    // kind 0: host -> device on pipe.in, 1: device -> host on pipe.out; pitches and width in elements
    auto copy = [&](void* dp, size_t dpitch, const void* hp, size_t hpitch, size_t width, size_t rows, int kind, bool pinned) {
        if (rc != DECX_HIP_OK || !width || !rows) return;
        if (pinned)
            rc = decx_hip_memcpy2d_async(kind == 0 ? dp : const_cast<void*>(hp), (kind == 0 ? dpitch : hpitch) * es,
                                         kind == 0 ? hp : dp, (kind == 0 ? hpitch : dpitch) * es, width * es, rows, kind,
                                         kind == 0 ? pipe.in : pipe.out);
        else if (kind == 0) rc = pipe.upload(dp, dpitch * es, (const char*)hp, hpitch * es, width * es, rows, true);
        else rc = pipe.download((char*)const_cast<void*>(hp), hpitch * es, dp, dpitch * es, width * es, rows, true);
    };
    const bool a_pinned = a->is_pinned(), b_pinned = b->is_pinned(), c_pinned = c && c->is_pinned(), d_pinned = d->is_pinned();
    copy(dB.data(), dB.Pitch(), b->data(), b->Pitch(), N, K, 0, b_pinned);
    for (uint32_t p = 0; p < panels && rc == DECX_HIP_OK; ++p) {
        const uint32_t r0 = p * rows_per, rows = (M - r0) < rows_per ? (M - r0) : rows_per;
        char* a_dev = (char*)dA.data() + (size_t)r0 * dA.Pitch() * es;
        char* d_dev = (char*)dD.data() + (size_t)r0 * dD.Pitch() * es;
        char* c_dev = c ? (char*)dC.data() + (size_t)r0 * dC.Pitch() * es : nullptr;
        copy(a_dev, dA.Pitch(), (const char*)a->data() + (size_t)r0 * a->Pitch() * es, a->Pitch(), K, rows, 0, a_pinned);
        if (c) copy(c_dev, dC.Pitch(), c_host + (size_t)r0 * c_host_pitch * es, c_host_pitch, N, rows, 0, c_pinned);
        void* arrived = events.make();
        void* done = events.make();
        if (!arrived || !done) { rc = DECX_HIP_E_INVALID_ARG; break; }
        if (rc == DECX_HIP_OK) rc = decx_hip_event_record(arrived, pipe.in);
        if (rc == DECX_HIP_OK) rc = decx_hip_stream_wait_event(S, arrived);
        if (rc == DECX_HIP_OK && a->Type() == de::_FP64_)
            rc = decx_hip_gemm_f64((const double*)a_dev, (const double*)dB.data(), (const double*)c_dev, (double*)d_dev, rows, N, K,
                                   dA.Pitch(), dB.Pitch(), c ? dC.Pitch() : 0, dD.Pitch(), 1.0, 1.0, S);
        else if (rc == DECX_HIP_OK)
            rc = f16 ? decx_hip_gemm_f16((const uint16_t*)a_dev, (const uint16_t*)dB.data(), (const uint16_t*)c_dev,
                                         (uint16_t*)d_dev, rows, N, K, dA.Pitch(), dB.Pitch(), c ? dC.Pitch() : 0,
                                         dD.Pitch(), 1.f, 1.f, S)
                     : decx_hip_gemm_f32((const float*)a_dev, (const float*)dB.data(), (const float*)c_dev,
                                         (float*)d_dev, rows, N, K, dA.Pitch(), dB.Pitch(), c ? dC.Pitch() : 0,
                                         dD.Pitch(), 1.f, 1.f, S);
        if (rc == DECX_HIP_OK) rc = decx_hip_event_record(done, S);
        if (rc == DECX_HIP_OK) rc = decx_hip_stream_wait_event(pipe.out, done);
        copy(d_dev, dD.Pitch(), (char*)d->data() + (size_t)r0 * d->Pitch() * es, d->Pitch(), N, rows, 1, d_pinned);
    }
    const int rf = pipe.flush();                           // the last pieces of a pageable dst
    if (rc == DECX_HIP_OK) rc = rf;
    // drain all three streams whatever happened, so that nothing is in flight when the device twins die
    const int r1 = decx_hip_stream_sync(pipe.in), r2 = decx_hip_stream_sync(S), r3 = decx_hip_stream_sync(pipe.out);
    if (rc == DECX_HIP_OK) rc = r1 != DECX_HIP_OK ? r1 : (r2 != DECX_HIP_OK ? r2 : r3);
    decx::err::from_hip(h, rc, "GEMM");
}

}  // namespace

_DECX_API_ void de::blas::cuda::GEMM(de::Matrix& A, de::Matrix& B, de::Matrix& dst) { gemm_host(A, B, nullptr, dst); }
_DECX_API_ void de::blas::cuda::GEMM(de::Matrix& A, de::Matrix& B, de::Matrix& C, de::Matrix& dst)
{
    gemm_host(A, B, &C, dst);
}
