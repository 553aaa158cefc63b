/*
 * DECX.h -- public C++ interface of the MI355X-native dense-GEMM module.
 *
 * Source- and ABI-compatible with the part of the DECX user API that the matrix
 * multiplication path touches, so code written against the original library
 * (samples/Matrix_Multiplication/MatMul.cpp) builds and links unchanged:
 *
 *   de::DH, de::GetLastError            srcs/includes/DECX/basic.h:84-98,127-159
 *   de::_DATA_TYPES_FLAGS_, formats     srcs/includes/DECX/classes/type_info.h:20-53
 *   de::Half, de::Point2D               srcs/includes/DECX/classes/class_utils.h:19-60
 *   de::Number, Float2Half, Half2Float  srcs/includes/DECX/classes/DecxNumber.h:17-188
 *   de::Matrix, de::MatrixLayout        srcs/includes/DECX/classes/Matrix.h:34-105
 *   de::GPU_Matrix, Pin/UnpinMemory     srcs/includes/DECX/classes/GPU_Matrix.h:19-65
 *   de::Memcpy (matrix form)            srcs/includes/DECX/classes/decx_memcpy.h:29-48
 *   de::blas::cuda::GEMM                srcs/includes/DECX/BLAS/BLAS.h:69-76
 *
 * Same class layouts (vtable order, the two shadow pointers of de::Matrix), same enum
 * values, same width-before-height argument order.  The namespace stays `cuda` because
 * it is part of the API's spelling; everything behind it is HIP on gfx950, reached
 * through the C ABI in decx_hip.h.
 *
 * Further down: the vector containers and the vector x matrix forms (de::Vector, de::GPU_Vector,
 * srcs/includes/DECX/classes/Vector.h, GPU_Vector.h, BLAS.h:79-80) and the tensor containers with
 * de::nn::cuda::Conv2D (Tensor.h, GPU_Tensor.h, TensorArray.h, BLAS.h:109-110), which call the same kernels.
 * Not provided here: de::blas::cpu::GEMM (the CPU path is not part of this module).
 */
#ifndef DECX_AMD_PUBLIC_H_
#define DECX_AMD_PUBLIC_H_

#ifndef __cplusplus
#error "DECX.h is a C++ header; C callers use decx_hip.h"
#endif

#include <cstdint>
#include <cstdio>

typedef unsigned char uchar;
typedef unsigned int uint;

#define _DECX_API_ __attribute__((visibility("default")))
#define _SHADOW_ATTRIBUTE_(__actual_type) __actual_type*

/* ------------------------------------------------------------------ status handle */
namespace de {

typedef struct DECX_Handle {
    int  error_type;           /* one of decx::DECX_error_types below */
    char error_string[100];
} DH;

/* The user-facing enum of the original header, kept value for value. */
enum DECX_error_types {
    DECX_SUCCESS = 0x00, DECX_FAIL_not_init = 0x01, DECX_FAIL_FFT_error_length = 0x02,
    DECX_FAIL_DimsNotMatching = 0x03, DECX_FAIL_Complex_comparing = 0x04, DECX_FAIL_ConvBadKernel = 0x05,
    DECX_FAIL_StepError = 0x06, DECX_FAIL_ChannelError = 0x07, DECX_FAIL_CVNLM_BadArea = 0x08,
    DECX_FAIL_FileNotExist = 0x09, DECX_GEMM_DimsError = 0x0a, DECX_FAIL_ErrorFlag = 0x0b,
    DECX_FAIL_DimError = 0x0c, DECX_FAIL_ErrorParams = 0x0d, DECX_FAIL_StoreError = 0x0e,
    DECX_FAIL_MNumNotMatching = 0x0f, DECX_FAIL_ALLOCATION = 0x10
};

_DECX_API_ void InitCuda();          /* selects GPU 0 and reads its properties; must precede Memcpy / GEMM */
_DECX_API_ void InitCPUInfo();       /* records the host's hardware concurrency */
_DECX_API_ DH*  GetLastError();      /* process-global status of the last failing call */
_DECX_API_ void ResetLastError();

namespace cuda { _DECX_API_ void DECX_CUDA_exit(); }
namespace cpu  { _DECX_API_ void DecxSetThreadingNum(const uint64_t _thread_num); }

}  // namespace de

/* The codes the library actually writes into de::DH::error_type: the original library
 * sets its *internal* numbering (srcs/common/Handle/decx_handle.h:47-179), which differs
 * from the user-facing enum above; both are kept. */
namespace decx {
enum DECX_error_types {
    DECX_SUCCESS = 0x00, DECX_FAIL_CPU_not_init = 0x01, DECX_FAIL_FFT_error_length = 0x02,
    DECX_FAIL_DimsNotMatching = 0x03, DECX_FAIL_Complex_comparing = 0x04, DECX_FAIL_ConvBadKernel = 0x05,
    DECX_FAIL_CVNLM_BadArea = 0x06, DECX_FAIL_ErrorFlag = 0x07, DECX_FAIL_ALLOCATION = 0x08,
    DECX_FAIL_CUDA_STREAM = 0x09, DECX_FAIL_CLASS_NOT_INIT = 0x0a, DECX_FAIL_TYPE_MOT_MATCH = 0x0b,
    DECX_FAIL_INVALID_PARAM = 0x0c, DECX_FAIL_IMAGE_LOAD_FAILED = 0x0d, DECX_FAIL_CUDA_EVENT = 0x0e,
    MULTIPLE_REFERENCES = 0x0f, CPU_HYPER_THREADING = 0x10, MEMCPY_DIFFERENT_TYPES = 0x11,
    DECX_FAIL_MEMCPY_OVERRANGED = 0x12, DECX_FAIL_UNSUPPORTED_TYPE = 0x13, DECX_FAIL_HOST_MEM_REGISTERED = 0x14,
    DECX_FAIL_HOST_MEM_UNREGISTERED = 0x15, DECX_FAIL_CUDA_not_init = 0x16, DECX_FAIL_CUDA_ALLOCATION = 0x17
};
}  // namespace decx

/* ------------------------------------------------------------------ element types */
namespace de {

enum _DATA_TYPES_FLAGS_ {
    _VOID_ = 0, _FP32_ = 1, _FP64_ = 2, _FP16_ = 3, _INT32_ = 4, _COMPLEX_F32_ = 5, _COMPLEX_F64_ = 6,
    _UINT64_ = 7, _UINT8_ = 8, _UCHAR4_ = 12, _VECTOR3F_ = 14, _VECTOR4F_ = 15
};

enum _DATA_FORMATS_ { _NA_ = 0, _RGB_ = 1, _YUV444_ = 2, _HSV_ = 3, _CPLX_CARTESIAN_ = 4, _CPLX_POLAR_ = 5 };

enum GEMM_properties { HALF_GEMM_DIRECT = 0, HALF_GEMM_ACCURATE = 1 };

struct Half { unsigned short val; };                 /* IEEE binary16 bit pattern */

typedef struct __attribute__((aligned(8))) complex_f {
    float real, image;
    complex_f(const float r, const float i) : real(r), image(i) {}
    complex_f() {}
} CPf;

typedef struct __attribute__((aligned(16))) complex_d {
    double real, image;
    complex_d(const double r, const double i) : real(r), image(i) {}
    complex_d() : real(0), image(0) {}
} CPd;

struct __attribute__((aligned(8))) Point2D {         /* [x = along the width, y = along the height] */
    int32_t x, y;
    Point2D(const int32_t _x, const int32_t _y) : x(_x), y(_y) {}
    Point2D(const uint32_t _x, const uint32_t _y) : x((int32_t)_x), y((int32_t)_y) {}
    Point2D() {}
};

struct __attribute__((aligned(16))) Point3D {        /* tensors: [x = depth, y = width, z = height] */
    int32_t x, y, z;
    Point3D(const int32_t _x, const int32_t _y, const int32_t _z) : x(_x), y(_y), z(_z) {}
    Point3D(const uint32_t _x, const uint32_t _y, const uint32_t _z) : x((int32_t)_x), y((int32_t)_y), z((int32_t)_z) {}
    Point3D() {}
};

/* How the borders of an image are treated by a convolution. */
enum extend_label { _EXTEND_NONE_ = 0, _EXTEND_REFLECT_ = 1, _EXTEND_CONSTANT_ = 2 };

_DECX_API_ Half  Float2Half(const float& __x);       /* round to nearest even */
_DECX_API_ float Half2Float(const Half& __x);

/* A tagged scalar: carries alpha / beta of the four-matrix GEMM. */
class _DECX_API_ Number {
    union __attribute__((aligned(16))) _data {
        float _fp32; double _fp64; CPf _cplxf32; CPd _cplxd64; uint8_t _u8; int32_t _i32; Half _fp16;
        _data() { _cplxd64.real = 0.0; _cplxd64.image = 0.0; }
    };
    _data   _number;
    int32_t _data_type_flag;

public:
    Number() : _data_type_flag(_VOID_) {}
    Number(const int32_t v) : _data_type_flag(_INT32_)       { _number._i32 = v; }
    Number(const uint8_t v) : _data_type_flag(_UINT8_)       { _number._u8 = v; }
    Number(const float v)   : _data_type_flag(_FP32_)        { _number._fp32 = v; }
    Number(const double v)  : _data_type_flag(_FP64_)        { _number._fp64 = v; }
    Number(const Half v)    : _data_type_flag(_FP16_)        { _number._fp16 = v; }
    Number(const CPf v)     : _data_type_flag(_COMPLEX_F32_) { _number._cplxf32 = v; }
    Number(const CPd v)     : _data_type_flag(_COMPLEX_F64_) { _number._cplxd64 = v; }

    int32_t Type() const { return _data_type_flag; }
    template <typename _Ty> _Ty get_data() { return *((_Ty*)&_number); }
    template <typename _Ty> const _Ty& get_data_ref() const { return *((const _Ty*)&_number); }

    Number& operator=(const float v)   { _number._fp32 = v;    _data_type_flag = _FP32_;        return *this; }
    Number& operator=(const double v)  { _number._fp64 = v;    _data_type_flag = _FP64_;        return *this; }
    Number& operator=(const CPf v)     { _number._cplxf32 = v; _data_type_flag = _COMPLEX_F32_; return *this; }
    Number& operator=(const CPd v)     { _number._cplxd64 = v; _data_type_flag = _COMPLEX_F64_; return *this; }
    Number& operator=(const uint8_t v) { _number._u8 = v;      _data_type_flag = _UINT8_;       return *this; }
    Number& operator=(const int32_t v) { _number._i32 = v;     _data_type_flag = _INT32_;       return *this; }
    Number& operator=(const Half v)    { _number._fp16 = v;    _data_type_flag = _FP16_;        return *this; }

    void Print() {
        switch (_data_type_flag) {
        case _FP32_:        printf("%f\n", get_data<float>()); break;
        case _FP16_:        printf("%f\n", Half2Float(get_data<Half>())); break;
        case _FP64_:        printf("%f\n", get_data<double>()); break;
        case _INT32_:       printf("%d\n", get_data<int32_t>()); break;
        case _UINT8_:       printf("%d\n", (int32_t)get_data<uint8_t>()); break;
        case _COMPLEX_F32_: printf("(%f, %f)\n", get_data<CPf>().real, get_data<CPf>().image); break;
        default: break;
        }
    }
};
typedef const Number& InputNumber;
typedef Number& OutputNumber;
typedef Number& InOutNumber;

/* ------------------------------------------------------------------ host matrix */

struct MatrixLayout {
    uint32_t width, height;
    uint32_t pitch;                    /* row stride in elements: width rounded up to 32 bytes */
    int32_t  _single_element_size;
};

class _DECX_API_ Matrix {
protected:
    _SHADOW_ATTRIBUTE_(void*)        _exp_data_ptr;        /* -> the implementation's data pointer */
    _SHADOW_ATTRIBUTE_(MatrixLayout) _exp_matrix_dscr;     /* -> the implementation's layout */

public:
    Matrix() {}
    virtual uint32_t Width() const = 0;
    virtual uint32_t Height() const = 0;

    template <typename _ptr_type> _ptr_type* ptr(const int row, const int col) {
        return ((_ptr_type*)*this->_exp_data_ptr) + this->_exp_matrix_dscr->pitch * row + col;
    }

    virtual void release() = 0;
    virtual Matrix& SoftCopy(Matrix& src) = 0;
    virtual _DATA_TYPES_FLAGS_ Type() const = 0;
    virtual void Reinterpret(const _DATA_TYPES_FLAGS_ _new_type) = 0;
    virtual _DATA_FORMATS_ Format() const = 0;
    ~Matrix() {}
};
typedef const Matrix& InputMatrix;
typedef Matrix& OutputMatrix;
typedef Matrix& InOutMatrix;

_DECX_API_ Matrix* CreateMatrixPtr();
_DECX_API_ Matrix& CreateMatrixRef();
_DECX_API_ Matrix* CreateMatrixPtr(const _DATA_TYPES_FLAGS_ type, const uint32_t _width, const uint32_t _height,
                                   const _DATA_FORMATS_ format = _NA_);
_DECX_API_ Matrix& CreateMatrixRef(const _DATA_TYPES_FLAGS_ type, const uint32_t _width, const uint32_t _height,
                                   const _DATA_FORMATS_ format = _NA_);

/* ------------------------------------------------------------------ device matrix */

class _DECX_API_ GPU_Matrix {
public:
    GPU_Matrix() {}
    virtual uint Width() const = 0;
    virtual uint Height() const = 0;
    virtual void release() = 0;
    virtual _DATA_TYPES_FLAGS_ Type() const = 0;
    virtual void Reinterpret(const _DATA_TYPES_FLAGS_ _new_type) = 0;
    virtual GPU_Matrix& SoftCopy(GPU_Matrix& src) = 0;
    virtual _DATA_FORMATS_ Format() const = 0;
    ~GPU_Matrix() {}
};
typedef const GPU_Matrix& InputGPUMatrix;
typedef GPU_Matrix& OutputGPUMatrix;
typedef GPU_Matrix& InOutGPUMatrix;

_DECX_API_ GPU_Matrix& CreateGPUMatrixRef();
_DECX_API_ GPU_Matrix* CreateGPUMatrixPtr();
_DECX_API_ GPU_Matrix* CreateGPUMatrixPtr(const _DATA_TYPES_FLAGS_ type, const uint32_t _width, const uint32_t _height,
                                          const _DATA_FORMATS_ format = _NA_);
_DECX_API_ GPU_Matrix& CreateGPUMatrixRef(const _DATA_TYPES_FLAGS_ type, const uint32_t _width, const uint32_t _height,
                                          const _DATA_FORMATS_ format = _NA_);

/* ------------------------------------------------------------------ host and device vectors */

/* A zero-filled array of Len() elements whose storage is rounded up to 32 bytes. */
class _DECX_API_ Vector {
protected:
    _SHADOW_ATTRIBUTE_(void*) _exp_data_ptr;               /* -> the implementation's data pointer */

public:
    Vector() {}
    virtual size_t Len() const = 0;

    template <typename _ptr_type> _ptr_type* ptr(const uint64_t _idx) { return ((_ptr_type*)*this->_exp_data_ptr) + _idx; }

    virtual void release() = 0;
    virtual Vector& SoftCopy(Vector& src) = 0;
    virtual _DATA_TYPES_FLAGS_ Type() const = 0;
    virtual void Reinterpret(const _DATA_TYPES_FLAGS_ _new_type) = 0;
    ~Vector() {}
};
typedef const Vector& InputVector;
typedef Vector& OutputVector;
typedef Vector& InOutVector;

_DECX_API_ Vector& CreateVectorRef();
_DECX_API_ Vector* CreateVectorPtr();
_DECX_API_ Vector& CreateVectorRef(const _DATA_TYPES_FLAGS_ _type, size_t len);
_DECX_API_ Vector* CreateVectorPtr(const _DATA_TYPES_FLAGS_ _type, size_t len);

class _DECX_API_ GPU_Vector {
public:
    GPU_Vector() {}
    virtual size_t Len() const = 0;
    virtual void release() = 0;
    virtual GPU_Vector& SoftCopy(GPU_Vector& src) = 0;
    virtual _DATA_TYPES_FLAGS_ Type() const = 0;
    virtual void Reinterpret(const _DATA_TYPES_FLAGS_ _new_type) = 0;
    ~GPU_Vector() {}
};

_DECX_API_ GPU_Vector& CreateGPUVectorRef();
_DECX_API_ GPU_Vector* CreateGPUVectorPtr();
_DECX_API_ GPU_Vector& CreateGPUVectorRef(const _DATA_TYPES_FLAGS_ _type, const size_t _length);
_DECX_API_ GPU_Vector* CreateGPUVectorPtr(const _DATA_TYPES_FLAGS_ _type, const size_t _length);

/* How fp16 vector products accumulate.  Every level accumulates in fp32 here (the most
 * accurate of the three); the level only selects the element type of the result, as it does
 * in the original: level 1 writes fp32, levels 2 and 3 write fp16 (rounded once). */
enum Fp16_Accuracy_Levels { Fp16_Accurate_L1 = 0, Fp16_Accurate_L2 = 1, Fp16_Accurate_L3 = 2 };

namespace cuda {
/* Makes the host matrix's storage page-locked (faster, asynchronous-capable transfers) and
 * back.  The storage is moved, not registered in place; pointers obtained from ptr<T>()
 * before the call must be re-read. */
_DECX_API_ DH PinMemory(Matrix& src);
_DECX_API_ DH UnpinMemory(Matrix& src);
_DECX_API_ DH PinMemory(Vector& src);
_DECX_API_ DH UnpinMemory(Vector& src);
}

/* ------------------------------------------------------------------ tensors (images with channels) */

/* Element (row x, column y, channel z) of a tensor lives at x * dp_x_wp + y * dpitch + z.  Host tensors pad
 * the width to 4 columns, device tensors to 8; both pad the depth to 16 bytes of elements; zero-filled. */
struct TensorLayout {
    uint32_t width, height, depth;
    uint32_t dpitch;               /* channel pitch in elements */
    uint32_t wpitch;               /* row pitch in columns */
    uint64_t dp_x_wp;              /* dpitch * wpitch */
    uint8_t  _single_element_size;
    uint64_t plane[3];             /* active elements of the WH, WD and HD planes */
};

class _DECX_API_ Tensor {
protected:
    _SHADOW_ATTRIBUTE_(void*)        _exp_data_ptr;
    _SHADOW_ATTRIBUTE_(TensorLayout) _exp_tensor_dscr;

public:
    Tensor() {}
    virtual uint32_t Width() const = 0;
    virtual uint32_t Height() const = 0;
    virtual uint32_t Depth() const = 0;

    template <typename _ptr_type> _ptr_type* ptr(const int x, const int y, const int z) {
        return ((_ptr_type*)(*this->_exp_data_ptr)) +
               (x * this->_exp_tensor_dscr->dp_x_wp + y * this->_exp_tensor_dscr->dpitch + z);
    }

    virtual Tensor& SoftCopy(Tensor& src) = 0;
    virtual void release() = 0;
    virtual _DATA_TYPES_FLAGS_ Type() const = 0;
    virtual void Reinterpret(const _DATA_TYPES_FLAGS_ _new_type) = 0;
};

_DECX_API_ Tensor* CreateTensorPtr();
_DECX_API_ Tensor& CreateTensorRef();
_DECX_API_ Tensor* CreateTensorPtr(const _DATA_TYPES_FLAGS_ _type, const uint _width, const uint _height, const uint _depth);
_DECX_API_ Tensor& CreateTensorRef(const _DATA_TYPES_FLAGS_ _type, const uint _width, const uint _height, const uint _depth);

class _DECX_API_ GPU_Tensor {
public:
    GPU_Tensor() {}
    virtual uint Width() const = 0;
    virtual uint Height() const = 0;
    virtual uint Depth() const = 0;
    virtual GPU_Tensor& SoftCopy(GPU_Tensor& src) = 0;
    virtual void release() = 0;
    virtual _DATA_TYPES_FLAGS_ Type() const = 0;
    virtual void Reinterpret(const _DATA_TYPES_FLAGS_ _new_type) = 0;
    virtual DH Extract_SoftCopy(const uint32_t index, GPU_Tensor& dst) const = 0;   /* one channel plane: not provided here */
};

_DECX_API_ GPU_Tensor* CreateGPUTensorPtr();
_DECX_API_ GPU_Tensor& CreateGPUTensorRef();
_DECX_API_ GPU_Tensor* CreateGPUTensorPtr(const _DATA_TYPES_FLAGS_ _type, const uint _width, const uint _height, const uint32_t _depth);
_DECX_API_ GPU_Tensor& CreateGPUTensorRef(const _DATA_TYPES_FLAGS_ _type, const uint _width, const uint _height, const uint32_t _depth);

/* tensor_num tensors of one shape in one allocation (a set of convolution kernels). */
class _DECX_API_ TensorArray {
protected:
    _SHADOW_ATTRIBUTE_(void**)       _exp_data_ptr;        /* -> the table of per-tensor pointers */
    _SHADOW_ATTRIBUTE_(TensorLayout) _exp_tensor_dscr;

public:
    TensorArray() {}
    virtual uint Width() const = 0;
    virtual uint Height() const = 0;
    virtual uint Depth() const = 0;
    virtual uint TensorNum() const = 0;

    template <typename _ptr_type> _ptr_type* ptr(const int x, const int y, const int z, const int tensor_id) {
        return ((_ptr_type*)(*this->_exp_data_ptr)[tensor_id]) + x * this->_exp_tensor_dscr->dp_x_wp +
               y * this->_exp_tensor_dscr->dpitch + z;
    }

    virtual TensorArray& SoftCopy(TensorArray& src) = 0;
    virtual _DATA_TYPES_FLAGS_ Type() const = 0;
    virtual void Reinterpret(const _DATA_TYPES_FLAGS_ _new_type) = 0;
    virtual DH Extract_SoftCopy(const uint32_t index, Tensor& dst) const = 0;        /* dst aliases tensor `index` */
    virtual void release() = 0;
};

_DECX_API_ TensorArray& CreateTensorArrayRef();
_DECX_API_ TensorArray* CreateTensorArrayPtr();
_DECX_API_ TensorArray& CreateTensorArrayRef(const _DATA_TYPES_FLAGS_ _type, const uint width, const uint height, const uint depth, const uint tensor_num);
_DECX_API_ TensorArray* CreateTensorArrayPtr(const _DATA_TYPES_FLAGS_ _type, const uint width, const uint height, const uint depth, const uint tensor_num);

class _DECX_API_ GPU_TensorArray {
public:
    GPU_TensorArray() {}
    virtual uint Width() const = 0;
    virtual uint Height() const = 0;
    virtual uint Depth() const = 0;
    virtual uint TensorNum() const = 0;
    virtual _DATA_TYPES_FLAGS_ Type() const = 0;
    virtual void Reinterpret(const _DATA_TYPES_FLAGS_ _new_type) = 0;
    virtual GPU_TensorArray& SoftCopy(const GPU_TensorArray& src) = 0;
    virtual DH Extract_SoftCopy(const uint32_t index, GPU_Tensor& dst) const = 0;    /* dst aliases tensor `index` */
    virtual void release() = 0;
};

_DECX_API_ GPU_TensorArray& CreateGPUTensorArrayRef();
_DECX_API_ GPU_TensorArray* CreateGPUTensorArrayPtr();
_DECX_API_ GPU_TensorArray& CreateGPUTensorArrayRef(const _DATA_TYPES_FLAGS_ _type, const uint width, const uint height, const uint depth, const uint32_t _array_length);
_DECX_API_ GPU_TensorArray* CreateGPUTensorArrayPtr(const _DATA_TYPES_FLAGS_ _type, const uint width, const uint height, const uint depth, const uint32_t _array_length);

/* ------------------------------------------------------------------ transfers */

enum DECX_Memcpy_Flags { DECX_MEMCPY_H2D = 0, DECX_MEMCPY_D2H = 1 };

/* Copies the cpy_size = [W, H] region that starts at start_src in the source object to
 * start_dst in the destination object; the source is the host matrix for H2D and the
 * device matrix for D2H.  Blocks until the copy has finished. */
_DECX_API_ DH Memcpy(Matrix& __host, GPU_Matrix& __device, const Point2D start_src, Point2D start_dst,
                     const Point2D cpy_size, const int _memcpy_flag);

/* Copies cpy_len elements from element start_src of the source to element start_dst of the
 * destination (source = host vector for H2D, device vector for D2H). */
_DECX_API_ DH Memcpy(Vector& __host, GPU_Vector& __device, const uint64_t start_src, const uint64_t start_dst,
                     const uint64_t cpy_len, const int _memcpy_flag);

/* Copies the cpy_size = [D, W, H] box that starts at start_src = [depth, column, row] of the source to start_dst
 * of the destination (source = host tensor for H2D, device tensor for D2H). */
_DECX_API_ DH Memcpy(Tensor& __host, GPU_Tensor& __device, const Point3D start_src, const Point3D start_dst,
                     const Point3D cpy_size, const int _memcpy_flag);

/* ------------------------------------------------------------------ the product */
namespace blas {
namespace cuda {
/* dst <- A . B.  dst is reshaped to B.Width() x A.Height() of A's type (its storage is
 * reallocated only when it has to grow).  Returns when the result is complete. */
_DECX_API_ void GEMM(GPU_Matrix& A, GPU_Matrix& B, GPU_Matrix& dst);
/* dst <- alpha . (A . B) + beta . C; alpha and beta must carry A's element type. */
_DECX_API_ void GEMM(GPU_Matrix& A, GPU_Matrix& B, GPU_Matrix& C, GPU_Matrix& dst,
                     const Number alpha, const Number beta);
/* Host-matrix forms: operands are staged through device memory around the same kernels. */
_DECX_API_ void GEMM(Matrix& A, Matrix& B, Matrix& dst);
_DECX_API_ void GEMM(Matrix& A, Matrix& B, Matrix& C, Matrix& dst);
/* Vector forms on host objects.  dst <- A . B with A a row vector of B.Height() elements
 * (result: B.Width() elements), or with B a column vector of A.Width() elements (result:
 * A.Height() elements).  For fp16 operands _fp16_accu (Fp16_Accuracy_Levels) selects an fp32
 * (level 1) or fp16 result.  dst keeps its storage when the result fits and is re-created
 * with the result's type and length otherwise. */
_DECX_API_ void GEMM(Vector& A, Matrix& B, Vector& dst, const uint32_t _fp16_accu = 0);
_DECX_API_ void GEMM(Matrix& A, Vector& B, Vector& dst, const uint32_t _fp16_accu = 0);
}  // namespace cuda
}  // namespace blas

/* ------------------------------------------------------------------ convolution on the product */
namespace nn {
namespace cuda {
/* dst(y, x, n) <- sum over kh, kw, c of src(y * strides.y + kh, x * strides.x + kw, c) * kernel_n(kh, kw, c)   (fp32).
 * _EXTEND_NONE_: dst is ((W - KW + 1) / strides.x) x ((H - KH + 1) / strides.y); _EXTEND_CONSTANT_: src is
 * zero-extended (KW / 2 columns on the left, KH / 2 rows on top) and dst is (W / strides.x) x (H / strides.y).
 * dst is reshaped to that size with depth = kernel.TensorNum().  Computed as one GEMM on the matrix cores whose
 * left operand is read straight out of the image (no im2col buffer). */
_DECX_API_ DH Conv2D(GPU_Tensor& src, GPU_TensorArray& kernel, GPU_Tensor& dst, const Point2D strides = {1, 1},
                     const extend_label extend = _EXTEND_NONE_);
}  // namespace cuda
}  // namespace nn

}  // namespace de

#endif  /* DECX_AMD_PUBLIC_H_ */
