// C-ABI entry points of libaiter_fp8bs.so: argument validation, error bridging and device
// selection.  All arithmetic lives in the kernel translation units.
//
// Contract mirrored from the reference's ctypes flavour: int status, thread-local message
// (csrc/include/aiter_ctypes_error.h:59-107), borrowed aiter_tensor_t descriptors
// (csrc/include/aiter_tensor.h:8-17), device guard around the launch
// (csrc/include/aiter_hip_common.h:538-552), work enqueued on the caller's stream.
#include "../../include/aiter_fp8bs.h"
#include "fp8bs_launch.h"

#include <exception>
#include <sstream>
#include <stdexcept>
#include <string>

static_assert(sizeof(aiter_tensor_t) == 160, "aiter_tensor_t must stay 160 bytes");

namespace {

thread_local std::string g_last_error;

struct ArgError : std::runtime_error
{
    using std::runtime_error::runtime_error;
};

template <typename... Ts>
[[noreturn]] void fail(const char* fn, Ts&&... parts)
{
    std::ostringstream os;
    os << fn << ": ";
    (os << ... << parts);
    throw ArgError(os.str());
}

#define FP8BS_CHECK(cond, ...)          \
    do                                  \
    {                                   \
        if(!(cond))                     \
            fail(__func__, __VA_ARGS__); \
    } while(0)

const char* dtype_name(int d)
{
    static const char* names[] = {"fp8", "fp8_e8m0", "fp16", "bf16", "fp32", "i4x2", "fp4x2",
                                  "u32", "i32", "i16", "i8", "u8", "i64", "u64"};
    return (d >= 0 && d < 14) ? names[d] : "unknown";
}

size_t dtype_size(int d)
{
    switch(d)
    {
    case AITER_DTYPE_fp8:
    case AITER_DTYPE_fp8_e8m0:
    case AITER_DTYPE_i4x2:
    case AITER_DTYPE_fp4x2:
    case AITER_DTYPE_i8:
    case AITER_DTYPE_u8: return 1;
    case AITER_DTYPE_fp16:
    case AITER_DTYPE_bf16:
    case AITER_DTYPE_i16: return 2;
    case AITER_DTYPE_fp32:
    case AITER_DTYPE_u32:
    case AITER_DTYPE_i32: return 4;
    case AITER_DTYPE_i64:
    case AITER_DTYPE_u64: return 8;
    default: return 0;
    }
}

// fp8 payloads may arrive typed as fp8 or as raw bytes (torch.uint8 views are common)
bool is_fp8_like(int d) { return d == AITER_DTYPE_fp8 || d == AITER_DTYPE_u8 || d == AITER_DTYPE_i8; }
bool is_f16_like(int d) { return d == AITER_DTYPE_bf16 || d == AITER_DTYPE_fp16; }

bool contiguous(const aiter_tensor_t* t)
{
    if(t->numel_ == 0)
        return true;
    int64_t expect = 1;
    for(int d = t->ndim - 1; d >= 0; --d)
    {
        if(t->shape[d] != 1 && t->strides[d] != expect)
            return false;
        expect *= t->shape[d];
    }
    return true;
}

void check_tensor(const char* fn, const aiter_tensor_t* t, const char* name)
{
    if(t == nullptr)
        fail(fn, name, " must not be null");
    if(t->ndim < 0 || t->ndim > 8)
        fail(fn, name, ".ndim ", t->ndim, " outside 0..8");
    size_t n = 1;
    for(int d = 0; d < t->ndim; ++d)
    {
        if(t->shape[d] < 0)
            fail(fn, name, " has a negative extent");
        n *= (size_t)t->shape[d];
    }
    if(n != t->numel_)
        fail(fn, name, ".numel ", t->numel_, " does not match its shape (", n, ")");
    if(dtype_size(t->dtype_) == 0)
        fail(fn, name, " has unknown dtype code ", t->dtype_);
    if(t->numel_ != 0 && t->ptr == nullptr)
        fail(fn, name, " has a null data pointer");
    if(t->numel_ != 0 && t->device_id < 0)
        fail(fn, name, " must live in GPU memory (device_id ", t->device_id, ")");
}

void check_aligned(const char* fn, const aiter_tensor_t* t, const char* name, size_t bytes)
{
    if(t->numel_ != 0 && ((uintptr_t)t->ptr % bytes) != 0)
        fail(fn, name, " must be ", bytes, "-byte aligned");
}

void same_device(const char* fn, std::initializer_list<const aiter_tensor_t*> ts)
{
    int dev = -2;
    for(const aiter_tensor_t* t : ts)
    {
        if(t == nullptr || t->numel_ == 0)
            continue;
        if(dev == -2)
            dev = t->device_id;
        else if(t->device_id != dev)
            fail(fn, "tensors live on different devices (", dev, " and ", t->device_id, ")");
    }
}

int64_t rows_of(const aiter_tensor_t* t)
{
    int64_t last = t->shape[t->ndim - 1];
    return last == 0 ? 0 : (int64_t)(t->numel_ / (size_t)last);
}

// all leading dims must collapse onto one row stride, last dim unit stride
int64_t row_stride_2d(const char* fn, const aiter_tensor_t* t, const char* name)
{
    if(t->ndim < 1)
        fail(fn, name, " must have at least one dimension");
    int last = t->ndim - 1;
    if(t->shape[last] > 1 && t->strides[last] != 1)
        fail(fn, name, " must be contiguous in its last dimension");
    if(t->ndim == 1)
        return t->shape[0];
    int64_t stride = t->strides[last - 1];
    int64_t expect = stride;
    for(int d = last - 1; d >= 0; --d)
    {
        if(t->shape[d] != 1 && t->strides[d] != expect)
            fail(fn, name, " has leading dimensions that do not collapse to one row stride");
        expect *= t->shape[d];
    }
    return stride;
}

struct DeviceGuard
{
    int  prev  = -1;
    bool moved = false;
    explicit DeviceGuard(int dev)
    {
        if(dev < 0)
            return;
        if(hipGetDevice(&prev) != hipSuccess)
            throw std::runtime_error("hipGetDevice failed (no usable HIP device?)");
        if(prev != dev)
        {
            hipError_t e = hipSetDevice(dev);
            if(e != hipSuccess)
                throw std::runtime_error(std::string("hipSetDevice failed: ") + hipGetErrorString(e));
            moved = true;
        }
    }
    ~DeviceGuard()
    {
        if(moved)
            (void)hipSetDevice(prev);
    }
};

void check_hip(const char* fn, hipError_t e, const char* extra = nullptr)
{
    if(e == hipSuccess)
        return;
    std::string msg = std::string(fn) + ": HIP error: " + hipGetErrorString(e);
    if(extra)
        msg += std::string(" (") + extra + ")";
    throw std::runtime_error(msg);
}

template <typename F>
int guarded(F&& body)
{
    g_last_error.clear();
    try
    {
        body();
        return 0;
    }
    catch(const std::exception& e)
    {
        g_last_error = e.what();
    }
    catch(...)
    {
        g_last_error = "unknown C++ exception";
    }
    return -1;
}

fp8bs::In16 in16_of(int d) { return d == AITER_DTYPE_bf16 ? fp8bs::In16::bf16 : fp8bs::In16::fp16; }

void rmsnorm_common(const char* fn, aiter_tensor_t* out, aiter_tensor_t* input,
                    aiter_tensor_t* residual_in, aiter_tensor_t* residual_out,
                    aiter_tensor_t* scale, aiter_tensor_t* weight, float epsilon, int64_t group_size,
                    int shuffle_scale, int gemma_norm, bool quant, bool add, hipStream_t stream)
{
    check_tensor(fn, out, "out");
    check_tensor(fn, input, "input");
    check_tensor(fn, weight, "weight");
    if(quant)
        check_tensor(fn, scale, "scale");
    if(add)
    {
        check_tensor(fn, residual_in, "residual_in");
        check_tensor(fn, residual_out, "residual_out");
    }
    same_device(fn, {out, input, weight, scale, residual_in, residual_out});
    if(!is_f16_like(input->dtype_))
        fail(fn, "input must be bf16 or fp16, got ", dtype_name(input->dtype_));
    if(weight->dtype_ != input->dtype_)
        fail(fn, "weight dtype ", dtype_name(weight->dtype_), " must match input dtype ",
             dtype_name(input->dtype_));
    if(input->ndim < 1)
        fail(fn, "input must have at least one dimension");
    const int64_t hidden = input->shape[input->ndim - 1];
    const int64_t rows   = rows_of(input);
    if(weight->numel_ != (size_t)hidden || !contiguous(weight))
        fail(fn, "weight must be a contiguous vector of ", hidden, " elements");
    if(hidden <= 0 || hidden > 8192)
        fail(fn, "hidden size ", hidden, " outside 1..8192");
    if(hidden % 8 != 0)
        fail(fn, "hidden size ", hidden, " must be a multiple of 8");
    if(out->numel_ != input->numel_ || out->shape[out->ndim - 1] != hidden)
        fail(fn, "out shape must match input shape");

    fp8bs::NormArgs a{};
    a.x        = input->ptr;
    a.x_stride = row_stride_2d(fn, input, "input");
    a.weight   = weight->ptr;
    a.rows     = rows;
    a.hidden   = (int32_t)hidden;
    a.eps      = epsilon;
    a.gemma_norm = gemma_norm != 0;
    a.dtype    = in16_of(input->dtype_);
    check_aligned(fn, input, "input", 16);
    check_aligned(fn, weight, "weight", 16);
    check_aligned(fn, out, "out", 16);
    if(a.x_stride % 8 != 0)
        fail(fn, "input row stride must be a multiple of 8 elements");
    if(add)
    {
        if(residual_in->dtype_ != input->dtype_ || residual_out->dtype_ != input->dtype_)
            fail(fn, "residual tensors must have the input dtype");
        if(residual_in->numel_ != input->numel_ || residual_out->numel_ != input->numel_)
            fail(fn, "residual tensors must have the input shape");
        a.residual_in    = residual_in->ptr;
        a.residual_out   = residual_out->ptr;
        a.res_in_stride  = row_stride_2d(fn, residual_in, "residual_in");
        a.res_out_stride = row_stride_2d(fn, residual_out, "residual_out");
        check_aligned(fn, residual_in, "residual_in", 16);
        check_aligned(fn, residual_out, "residual_out", 16);
        if(a.res_in_stride % 8 != 0 || a.res_out_stride % 8 != 0)
            fail(fn, "residual row strides must be multiples of 8 elements");
    }
    if(quant)
    {
        if(group_size != 32 && group_size != 64 && group_size != 128)
            fail(fn, "group_size ", group_size,
                 " is not supported: this library implements the grouped path only (32, 64, 128)");
        if(hidden % group_size != 0)
            fail(fn, "hidden size ", hidden, " is not a multiple of group_size ", group_size);
        if(!is_fp8_like(out->dtype_))
            fail(fn, "out must be fp8, got ", dtype_name(out->dtype_));
        if(!contiguous(out))
            fail(fn, "out must be contiguous");
        if(scale->dtype_ != AITER_DTYPE_fp32)
            fail(fn, "scale must be fp32, got ", dtype_name(scale->dtype_));
        if(scale->numel_ != (size_t)(rows * (hidden / group_size)) || !contiguous(scale))
            fail(fn, "scale must be contiguous with rows*hidden/group_size = ",
                 rows * (hidden / group_size), " elements, got ", scale->numel_);
        a.out8            = (uint8_t*)out->ptr;
        a.out_stride      = hidden;
        a.scale           = (float*)scale->ptr;
        a.group           = (int32_t)group_size;
        a.transpose_scale = shuffle_scale != 0;
    }
    else
    {
        if(out->dtype_ != input->dtype_)
            fail(fn, "out dtype must match input dtype");
        a.out16      = out->ptr;
        a.out_stride = row_stride_2d(fn, out, "out");
        if(a.out_stride % 8 != 0)
            fail(fn, "out row stride must be a multiple of 8 elements");
    }
    if(rows == 0)
        return;
    if(rows > 0x7fffffffLL)
        fail(fn, "too many rows");
    DeviceGuard guard(input->device_id);
    check_hip(fn, fp8bs::launch_rmsnorm(a, stream));
}

} // namespace

static int gemm_blockscale_common(const char* fn, bool preshuffled, aiter_tensor_t* XQ, aiter_tensor_t* WQ,
                                  aiter_tensor_t* x_scale, aiter_tensor_t* w_scale, aiter_tensor_t* Out,
                                  int64_t splitK, const char* kernelName, aiter_stream_t stream)
{
    return guarded([&] {
        check_tensor(fn, XQ, "XQ");
        check_tensor(fn, WQ, "WQ");
        check_tensor(fn, x_scale, "x_scale");
        check_tensor(fn, w_scale, "w_scale");
        check_tensor(fn, Out, "Out");
        same_device(fn, {XQ, WQ, x_scale, w_scale, Out});
        // csrc/ck_gemm_a8w8_blockscale/gemm_a8w8_blockscale.cu:90-97
        if(!is_fp8_like(XQ->dtype_) || !is_fp8_like(WQ->dtype_))
            fail(fn, "XQ and WQ must be fp8, got ", dtype_name(XQ->dtype_), " and ",
                 dtype_name(WQ->dtype_));
        if(XQ->dtype_ != WQ->dtype_)
            fail(fn, "Weights and activations should have the same dtype!");
        if(x_scale->dtype_ != w_scale->dtype_)
            fail(fn, "Scales should have the same dtype!");
        if(x_scale->dtype_ != AITER_DTYPE_fp32)
            fail(fn, "scales must be fp32, got ", dtype_name(x_scale->dtype_));
        if(!is_f16_like(Out->dtype_))
            fail(fn, "Out must be bf16 or fp16, got ", dtype_name(Out->dtype_));
        if(XQ->ndim != 2 || WQ->ndim != 2 || Out->ndim != 2)
            fail(fn, "XQ, WQ and Out must be 2-D");
        const int64_t M = XQ->shape[0], K = XQ->shape[1], N = WQ->shape[0];
        if(WQ->shape[1] != K)
            fail(fn, "XQ is [", M, ",", K, "] but WQ is [", N, ",", WQ->shape[1], "]");
        if(K % 128 != 0)
            fail(fn, "K = ", K, " must be a multiple of the 128-wide scale block");
        if(Out->shape[0] != M || Out->shape[1] != N || !contiguous(Out))
            fail(fn, "Out must be a contiguous [", M, ",", N, "] tensor");
        const int64_t kb = K / 128, nb = (N + 127) / 128;
        if(!preshuffled)
        {
            if((int64_t)x_scale->numel_ != M * kb || !contiguous(x_scale))
                fail(fn, "x_scale must be contiguous [", M, ",", kb, "], got ", x_scale->numel_,
                     " elements");
        }
        else
        {
            // The pre-shuffled kernels read x_scale as [K/128][M] (column-major); callers pass
            // either that buffer viewed as a contiguous [M, K/128] tensor or an [M, K/128] view
            // with strides (1, M) (op_tests/test_gemm_a8w8_blockscale.py:112-125).  Both put
            // element (m, kb) at kb * M + m.
            const bool as_view = x_scale->ndim == 2 && x_scale->shape[0] == M && x_scale->shape[1] == kb &&
                                 (M <= 1 || x_scale->strides[0] == 1) && (kb <= 1 || x_scale->strides[1] == M);
            if((int64_t)x_scale->numel_ != M * kb || !(contiguous(x_scale) || as_view))
                fail(fn, "x_scale must hold M*K/128 = ", M * kb,
                     " column-major values (contiguous buffer, or [M,K/128] view with strides (1,M))");
            if(N % 16 != 0)
                fail(fn, "pre-shuffled weights need N % 16 == 0, got N = ", N);
            if(N > 1 && WQ->strides[0] != K)
                fail(fn, "pre-shuffled weights must be a contiguous [N, K] buffer");
        }
        if((int64_t)w_scale->numel_ != nb * kb || !contiguous(w_scale))
            fail(fn, "w_scale must be contiguous [", nb, ",", kb, "], got ", w_scale->numel_,
                 " elements");
        if((K > 1 && XQ->strides[1] != 1) || (K > 1 && WQ->strides[1] != 1))
            fail(fn, "XQ and WQ must be contiguous in K");
        const int64_t lda = M > 1 ? XQ->strides[0] : K, ldb = N > 1 ? WQ->strides[0] : K;
        if(lda < K || ldb < K || lda % 16 != 0 || ldb % 16 != 0)
            fail(fn, "row strides of XQ/WQ must be >= K and multiples of 16 bytes");
        check_aligned(fn, XQ, "XQ", 16);
        check_aligned(fn, WQ, "WQ", 16);
        check_aligned(fn, Out, "Out", 8);
        check_aligned(fn, x_scale, "x_scale", 4);
        check_aligned(fn, w_scale, "w_scale", 4);
        if(M > 0x7fffffffLL / 2 || N > 0x7fffffffLL / 2 || K > 0x7fffffffLL / 2)
            fail(fn, "problem too large");
        if(splitK < -1 || splitK > 4)
            fail(fn, "splitK = ", splitK, " outside -1..4");
        if(M == 0 || N == 0)
            return;

        fp8bs::GemmArgs a{};
        a.xq           = (const uint8_t*)XQ->ptr;
        a.wq           = (const uint8_t*)WQ->ptr;
        a.xs           = (const float*)x_scale->ptr;
        a.ws           = (const float*)w_scale->ptr;
        a.out          = Out->ptr;
        a.M            = M;
        a.N            = N;
        a.K            = K;
        a.lda          = lda;
        a.ldb          = ldb;
        a.out_dtype    = in16_of(Out->dtype_);
        a.split_k_log2 = (int)splitK;
        a.kernel_name  = kernelName;
        a.device_id    = XQ->device_id;
        a.w_shuffled   = preshuffled;
        a.xs_col_major = preshuffled;
        DeviceGuard guard(XQ->device_id);
        const char* why = nullptr;
        hipError_t  e   = fp8bs::launch_gemm_blockscale(a, (hipStream_t)stream, &why);
        check_hip(fn, e, why);
    });
}

extern "C" {

int aiter_ctypes_abi_version(void) { return 2; }

const char* aiter_get_last_error(void)
{
    return g_last_error.empty() ? nullptr : g_last_error.c_str();
}

void aiter_clear_last_error(void) { g_last_error.clear(); }

const char* aiter_fp8bs_gemm_kernel_names(void) { return fp8bs::gemm_kernel_names(); }

int dynamic_per_token_scaled_quant(aiter_tensor_t* out, aiter_tensor_t* input,
                                   aiter_tensor_t* scales, aiter_tensor_t* scale_ub,
                                   int shuffle_scale, aiter_tensor_t* num_rows,
                                   int64_t num_rows_factor, aiter_stream_t stream)
{
    return guarded([&] {
        const char* fn = "dynamic_per_token_scaled_quant";
        check_tensor(fn, out, "out");
        check_tensor(fn, input, "input");
        check_tensor(fn, scales, "scales");
        if(scale_ub != nullptr)
            fail(fn, "scale_ub is not supported by the group quant path");
        if(num_rows != nullptr)
        {
            check_tensor(fn, num_rows, "num_rows");
            if(num_rows->dtype_ != AITER_DTYPE_i32 || num_rows->numel_ < 1)
                fail(fn, "num_rows must be an int32 device scalar");
        }
        same_device(fn, {out, input, scales, num_rows});
        if(!contiguous(input) || !contiguous(out))
            fail(fn, "input and out must be contiguous");
        if(!is_f16_like(input->dtype_))
            fail(fn, "input must be bf16 or fp16, got ", dtype_name(input->dtype_));
        if(!is_fp8_like(out->dtype_))
            fail(fn, "out must be fp8, got ", dtype_name(out->dtype_),
                 " (only the fp8 group quant is implemented)");
        if(input->ndim < 1 || out->ndim < 1)
            fail(fn, "input and out must have at least one dimension");
        const int64_t group = input->shape[input->ndim - 1];
        if(group != 32 && group != 64 && group != 128)
            fail(fn, "input must be viewed as [-1, group] with group in {32, 64, 128}; got last "
                     "dimension ",
                 group, " (per-token quant over whole rows is not part of this library)");
        if(out->numel_ != input->numel_)
            fail(fn, "out and input must hold the same number of elements");
        const int64_t K = out->shape[out->ndim - 1];
        if(K <= 0 || K % group != 0)
            fail(fn, "out last dimension ", K, " is not a multiple of the group size ", group);
        const int64_t n_groups = (int64_t)(input->numel_ / (size_t)group);
        const int64_t rows     = (int64_t)(out->numel_ / (size_t)K);
        if(scales->dtype_ != AITER_DTYPE_fp32)
            fail(fn, "scales must be fp32, got ", dtype_name(scales->dtype_),
                 " (e8m0 scales are not part of this library)");
        if((int64_t)scales->numel_ != n_groups || !contiguous(scales))
            fail(fn, "scales must be contiguous with one element per group (", n_groups, "), got ",
                 scales->numel_);
        if(n_groups >= (1LL << 31))
            fail(fn, "too many groups (", n_groups, ")");
        if(num_rows_factor < 0 || num_rows_factor > 0x7fffffffLL)
            fail(fn, "num_rows_factor out of range");
        check_aligned(fn, input, "input", 16);
        check_aligned(fn, out, "out", 16);
        check_aligned(fn, scales, "scales", 4);

        fp8bs::QuantArgs a{};
        a.x               = input->ptr;
        a.y               = (uint8_t*)out->ptr;
        a.scale           = (float*)scales->ptr;
        a.rows            = rows;
        a.groups_per_row  = (int32_t)(K / group);
        a.group           = (int32_t)group;
        a.transpose_scale = shuffle_scale != 0;
        a.num_rows        = num_rows ? (const int32_t*)num_rows->ptr : nullptr;
        a.num_rows_factor = (int32_t)num_rows_factor;
        a.dtype           = in16_of(input->dtype_);
        if(n_groups == 0)
            return;
        DeviceGuard guard(input->device_id);
        check_hip(fn, fp8bs::launch_group_quant(a, (hipStream_t)stream));
    });
}

int rmsnorm(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* weight, float epsilon,
            int gemma_norm, aiter_stream_t stream)
{
    return guarded([&] {
        rmsnorm_common("rmsnorm", out, input, nullptr, nullptr, nullptr, weight, epsilon, 0, 0,
                       gemma_norm, false, false, (hipStream_t)stream);
    });
}

int rmsnorm_quant(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* scale,
                  aiter_tensor_t* weight, float epsilon, int64_t group_size, int shuffle_scale,
                  int gemma_norm, aiter_stream_t stream)
{
    return guarded([&] {
        rmsnorm_common("rmsnorm_quant", out, input, nullptr, nullptr, scale, weight, epsilon,
                       group_size, shuffle_scale, gemma_norm, true, false, (hipStream_t)stream);
    });
}

int add_rmsnorm(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* residual_in,
                aiter_tensor_t* residual_out, aiter_tensor_t* weight, float epsilon,
                int gemma_norm, aiter_stream_t stream)
{
    return guarded([&] {
        rmsnorm_common("add_rmsnorm", out, input, residual_in, residual_out, nullptr, weight,
                       epsilon, 0, 0, gemma_norm, false, true, (hipStream_t)stream);
    });
}

int add_rmsnorm_quant(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* residual_in,
                      aiter_tensor_t* residual_out, aiter_tensor_t* scale,
                      aiter_tensor_t* weight, float epsilon, int64_t group_size,
                      int shuffle_scale, int gemma_norm, aiter_stream_t stream)
{
    return guarded([&] {
        rmsnorm_common("add_rmsnorm_quant", out, input, residual_in, residual_out, scale, weight,
                       epsilon, group_size, shuffle_scale, gemma_norm, true, true,
                       (hipStream_t)stream);
    });
}

int weight_per_128x128_quant(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* scales,
                             aiter_stream_t stream)
{
    return guarded([&] {
        const char* fn = "weight_per_128x128_quant";
        check_tensor(fn, out, "out");
        check_tensor(fn, input, "input");
        check_tensor(fn, scales, "scales");
        same_device(fn, {out, input, scales});
        if(!is_f16_like(input->dtype_))
            fail(fn, "input must be bf16 or fp16, got ", dtype_name(input->dtype_));
        if(!is_fp8_like(out->dtype_))
            fail(fn, "out must be fp8, got ", dtype_name(out->dtype_));
        if(scales->dtype_ != AITER_DTYPE_fp32)
            fail(fn, "scales must be fp32, got ", dtype_name(scales->dtype_));
        if(input->ndim != 2 || out->ndim != 2)
            fail(fn, "input and out must be 2-D [N, K]");
        const int64_t N = input->shape[0], K = input->shape[1];
        if(out->shape[0] != N || out->shape[1] != K)
            fail(fn, "out must have the shape of input, [", N, ",", K, "]");
        if(K % 128 != 0)
            fail(fn, "K = ", K, " must be a multiple of 128");
        if((K > 1 && input->strides[1] != 1) || (K > 1 && out->strides[1] != 1))
            fail(fn, "input and out must be contiguous in K");
        const int64_t ldw = N > 1 ? input->strides[0] : K, ldq = N > 1 ? out->strides[0] : K;
        if(ldw < K || ldq < K || ldw % 8 != 0 || ldq % 16 != 0)
            fail(fn, "row strides must be >= K and multiples of 16 bytes");
        const int64_t nb = (N + 127) / 128, kb = K / 128;
        if((int64_t)scales->numel_ != nb * kb || !contiguous(scales))
            fail(fn, "scales must be contiguous [", nb, ",", kb, "], got ", scales->numel_, " elements");
        if(N >= (1LL << 31) || K >= (1LL << 31) || nb > 65535)
            fail(fn, "matrix too large");
        check_aligned(fn, input, "input", 16);
        check_aligned(fn, out, "out", 16);
        check_aligned(fn, scales, "scales", 4);
        fp8bs::WeightQuantArgs a{};
        a.w     = input->ptr;
        a.q     = (uint8_t*)out->ptr;
        a.scale = (float*)scales->ptr;
        a.N     = N;
        a.K     = K;
        a.ldw   = ldw;
        a.ldq   = ldq;
        a.dtype = in16_of(input->dtype_);
        DeviceGuard guard(input->device_id);
        check_hip(fn, fp8bs::launch_weight_block_quant(a, (hipStream_t)stream), nullptr);
    });
}

int gemm_a8w8_blockscale(aiter_tensor_t* XQ, aiter_tensor_t* WQ, aiter_tensor_t* x_scale,
                         aiter_tensor_t* w_scale, aiter_tensor_t* Out, int64_t splitK,
                         const char* kernelName, aiter_stream_t stream)
{
    return gemm_blockscale_common("gemm_a8w8_blockscale", false, XQ, WQ, x_scale, w_scale, Out, splitK,
                                  kernelName, stream);
}

int gemm_a8w8_blockscale_bpreshuffle(aiter_tensor_t* XQ, aiter_tensor_t* WQ, aiter_tensor_t* x_scale,
                                     aiter_tensor_t* w_scale, aiter_tensor_t* Out, const char* kernelName,
                                     aiter_stream_t stream)
{
    return gemm_blockscale_common("gemm_a8w8_blockscale_bpreshuffle", true, XQ, WQ, x_scale, w_scale, Out,
                                  -1, kernelName, stream);
}

} // extern "C"
