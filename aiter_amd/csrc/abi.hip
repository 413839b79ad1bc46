// C-ABI entry points of libaiter_fp8bs.so: argument validation, error bridging and device
// selection.  All arithmetic lives in the kernel translation units.
//
// Contract mirrored from the reference's ctypes flavour: int status, thread-local message
// (csrc/include/aiter_ctypes_error.h:59-107), borrowed aiter_tensor_t descriptors
// (csrc/include/aiter_tensor.h:8-17), device guard around the launch
// (csrc/include/aiter_hip_common.h:538-552), work enqueued on the caller's stream.
#include "../../include/aiter_fp8bs.h"
#include "fp8bs_launch.h"
#include "moe_launch.h"

#include <cstdlib>
#include <cstring>
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
                                  int64_t splitK, const char* kernelName, aiter_stream_t stream,
                                  bool static_scratch = false, aiter_tensor_t* bias = nullptr)
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
        // csrc/ck_gemm_a8w8_blockscale/gemm_a8w8_blockscale.cu:82-114 takes 0..30 (KBatch = 1 << splitK)
        if(splitK < -1 || splitK > 30)
            fail(fn, "splitK = ", splitK, " outside -1..30");
        if(bias)
        {
            check_tensor(fn, bias, "bias");
            same_device(fn, {XQ, bias});
            if(bias->dtype_ != AITER_DTYPE_fp32 || (int64_t)bias->numel_ != N || !contiguous(bias))
                fail(fn, "bias must be a contiguous fp32 tensor of N = ", N, " elements, got ", bias->numel_, " of ",
                     dtype_name(bias->dtype_));
            if(N % 4 != 0)
                fail(fn, "a bias needs N % 4 == 0, got N = ", N);
            check_aligned(fn, bias, "bias", 16);
        }
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
        a.static_scratch = static_scratch;
        DeviceGuard guard(XQ->device_id);
        const char* why = nullptr;
        hipError_t  e   = fp8bs::launch_gemm_blockscale(a, (hipStream_t)stream, &why);
        check_hip(fn, e, why);
        if(bias)
            check_hip(fn, fp8bs::launch_gemm_bias_add(Out->ptr, a.out_dtype, (const float*)bias->ptr, M, N,
                                                      (hipStream_t)stream), nullptr);
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

int aiter_fp8bs_gemm_choice(int64_t M, int64_t N, int64_t K, int preshuffled, char* out, int64_t out_len)
{
    return guarded([&] {
        const char* fn = "aiter_fp8bs_gemm_choice";
        if(out == nullptr || out_len < 32)
            fail(fn, "out must hold at least 32 characters");
        if(M < 1 || N < 1 || K < 128 || K % 128 != 0 || M > 0x7fffffffLL / 2 || N > 0x7fffffffLL / 2 ||
           K > 0x7fffffffLL / 2)
            fail(fn, "M and N must be positive and K a positive multiple of 128, got ", M, " x ", N, " x ", K);
        fp8bs::gemm_describe_choice(M, N, K, preshuffled != 0, out, (size_t)out_len);
    });
}

int aiter_fp8bs_gemm_resolve(int64_t M, int64_t N, int64_t K, int preshuffled, int64_t splitK, const char* kernelName,
                             char* out, int64_t out_len)
{
    return guarded([&] {
        const char* fn = "aiter_fp8bs_gemm_resolve";
        if(out == nullptr || out_len < 64)
            fail(fn, "out must hold at least 64 characters");
        if(M < 1 || N < 1 || K < 128 || K % 128 != 0 || M > 0x7fffffffLL / 2 || N > 0x7fffffffLL / 2 ||
           K > 0x7fffffffLL / 2)
            fail(fn, "M and N must be positive and K a positive multiple of 128, got ", M, " x ", N, " x ", K);
        if(splitK < -1 || splitK > 30)
            fail(fn, "splitK = ", splitK, " outside -1..30");
        const char* why = nullptr;
        if(!fp8bs::gemm_describe_request(M, N, K, preshuffled != 0, (int)splitK, kernelName, out, (size_t)out_len, &why))
            fail(fn, why ? why : "cannot resolve the request");
    });
}

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

int gemm_a8w8_blockscale_noalloc(aiter_tensor_t* XQ, aiter_tensor_t* WQ, aiter_tensor_t* x_scale,
                                 aiter_tensor_t* w_scale, aiter_tensor_t* Out, int64_t splitK,
                                 const char* kernelName, aiter_stream_t stream)
{
    return gemm_blockscale_common("gemm_a8w8_blockscale_noalloc", false, XQ, WQ, x_scale, w_scale, Out, splitK,
                                  kernelName, stream, true);
}

int gemm_a8w8_blockscale_bpreshuffle(aiter_tensor_t* XQ, aiter_tensor_t* WQ, aiter_tensor_t* x_scale,
                                     aiter_tensor_t* w_scale, aiter_tensor_t* Out, const char* kernelName,
                                     aiter_stream_t stream)
{
    return gemm_blockscale_common("gemm_a8w8_blockscale_bpreshuffle", true, XQ, WQ, x_scale, w_scale, Out,
                                  -1, kernelName, stream);
}

int gemm_a8w8_blockscale_bpreshuffle_asm(aiter_tensor_t* A, aiter_tensor_t* B, aiter_tensor_t* out,
                                         aiter_tensor_t* A_scale, aiter_tensor_t* B_scale, aiter_tensor_t* bias,
                                         int splitK, const char* kernelName, int bpreshuffle,
                                         aiter_tensor_t* zero_bias_buf, aiter_stream_t stream)
{
    (void)zero_bias_buf; // the reference's kernel always reads a bias and wants zeros when there is none
    if(!bpreshuffle)
        return guarded([&] {
            fail("gemm_a8w8_blockscale_bpreshuffle_asm",
                 "bpreshuffle = 0 is not supported: row-major weights go through gemm_a8w8_blockscale");
        });
    // splitK and kernelName tune the reference's kernel: the name is foreign here and dropped with its split
    (void)splitK;
    (void)kernelName;
    return gemm_blockscale_common("gemm_a8w8_blockscale_bpreshuffle_asm", true, A, B, A_scale, B_scale, out, -1,
                                  nullptr, stream, false, bias);
}

// ---- mixture of experts -------------------------------------------------------------------

int topk_softmax(aiter_tensor_t* topk_weights, aiter_tensor_t* topk_indices,
                 aiter_tensor_t* token_expert_indices, aiter_tensor_t* gating_output, int need_renorm,
                 aiter_stream_t stream)
{
    return guarded([&] {
        const char* fn = "topk_softmax";
        check_tensor(fn, topk_weights, "topk_weights");
        check_tensor(fn, topk_indices, "topk_indices");
        check_tensor(fn, gating_output, "gating_output");
        if(token_expert_indices)
            check_tensor(fn, token_expert_indices, "token_expert_indices");
        same_device(fn, {topk_weights, topk_indices, token_expert_indices, gating_output});
        if(gating_output->ndim != 2 || !contiguous(gating_output))
            fail(fn, "gating_output must be a contiguous [tokens, experts] matrix");
        const int64_t tokens = gating_output->shape[0], experts = gating_output->shape[1];
        if(topk_weights->ndim != 2 || topk_indices->ndim != 2 || topk_weights->shape[0] != tokens ||
           topk_indices->shape[0] != tokens || topk_weights->shape[1] != topk_indices->shape[1])
            fail(fn, "topk_weights and topk_indices must both be [tokens, topk]");
        const int64_t topk = topk_weights->shape[1];
        if(experts < 1 || experts > 1024)
            fail(fn, "experts = ", experts, " outside 1..1024");
        if(topk < 1 || topk > 32 || topk > experts)
            fail(fn, "topk = ", topk, " outside 1..min(32, experts)");
        if(topk_weights->dtype_ != AITER_DTYPE_fp32 || topk_indices->dtype_ != AITER_DTYPE_i32)
            fail(fn, "topk_weights must be fp32 and topk_indices int32");
        if((topk > 1 && topk_weights->strides[1] != 1) || (topk > 1 && topk_indices->strides[1] != 1))
            fail(fn, "topk_weights and topk_indices must be contiguous in their last dimension");
        if(token_expert_indices &&
           (token_expert_indices->dtype_ != AITER_DTYPE_i32 || !contiguous(token_expert_indices) ||
            (int64_t)token_expert_indices->numel_ != tokens * topk))
            fail(fn, "token_expert_indices must be contiguous int32 [tokens, topk]");
        if(tokens >= (1LL << 24))
            fail(fn, "too many tokens");
        fp8bs::TopkSoftmaxArgs a{};
        a.gating = gating_output->ptr;
        switch(gating_output->dtype_)
        {
        case AITER_DTYPE_bf16: a.gating_dtype = 0; break;
        case AITER_DTYPE_fp16: a.gating_dtype = 1; break;
        case AITER_DTYPE_fp32: a.gating_dtype = 2; break;
        default: fail(fn, "gating_output must be bf16, fp16 or fp32, got ", dtype_name(gating_output->dtype_));
        }
        a.weights   = (float*)topk_weights->ptr;
        a.ids       = (int32_t*)topk_indices->ptr;
        a.src_rows  = token_expert_indices ? (int32_t*)token_expert_indices->ptr : nullptr;
        a.tokens    = (int32_t)tokens;
        a.experts   = (int32_t)experts;
        a.topk      = (int32_t)topk;
        a.w_stride  = tokens > 1 ? topk_weights->strides[0] : topk;
        a.id_stride = tokens > 1 ? topk_indices->strides[0] : topk;
        a.renorm    = need_renorm != 0;
        if(tokens == 0)
            return;
        DeviceGuard guard(gating_output->device_id);
        check_hip(fn, fp8bs::launch_topk_softmax(a, (hipStream_t)stream), nullptr);
    });
}

int moe_sorting_fwd(aiter_tensor_t* topk_ids, aiter_tensor_t* topk_weights, aiter_tensor_t* sorted_token_ids,
                    aiter_tensor_t* sorted_weights, aiter_tensor_t* sorted_expert_ids,
                    aiter_tensor_t* num_valid_ids, aiter_tensor_t* moe_buf, int64_t num_experts,
                    int64_t unit_size, aiter_tensor_t* local_expert_mask, aiter_tensor_t* num_local_tokens,
                    int64_t dispatch_policy, aiter_stream_t stream)
{
    return guarded([&] {
        const char* fn = "moe_sorting_fwd";
        check_tensor(fn, topk_ids, "topk_ids");
        check_tensor(fn, topk_weights, "topk_weights");
        check_tensor(fn, sorted_token_ids, "sorted_token_ids");
        check_tensor(fn, sorted_weights, "sorted_weights");
        check_tensor(fn, sorted_expert_ids, "sorted_expert_ids");
        check_tensor(fn, num_valid_ids, "num_valid_ids");
        if(moe_buf)
            check_tensor(fn, moe_buf, "moe_buf");
        if(local_expert_mask)
            check_tensor(fn, local_expert_mask, "local_expert_mask");
        if(num_local_tokens)
            check_tensor(fn, num_local_tokens, "num_local_tokens");
        same_device(fn, {topk_ids, topk_weights, sorted_token_ids, sorted_weights, sorted_expert_ids, num_valid_ids,
                         moe_buf, local_expert_mask, num_local_tokens});
        (void)dispatch_policy; // a tuning hint of the reference's kernels
        // with num_local_tokens the ids may carry more rows than are in use, and than the weights have
        // (op_tests/test_moe_sorting.py:180-187)
        if(topk_ids->ndim != 2 || topk_weights->ndim != 2 || topk_ids->shape[1] != topk_weights->shape[1] ||
           (num_local_tokens ? topk_weights->shape[0] > topk_ids->shape[0]
                             : topk_weights->shape[0] != topk_ids->shape[0]))
            fail(fn, "topk_ids and topk_weights must both be [tokens, topk] (topk_weights may have fewer rows when "
                     "num_local_tokens is given)");
        const int64_t M = topk_ids->shape[0], topk = topk_ids->shape[1];
        if(topk_ids->dtype_ != AITER_DTYPE_i32 || topk_weights->dtype_ != AITER_DTYPE_fp32)
            fail(fn, "topk_ids must be int32 and topk_weights fp32");
        if((topk > 1 && topk_ids->strides[1] != 1) || (topk > 1 && topk_weights->strides[1] != 1))
            fail(fn, "topk_ids and topk_weights must be contiguous in their last dimension");
        if(num_experts < 1 || num_experts > 1024)
            fail(fn, "num_experts = ", num_experts, " outside 1..1024");
        if(unit_size < 1 || unit_size > 1024)
            fail(fn, "unit_size = ", unit_size, " outside 1..1024");
        if(topk < 1 || topk > 255)
            fail(fn, "topk = ", topk, " outside 1..255 (the sorted ids keep the slot in 8 bits)");
        if(M >= (1LL << 24))
            fail(fn, "tokens = ", M, " do not fit the 24 bits the sorted ids keep for them");
        const int64_t max_padded = M * topk + num_experts * unit_size - topk;
        const int64_t max_blocks = (max_padded + unit_size - 1) / unit_size;
        if(sorted_token_ids->dtype_ != AITER_DTYPE_i32 || !contiguous(sorted_token_ids) ||
           (int64_t)sorted_token_ids->numel_ < max_padded)
            fail(fn, "sorted_token_ids must be contiguous int32 with at least ", max_padded, " elements");
        if(sorted_weights->dtype_ != AITER_DTYPE_fp32 || !contiguous(sorted_weights) ||
           (int64_t)sorted_weights->numel_ < max_padded)
            fail(fn, "sorted_weights must be contiguous fp32 with at least ", max_padded, " elements");
        if(sorted_expert_ids->dtype_ != AITER_DTYPE_i32 || !contiguous(sorted_expert_ids) ||
           (int64_t)sorted_expert_ids->numel_ < max_blocks)
            fail(fn, "sorted_expert_ids must be contiguous int32 with at least ", max_blocks, " elements");
        if(num_valid_ids->dtype_ != AITER_DTYPE_i32 || num_valid_ids->numel_ < 2 || !contiguous(num_valid_ids))
            fail(fn, "num_valid_ids must be contiguous int32 with 2 elements");
        if(local_expert_mask && (local_expert_mask->dtype_ != AITER_DTYPE_i32 || !contiguous(local_expert_mask) ||
                                 (int64_t)local_expert_mask->numel_ != num_experts))
            fail(fn, "local_expert_mask must be contiguous int32 [num_experts]");
        if(num_local_tokens && (num_local_tokens->dtype_ != AITER_DTYPE_i32 || num_local_tokens->numel_ < 1))
            fail(fn, "num_local_tokens must be an int32 scalar on the device");
        size_t buf_bytes = 0;
        if(moe_buf && moe_buf->numel_)
        {
            if(!contiguous(moe_buf))
                fail(fn, "moe_buf must be contiguous");
            buf_bytes = moe_buf->numel_ * dtype_size(moe_buf->dtype_);
            if(buf_bytes % 16 != 0)
                fail(fn, "moe_buf must span a multiple of 16 bytes");
            check_aligned(fn, moe_buf, "moe_buf", 16);
        }
        fp8bs::MoeSortArgs a{};
        a.topk_ids          = (const int32_t*)topk_ids->ptr;
        a.topk_weights      = (const float*)topk_weights->ptr;
        a.expert_mask       = local_expert_mask ? (const int32_t*)local_expert_mask->ptr : nullptr;
        a.num_local_tokens  = num_local_tokens ? (const int32_t*)num_local_tokens->ptr : nullptr;
        a.sorted_ids        = (int32_t*)sorted_token_ids->ptr;
        a.sorted_weights    = (float*)sorted_weights->ptr;
        a.sorted_expert_ids = (int32_t*)sorted_expert_ids->ptr;
        a.num_valid_ids     = (int32_t*)num_valid_ids->ptr;
        a.moe_buf           = buf_bytes ? moe_buf->ptr : nullptr;
        a.moe_buf_bytes     = buf_bytes;
        a.M                 = (int32_t)M;
        a.w_rows            = (int32_t)topk_weights->shape[0];
        a.topk              = (int32_t)topk;
        a.experts           = (int32_t)num_experts;
        a.unit              = (int32_t)unit_size;
        a.max_padded        = (int32_t)max_padded;
        a.max_blocks        = (int32_t)max_blocks;
        a.id_stride         = M > 1 ? topk_ids->strides[0] : topk;
        a.w_stride          = topk_weights->shape[0] > 1 ? topk_weights->strides[0] : topk;
        a.device_id         = topk_ids->device_id;
        if(max_padded >= (1LL << 31))
            fail(fn, "problem too large");
        DeviceGuard guard(topk_ids->device_id);
        const char* why = nullptr;
        hipError_t  e   = fp8bs::launch_moe_sorting(a, (hipStream_t)stream, &why);
        check_hip(fn, e, why);
    });
}

int fmoe_fp8_blockscale_g1u1(aiter_tensor_t* out, aiter_tensor_t* input, aiter_tensor_t* gate, aiter_tensor_t* down,
                             aiter_tensor_t* sorted_token_ids, aiter_tensor_t* sorted_weights,
                             aiter_tensor_t* sorted_expert_ids, aiter_tensor_t* num_valid_ids, int64_t topk,
                             aiter_tensor_t* input_scale, aiter_tensor_t* fc1_scale, aiter_tensor_t* fc2_scale,
                             const char* kernel_name, int64_t fc_scale_blkn, int64_t fc_scale_blkk,
                             aiter_tensor_t* fc2_smooth_scale, int64_t activation, int64_t block_size_M,
                             aiter_stream_t stream)
{
    return guarded([&] {
        const char* fn = "fmoe_fp8_blockscale_g1u1";
        check_tensor(fn, out, "out");
        check_tensor(fn, input, "input");
        check_tensor(fn, gate, "gate");
        check_tensor(fn, down, "down");
        check_tensor(fn, sorted_token_ids, "sorted_token_ids");
        check_tensor(fn, sorted_weights, "sorted_weights");
        check_tensor(fn, sorted_expert_ids, "sorted_expert_ids");
        check_tensor(fn, num_valid_ids, "num_valid_ids");
        check_tensor(fn, fc1_scale, "fc1_scale");
        check_tensor(fn, fc2_scale, "fc2_scale");
        if(input_scale)
            check_tensor(fn, input_scale, "input_scale");
        same_device(fn, {out, input, gate, down, sorted_token_ids, sorted_weights, sorted_expert_ids, num_valid_ids,
                         input_scale, fc1_scale, fc2_scale});
        if(fc2_smooth_scale)
            fail(fn, "fc2_smooth_scale is not supported");
        if(fc_scale_blkn != 128 || fc_scale_blkk != 128)
            fail(fn, "only 128 x 128 weight scale blocks are supported, got ", fc_scale_blkn, " x ", fc_scale_blkk);
        // the block size the arrays were sorted with (the reference's kernels exist for 16, 32 and 64:
        // hsa/gfx950/fmoe/silu/fmoe_bf16_blockscaleFp8_g1u1_silu.csv, column subGU_m)
        if(block_size_M != 16 && block_size_M != 32 && block_size_M != 64 && block_size_M != 128)
            fail(fn, "block_size_M must be 16, 32, 64 or 128, got ", block_size_M);
        if(activation != 0 && activation != 1)
            fail(fn, "activation must be 0 (silu) or 1 (gelu), got ", activation);
        if(!is_f16_like(out->dtype_))
            fail(fn, "out must be bf16 or fp16, got ", dtype_name(out->dtype_));
        if(input->ndim != 2 || out->ndim != 2 || gate->ndim != 3 || down->ndim != 3)
            fail(fn, "input/out must be 2-D [tokens, dim], gate/down 3-D [experts, n, k]");
        const int64_t M = input->shape[0], dim = input->shape[1];
        const int64_t E = gate->shape[0], inter = down->shape[2];
        if(out->shape[0] != M || out->shape[1] != dim)
            fail(fn, "out must be [", M, ",", dim, "]");
        if(gate->shape[1] != 2 * inter || gate->shape[2] != dim)
            fail(fn, "gate must be [experts, 2*inter_dim, dim] = [", E, ",", 2 * inter, ",", dim, "] (gate then up rows)");
        if(down->shape[0] != E || down->shape[1] != dim)
            fail(fn, "down must be [", E, ",", dim, ",", inter, "]");
        if(!is_fp8_like(gate->dtype_) || !is_fp8_like(down->dtype_))
            fail(fn, "gate and down must be fp8");
        if(!contiguous(gate) || !contiguous(down))
            fail(fn, "gate and down must be contiguous (pre-shuffled with layout (16,16))");
        if(dim % 128 != 0 || inter % 128 != 0 || dim < 128 || inter < 128)
            fail(fn, "dim = ", dim, " and inter_dim = ", inter, " must be positive multiples of 128");
        if(dim % 256 != 0)
            fail(fn, "dim = ", dim, " must be a multiple of 256");
        if(topk < 1 || topk > 255)
            fail(fn, "topk = ", topk, " outside 1..255");
        if(M >= (1LL << 24) || E > 1024 || E < 1)
            fail(fn, "tokens or experts out of range");
        const int64_t kb1 = dim / 128, kb2 = inter / 128;
        if(fc1_scale->dtype_ != AITER_DTYPE_fp32 || !contiguous(fc1_scale) ||
           (int64_t)fc1_scale->numel_ != E * (2 * inter / 128) * kb1)
            fail(fn, "fc1_scale must be contiguous fp32 with experts * (2*inter_dim/128) * (dim/128) = ",
                 E * (2 * inter / 128) * kb1, " elements, got ", fc1_scale->numel_);
        if(fc2_scale->dtype_ != AITER_DTYPE_fp32 || !contiguous(fc2_scale) ||
           (int64_t)fc2_scale->numel_ != E * (dim / 128) * kb2)
            fail(fn, "fc2_scale must be contiguous fp32 with experts * (dim/128) * (inter_dim/128) = ",
                 E * (dim / 128) * kb2, " elements, got ", fc2_scale->numel_);
        if(sorted_token_ids->dtype_ != AITER_DTYPE_i32 || sorted_expert_ids->dtype_ != AITER_DTYPE_i32 ||
           num_valid_ids->dtype_ != AITER_DTYPE_i32 || sorted_weights->dtype_ != AITER_DTYPE_fp32)
            fail(fn, "sorted_token_ids / sorted_expert_ids / num_valid_ids must be int32, sorted_weights fp32");
        if(!contiguous(sorted_token_ids) || !contiguous(sorted_expert_ids) || !contiguous(sorted_weights) ||
           num_valid_ids->numel_ < 1)
            fail(fn, "the sorted arrays must be contiguous");
        const int64_t unit       = block_size_M;
        const int64_t block_rows = unit < 32 ? unit : 32; // rows of the blocks the kernels walk
        const int64_t max_blocks = (int64_t)sorted_expert_ids->numel_;
        const int64_t max_padded = max_blocks * unit;
        if((int64_t)sorted_token_ids->numel_ < max_padded - (unit - 1) ||
           (int64_t)sorted_weights->numel_ < max_padded - (unit - 1))
            fail(fn, "sorted_token_ids and sorted_weights must cover the ", max_blocks,
                 " blocks of sorted_expert_ids");
        // the kernels read whole blocks: the last block may only be addressed if it is backed
        const int64_t backed = (int64_t)sorted_token_ids->numel_ < (int64_t)sorted_weights->numel_
                                   ? (int64_t)sorted_token_ids->numel_
                                   : (int64_t)sorted_weights->numel_;
        const int64_t use_sorted = backed / unit < max_blocks ? backed / unit : max_blocks;
        const int64_t use_blocks = use_sorted * (unit / block_rows);
        if(max_padded >= (1LL << 31) || max_padded * dim >= (1LL << 40))
            fail(fn, "problem too large");

        fp8bs::MoeArgs a{};
        if(is_fp8_like(input->dtype_))
        {
            if(!input_scale)
                fail(fn, "fp8 input needs input_scale");
            if(input_scale->dtype_ != AITER_DTYPE_fp32 || !contiguous(input_scale) ||
               (int64_t)input_scale->numel_ != M * kb1)
                fail(fn, "input_scale must be contiguous fp32 [dim/128, tokens] = [", kb1, ",", M, "]");
            if(input_scale->ndim == 2 && M > 1 && kb1 > 1 &&
               !(input_scale->shape[0] == kb1 && input_scale->shape[1] == M))
                fail(fn, "input_scale must be laid out [dim/128, tokens] (the transposed scale of the 1x128 quant)");
            if(dim > 1 && input->strides[1] != 1)
                fail(fn, "input must be contiguous in its last dimension");
            a.lda = M > 1 ? input->strides[0] : dim;
            if(a.lda < dim || a.lda % 16 != 0)
                fail(fn, "input row stride must be >= dim and a multiple of 16");
            check_aligned(fn, input, "input", 16);
            a.xq = (const uint8_t*)input->ptr;
            a.xs = (const float*)input_scale->ptr;
        }
        else if(is_f16_like(input->dtype_))
        {
            if(!contiguous(input))
                fail(fn, "16-bit input must be contiguous");
            check_aligned(fn, input, "input", 16);
            a.x16       = input->ptr;
            a.x16_dtype = in16_of(input->dtype_);
            a.lda       = dim;
        }
        else
            fail(fn, "input must be fp8 (with input_scale) or bf16/fp16, got ", dtype_name(input->dtype_));
        if(dim > 1 && out->strides[1] != 1)
            fail(fn, "out must be contiguous in its last dimension");
        a.out_stride = M > 1 ? out->strides[0] : dim;
        if(a.out_stride < dim || a.out_stride % 4 != 0)
            fail(fn, "out row stride must be >= dim and a multiple of 4");
        check_aligned(fn, out, "out", 8);
        check_aligned(fn, gate, "gate", 16);
        check_aligned(fn, down, "down", 16);
        a.w1                = (const uint8_t*)gate->ptr;
        a.w1_scale          = (const float*)fc1_scale->ptr;
        a.w2                = (const uint8_t*)down->ptr;
        a.w2_scale          = (const float*)fc2_scale->ptr;
        a.sorted_ids        = (const int32_t*)sorted_token_ids->ptr;
        a.sorted_weights    = (const float*)sorted_weights->ptr;
        a.sorted_expert_ids = (const int32_t*)sorted_expert_ids->ptr;
        a.num_valid         = (const int32_t*)num_valid_ids->ptr;
        a.out               = out->ptr;
        a.out_dtype         = in16_of(out->dtype_);
        a.M                 = (int32_t)M;
        a.dim               = (int32_t)dim;
        a.inter             = (int32_t)inter;
        a.experts           = (int32_t)E;
        a.topk              = (int32_t)topk;
        a.max_blocks        = (int32_t)use_blocks;
        a.max_padded        = (int32_t)(use_blocks * block_rows);
        a.block_rows        = (int32_t)block_rows;
        a.expert_shift      = unit == 128 ? 2 : unit == 64 ? 1 : 0;
        a.activation        = (int32_t)activation;
        // the reference's names pick among its tuned kernels; here "nt=1|2|4" pins the first GEMM's
        // columns per workgroup, "dw=" / "dc=" / "down=rows" pick the second GEMM that writes rows
        // (and its shape), "down=cols" the one that sums per token in LDS, "pair=0|1" whether consecutive
        // blocks of one expert are multiplied in pairs, "tail=0" keeps the first GEMM's last blocks as wide as the rest, "stage=0" stores the second GEMM's 16-bit rows straight from the lanes instead of through LDS, "ring=0" has the first GEMM's pairs of blocks request and wait for every K block in turn instead of keeping the weights two K blocks ahead; several hints are joined by commas; anything else
        // means choose
        a.gate_tiles     = 0;
        a.down_waves     = 0;
        a.down_wave_cols = 0;
        a.down_mode      = 0;
        a.pair_blocks    = -1;
        a.fine_tail      = -1;
        a.down_staged    = -1;
        a.gate_ring      = -1;
        for(const char* hint = kernel_name; hint && *hint;)
        {
            const char*  end = strchr(hint, ',');
            const size_t len = end ? (size_t)(end - hint) : strlen(hint);
            auto         is  = [&](const char* word) { return len == strlen(word) && strncmp(hint, word, len) == 0; };
            if(len > 3 && strncmp(hint, "nt=", 3) == 0)
                a.gate_tiles = atoi(hint + 3);
            else if(len > 3 && strncmp(hint, "dw=", 3) == 0)
            {
                a.down_waves = atoi(hint + 3);
                a.down_mode  = 1; // these hints are about the kernel that writes rows
            }
            else if(len > 3 && strncmp(hint, "dc=", 3) == 0)
            {
                a.down_wave_cols = 64;
                a.down_waves     = atoi(hint + 3);
                a.down_mode      = 1;
            }
            else if(is("down=rows"))
                a.down_mode = 1;
            else if(is("down=cols"))
                a.down_mode = 2;
            else if(len > 5 && strncmp(hint, "pair=", 5) == 0)
                a.pair_blocks = atoi(hint + 5) != 0 ? 1 : 0;
            else if(is("tail=0"))
                a.fine_tail = 0;
            else if(is("stage=0"))
                a.down_staged = 0;
            else if(is("ring=0"))
                a.gate_ring = 0;
            hint = end ? end + 1 : nullptr;
        }
        a.device_id         = input->device_id;
        if(M == 0)
            return; // nothing to do, and no device needed to say so
        DeviceGuard guard(input->device_id);
        const char* why = nullptr;
        hipError_t  e   = fp8bs::launch_fmoe_blockscale(a, (hipStream_t)stream, &why);
        check_hip(fn, e, why);
    });
}

} // extern "C"
