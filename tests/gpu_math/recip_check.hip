// Test-only kernels (not part of the product library): the short forms of fp8bs_math.h against the
// operations they stand for, on the GPU, through the same header the kernels include.
//   gpu_math_recip_sweep   every float with bits in [lo_bits, hi_bits): recip_in_range(s) vs 1.0f / s
//   gpu_math_mean_sweep    div_by_count(a, n, RN(1/n)) vs a / n for n = 1 .. max_n and `per_n` values of a
// Both return a hipError_t and write the number of mismatches (and one example) to host memory.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../aiter_amd/csrc/fp8bs_math.h"

namespace
{

__global__ void recip_sweep_kernel(uint32_t lo, uint32_t hi, unsigned long long* bad, uint32_t* example)
{
    unsigned long long n = 0;
    for(uint64_t u = (uint64_t)lo + blockIdx.x * (uint64_t)blockDim.x + threadIdx.x; u < hi;
        u += (uint64_t)gridDim.x * blockDim.x)
    {
        const float s = __uint_as_float((uint32_t)u);
        if(__float_as_uint(fp8bs::recip_in_range(s)) != __float_as_uint(1.0f / s))
        {
            ++n;
            atomicMax(example, (uint32_t)u);
        }
        if(__float_as_uint(fp8bs::recip_in_range(-s)) != __float_as_uint(1.0f / -s))
        {
            ++n;
            atomicMax(example, (uint32_t)u | 0x80000000u);
        }
    }
    if(n)
        atomicAdd(bad, n);
}

__device__ uint64_t mix(uint64_t x)
{
    x ^= x >> 33;
    x *= 0xff51afd7ed558ccdull;
    x ^= x >> 33;
    x *= 0xc4ceb9fe1a85ec53ull;
    return x ^ (x >> 33);
}

__global__ void mean_sweep_kernel(uint32_t max_n, uint32_t per_n, unsigned long long* bad, uint32_t* example)
{
    unsigned long long wrong = 0;
    for(uint32_t n = 1 + blockIdx.x; n <= max_n; n += gridDim.x)
    {
        const double dn = (double)n, inv = 1.0 / dn;
        for(uint32_t i = threadIdx.x; i < per_n; i += blockDim.x)
        {
            // significands from a hash, exponents across the range a sum of squares of 16-bit floats spans,
            // and the special values
            const uint64_t h = mix(((uint64_t)n << 32) | i);
            double         a = __longlong_as_double((long long)((h & 0x000fffffffffffffull) | ((uint64_t)(1023 - 280 + (h >> 52) % 560) << 52)));
            if(i == 0)
                a = 0.0;
            if(i == 1)
                a = __longlong_as_double(0x7ff0000000000000ll);
            if(i == 2)
                a = dn; // exact quotient 1
            if(__double_as_longlong(fp8bs::div_by_count(a, dn, inv)) != __double_as_longlong(a / dn))
            {
                ++wrong;
                atomicMax(example, n);
            }
        }
    }
    if(wrong)
        atomicAdd(bad, wrong);
}

int run(void (*launch)(unsigned long long*, uint32_t*, const uint32_t*), const uint32_t* args,
        unsigned long long* mismatches, uint32_t* example)
{
    unsigned long long* d_bad = nullptr;
    uint32_t*           d_ex  = nullptr;
    hipError_t          e     = hipMalloc((void**)&d_bad, sizeof(*d_bad));
    if(e == hipSuccess)
        e = hipMalloc((void**)&d_ex, sizeof(*d_ex));
    if(e == hipSuccess)
        e = hipMemset(d_bad, 0, sizeof(*d_bad));
    if(e == hipSuccess)
        e = hipMemset(d_ex, 0, sizeof(*d_ex));
    if(e == hipSuccess)
    {
        launch(d_bad, d_ex, args);
        e = hipGetLastError();
    }
    if(e == hipSuccess)
        e = hipDeviceSynchronize();
    if(e == hipSuccess)
        e = hipMemcpy(mismatches, d_bad, sizeof(*d_bad), hipMemcpyDeviceToHost);
    if(e == hipSuccess)
        e = hipMemcpy(example, d_ex, sizeof(*d_ex), hipMemcpyDeviceToHost);
    (void)hipFree(d_bad);
    (void)hipFree(d_ex);
    return (int)e;
}

} // namespace

extern "C" {

int gpu_math_recip_sweep(uint32_t lo_bits, uint32_t hi_bits, unsigned long long* mismatches, uint32_t* example)
{
    const uint32_t args[2] = {lo_bits, hi_bits};
    return run([](unsigned long long* bad, uint32_t* ex, const uint32_t* a) {
        hipLaunchKernelGGL(recip_sweep_kernel, dim3(4096), dim3(256), 0, 0, a[0], a[1], bad, ex);
    }, args, mismatches, example);
}

int gpu_math_mean_sweep(uint32_t max_n, uint32_t per_n, unsigned long long* mismatches, uint32_t* example)
{
    const uint32_t args[2] = {max_n, per_n};
    return run([](unsigned long long* bad, uint32_t* ex, const uint32_t* a) {
        hipLaunchKernelGGL(mean_sweep_kernel, dim3(2048), dim3(256), 0, 0, a[0], a[1], bad, ex);
    }, args, mismatches, example);
}

uint32_t gpu_math_recip_min_bits() { return fp8bs::kRecipMinBits; }
uint32_t gpu_math_recip_max_bits() { return fp8bs::kRecipMaxBits; }

} // extern "C"
