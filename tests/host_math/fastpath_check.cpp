// Host-side exhaustive check of the quantiser's fast division path.  Compiles the SAME header
// the HIP kernels use (aiter_amd/csrc/fp8bs_math.h) with g++ and compares, for 16-bit-float
// inputs, the FMA-based division against IEEE division, and the software e4m3fn conversion
// against the oracle's.
//
//   fastpath_check <mode>
//     bf16  every bf16 amax in the fast range x every bf16 |x| <= amax  (sampled exponents: all
//           128 significands of amax at each of a set of exponents, all x codes)
//     fp16  every fp16 amax x every fp16 |x| <= amax
//     scale amax / 448 by multiplication and correction vs the IEEE division, every bf16 and fp16 amax
//     mean  sum / row length by multiplication and correction vs the fp64 division, row lengths 1 .. 16384
//     cvt   software conversion vs oracle on structured fp32 inputs
// Prints "OK <count>" or the first mismatches and exits non-zero.
#include "../../aiter_amd/csrc/fp8bs_math.h"
#include "../../oracle/fp8bs_oracle.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>

static float bf16f(uint16_t h) { return fp8bs::bits_f32((uint32_t)h << 16); }

static long check_pair(float x, float amax, long& bad)
{
    float s = amax / 448.0f;
    float r = 1.0f / s;
    long  n = 0;
    for(int sign = 0; sign < 2; ++sign)
    {
        float xv   = sign ? -x : x;
        float want = xv / s;
        float got  = fp8bs::div_by_scale(xv, s, r);
        ++n;
        // requirement: identical fp8 code always, and the identical fp32 quotient wherever it
        // is large enough to reach the fp8 grid (|q| >= 2^-12)
        uint8_t cw = oracle_f32_to_e4m3fn(want), cg = oracle_f32_to_e4m3fn(got);
        bool    q_differs = fp8bs::f32_bits(want) != fp8bs::f32_bits(got);
        if(cw != cg || (q_differs && (want >= 0x1p-12f || want <= -0x1p-12f)))
        {
            if(bad < 10)
                fprintf(stderr, "x=%a amax=%a want=%a got=%a codes %02x %02x\n", xv, amax, want, got, cw, cg);
            ++bad;
        }
    }
    return n;
}

int main(int argc, char** argv)
{
    const char* mode = argc > 1 ? argv[1] : "bf16";
    long        n = 0, bad = 0;
    if(strcmp(mode, "bf16") == 0)
    {
        // exponents of amax: edges of the fast range, around 1, and where quotients hit the
        // fp8 subnormal range for small x
        const int exps[] = {-80, -79, -64, -1, 0, 1, 8, 63, 99, 100};
        for(int e : exps)
            for(int m = 0; m < 128; ++m)
            {
                if(e == 100 && m != 0)
                    continue; // 2^100 itself is the last admissible amax
                uint16_t acode = (uint16_t)(((e + 127) << 7) | m);
                float    amax  = bf16f(acode);
                if(!fp8bs::amax_allows_fast_path(fp8bs::f32_bits(amax)))
                {
                    fprintf(stderr, "amax %a unexpectedly outside the fast range\n", amax);
                    return 2;
                }
                for(uint32_t xc = 0; xc <= acode; ++xc) // every bf16 magnitude up to amax, subnormals too
                    n += check_pair(bf16f((uint16_t)xc), amax, bad);
            }
    }
    else if(strcmp(mode, "fp16") == 0)
    {
        for(uint32_t ac = 1; ac < 0x7c00; ++ac)
        {
            float amax = oracle_f16_to_f32((uint16_t)ac);
            if(!fp8bs::amax_allows_fast_path(fp8bs::f32_bits(amax)))
            {
                fprintf(stderr, "fp16 amax %a outside the fast range\n", amax);
                return 2;
            }
            // all x would be 5e8 pairs; take every x that shares the top or is within 2^-13 of amax,
            // plus a stride over the rest
            uint32_t step = ac > 4096 ? 7 : 1;
            for(uint32_t xc = 0; xc <= ac; xc += step)
                n += check_pair(oracle_f16_to_f32((uint16_t)xc), amax, bad);
            n += check_pair(amax, amax, bad);
        }
    }
    else if(strcmp(mode, "scale") == 0)
    {
        // amax / 448 without the division: every bf16 and every fp16 amax inside the fast range
        for(int kind = 0; kind < 2; ++kind)
            for(uint32_t ac = 1; ac < (kind == 0 ? 0x7f80u : 0x7c00u); ++ac)
            {
                const float amax = kind == 0 ? bf16f((uint16_t)ac) : oracle_f16_to_f32((uint16_t)ac);
                if(!fp8bs::amax_allows_fast_path(fp8bs::f32_bits(amax)))
                    continue;
                const float want = amax / 448.0f, got = fp8bs::amax_over_448(amax);
                ++n;
                if(fp8bs::f32_bits(want) != fp8bs::f32_bits(got))
                {
                    if(bad < 10)
                        fprintf(stderr, "amax=%a want=%a got=%a\n", amax, want, got);
                    ++bad;
                }
            }
    }
    else if(strcmp(mode, "mean") == 0)
    {
        // sum of squares / row length: significands from a hash over the exponents such sums span, plus 0,
        // inf and the exact quotient 1
        for(uint32_t len = 1; len <= 16384; ++len)
        {
            const double dn = (double)len, inv = 1.0 / dn;
            for(uint32_t i = 0; i < 256; ++i)
            {
                uint64_t h = ((uint64_t)len << 32) | i;
                h ^= h >> 33; h *= 0xff51afd7ed558ccdull; h ^= h >> 33; h *= 0xc4ceb9fe1a85ec53ull; h ^= h >> 33;
                const uint64_t bits = (h & 0x000fffffffffffffull) | ((uint64_t)(1023 - 280 + (h >> 52) % 560) << 52);
                double a;
                memcpy(&a, &bits, 8);
                if(i == 0) a = 0.0;
                if(i == 1) a = __builtin_inf();
                if(i == 2) a = dn;
                const double want = a / dn, got = fp8bs::div_by_count(a, dn, inv);
                ++n;
                if(memcmp(&want, &got, 8) != 0)
                {
                    if(bad < 10)
                        fprintf(stderr, "a=%a len=%u want=%a got=%a\n", a, len, want, got);
                    ++bad;
                }
            }
        }
    }
    else if(strcmp(mode, "cvt") == 0)
    {
        for(uint64_t hi = 0; hi < (1u << 20); ++hi)
        {
            const uint32_t lows[] = {0x000, 0x001, 0x7ff, 0x800, 0x801, 0xfff};
            for(uint32_t lo : lows)
            {
                float   f = fp8bs::bits_f32((uint32_t)(hi << 12) | lo);
                uint8_t a = fp8bs::f32_to_e4m3fn_sw(f), b = oracle_f32_to_e4m3fn(f);
                ++n;
                if(a != b)
                {
                    if(bad < 10)
                        fprintf(stderr, "cvt %a: sw %02x oracle %02x\n", f, a, b);
                    ++bad;
                }
            }
        }
    }
    else
    {
        fprintf(stderr, "unknown mode %s\n", mode);
        return 2;
    }
    if(bad)
    {
        printf("FAIL %ld of %ld\n", bad, n);
        return 1;
    }
    printf("OK %ld\n", n);
    return 0;
}
