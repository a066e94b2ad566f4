// std::numeric_limits for the 16-bit element types, bit-level views of them, and the largest
// integer each type counts exactly.  Same names as the reference's
// library/include/hiptensor/internal/type_traits.hpp:34-318.
#ifndef HIPTENSOR_TYPE_TRAITS_HPP
#define HIPTENSOR_TYPE_TRAITS_HPP

#include <limits>
#include <type_traits>

#include "native_types.hpp"

namespace hiptensor
{
    namespace detail
    {
        // one 16-bit pattern seen as any of the 16-bit element types
        union Fp16Bits
        {
            uint16_t   i16;
            float16_t  f16;
            bfloat16_t b16;
#if !HIPTENSOR_NO_HALF
            hfloat16_t h16;
#endif
            constexpr Fp16Bits(uint16_t bits)
                : i16(bits)
            {
            }
            constexpr Fp16Bits(float16_t v)
                : f16(v)
            {
            }
            constexpr Fp16Bits(bfloat16_t v)
                : b16(v)
            {
            }
#if !HIPTENSOR_NO_HALF
            constexpr Fp16Bits(hfloat16_t v)
                : h16(v)
            {
            }
#endif
        };

        union Fp32Bits
        {
            uint32_t  i32;
            float32_t f32;
            constexpr Fp32Bits(uint32_t bits)
                : i32(bits)
            {
            }
            constexpr Fp32Bits(float32_t v)
                : f32(v)
            {
            }
        };

        // IEEE-754 layouts: binary16 has 10 stored mantissa bits, bfloat16 has 7
        struct HalfPatterns
        {
            static constexpr uint16_t kEpsilon = 0x1400, kInf = 0x7C00, kLowest = 0xFBFF, kMax = 0x7BFF, kMin = 0x0400,
                                      kQnan = 0x7FFF, kSnan = 0x7DFF;
        };
        struct BFloatPatterns
        {
            static constexpr uint16_t kEpsilon = 0x3C00, kInf = 0x7F80, kLowest = 0xFF7F, kMax = 0x7F7F, kMin = 0x0080,
                                      kQnan = 0x7FC0, kSnan = 0x7FA0;
        };
    }
}

namespace std
{
#define HIPTENSOR_LIMIT(TYPE, FIELD, PAT, NAME, VALUE)                              \
    template <>                                                                     \
    HIPTENSOR_HOST_DEVICE constexpr TYPE numeric_limits<TYPE>::NAME() noexcept      \
    {                                                                               \
        return hiptensor::detail::Fp16Bits(static_cast<uint16_t>(hiptensor::detail::PAT::VALUE)).FIELD; \
    }
#define HIPTENSOR_LIMITS_OF(TYPE, FIELD, PAT)             \
    HIPTENSOR_LIMIT(TYPE, FIELD, PAT, epsilon, kEpsilon)   \
    HIPTENSOR_LIMIT(TYPE, FIELD, PAT, infinity, kInf)      \
    HIPTENSOR_LIMIT(TYPE, FIELD, PAT, lowest, kLowest)     \
    HIPTENSOR_LIMIT(TYPE, FIELD, PAT, max, kMax)           \
    HIPTENSOR_LIMIT(TYPE, FIELD, PAT, min, kMin)           \
    HIPTENSOR_LIMIT(TYPE, FIELD, PAT, quiet_NaN, kQnan)    \
    HIPTENSOR_LIMIT(TYPE, FIELD, PAT, signaling_NaN, kSnan)

    HIPTENSOR_LIMITS_OF(hiptensor::float16_t, f16, HalfPatterns)
#if !HIPTENSOR_NO_HALF
    HIPTENSOR_LIMITS_OF(hiptensor::hfloat16_t, h16, HalfPatterns)
#endif
    HIPTENSOR_LIMITS_OF(hiptensor::bfloat16_t, b16, BFloatPatterns)

#undef HIPTENSOR_LIMITS_OF
#undef HIPTENSOR_LIMIT
}

namespace hiptensor
{
    // The largest integer n such that every integer in [0, n] is a value of T: all of an integer
    // type's range, 2^(mantissa bits + 1) for a floating-point type.
    template <typename T>
    constexpr auto maxExactInteger()
    {
        if constexpr(std::is_integral<T>::value)
            return std::numeric_limits<T>::max();
        else if constexpr(std::is_same<T, float64_t>::value)
            return static_cast<int64_t>(1ll << std::numeric_limits<float64_t>::digits);
        else if constexpr(std::is_same<T, float32_t>::value)
            return static_cast<int32_t>(1 << std::numeric_limits<float32_t>::digits);
        else if constexpr(std::is_same<T, bfloat16_t>::value)
            return static_cast<int32_t>(1 << 8); // 7 stored + 1 implied bit
        else
            return static_cast<int32_t>(1 << 11); // binary16: 10 stored + 1 implied bit
    }
}

#endif // HIPTENSOR_TYPE_TRAITS_HPP
