// Conversions, host-side arithmetic for __half, and stream output of the 16-bit element types
// (names as in the reference's library/include/hiptensor/internal/types_ext.hpp:38-179).
#ifndef HIPTENSOR_TYPES_EXT_HPP
#define HIPTENSOR_TYPES_EXT_HPP

#include <cmath>
#include <ostream>

#include "type_traits.hpp"

namespace hiptensor
{
    // convert<To>(from): a static_cast, except that __half goes through _Float16 bit patterns when
    // HIP's implicit __half conversions are switched off
    template <typename To, typename From>
    HIPTENSOR_HOST_DEVICE inline To convert(const From& value)
    {
        if constexpr(std::is_same<To, From>::value)
            return value;
#if !HIPTENSOR_NO_HALF && defined(__HIP_NO_HALF_CONVERSIONS__)
        else if constexpr(std::is_same<To, hfloat16_t>::value)
            return detail::Fp16Bits(static_cast<float16_t>(value)).h16;
        else if constexpr(std::is_same<From, hfloat16_t>::value)
            return static_cast<To>(detail::Fp16Bits(value).f16);
#endif
        else
            return static_cast<To>(value);
    }

#if !HIPTENSOR_NO_HALF
// HIP defines the __half operators for device code only (for host and device when they are
// switched off altogether): supply what is missing, computed in _Float16.
#if defined(__HIP_NO_HALF_OPERATORS__)
#define HIPTENSOR_HALF_OP_ATTR HIPTENSOR_HOST_DEVICE
#else
#define HIPTENSOR_HALF_OP_ATTR HIPTENSOR_HOST
#endif
#define HIPTENSOR_HALF_BINARY(OP)                                                               \
    HIPTENSOR_HALF_OP_ATTR inline hfloat16_t operator OP(const hfloat16_t& a, const hfloat16_t& b) \
    {                                                                                           \
        return convert<hfloat16_t>(convert<float16_t>(a) OP convert<float16_t>(b));             \
    }                                                                                           \
    HIPTENSOR_HALF_OP_ATTR inline hfloat16_t& operator OP##=(hfloat16_t& a, const hfloat16_t& b) \
    {                                                                                           \
        a = a OP b;                                                                             \
        return a;                                                                               \
    }
    HIPTENSOR_HALF_BINARY(+)
    HIPTENSOR_HALF_BINARY(-)
    HIPTENSOR_HALF_BINARY(*)
    HIPTENSOR_HALF_BINARY(/)
#undef HIPTENSOR_HALF_BINARY

    HIPTENSOR_HALF_OP_ATTR inline hfloat16_t operator-(const hfloat16_t& a)
    {
        return detail::Fp16Bits(static_cast<uint16_t>(detail::Fp16Bits(a).i16 ^ 0x8000u)).h16;
    }
    // equality within two units of the last place (or below the smallest normal), as the reference's
    // test helpers expect of this operator
    HIPTENSOR_HALF_OP_ATTR inline bool operator==(const hfloat16_t& a, const hfloat16_t& b)
    {
        const float fa = __half2float(a), fb = __half2float(b);
        const float diff = std::fabs(fa - fb);
        return diff <= 2.0f * __half2float(std::numeric_limits<hfloat16_t>::epsilon()) * std::fabs(fa + fb)
               || diff < __half2float(std::numeric_limits<hfloat16_t>::min());
    }
    HIPTENSOR_HALF_OP_ATTR inline bool operator!=(const hfloat16_t& a, const hfloat16_t& b)
    {
        return !(a == b);
    }
#endif // !HIPTENSOR_NO_HALF
}

namespace std
{
// (internal/hiptensor_utility.hpp offers the same inserter: whichever header comes first defines it)
#ifndef HIPTENSOR_FLOAT16_INSERTER_DEFINED
#define HIPTENSOR_FLOAT16_INSERTER_DEFINED
    inline ostream& operator<<(ostream& os, const hiptensor::float16_t& v)
    {
        return os << static_cast<float>(v);
    }
#endif
#if !HIPTENSOR_NO_HALF
    inline ostream& operator<<(ostream& os, const hiptensor::hfloat16_t& v)
    {
        return os << __half2float(v);
    }
#endif
}

#endif // HIPTENSOR_TYPES_EXT_HPP
