// Element type names used by applications written against the reference's headers
// (library/include/hiptensor/internal/native_types.hpp:40-85).
#ifndef HIPTENSOR_NATIVE_TYPES_HPP
#define HIPTENSOR_NATIVE_TYPES_HPP

#include <cstdint>

#include <hip/hip_bfloat16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_vector_types.h>

#include "config.hpp"

namespace hiptensor
{
    // types the compiler computes with directly
    typedef _Float16 float16_t;
    typedef float    float32_t;
    typedef double   float64_t;
    using ::int8_t;
    using ::int16_t;
    using ::int32_t;
    using ::int64_t;
    using ::uint8_t;
    using ::uint16_t;
    using ::uint32_t;
    using ::uint64_t;
    typedef ::int32_t index_t;
    typedef ::int64_t index64_t;

    // types that come as classes from the HIP headers
    typedef hip_bfloat16 bfloat16_t;
#if !HIPTENSOR_NO_HALF
    typedef __half hfloat16_t;
#endif
}

#include "native_types_impl.hpp"

#endif // HIPTENSOR_NATIVE_TYPES_HPP
