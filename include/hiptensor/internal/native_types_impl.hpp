// Kept for source compatibility with library/include/hiptensor/internal/native_types_impl.hpp:
// the element types need no out-of-line definitions here.
#ifndef HIPTENSOR_NATIVE_TYPES_IMPL_HPP
#define HIPTENSOR_NATIVE_TYPES_IMPL_HPP
#include "native_types.hpp"
#endif // HIPTENSOR_NATIVE_TYPES_IMPL_HPP
