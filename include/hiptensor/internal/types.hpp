// All element-type support headers at once (library/include/hiptensor/internal/types.hpp).
#ifndef HIPTENSOR_INTERNAL_TYPES_HPP
#define HIPTENSOR_INTERNAL_TYPES_HPP
#include "native_types.hpp"
#include "type_traits.hpp"
#include "types_ext.hpp"
#endif // HIPTENSOR_INTERNAL_TYPES_HPP
