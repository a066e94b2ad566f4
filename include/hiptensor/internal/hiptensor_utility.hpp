// Convenience macros and printers that programs written against hipTensor 1.4 pick
// up through <hiptensor/hiptensor.hpp> (library/include/hiptensor/internal/
// hiptensor_utility.hpp:37-159).  Names and behaviour match; the bodies are this
// library's own.
#ifndef HIPTENSOR_UTILITY_INTERNAL_HPP
#define HIPTENSOR_UTILITY_INTERNAL_HPP

#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <string>
#include <vector>

#include <hip/hip_bfloat16.h>
#include <hip/hip_complex.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include "../hiptensor_types.hpp"

const char* hiptensorGetErrorString(const hiptensorStatus_t error);

namespace hiptensor_detail
{
    [[noreturn]] inline void die(const char* what, const char* text, int code, const char* file, int line)
    {
        std::fprintf(stderr, "%s error: '%s'(%d) at %s:%d\n", what, text, code, file, line);
        std::exit(EXIT_FAILURE);
    }
}

// Abort the process on a failed HIP call (reference: hiptensor_utility.hpp:37-49).
#ifndef CHECK_HIP_ERROR
#define CHECK_HIP_ERROR(expression)                                                              \
    do                                                                                           \
    {                                                                                            \
        hipError_t hiptensor_chk_ = (expression);                                                \
        if(hiptensor_chk_ != hipSuccess)                                                         \
            hiptensor_detail::die(                                                               \
                "hip", hipGetErrorString(hiptensor_chk_), (int)hiptensor_chk_, __FILE__, __LINE__); \
    } while(0)
#endif

// Abort the process on a failed hipTensor call (reference: hiptensor_utility.hpp:51-63).
#ifndef CHECK_HIPTENSOR_ERROR
#define CHECK_HIPTENSOR_ERROR(expression)                                                 \
    do                                                                                    \
    {                                                                                     \
        hiptensorStatus_t hiptensor_chk_ = (expression);                                  \
        if(hiptensor_chk_ != HIPTENSOR_STATUS_SUCCESS)                                    \
            hiptensor_detail::die("hipTensor",                                            \
                                  hiptensorGetErrorString(hiptensor_chk_),                \
                                  (int)hiptensor_chk_,                                    \
                                  __FILE__,                                               \
                                  __LINE__);                                              \
    } while(0)
#endif

// Half-precision values print as float (the stream has no inserter of its own for them).
// (internal/types_ext.hpp offers the same inserter: whichever header comes first defines it)
#if defined(__FLT16_MANT_DIG__) && !defined(HIPTENSOR_FLOAT16_INSERTER_DEFINED)
#define HIPTENSOR_FLOAT16_INSERTER_DEFINED
namespace std
{
    inline ostream& operator<<(ostream& os, const _Float16& v)
    {
        return os << static_cast<float>(v);
    }
}
#endif

// "re + imi" / "re-imi" formatting of complex scalars.
inline std::ostream& operator<<(std::ostream& os, const hipFloatComplex& z)
{
    os << hipCrealf(z);
    if(hipCimagf(z) >= 0)
        os << " + ";
    return os << hipCimagf(z) << "i";
}

inline std::ostream& operator<<(std::ostream& os, const hipDoubleComplex& z)
{
    os << hipCreal(z);
    if(hipCimag(z) >= 0)
        os << " + ";
    return os << hipCimag(z) << "i";
}

// Comma-separated dump of an array to a stream.
template <typename T>
void hiptensorPrintArrayElements(std::ostream& stream, T* vec, size_t size)
{
    for(size_t i = 0; i < size; ++i)
        stream << vec[i] << (i + 1 < size ? ", " : "");
}

// Separator-joined dump of a vector to stdout.
template <typename S>
void hiptensorPrintVectorElements(const std::vector<S>& vec, std::string sep = " ")
{
    for(size_t i = 0; i < vec.size(); ++i)
        std::cout << vec[i] << (i + 1 < vec.size() ? sep : std::string());
}

// Separator-joined dump of an array to an open file.
template <typename F>
void hiptensorPrintElementsToFile(std::ofstream& fs, F* output, size_t size, std::string sep = " ")
{
    if(!fs.is_open())
    {
        std::cout << "File not found!\n";
        return;
    }
    for(size_t i = 0; i < size; ++i)
        fs << static_cast<F>(output[i]) << (i + 1 < size ? sep : std::string());
}

inline bool operator==(const hiptensorTensorDescriptor_t& a, const hiptensorTensorDescriptor_t& b)
{
    return a.mType == b.mType && a.mUnaryOp == b.mUnaryOp && a.mLengths == b.mLengths
           && a.mStrides == b.mStrides;
}

inline bool operator!=(const hiptensorTensorDescriptor_t& a, const hiptensorTensorDescriptor_t& b)
{
    return !(a == b);
}

// "dim N, lengths {..}, strides {..}" (reference: hiptensor_utility.hpp:140-157).
inline std::ostream& operator<<(std::ostream& os, const hiptensorTensorDescriptor_t& desc)
{
    os << "dim " << desc.mLengths.size() << ", lengths {";
    for(size_t i = 0; i < desc.mLengths.size(); ++i)
        os << desc.mLengths[i] << (i + 1 < desc.mLengths.size() ? ", " : "");
    os << "}, strides {";
    for(size_t i = 0; i < desc.mStrides.size(); ++i)
        os << desc.mStrides[i] << (i + 1 < desc.mStrides.size() ? ", " : "");
    return os << "}";
}

#endif // HIPTENSOR_UTILITY_INTERNAL_HPP
