// Build configuration macros of the public headers.  Same macro names as the reference's
// library/include/hiptensor/internal/config.hpp:32-102; this library's device code exists for
// gfx950 only, so that is the one architecture symbol that can be non-zero in a device pass.
#ifndef HIPTENSOR_CONFIG_HPP
#define HIPTENSOR_CONFIG_HPP

// ---- architecture of the current compilation pass ----
#if defined(__gfx950__)
#define HIPTENSOR_ARCH_GFX950 __gfx950__
#define HIPTENSOR_ARCH_HOST 0
#elif defined(__HIP_DEVICE_COMPILE__) && __HIP_DEVICE_COMPILE__
#define HIPTENSOR_ARCH_GFX950 0
#define HIPTENSOR_ARCH_HOST 0
#else
#define HIPTENSOR_ARCH_GFX950 0
#define HIPTENSOR_ARCH_HOST 1
#endif
// the architectures the reference names: never the target of this library
#define HIPTENSOR_ARCH_GFX908 0
#define HIPTENSOR_ARCH_GFX90A 0
#define HIPTENSOR_ARCH_GFX940 0
#define HIPTENSOR_ARCH_GFX941 0
#define HIPTENSOR_ARCH_GFX942 0

// ---- function attributes ----
#define HIPTENSOR_HOST __host__
#define HIPTENSOR_DEVICE __device__
#define HIPTENSOR_HOST_DEVICE __host__ __device__
#define HIPTENSOR_KERNEL __global__

// marks an entry point that exists for source compatibility but has no implementation here
#ifdef NDEBUG
#define HIPTENSOR_UNSUPPORTED_IMPL(MSG)
#else
#define HIPTENSOR_UNSUPPORTED_IMPL(MSG) __attribute__((deprecated(MSG)))
#endif

// ---- __half availability (HIP's own switches) ----
#ifdef HIP_NO_HALF
#define HIPTENSOR_NO_HALF 1
#else
#define HIPTENSOR_NO_HALF 0
#endif
#if HIPTENSOR_NO_HALF || defined(__HIP_NO_HALF_CONVERSIONS__)
#define HIPTENSOR_TESTS_NO_HALF 1
#else
#define HIPTENSOR_TESTS_NO_HALF 0
#endif

#endif // HIPTENSOR_CONFIG_HPP
