// Host-only check of <hiptensor/internal/*.hpp>: the headers compile together with the public
// header and their constants and operators hold the values their names promise.
#include <hiptensor/internal/types.hpp>
#include <hiptensor/internal/config.hpp>
#include <hiptensor/hiptensor.hpp>
#include <iostream>
#include <sstream>
int main()
{
    using namespace hiptensor;
    static_assert(maxExactInteger<float32_t>() == (1 << 24), "");
    static_assert(maxExactInteger<float16_t>() == 2048, "");
    static_assert(maxExactInteger<bfloat16_t>() == 256, "");
    static_assert(maxExactInteger<int32_t>() == 2147483647, "");
    static_assert(maxExactInteger<float64_t>() == (1ll << 53), "");
    int bad = 0;
    bad += (float)std::numeric_limits<float16_t>::max() != 65504.f;
    bad += (float)std::numeric_limits<float16_t>::epsilon() != 0.0009765625f;
    bad += (float)std::numeric_limits<float16_t>::min() != 6.103515625e-05f;
    bad += (float)std::numeric_limits<float16_t>::lowest() != -65504.f;
    bad += !std::isinf((float)std::numeric_limits<float16_t>::infinity());
    bad += !std::isnan((float)std::numeric_limits<float16_t>::quiet_NaN());
    bad += (float)std::numeric_limits<bfloat16_t>::epsilon() != 0.0078125f;
    bad += (float)std::numeric_limits<bfloat16_t>::max() != 3.3895313892515355e+38f;
    bad += __half2float(std::numeric_limits<hfloat16_t>::max()) != 65504.f;
    hfloat16_t a = convert<hfloat16_t>(1.5f), b = convert<hfloat16_t>(2.25f);
    bad += convert<float>(a + b) != 3.75f;
    bad += convert<float>(a * b) != 3.375f;
    bad += convert<float>(-a) != -1.5f;
    bad += !(a == convert<hfloat16_t>(1.5f)) || (a == b) || !(a != b);
    a += b;
    bad += convert<float>(a) != 3.75f;
    std::ostringstream os;
    os << float16_t(0.5f) << " " << b;
    bad += os.str() != "0.5 2.25";
    bad += HIPTENSOR_ARCH_HOST != 1;
    std::cout << (bad ? "FAIL " : "ok ") << bad << std::endl;
    return bad;
}
