// Drop-in check of hiptensorPermutation through the C++ API: the call sequence of the reference's
// samples/02_permutation/permutation.cpp:60-150 (create, two tensor descriptors with NULL strides,
// one hiptensorPermutation call on the null stream), built against <hiptensor/hiptensor.hpp> of
// this repository and linked against libhiptensor_amd.so.  The result is checked against a host
// loop over A's multi-index (both tensors packed with their first listed mode fastest).
//
//   B[c,n,h,w] = alpha * A[w,h,c,n]
#include <cstdio>
#include <cstdlib>
#include <unordered_map>
#include <vector>

#include <hip/hip_runtime.h>
#include <hiptensor/hiptensor.hpp>

template <typename T>
static int run(hipDataType type, float alphaValue, hiptensorOperator_t opA, const char* name)
{
    std::vector<int32_t>                 modeA{'w', 'h', 'c', 'n'}, modeB{'c', 'n', 'h', 'w'};
    std::unordered_map<int32_t, int64_t> extent{{'h', 32}, {'w', 33}, {'c', 34}, {'n', 35}};
    std::vector<int64_t>                 lenA, lenB;
    for(auto m : modeA)
        lenA.push_back(extent[m]);
    for(auto m : modeB)
        lenB.push_back(extent[m]);
    size_t n = 1;
    for(auto l : lenA)
        n *= (size_t)l;

    std::vector<T> hA(n), hB(n), want(n);
    for(size_t i = 0; i < n; i++)
        hA[i] = (T)(float)((int)(i % 257) - 128) / (T)64.0f;
    // B offset of A's multi-index (w, h, c, n): c + 34 * (n + 35 * (h + 32 * w))
    const T alphaT = (T)alphaValue;
    for(int64_t in = 0; in < 35; in++)
        for(int64_t ic = 0; ic < 34; ic++)
            for(int64_t ih = 0; ih < 32; ih++)
                for(int64_t iw = 0; iw < 33; iw++)
                {
                    T x = hA[iw + 33 * (ih + 32 * (ic + 34 * in))];
                    if(opA == HIPTENSOR_OP_SQRT) // bound to "square" in the reference
                        x = x * x;
                    want[ic + 34 * (in + 35 * (ih + 32 * iw))] = alphaT * x;
                }

    void *dA = nullptr, *dB = nullptr;
    if(hipMalloc(&dA, n * sizeof(T)) != hipSuccess || hipMalloc(&dB, n * sizeof(T)) != hipSuccess)
        return 1;
    (void)hipMemcpy(dA, hA.data(), n * sizeof(T), hipMemcpyHostToDevice);
    (void)hipMemset(dB, 0xFF, n * sizeof(T));

    hiptensorHandle_t* handle = nullptr;
    if(hiptensorCreate(&handle) != HIPTENSOR_STATUS_SUCCESS)
        return 1;
    hiptensorTensorDescriptor_t descA, descB;
    if(hiptensorInitTensorDescriptor(handle, &descA, 4, lenA.data(), nullptr, type, opA) != HIPTENSOR_STATUS_SUCCESS
       || hiptensorInitTensorDescriptor(handle, &descB, 4, lenB.data(), nullptr, type, HIPTENSOR_OP_IDENTITY) != HIPTENSOR_STATUS_SUCCESS)
        return 1;
    const float alpha = alphaValue;
    auto        st    = hiptensorPermutation(handle, &alpha, dA, &descA, modeA.data(), dB, &descB, modeB.data(), HIP_R_32F, 0);
    if(st != HIPTENSOR_STATUS_SUCCESS)
    {
        std::printf("%s: hiptensorPermutation returned %s\n", name, hiptensorGetErrorString(st));
        return 1;
    }
    (void)hipDeviceSynchronize();
    (void)hipMemcpy(hB.data(), dB, n * sizeof(T), hipMemcpyDeviceToHost);
    size_t bad = 0;
    for(size_t i = 0; i < n; i++)
        bad += !(hB[i] == want[i]);
    std::printf("%s: %s (%zu of %zu elements differ)\n", name, bad ? "FAIL" : "PASS", bad, n);
    (void)hiptensorDestroy(handle);
    (void)hipFree(dA);
    (void)hipFree(dB);
    return bad ? 1 : 0;
}

int main()
{
    int fails = 0;
    fails += run<float>(HIP_R_32F, 1.0f, HIPTENSOR_OP_IDENTITY, "f32 identity alpha=1");
    fails += run<float>(HIP_R_32F, 2.5f, HIPTENSOR_OP_SQRT, "f32 square alpha=2.5");
    fails += run<_Float16>(HIP_R_16F, 0.5f, HIPTENSOR_OP_IDENTITY, "f16 identity alpha=0.5");
    std::printf(fails ? "dropin_permutation: %d case(s) failed\n" : "dropin_permutation: ok\n", fails);
    return fails ? 1 : 0;
}
