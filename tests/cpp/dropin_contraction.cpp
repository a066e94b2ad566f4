// Drop-in check of the C++ API: a program written the way a user of hipTensor 1.4 writes
// one (the call sequence of the reference's samples/01_contraction/simple_bilinear_contraction.hpp:
// 86-271: create, three tensor descriptors, alignment requirements, contraction descriptor,
// find, workspace size, plan, contraction), built against <hiptensor/hiptensor.hpp> of this
// repository and linked against libhiptensor_amd.so.  It checks the result against a plain
// host loop and prints PASS / FAIL per case.
//
//   C[m,u,n,v] = alpha * A[m,h,k,n] * B[u,k,v,h] + beta * C[m,u,n,v]   (D aliases C)
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <numeric>
#include <unordered_map>
#include <vector>

#include <hip/hip_runtime.h>
#include <hiptensor/hiptensor.hpp>

template <typename T, typename S>
static int run(hipDataType type, hiptensorComputeType_t compute, S alpha, S beta, double tol, const char* name)
{
    std::vector<int32_t> modeC{'m', 'u', 'n', 'v'}, modeA{'m', 'h', 'k', 'n'}, modeB{'u', 'k', 'v', 'h'};
    std::unordered_map<int32_t, int64_t> extent{{'m', 5}, {'n', 6}, {'u', 3}, {'v', 4}, {'h', 3}, {'k', 8}};
    auto lens = [&](const std::vector<int32_t>& m) {
        std::vector<int64_t> l;
        for(auto x : m)
            l.push_back(extent[x]);
        return l;
    };
    auto aLen = lens(modeA), bLen = lens(modeB), cLen = lens(modeC);
    auto count = [](const std::vector<int64_t>& l) { return (size_t)std::accumulate(l.begin(), l.end(), int64_t{1}, std::multiplies<int64_t>()); };
    size_t nA = count(aLen), nB = count(bLen), nC = count(cLen);

    std::vector<T> hA(nA), hB(nB), hC(nC), hOut(nC);
    for(size_t i = 0; i < nA; i++)
        hA[i] = (T)(((double)std::rand() / RAND_MAX - 0.5) * 2);
    for(size_t i = 0; i < nB; i++)
        hB[i] = (T)(((double)std::rand() / RAND_MAX - 0.5) * 2);
    for(size_t i = 0; i < nC; i++)
        hC[i] = (T)(((double)std::rand() / RAND_MAX - 0.5) * 2);

    T *dA, *dB, *dC;
    CHECK_HIP_ERROR(hipMalloc((void**)&dA, nA * sizeof(T)));
    CHECK_HIP_ERROR(hipMalloc((void**)&dB, nB * sizeof(T)));
    CHECK_HIP_ERROR(hipMalloc((void**)&dC, nC * sizeof(T)));
    CHECK_HIP_ERROR(hipMemcpy(dA, hA.data(), nA * sizeof(T), hipMemcpyHostToDevice));
    CHECK_HIP_ERROR(hipMemcpy(dB, hB.data(), nB * sizeof(T), hipMemcpyHostToDevice));
    CHECK_HIP_ERROR(hipMemcpy(dC, hC.data(), nC * sizeof(T), hipMemcpyHostToDevice));

    hiptensorHandle_t* handle;
    CHECK_HIPTENSOR_ERROR(hiptensorCreate(&handle));
    hiptensorTensorDescriptor_t descA, descB, descC;
    CHECK_HIPTENSOR_ERROR(hiptensorInitTensorDescriptor(handle, &descA, aLen.size(), aLen.data(), nullptr, type, HIPTENSOR_OP_IDENTITY));
    CHECK_HIPTENSOR_ERROR(hiptensorInitTensorDescriptor(handle, &descB, bLen.size(), bLen.data(), nullptr, type, HIPTENSOR_OP_IDENTITY));
    CHECK_HIPTENSOR_ERROR(hiptensorInitTensorDescriptor(handle, &descC, cLen.size(), cLen.data(), nullptr, type, HIPTENSOR_OP_IDENTITY));
    uint32_t alA, alB, alC;
    CHECK_HIPTENSOR_ERROR(hiptensorGetAlignmentRequirement(handle, dA, &descA, &alA));
    CHECK_HIPTENSOR_ERROR(hiptensorGetAlignmentRequirement(handle, dB, &descB, &alB));
    CHECK_HIPTENSOR_ERROR(hiptensorGetAlignmentRequirement(handle, dC, &descC, &alC));
    hiptensorContractionDescriptor_t desc;
    CHECK_HIPTENSOR_ERROR(hiptensorInitContractionDescriptor(handle, &desc, &descA, modeA.data(), alA, &descB, modeB.data(), alB,
                                                             &descC, modeC.data(), alC, &descC, modeC.data(), alC, compute));
    hiptensorContractionFind_t find;
    CHECK_HIPTENSOR_ERROR(hiptensorInitContractionFind(handle, &find, HIPTENSOR_ALGO_DEFAULT));
    uint64_t worksize = 0;
    CHECK_HIPTENSOR_ERROR(hiptensorContractionGetWorkspaceSize(handle, &desc, &find, HIPTENSOR_WORKSPACE_RECOMMENDED, &worksize));
    void* work = nullptr;
    if(worksize > 0)
        CHECK_HIP_ERROR(hipMalloc(&work, worksize));
    hiptensorContractionPlan_t plan;
    CHECK_HIPTENSOR_ERROR(hiptensorInitContractionPlan(handle, &plan, &desc, &find, worksize));
    CHECK_HIPTENSOR_ERROR(hiptensorContraction(handle, &plan, &alpha, dA, dB, &beta, dC, dC, work, worksize, 0));
    CHECK_HIP_ERROR(hipDeviceSynchronize());
    CHECK_HIP_ERROR(hipMemcpy(hOut.data(), dC, nC * sizeof(T), hipMemcpyDeviceToHost));

    // host check: default strides are packed with the last mode fastest
    auto stride = [&](const std::vector<int64_t>& l) {
        std::vector<int64_t> s(l.size(), 1);
        for(int i = (int)l.size() - 2; i >= 0; i--)
            s[i] = s[i + 1] * l[i + 1];
        return s;
    };
    auto sA = stride(aLen), sB = stride(bLen), sC = stride(cLen);
    double worst = 0;
    for(int64_t m = 0; m < extent['m']; m++)
        for(int64_t u = 0; u < extent['u']; u++)
            for(int64_t n = 0; n < extent['n']; n++)
                for(int64_t v = 0; v < extent['v']; v++)
                {
                    double acc = 0;
                    for(int64_t h = 0; h < extent['h']; h++)
                        for(int64_t k = 0; k < extent['k']; k++)
                            acc += (double)hA[m * sA[0] + h * sA[1] + k * sA[2] + n * sA[3]]
                                   * (double)hB[u * sB[0] + k * sB[1] + v * sB[2] + h * sB[3]];
                    size_t ic  = m * sC[0] + u * sC[1] + n * sC[2] + v * sC[3];
                    double ref = (double)alpha * acc + (double)beta * (double)hC[ic];
                    worst      = std::fmax(worst, std::fabs(ref - (double)hOut[ic]) / (std::fabs(ref) + 1.0));
                }
    CHECK_HIPTENSOR_ERROR(hiptensorDestroy(handle));
    CHECK_HIP_ERROR(hipFree(dA));
    CHECK_HIP_ERROR(hipFree(dB));
    CHECK_HIP_ERROR(hipFree(dC));
    if(work)
        CHECK_HIP_ERROR(hipFree(work));
    const bool ok = worst <= tol;
    std::printf("%s %s: max error %.3e (tolerance %.1e)\n", ok ? "PASS" : "FAIL", name, worst, tol);
    return ok ? 0 : 1;
}

int main()
{
    int bad = 0;
    bad += run<float, float>(HIP_R_32F, HIPTENSOR_COMPUTE_32F, 1.1f, 1.2f, 1e-5, "f32 bilinear");
    bad += run<double, double>(HIP_R_64F, HIPTENSOR_COMPUTE_64F, 2.0, -0.5, 1e-12, "f64 bilinear");
    bad += run<_Float16, float>(HIP_R_16F, HIPTENSOR_COMPUTE_32F, 1.0f, 1.0f, 1e-2, "f16 bilinear");
    std::printf(bad ? "dropin_contraction: FAILED\n" : "dropin_contraction: ok\n");
    return bad;
}
