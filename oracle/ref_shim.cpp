// C-ABI shim around the reference's hiptensorContractionReference
// (library/src/contraction/contraction_cpu_reference.hpp:35-58) so that the
// checker scripts can call the *compiled reference* through ctypes.
// TEST INFRASTRUCTURE ONLY; compiled by oracle/build_ref.sh against the
// reference headers in place; never linked into the product library.
#include <cstdint>
#include <vector>

#include <hiptensor/hiptensor.hpp>

#include "contraction_cpu_reference.hpp"

extern "C" int ref_contraction(int            computeType,
                               const void*    alpha,
                               const void*    A,
                               const void*    B,
                               const void*    beta,
                               const void*    C,
                               void*          D,
                               int            nA,
                               const int64_t* lenA,
                               const int64_t* strA,
                               const int32_t* modeA,
                               int            nB,
                               const int64_t* lenB,
                               const int64_t* strB,
                               const int32_t* modeB,
                               int            nD,
                               const int64_t* lenC,
                               const int64_t* strC,
                               const int64_t* lenD,
                               const int64_t* strD,
                               const int32_t* modeD,
                               int            typeA,
                               int            typeB,
                               int            typeC,
                               int            typeD)
{
    // contraction_cpu_reference.cpp:57 reads only mContractionDesc.mComputeType.
    hiptensorContractionPlan_t plan;
    plan.mSolution                     = nullptr;
    plan.mContractionDesc.mComputeType = (hiptensorComputeType_t)computeType;

    auto vec = [](const int64_t* p, int n) {
        return p ? std::vector<size_t>(p, p + n) : std::vector<size_t>(n, 0);
    };
    std::vector<int32_t> mA(modeA, modeA + nA), mB(modeB, modeB + nB), mD(modeD, modeD + nD);

    // The library passes the D mode list for both C and D
    // (hiptensor_contraction.cpp:772 uses mTensorMode[2] twice).
    return (int)hiptensorContractionReference(&plan,
                                              alpha,
                                              A,
                                              B,
                                              beta,
                                              C,
                                              D,
                                              vec(lenA, nA),
                                              vec(strA, nA),
                                              mA,
                                              vec(lenB, nB),
                                              vec(strB, nB),
                                              mB,
                                              vec(lenC, nD),
                                              vec(strC, nD),
                                              mD,
                                              vec(lenD, nD),
                                              vec(strD, nD),
                                              mD,
                                              (hipDataType)typeA,
                                              (hipDataType)typeB,
                                              (hipDataType)typeC,
                                              (hipDataType)typeD,
                                              nullptr);
}

#include "permutation_cpu_reference.hpp"

// The reference's hiptensorPermutationReference
// (library/src/permutation/permutation_cpu_reference.hpp:33-43).  The handle is not read
// (permutation_cpu_reference.cpp:31-83); the descriptors are built here the way
// hiptensorInitTensorDescriptor fills them for NULL strides (library/src/hiptensor.cpp:199-206).
extern "C" int ref_permutation(const void*    alpha,
                               const void*    A,
                               void*          B,
                               int            rank,
                               const int64_t* lenA,
                               const int32_t* modeA,
                               const int64_t* lenB,
                               const int32_t* modeB,
                               int            typeA,
                               int            typeB,
                               int            opA,
                               int            opB,
                               int            typeScalar)
{
    auto desc = [rank](const int64_t* len, int type, int op) {
        std::vector<size_t> l(len, len + rank), s(rank, 1);
        for(int i = rank - 2; i >= 0; --i)
            s[i] = s[i + 1] * l[i + 1];
        return hiptensorTensorDescriptor_t{(hipDataType)type, l, s, (hiptensorOperator_t)op};
    };
    auto dA = desc(lenA, typeA, opA);
    auto dB = desc(lenB, typeB, opB);
    return (int)hiptensorPermutationReference(
        nullptr, alpha, A, &dA, modeA, B, &dB, modeB, (hipDataType)typeScalar, nullptr);
}
