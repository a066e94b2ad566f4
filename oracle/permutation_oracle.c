/*
 * CPU oracle for the tensor-permutation path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a checker: only tests, the smoke check and the cpu_baseline leg
 * of the benchmark may load it.  The product library never links or calls it.
 *
 * It restates, in plain C, what the reference's permutation computes:
 *   - argument set-up: library/src/permutation/permutation_solution_impl.hpp:108-160.
 *     alpha is read as the scalar type and widened to float (:108-113).  The strides held
 *     by the two descriptors are NOT used: both tensors are taken as packed with the FIRST
 *     mode fastest (:125-128, with the build's default HIPTENSOR_DATA_LAYOUT_COL_MAJOR=1,
 *     CMakeLists.txt:69), and B's stride of mode modeB[i] is attached to the position that
 *     mode has in A (:129-132; the look-up table is keyed by `char`, so mode labels are
 *     compared modulo 256).
 *   - element loop: library/src/permutation/permutation_cpu_reference_impl.hpp:112-141:
 *     every multi-index over A's lengths, B[offB] = op(A[offA]).
 *   - element operation: the third-party Composable Kernel functor
 *     UnaryCombinedOp<Aop, Scale, Bop> (ck/tensor_operation/gpu/element/
 *     combined_element_wise_operation.hpp:14-32): y = Aop(x); y = Scale(y); y = Bop(y), each
 *     step stored in the element type.  PassThrough copies; HIPTENSOR_OP_SQRT is bound to
 *     UnarySquare, y = x*x (library/src/permutation/permutation_types_impl.hpp:46-48,
 *     unary_element_wise_operation.hpp:746-761) - a square, whatever the name says;
 *     Scale is `alpha * y` in float for f32 and `half(alpha) * y` in half arithmetic for
 *     f16 (unary_element_wise_operation.hpp:635-665).
 *   - supported: ranks 2..6, f16 or f32 data (A and B alike), f16 or f32 scalar
 *     (library/src/permutation/hiptensor_permutation.cpp:120-155,
 *     permutation_solution_rank2..6_instances.cpp).
 *
 * Parity status: pinned against the reference's own known-answer vector
 * (test/02_permutation/permutation_cpu_impl_test.cpp:82-93, held as a fixture under
 * tests/golden/), bit-for-bit against the compiled reference (oracle/_ref, built by
 * oracle/build_ref.sh) by tests/test_permutation_oracle.py where that library is present,
 * and against committed outputs of that library elsewhere.
 *
 * Element types use the hipDataType numbering: 0 f32, 2 f16.  Operators use
 * hiptensorOperator_t: 1 identity, 2 "sqrt" (= square, see above).
 */
#include <stdint.h>
#include <string.h>

uint16_t oracle_f32_to_f16(float f);
float    oracle_f16_to_f32(uint16_t h);

#define MAX_RANK 6

/* half * half rounded to half: the float product of two halves is exact (22 significant
 * bits), so one rounding to half gives the correctly rounded half product. */
static uint16_t hmul(uint16_t a, uint16_t b)
{
    return oracle_f32_to_f16(oracle_f16_to_f32(a) * oracle_f16_to_f32(b));
}

int oracle_permutation(int            dtype,
                       int            scalar_type,
                       const void*    alpha,
                       const void*    A,
                       void*          B,
                       int            rank,
                       const int64_t* lenA,
                       const int32_t* modeA,
                       const int64_t* lenB,
                       const int32_t* modeB,
                       int            opA,
                       int            opB)
{
    if(rank < 2 || rank > MAX_RANK)
        return 14; /* no instance: HIPTENSOR_STATUS_INTERNAL_ERROR */
    if((dtype != 0 && dtype != 2) || (scalar_type != 0 && scalar_type != 2))
        return 15; /* HIPTENSOR_STATUS_NOT_SUPPORTED */
    if((opA != 1 && opA != 2) || (opB != 1 && opB != 2))
        return 14;

    float alphaF;
    if(scalar_type == 2)
    {
        uint16_t h;
        memcpy(&h, alpha, 2);
        alphaF = oracle_f16_to_f32(h);
    }
    else
        memcpy(&alphaF, alpha, 4);
    const uint16_t alphaH = oracle_f32_to_f16(alphaF);

    /* packed strides, first mode fastest */
    int32_t aStr[MAX_RANK], bStr[MAX_RANK], bStrInA[MAX_RANK];
    int32_t s = 1;
    for(int i = 0; i < rank; i++)
    {
        aStr[i] = s;
        s *= (int32_t)lenA[i];
    }
    s = 1;
    for(int i = 0; i < rank; i++)
    {
        bStr[i] = s;
        s *= (int32_t)lenB[i];
    }
    /* the reference's map<char, index>: a later duplicate label overwrites an earlier one,
     * a label absent from A maps to position 0 (operator[] default-inserts 0) */
    for(int i = 0; i < rank; i++)
        bStrInA[i] = 0;
    for(int i = 0; i < rank; i++)
    {
        int pos = 0;
        for(int j = 0; j < rank; j++)
            if((char)modeA[j] == (char)modeB[i])
                pos = j;
        bStrInA[pos] = bStr[i];
    }

    int64_t count = 1;
    for(int i = 0; i < rank; i++)
        count *= lenA[i];

    int32_t idx[MAX_RANK] = {0};
    for(int64_t e = 0; e < count; e++)
    {
        int32_t offA = 0, offB = 0;
        for(int i = 0; i < rank; i++)
        {
            offA += idx[i] * aStr[i];
            offB += idx[i] * bStrInA[i];
        }
        /* last index fastest, as the reference steps it */
        for(int i = rank - 1; i >= 0; --i)
        {
            if(idx[i] < lenA[i] - 1)
            {
                ++idx[i];
                break;
            }
            idx[i] = 0;
        }
        if(dtype == 0)
        {
            float y = ((const float*)A)[offA];
            if(opA == 2)
                y = y * y;
            y = alphaF * y;
            if(opB == 2)
                y = y * y;
            ((float*)B)[offB] = y;
        }
        else
        {
            uint16_t y = ((const uint16_t*)A)[offA];
            if(opA == 2)
                y = hmul(y, y);
            y = hmul(alphaH, y);
            if(opB == 2)
                y = hmul(y, y);
            ((uint16_t*)B)[offB] = y;
        }
    }
    return 0;
}
