/*
 * CPU oracle for the tensor-contraction path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is a checker: only tests, the smoke check and the cpu_baseline leg
 * of the benchmark may load it.  The product library never links or calls it.
 *
 * It restates, in plain C, the algorithm of the reference's CPU contraction:
 *   - mode normalisation: library/src/contraction/contraction_solution.cpp:34-160
 *     (M group = D's modes found in A, in D's order; N group = the remaining D
 *      modes, in D's order; K group = A's modes found in B, in A's order)
 *   - loop nest, accumulate type, "round to the output type, then apply
 *     alpha/beta": library/src/contraction/contraction_cpu_reference_impl.hpp:152-445
 *   - accumulate / compute type per data-type row:
 *     library/src/contraction/contraction_cpu_reference_instances.cpp:32-298
 *   - alpha/beta read as the compute type and narrowed to float:
 *     library/src/contraction/contraction_solution_impl.hpp:111-123 and the
 *     float constructors of the third-party Composable Kernel functors
 *     Bilinear / Scale (ck/tensor_operation/gpu/element/
 *     binary_element_wise_operation.hpp:292-366, unary_element_wise_operation.hpp:635-680)
 *   - complex alpha/beta kept as double complex then narrowed:
 *     library/src/contraction/device/device_element_wise_operation_complex.hpp:38-91
 *   - threading: contiguous chunks of the row-major flattened normalised output
 *     index (ck/library/utility/host_tensor.hpp:633-690); every output element
 *     is produced by one sequential K loop, so results do not depend on the
 *     thread count.
 *
 * Parity status: every data-type row below is pinned bit-for-bit against the
 * compiled reference (oracle/_ref, built by oracle/build_ref.sh) by
 * tests/test_oracle_vs_ref.py where that library is present, and against the
 * committed fixtures under tests/golden/ (written from that library) elsewhere.
 *
 * Element types use the hipDataType numbering: 0 f32, 1 f64, 2 f16, 14 bf16,
 * 4 complex f32, 5 complex f64.  Compute types use hiptensorComputeType_t:
 * 1 f16, 4 f32, 16 f64, 1024 bf16, 2048 complex f32, 4096 complex f64.
 */
#include <math.h>
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define MAX_MODES 32

enum { T_F32 = 0, T_F64 = 1, T_F16 = 2, T_C32 = 4, T_C64 = 5, T_BF16 = 14 };
enum { CT_16F = 1, CT_32F = 4, CT_64F = 16, CT_16BF = 1024, CT_C32F = 2048, CT_C64F = 4096 };

/* ---------- 16-bit float conversions (round to nearest even) ---------- */

static float f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp  = (h >> 10) & 0x1Fu;
    uint32_t man  = h & 0x3FFu;
    uint32_t bits;
    if(exp == 0)
    {
        if(man == 0)
            bits = sign;
        else
        {
            int e = -1;
            do
            {
                man <<= 1;
                e++;
            } while(!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    }
    else if(exp == 31)
        bits = sign | 0x7F800000u | (man << 13);
    else
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static uint16_t f32_to_f16(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t abs  = x & 0x7FFFFFFFu;
    if(abs >= 0x7F800000u) /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (abs > 0x7F800000u ? 0x200u | ((abs >> 13) & 0x3FFu) : 0));
    if(abs >= 0x477FF000u) /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    if(abs < 0x33000001u) /* < 2^-25 (or == 2^-25 which ties to even 0) */
        return (uint16_t)sign;
    int32_t  e   = (int32_t)(abs >> 23) - 127;
    uint32_t man = (abs & 0x7FFFFFu) | 0x800000u;
    int      shift;
    uint32_t base;
    if(e < -14)
    { /* subnormal half */
        shift = 13 + (-14 - e);
        base  = 0;
    }
    else
    {
        shift = 13;
        base  = ((uint32_t)(e + 15) << 10) - 0x400u; /* hidden bit adds 0x400 */
    }
    uint32_t q   = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t hlf = 1u << (shift - 1);
    if(rem > hlf || (rem == hlf && (q & 1u)))
        q++;
    return (uint16_t)(sign | (base + q));
}

static float bf16_to_f32(uint16_t h)
{
    uint32_t bits = (uint32_t)h << 16;
    float    f;
    memcpy(&f, &bits, 4);
    return f;
}

/* ck/utility/type_convert.hpp, bf16_convert_rtn: RNE, NaN kept quiet. */
static uint16_t f32_to_bf16(float f)
{
    uint32_t x;
    memcpy(&x, &f, 4);
    if((~x & 0x7F800000u) == 0)
    {
        if(x & 0xFFFFu)
            x |= 0x10000u; /* keep NaN a NaN */
    }
    else
        x += 0x7FFFu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
}

/* ---------- problem description ---------- */

typedef struct
{
    int     dtype, ctype, bilinear;
    int     nM, nN, nK;
    int64_t lenM[MAX_MODES], lenN[MAX_MODES], lenK[MAX_MODES];
    int64_t aM[MAX_MODES], aK[MAX_MODES];
    int64_t bN[MAX_MODES], bK[MAX_MODES];
    int64_t cM[MAX_MODES], cN[MAX_MODES];
    int64_t dM[MAX_MODES], dN[MAX_MODES];
    int64_t M, N, K;
    /* K offset tables, K-loop order = normalised order, last K mode innermost */
    int64_t *akoff, *bkoff;
    const void *A, *B, *C;
    void*       D;
    double      alpha[2], beta[2];
    int64_t     begin, end, step;
    /* optional pre-converted float copies of A and B (real 16/32-bit rows) */
    const float *Af, *Bf;
} problem_t;

static int find_mode(const int32_t* modes, int n, int32_t m)
{
    for(int i = 0; i < n; i++)
        if(modes[i] == m)
            return i;
    return -1;
}

static int64_t extent_of(int n, const int64_t* len, const int64_t* str)
{
    int64_t e = 1;
    for(int i = 0; i < n; i++)
    {
        if(len[i] == 0)
            return 0;
        e += (len[i] - 1) * str[i];
    }
    return e;
}

/* read alpha/beta the way readVal<ScalarData>(ptr, computeType) does
 * (library/src/data_types.cpp:153-204) */
static void read_scalar(const void* p, int ctype, double out[2])
{
    out[0] = 0;
    out[1] = 0;
    if(!p)
        return;
    switch(ctype)
    {
    case CT_16F: out[0] = f16_to_f32(*(const uint16_t*)p); break;
    case CT_16BF: out[0] = bf16_to_f32(*(const uint16_t*)p); break;
    case CT_32F: out[0] = *(const float*)p; break;
    case CT_64F: out[0] = *(const double*)p; break;
    case CT_C32F:
        out[0] = ((const float*)p)[0];
        out[1] = ((const float*)p)[1];
        break;
    case CT_C64F:
        out[0] = ((const double*)p)[0];
        out[1] = ((const double*)p)[1];
        break;
    default: break;
    }
}

/* ---------- per-element kernels ---------- */

static inline float load_as_float(const void* base, int dtype, int64_t off)
{
    switch(dtype)
    {
    case T_F16: return f16_to_f32(((const uint16_t*)base)[off]);
    case T_BF16: return bf16_to_f32(((const uint16_t*)base)[off]);
    case T_F32: return ((const float*)base)[off];
    default: return (float)((const double*)base)[off];
    }
}

/* ComputeDataType conversion applied to each A/B element before the multiply
 * (contraction_cpu_reference_impl.hpp:392-397) */
static inline float to_compute_f32(float v, int ctype)
{
    if(ctype == CT_16F)
        return f16_to_f32(f32_to_f16(v));
    if(ctype == CT_16BF)
        return bf16_to_f32(f32_to_bf16(v));
    return v;
}

static void one_output(const problem_t* p, int64_t idx)
{
    /* idx -> (m.., n..) row-major over the normalised output modes */
    int64_t r    = idx;
    int64_t offA = 0, offB = 0, offC = 0, offD = 0;
    for(int i = p->nN - 1; i >= 0; i--)
    {
        int64_t n = r % p->lenN[i];
        r /= p->lenN[i];
        offB += n * p->bN[i];
        offC += n * p->cN[i];
        offD += n * p->dN[i];
    }
    for(int i = p->nM - 1; i >= 0; i--)
    {
        int64_t m = r % p->lenM[i];
        r /= p->lenM[i];
        offA += m * p->aM[i];
        offC += m * p->cM[i];
        offD += m * p->dM[i];
    }
    const int64_t  K  = p->K;
    const int64_t* ak = p->akoff;
    const int64_t* bk = p->bkoff;
    const float    alphaF = (float)p->alpha[0], betaF = (float)p->beta[0];

    switch(p->dtype)
    {
    case T_F16:
    case T_BF16:
    case T_F32:
    {
        float acc = 0.f;
        if(p->Af)
        {
            const float* a = p->Af + offA;
            const float* b = p->Bf + offB;
            for(int64_t k = 0; k < K; k++)
                acc += a[ak[k]] * b[bk[k]];
        }
        else
        {
            for(int64_t k = 0; k < K; k++)
                acc += to_compute_f32(load_as_float(p->A, p->dtype, offA + ak[k]), p->ctype)
                       * to_compute_f32(load_as_float(p->B, p->dtype, offB + bk[k]), p->ctype);
        }
        if(p->dtype == T_F32)
        {
            float d = p->bilinear ? betaF * ((const float*)p->C)[offC] : 0.f;
            ((float*)p->D)[offD] = p->bilinear ? alphaF * acc + d : alphaF * acc;
        }
        else if(p->dtype == T_BF16)
        {
            /* x rounded to bf16 first, then float math, then RNE to bf16 */
            float x = bf16_to_f32(f32_to_bf16(acc));
            float y = p->bilinear
                          ? alphaF * x + betaF * bf16_to_f32(((const uint16_t*)p->C)[offC])
                          : alphaF * x;
            ((uint16_t*)p->D)[offD] = f32_to_bf16(y);
        }
        else
        {
            /* half(alpha) * x (+ half(beta) * d) on _Float16 operands.  The host
             * compiler evaluates the expression with excess precision: the
             * products (exact in float) and their sum are formed in float and
             * rounded to half once, at the assignment. */
            float x  = f16_to_f32(f32_to_f16(acc));
            float ha = f16_to_f32(f32_to_f16(alphaF));
            float hb = f16_to_f32(f32_to_f16(betaF));
            float y  = p->bilinear ? ha * x + hb * f16_to_f32(((const uint16_t*)p->C)[offC])
                                   : ha * x;
            ((uint16_t*)p->D)[offD] = f32_to_f16(y);
        }
        break;
    }
    case T_F64:
    {
        const double* A = (const double*)p->A;
        const double* B = (const double*)p->B;
        double        x;
        if(p->ctype == CT_64F)
        {
            double acc = 0.0;
            for(int64_t k = 0; k < K; k++)
                acc += A[offA + ak[k]] * B[offB + bk[k]];
            x = acc;
        }
        else
        { /* f64 data, f32 compute: inputs narrowed, float accumulate */
            float acc = 0.f;
            for(int64_t k = 0; k < K; k++)
                acc += (float)A[offA + ak[k]] * (float)B[offB + bk[k]];
            x = (double)acc;
        }
        /* float alpha_/beta_ promoted in a double expression */
        double y = p->bilinear ? (double)alphaF * x + (double)betaF * ((const double*)p->C)[offC]
                               : (double)alphaF * x;
        ((double*)p->D)[offD] = y;
        break;
    }
    case T_C32:
    {
        const float* A  = (const float*)p->A;
        const float* B  = (const float*)p->B;
        float        ar = 0.f, ai = 0.f;
        for(int64_t k = 0; k < K; k++)
        {
            const float* a  = A + 2 * (offA + ak[k]);
            const float* b  = B + 2 * (offB + bk[k]);
            float        pr = a[0] * b[0] - a[1] * b[1];
            float        pi = a[1] * b[0] + a[0] * b[1];
            ar              = ar + pr;
            ai              = ai + pi;
        }
        float alr = (float)p->alpha[0], ali = (float)p->alpha[1];
        float yr  = alr * ar - ali * ai;
        float yi  = ali * ar + alr * ai;
        if(p->bilinear)
        {
            const float* c   = (const float*)p->C + 2 * offC;
            float        ber = (float)p->beta[0], bei = (float)p->beta[1];
            float        cr  = ber * c[0] - bei * c[1];
            float        ci  = bei * c[0] + ber * c[1];
            yr               = yr + cr;
            yi               = yi + ci;
        }
        ((float*)p->D)[2 * offD]     = yr;
        ((float*)p->D)[2 * offD + 1] = yi;
        break;
    }
    case T_C64:
    {
        const double* A  = (const double*)p->A;
        const double* B  = (const double*)p->B;
        double        ar = 0.0, ai = 0.0;
        for(int64_t k = 0; k < K; k++)
        {
            const double* a  = A + 2 * (offA + ak[k]);
            const double* b  = B + 2 * (offB + bk[k]);
            double        pr = a[0] * b[0] - a[1] * b[1];
            double        pi = a[1] * b[0] + a[0] * b[1];
            ar               = ar + pr;
            ai               = ai + pi;
        }
        double alr = p->alpha[0], ali = p->alpha[1];
        double yr  = alr * ar - ali * ai;
        double yi  = ali * ar + alr * ai;
        if(p->bilinear)
        {
            const double* c   = (const double*)p->C + 2 * offC;
            double        ber = p->beta[0], bei = p->beta[1];
            double        cr  = ber * c[0] - bei * c[1];
            double        ci  = bei * c[0] + ber * c[1];
            yr                = yr + cr;
            yi                = yi + ci;
        }
        ((double*)p->D)[2 * offD]     = yr;
        ((double*)p->D)[2 * offD + 1] = yi;
        break;
    }
    default: break;
    }
}

typedef struct
{
    const problem_t* p;
    int64_t          first, count; /* in units of "selected outputs" */
} job_t;

static void* worker(void* arg)
{
    job_t*           j = (job_t*)arg;
    const problem_t* p = j->p;
    for(int64_t s = j->first; s < j->first + j->count; s++)
        one_output(p, p->begin + s * p->step);
    return NULL;
}

static float* convert_to_float(const void* src, int dtype, int ctype, int64_t n)
{
    float* f = (float*)malloc((size_t)(n > 0 ? n : 1) * sizeof(float));
    if(!f)
        return NULL;
    for(int64_t i = 0; i < n; i++)
        f[i] = to_compute_f32(load_as_float(src, dtype, i), ctype);
    return f;
}

/*
 * Returns 0 on success, negative on a malformed problem.
 *
 * dtype     element type of A, B, C and D (one type for all, as in every row
 *           the reference registers)
 * ctype     compute type
 * C == NULL selects the scale op, otherwise bilinear
 * strC      may be NULL (then strD is used, as the reference does)
 * out_begin/out_end/out_step select which outputs are computed, as positions
 *           in the row-major flattened normalised output index
 *           [M modes in D's order][N modes in D's order]; pass 0, -1, 1 for all.
 *           Outputs that are not selected are left untouched in D.
 * nthreads  <= 0 means one thread
 */
int oracle_contraction(int            dtype,
                       int            ctype,
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
                       const int64_t* lenD,
                       const int64_t* strC,
                       const int64_t* strD,
                       const int32_t* modeD,
                       int64_t        out_begin,
                       int64_t        out_end,
                       int64_t        out_step,
                       int            nthreads)
{
    if(nA > MAX_MODES || nB > MAX_MODES || nD > MAX_MODES || nA < 0 || nB < 0 || nD < 0)
        return -1;
    problem_t p;
    memset(&p, 0, sizeof(p));
    p.dtype    = dtype;
    p.ctype    = ctype;
    p.bilinear = (C != NULL);
    p.A        = A;
    p.B        = B;
    p.C        = C;
    p.D        = D;
    if(!strC)
        strC = strD;
    read_scalar(alpha, ctype, p.alpha);
    read_scalar(beta, ctype, p.beta);

    /* M / N groups in D's order */
    for(int i = 0; i < nD; i++)
    {
        int ia = find_mode(modeA, nA, modeD[i]);
        if(ia >= 0)
        {
            p.lenM[p.nM] = lenA[ia];
            p.aM[p.nM]   = strA[ia];
            p.cM[p.nM]   = strC[i];
            p.dM[p.nM]   = strD[i];
            if(lenA[ia] != lenD[i])
                return -2;
            p.nM++;
        }
        else
        {
            int ib = find_mode(modeB, nB, modeD[i]);
            if(ib < 0)
                return -3;
            p.lenN[p.nN] = lenB[ib];
            p.bN[p.nN]   = strB[ib];
            p.cN[p.nN]   = strC[i];
            p.dN[p.nN]   = strD[i];
            if(lenB[ib] != lenD[i])
                return -2;
            p.nN++;
        }
    }
    /* K group in A's order */
    for(int i = 0; i < nA; i++)
    {
        int ib = find_mode(modeB, nB, modeA[i]);
        if(ib >= 0)
        {
            if(find_mode(modeD, nD, modeA[i]) >= 0)
                return -4; /* batch modes are not part of this path */
            if(lenA[i] != lenB[ib])
                return -2;
            p.lenK[p.nK] = lenA[i];
            p.aK[p.nK]   = strA[i];
            p.bK[p.nK]   = strB[ib];
            p.nK++;
        }
    }
    p.M = p.N = p.K = 1;
    for(int i = 0; i < p.nM; i++)
        p.M *= p.lenM[i];
    for(int i = 0; i < p.nN; i++)
        p.N *= p.lenN[i];
    for(int i = 0; i < p.nK; i++)
        p.K *= p.lenK[i];

    p.akoff = (int64_t*)malloc(sizeof(int64_t) * (size_t)(p.K > 0 ? p.K : 1));
    p.bkoff = (int64_t*)malloc(sizeof(int64_t) * (size_t)(p.K > 0 ? p.K : 1));
    if(!p.akoff || !p.bkoff)
        return -5;
    for(int64_t k = 0; k < p.K; k++)
    {
        int64_t r = k, oa = 0, ob = 0;
        for(int i = p.nK - 1; i >= 0; i--)
        {
            int64_t kk = r % p.lenK[i];
            r /= p.lenK[i];
            oa += kk * p.aK[i];
            ob += kk * p.bK[i];
        }
        p.akoff[k] = oa;
        p.bkoff[k] = ob;
    }

    int64_t total = p.M * p.N;
    if(out_end < 0 || out_end > total)
        out_end = total;
    if(out_begin < 0)
        out_begin = 0;
    if(out_step <= 0)
        out_step = 1;
    p.begin = out_begin;
    p.end   = out_end;
    p.step  = out_step;
    int64_t nsel = out_end > out_begin ? (out_end - out_begin + out_step - 1) / out_step : 0;

    float *Af = NULL, *Bf = NULL;
    if((dtype == T_F16 || dtype == T_BF16 || dtype == T_F32) && nsel * p.K > (1 << 22))
    {
        Af = convert_to_float(A, dtype, ctype, extent_of(nA, lenA, strA));
        Bf = convert_to_float(B, dtype, ctype, extent_of(nB, lenB, strB));
        if(Af && Bf)
        {
            p.Af = Af;
            p.Bf = Bf;
        }
    }

    if(nthreads <= 0)
        nthreads = 1;
    if(nthreads > 256)
        nthreads = 256;
    if((int64_t)nthreads > nsel)
        nthreads = nsel > 0 ? (int)nsel : 1;
    pthread_t th[256];
    job_t     jobs[256];
    int64_t   per = (nsel + nthreads - 1) / nthreads;
    int       started = 0;
    for(int t = 0; t < nthreads; t++)
    {
        int64_t first = (int64_t)t * per;
        int64_t cnt   = first >= nsel ? 0 : (first + per > nsel ? nsel - first : per);
        jobs[t].p     = &p;
        jobs[t].first = first;
        jobs[t].count = cnt;
        if(t == nthreads - 1 || cnt == 0)
        {
            /* run the last chunk on the calling thread */
            worker(&jobs[t]);
            break;
        }
        if(pthread_create(&th[t], NULL, worker, &jobs[t]) != 0)
        {
            worker(&jobs[t]);
            continue;
        }
        started = t + 1;
    }
    for(int t = 0; t < started; t++)
        pthread_join(th[t], NULL);

    free(Af);
    free(Bf);
    free(p.akoff);
    free(p.bkoff);
    return 0;
}

/* exposed so that tests can pin the conversions against numpy / torch */
uint16_t oracle_f32_to_f16(float f) { return f32_to_f16(f); }
uint16_t oracle_f32_to_bf16(float f) { return f32_to_bf16(f); }
float    oracle_f16_to_f32(uint16_t h) { return f16_to_f32(h); }
float    oracle_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

/* Seeded input generator of the reference's test harness
 * (test/device/common.hpp:68-81): value(i) = (float(pcg(i)) / 2^32 - 0.5) * 2 */
static uint32_t pcg_hash(uint32_t input)
{
    uint32_t state = input * 747796405u + 2891336453u;
    uint32_t word  = ((state >> ((state >> 28u) + 4u)) ^ state) * 277803737u;
    return (word >> 22u) ^ word;
}

float oracle_gen_value(uint32_t seeded_index)
{
    return ((float)pcg_hash(seeded_index) / 4294967296.0f - 0.5f) * 2.0f;
}
