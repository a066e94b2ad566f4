// Tensor permutation kernels, B[perm(index)] = opB(alpha * opA(A[index])), and their launcher.
//
// The work is a stream of bytes through HBM, so the kernels are built around memory
// coalescing, not arithmetic:
//   * COPY    one fused mode left: a scaled vector copy.
//   * TILED   A's fastest mode i and B's fastest mode j differ.  A workgroup moves a
//             two-dimensional tile of those two modes: it reads rows along i (contiguous in A),
//             applies the element operation, parks the tile in LDS, and writes it out along j
//             (contiguous in B).  The other modes only choose the tile's base offsets, once per
//             workgroup on the scalar unit.
//   * ROWS    A and B share the fastest mode: runs of it are contiguous on both sides and go
//             from registers straight back to memory, no LDS.
//   * STRIP   like TILED, for a tile mode too short to give long runs (the 3 of an RGB image,
//             say) when the other tile mode follows it directly in memory on that side: a
//             workgroup takes a strip of the long mode times the whole short mode, which is one
//             contiguous run on the short mode's side, and moves it linearly there.
//   * GROUPED TILED for tensors of many short modes: a tile row spans A's two fastest modes, a
//             tile column B's two fastest modes, so that runs stay long when no single mode is.
//   * SHARED  ROWS for a short shared fastest mode (interleaved channels): tiles of that mode
//             times a chunk of A's next mode times a chunk of B's next mode, through LDS.
//   * GATHER  one thread per element of B; covers tiny tensors and awkward extents.
// Element operation per Composable Kernel's UnaryCombinedOp<Aop, Scale, Bop>
// (ck/tensor_operation/gpu/element/combined_element_wise_operation.hpp:14-32): every step is
// rounded to the element type; for f16 alpha is rounded to half first
// (unary_element_wise_operation.hpp:647-651).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>
#include <cstdio>
#include <cstring>

#include "hiptk_kernels.h"

namespace hiptk
{
    namespace
    {
        constexpr int PERM_THREADS = 256;
        constexpr int PERM_BATCH   = HIPTK_PERM_MAX_RANK - 2;

        struct PArgs
        {
            const void* A;
            void*       B;
            uint32_t    e_i, e_j; // extents of the two tile modes
            uint32_t    a_j; // A stride of mode j (mode i has stride 1 in A)
            uint32_t    b_i, b_j; // B strides (TILED: b_j == 1, ROWS: b_i == 1)
            uint32_t    nt_i, nt_j; // tiles along i and j
            uint32_t    group; // tile order: bands of `group` tiles along j, walked j-first
            int32_t     nb; // modes that only pick the tile's base
            uint32_t    bext[PERM_BATCH], ba[PERM_BATCH], bb[PERM_BATCH];
            float       alpha;
            int32_t     op_a, op_b;
        };

        struct GArgs
        {
            const void* A;
            void*       B;
            uint32_t    n;
            int32_t     rank;
            uint32_t    ext[HIPTK_PERM_MAX_RANK]; // in B's order, fastest first; extents of 1 left out
            uint32_t    astr[HIPTK_PERM_MAX_RANK];
            uint32_t    magic[HIPTK_PERM_MAX_RANK]; // floor(2^32 / ext) + 1
            float       alpha;
            int32_t     op_a, op_b;
        };

        template <typename T, int V>
        struct alignas(sizeof(T) * V) Vec
        {
            T v[V];
        };

        // Every element is read once and written once: loads and stores are marked non-temporal so
        // that the stream does not displace itself in the caches (measured: a plain 1 GiB copy
        // 5.8 TB/s, with non-temporal loads and stores 6.2 TB/s).
        template <int BYTES>
        struct RawBits;
        template <>
        struct RawBits<2>
        {
            using type = uint16_t;
        };
        template <>
        struct RawBits<4>
        {
            using type = uint32_t;
        };
        template <>
        struct RawBits<8>
        {
            using type = uint32_t __attribute__((ext_vector_type(2)));
        };
        template <>
        struct RawBits<16>
        {
            using type = uint32_t __attribute__((ext_vector_type(4)));
        };

        template <typename T, int V>
        __device__ inline Vec<T, V> load_stream(const T* p)
        {
            using R = typename RawBits<sizeof(T) * V>::type;
            const R r = __builtin_nontemporal_load(reinterpret_cast<const R*>(p));
            return __builtin_bit_cast(Vec<T, V>, r);
        }

        template <typename T, int V>
        __device__ inline void store_stream(T* p, const Vec<T, V>& v)
        {
            using R = typename RawBits<sizeof(T) * V>::type;
            __builtin_nontemporal_store(__builtin_bit_cast(R, v), reinterpret_cast<R*>(p));
        }

        template <typename T>
        __device__ inline T element_op(T x, T alpha, int op_a, int op_b)
        {
            if(op_a == HIPTK_PERM_OP_RAW)
                return x; // a plain move: every bit pattern, NaN payloads included, arrives unchanged
            T y = x;
            if(op_a)
                y = y * y;
            y = alpha * y;
            if(op_b)
                y = y * y;
            return y;
        }

        // The tile in LDS is [TJ][TI].  Column reads must spread over the 64 banks: the small
        // tiles pad each row by one element; the 64 KiB tiles have no room for padding and XOR
        // the column index with the row number instead (in units of one 32-bit word).
        template <typename T, int TI, int TJ, int VR, int VW, bool TRANSPOSE, int NT = PERM_THREADS, bool SWZ = false>
        __global__ __launch_bounds__(NT) void permute_tile_kernel(PArgs a)
        {
            constexpr int PITCH = SWZ ? TI : TI + 4 / (int)sizeof(T); // an odd number of 32-bit words
            constexpr int VPR   = TI / VR; // vectors per tile row
            constexpr int NRV   = VPR * TJ / NT; // vectors per thread, read side
            static_assert(TI % VR == 0 && (VPR * TJ) % NT == 0 && NRV >= 1, "read shape");
            static_assert(!SWZ || TI * sizeof(T) >= 256, "a swizzled row spans all 64 banks");
            __shared__ T tile[TRANSPOSE ? TJ * PITCH : 1];
            auto         at = [](uint32_t j, uint32_t i) -> uint32_t {
                return SWZ ? j * TI + (i ^ ((j & 63u) * (4u / sizeof(T)))) : j * PITCH + i;
            };

            const T* __restrict__ A = static_cast<const T*>(a.A);
            T* __restrict__ B       = static_cast<T*>(a.B);
            const int tid           = threadIdx.x;

            // Workgroups that run at the same time should spread over both tile modes: tiles that
            // are neighbours along i touch neighbouring addresses of A, neighbours along j
            // neighbouring addresses of B.  The tile plane is cut into bands of `group` tiles
            // along j; inside a band the walk is j-first.
            const uint32_t plane = a.nt_i * a.nt_j;
            uint32_t       blk   = blockIdx.x / plane;
            const uint32_t lin   = blockIdx.x - blk * plane;
            uint32_t ti, tj;
            if(a.group == 0)
            {
                // diagonal walk: consecutive workgroups differ in both tile coordinates, so that
                // with power-of-two strides neither side keeps hitting the same memory channels
                ti                = lin % a.nt_i;
                const uint32_t rj = lin / a.nt_i;
                tj                = (rj + ti) % a.nt_j;
            }
            else
            {
                const uint32_t band = lin / (a.group * a.nt_i);
                const uint32_t rem  = lin - band * (a.group * a.nt_i);
                const uint32_t left = a.nt_j - band * a.group;
                const uint32_t rows = left < a.group ? left : a.group;
                ti                  = rem / rows;
                tj                  = band * a.group + (rem - ti * rows);
            }
            uint32_t       aoff = 0, boff = 0;
            for(int d = 0; d < a.nb; ++d)
            {
                const uint32_t c = blk % a.bext[d];
                blk /= a.bext[d];
                aoff += c * a.ba[d];
                boff += c * a.bb[d];
            }
            const uint32_t i0 = ti * TI, j0 = tj * TJ;
            aoff += i0 + j0 * a.a_j;
            boff += i0 * a.b_i + j0 * a.b_j;

            const T alpha = static_cast<T>(a.alpha);

            Vec<T, VR> r[NRV];
#pragma unroll
            for(int k = 0; k < NRV; ++k)
            {
                // Lanes outside the extents load the tile's first element instead of branching
                // around the load: a branch per load would make the compiler wait for each load
                // before issuing the next, and the loads must all be in flight together.
                const uint32_t v = tid + k * NT, iv = v % VPR, j = v / VPR;
                const bool     ok = (i0 + iv * VR < a.e_i) && (j0 + j < a.e_j);
                r[k] = load_stream<T, VR>(A + aoff + (ok ? iv * VR + j * a.a_j : 0u));
            }
#pragma unroll
            for(int k = 0; k < NRV; ++k)
            {
                const uint32_t v = tid + k * NT, iv = v % VPR, j = v / VPR;
#pragma unroll
                for(int e = 0; e < VR; ++e)
                    r[k].v[e] = element_op(r[k].v[e], alpha, a.op_a, a.op_b);
                if constexpr(TRANSPOSE)
                {
#pragma unroll
                    for(int e = 0; e < VR; ++e)
                        tile[at(j, iv * VR + e)] = r[k].v[e];
                }
                else
                {
                    const bool ok = (i0 + iv * VR < a.e_i) && (j0 + j < a.e_j);
                    if(ok)
                        store_stream<T, VR>(B + boff + iv * VR + j * a.b_j, r[k]);
                }
            }
            if constexpr(TRANSPOSE)
            {
                constexpr int VPC = TJ / VW; // vectors per tile column
                constexpr int NWV = VPC * TI / NT;
                static_assert(TJ % VW == 0 && (VPC * TI) % NT == 0 && NWV >= 1, "write shape");
                __syncthreads();
#pragma unroll
                for(int k = 0; k < NWV; ++k)
                {
                    const uint32_t v = tid + k * NT, jv = v % VPC, i = v / VPC;
                    const bool     ok = (j0 + jv * VW < a.e_j) && (i0 + i < a.e_i);
                    Vec<T, VW>     o;
#pragma unroll
                    for(int e = 0; e < VW; ++e)
                        o.v[e] = tile[at(jv * VW + e, i)];
                    if(ok)
                        store_stream<T, VW>(B + boff + jv * VW + i * a.b_i, o);
                }
            }
        }

        struct SArgs
        {
            const void* A;
            void*       B;
            uint32_t    e_s, e_l; // extents of the short and of the long tile mode
            uint32_t    row_stride; // stride of the short mode on the side that is walked in rows
            uint32_t    magic; // floor(2^32 / e_s) + 1: v / e_s == umulhi(v, magic) for v < 2^28
            uint32_t    nt; // strips along the long mode
            int32_t     nb;
            uint32_t    bext[PERM_BATCH], ba[PERM_BATCH], bb[PERM_BATCH];
            float       alpha;
            int32_t     op_a, op_b;
        };

        // LINEAR_WRITE: the long mode is A's fastest, the short one B's fastest, and B holds the
        // long mode right after the short one, so a strip is one run of cnt * e_s elements of B.
        // It is read in e_s rows of A and written linearly.  !LINEAR_WRITE is the mirror image:
        // the short mode is A's fastest with the long one right after it; the strip is read
        // linearly from A and written in e_s rows of B.
        // Position of a linear index v of a strip: v = x * e_s + s.  One division per thread finds
        // the first position; afterwards the walk only adds (32-bit integer multiplies and
        // divides run at a quarter of the add rate, and this kernel has one per element to spare).
        struct StripPos
        {
            uint32_t s, x;
            __device__ void advance(uint32_t ds, uint32_t dx, uint32_t e_s)
            {
                s += ds;
                x += dx;
                if(s >= e_s)
                {
                    s -= e_s;
                    ++x;
                }
            }
        };

        template <typename T, int TL, int VL, int VS, bool LINEAR_WRITE>
        __global__ __launch_bounds__(PERM_THREADS) void permute_strip_kernel(SArgs a)
        {
            constexpr int NT    = PERM_THREADS;
            constexpr int U     = 8; // loads in flight per thread: a whole 32 KiB strip of full vectors
            constexpr int PITCH = TL + 4 / (int)sizeof(T); // an odd number of 32-bit words: rows start in different banks
            constexpr int VPR   = TL / VS; // row vectors per strip row
            static_assert(TL % VS == 0 && TL % VL == 0, "strip shape");
            extern __shared__ unsigned char strip_smem[];
            T* tile = reinterpret_cast<T*>(strip_smem); // [e_s][PITCH]

            const T* __restrict__ A = static_cast<const T*>(a.A);
            T* __restrict__ B       = static_cast<T*>(a.B);
            const uint32_t tid      = threadIdx.x;

            uint32_t       blk = blockIdx.x;
            const uint32_t t   = blk % a.nt;
            blk /= a.nt;
            uint32_t aoff = 0, boff = 0;
            for(int d = 0; d < a.nb; ++d)
            {
                const uint32_t c = blk % a.bext[d];
                blk /= a.bext[d];
                aoff += c * a.ba[d];
                boff += c * a.bb[d];
            }
            const uint32_t l0  = t * TL;
            const uint32_t cnt = (a.e_l - l0) < (uint32_t)TL ? (a.e_l - l0) : (uint32_t)TL;
            const T        alpha = static_cast<T>(a.alpha);
            const uint32_t nrv   = a.e_s * VPR; // row vectors of the strip (tail rows included)
            const uint32_t nlv   = cnt * a.e_s / VL; // linear vectors of the strip

            // the walk over linear vectors u = tid, tid + NT, ...: first element v = u * VL
            StripPos pos;
            pos.x = __umulhi(tid * VL, a.magic);
            pos.s = tid * VL - pos.x * a.e_s;
            const uint32_t step_x = __umulhi((uint32_t)(NT * VL), a.magic); // scalar
            const uint32_t step_s = NT * VL - step_x * a.e_s;

            if constexpr(LINEAR_WRITE)
            {
                aoff += l0;
                boff += l0 * a.e_s;
                for(uint32_t u0 = 0; u0 < nrv; u0 += NT * U)
                {
                    Vec<T, VS> r[U];
#pragma unroll
                    for(int k = 0; k < U; ++k)
                    {
                        // out-of-range lanes load the strip's first element (no branch: see the tile kernel)
                        const uint32_t u = u0 + tid + k * NT, s = u / VPR, xv = u % VPR;
                        const bool     ok = u < nrv && xv * VS < cnt;
                        r[k] = load_stream<T, VS>(A + aoff + (ok ? xv * VS + s * a.row_stride : 0u));
                    }
#pragma unroll
                    for(int k = 0; k < U; ++k)
                    {
                        const uint32_t u = u0 + tid + k * NT, s = u / VPR, xv = u % VPR;
                        if(u < nrv)
                        {
#pragma unroll
                            for(int e = 0; e < VS; ++e)
                                tile[s * PITCH + xv * VS + e] = element_op(r[k].v[e], alpha, a.op_a, a.op_b);
                        }
                    }
                }
                __syncthreads();
                for(uint32_t u = tid; u < nlv; u += NT)
                {
                    Vec<T, VL> o;
                    StripPos   q = pos;
#pragma unroll
                    for(int e = 0; e < VL; ++e)
                    {
                        o.v[e] = tile[q.s * PITCH + q.x];
                        q.advance(1, 0, a.e_s);
                    }
                    store_stream<T, VL>(B + boff + u * VL, o);
                    pos.advance(step_s, step_x, a.e_s);
                }
            }
            else
            {
                aoff += l0 * a.e_s;
                boff += l0;
                for(uint32_t u0 = 0; u0 < nlv; u0 += NT * U)
                {
                    Vec<T, VL> r[U];
#pragma unroll
                    for(int k = 0; k < U; ++k)
                    {
                        const uint32_t u = u0 + tid + k * NT;
                        r[k] = load_stream<T, VL>(A + aoff + (u < nlv ? u * VL : 0u));
                    }
#pragma unroll
                    for(int k = 0; k < U; ++k)
                    {
                        const uint32_t u = u0 + tid + k * NT;
                        if(u < nlv)
                        {
                            StripPos q = pos;
#pragma unroll
                            for(int e = 0; e < VL; ++e)
                            {
                                tile[q.s * PITCH + q.x] = element_op(r[k].v[e], alpha, a.op_a, a.op_b);
                                q.advance(1, 0, a.e_s);
                            }
                        }
                        pos.advance(step_s, step_x, a.e_s);
                    }
                }
                __syncthreads();
                for(uint32_t u = tid; u < nrv; u += NT)
                {
                    const uint32_t s = u / VPR, xv = u % VPR;
                    if(xv * VS < cnt)
                    {
                        Vec<T, VS> o;
#pragma unroll
                        for(int e = 0; e < VS; ++e)
                            o.v[e] = tile[s * PITCH + xv * VS + e];
                        store_stream<T, VS>(B + boff + xv * VS + s * a.row_stride, o);
                    }
                }
            }
        }

        struct QArgs
        {
            const void* A;
            void*       B;
            uint32_t    e_i0, e_i1, e_j0, e_j1; // extents of the row modes (0, i2) and the column modes (j, j2); 1 if absent
            uint32_t    w_i, w_j; // elements of mode 0 / mode j per tile (== the extent when c > 1)
            uint32_t    c_i, c_j; // indices of i2 / j2 per tile
            uint32_t    a_j0, a_j1, b_i0, b_i1; // A strides of the column modes, B strides of the row modes
            uint32_t    nt_i0, nt_j0, nt_i, nt_j; // tiles along mode 0, mode j, i2 and j2
            uint32_t    pitch; // LDS row pitch in elements: an odd number of 32-bit words
            uint32_t    m_rv, m_wj, m_cv, m_wi; // floor(2^32 / d) + 1 for d = TI / VR, w_j, TJ / VW, w_i
            int32_t     nb;
            uint32_t    bext[PERM_BATCH], ba[PERM_BATCH], bb[PERM_BATCH];
            float       alpha;
            int32_t     op_a, op_b;
        };

        // Row x of a tile is (x0, x1) = (x mod w_i, x div w_i): x0 walks w_i elements of mode 0 and,
        // when the tile takes all of mode 0, x1 walks c_i indices of A's next mode - the two are
        // contiguous in A, so a row is one run of A.  Column y is (y0, y1) over mode j and B's next
        // mode in the same way, one run of B.  Rows are read along x, the tile is parked in LDS as
        // [y][x], and columns are written along y.
        template <typename T, int VR, int VW>
        __global__ __launch_bounds__(PERM_THREADS) void permute_group_kernel(QArgs a)
        {
            constexpr int NT = PERM_THREADS;
            constexpr int U  = 8;
            extern __shared__ unsigned char group_smem[];
            T* tile = reinterpret_cast<T*>(group_smem);

            const T* __restrict__ A = static_cast<const T*>(a.A);
            T* __restrict__ B       = static_cast<T*>(a.B);
            const uint32_t tid      = threadIdx.x;

            uint32_t       blk = blockIdx.x;
            const uint32_t ti0 = blk % a.nt_i0;
            blk /= a.nt_i0;
            const uint32_t tj0 = blk % a.nt_j0;
            blk /= a.nt_j0;
            const uint32_t ti = blk % a.nt_i;
            blk /= a.nt_i;
            const uint32_t tj = blk % a.nt_j;
            blk /= a.nt_j;
            uint32_t aoff = 0, boff = 0;
            for(int d = 0; d < a.nb; ++d)
            {
                const uint32_t c = blk % a.bext[d];
                blk /= a.bext[d];
                aoff += c * a.ba[d];
                boff += c * a.bb[d];
            }
            const uint32_t i0s = ti0 * a.w_i, j0s = tj0 * a.w_j;
            const uint32_t wi = (a.e_i0 - i0s) < a.w_i ? (a.e_i0 - i0s) : a.w_i;
            const uint32_t wj = (a.e_j0 - j0s) < a.w_j ? (a.e_j0 - j0s) : a.w_j;
            const uint32_t i1s = ti * a.c_i, j1s = tj * a.c_j;
            const uint32_t ci = (a.e_i1 - i1s) < a.c_i ? (a.e_i1 - i1s) : a.c_i;
            const uint32_t cj = (a.e_j1 - j1s) < a.c_j ? (a.e_j1 - j1s) : a.c_j;
            // rows and columns inside the extents (c > 1 only with the whole first mode: w == e)
            const uint32_t nx = a.w_i * (ci - 1) + wi, ny = a.w_j * (cj - 1) + wj;
            const uint32_t RV = a.w_i * a.c_i / VR, CV = a.w_j * a.c_j / VW; // vectors per nominal row / column
            aoff += i0s + i1s * a.e_i0 + j0s * a.a_j0 + j1s * a.a_j1;
            boff += i0s * a.b_i0 + i1s * a.b_i1 + j0s + j1s * a.e_j0;
            const T alpha = static_cast<T>(a.alpha);

            const uint32_t total_r = RV * ny;
            for(uint32_t u0 = 0; u0 < total_r; u0 += NT * U)
            {
                Vec<T, VR> r[U];
                uint32_t   at[U];
#pragma unroll
                for(int k = 0; k < U; ++k)
                {
                    const uint32_t v  = u0 + tid + k * NT;
                    const uint32_t y  = __umulhi(v, a.m_rv), xv = v - y * RV;
                    const uint32_t y1 = __umulhi(y, a.m_wj), y0 = y - y1 * a.w_j;
                    const bool     ok = v < total_r && xv * VR < nx;
                    at[k]             = ok ? y * a.pitch + xv * VR : 0xFFFFFFFFu;
                    // out-of-range lanes load the tile's first element: no branch, all loads in flight
                    r[k] = load_stream<T, VR>(A + aoff + (ok ? xv * VR + y0 * a.a_j0 + y1 * a.a_j1 : 0u));
                }
#pragma unroll
                for(int k = 0; k < U; ++k)
                {
                    if(at[k] != 0xFFFFFFFFu)
                    {
#pragma unroll
                        for(int e = 0; e < VR; ++e)
                            tile[at[k] + e] = element_op(r[k].v[e], alpha, a.op_a, a.op_b);
                    }
                }
            }
            __syncthreads();
            const uint32_t total_w = CV * nx;
            for(uint32_t v = tid; v < total_w; v += NT)
            {
                const uint32_t x = __umulhi(v, a.m_cv), yv = v - x * CV;
                if(yv * VW < ny)
                {
                    const uint32_t x1 = __umulhi(x, a.m_wi), x0 = x - x1 * a.w_i;
                    Vec<T, VW>     o;
#pragma unroll
                    for(int e = 0; e < VW; ++e)
                        o.v[e] = tile[(yv * VW + e) * a.pitch + x];
                    store_stream<T, VW>(B + boff + yv * VW + x0 * a.b_i0 + x1 * a.b_i1, o);
                }
            }
        }

        struct HArgs
        {
            const void* A;
            void*       B;
            uint32_t    e_c, e_i, e_j; // extents of mode 0, of A's next mode i and of B's next mode j
            uint32_t    c_i, c_j; // indices of i / j per tile
            uint32_t    a_j, b_i; // A stride of j, B stride of i (a_i == b_j == e_c)
            uint32_t    nt_i, nt_j;
            uint32_t    pitch; // LDS row pitch in elements: an odd number of 32-bit words
            uint32_t    m_rv, m_cv, m_ec; // floor(2^32 / d) + 1 for d = e_c * c_i / VR, e_c * c_j / VW, e_c
            int32_t     nb;
            uint32_t    bext[PERM_BATCH], ba[PERM_BATCH], bb[PERM_BATCH];
            float       alpha;
            int32_t     op_a, op_b;
        };

        // A and B share the fastest mode c.  The tile (c, i-chunk, j-chunk) is read as c_j runs of
        // e_c * c_i elements (c and i are contiguous in A), parked in LDS as [j][i * e_c + c], and
        // written as c_i runs of e_c * c_j elements (c and j are contiguous in B).
        template <typename T, int VR, int VW>
        __global__ __launch_bounds__(PERM_THREADS) void permute_shared_kernel(HArgs a)
        {
            constexpr int NT = PERM_THREADS;
            constexpr int U  = 8;
            extern __shared__ unsigned char shared_smem[];
            T* tile = reinterpret_cast<T*>(shared_smem);

            const T* __restrict__ A = static_cast<const T*>(a.A);
            T* __restrict__ B       = static_cast<T*>(a.B);
            const uint32_t tid      = threadIdx.x;

            uint32_t       blk = blockIdx.x;
            const uint32_t ti  = blk % a.nt_i;
            blk /= a.nt_i;
            const uint32_t tj = blk % a.nt_j;
            blk /= a.nt_j;
            uint32_t aoff = 0, boff = 0;
            for(int d = 0; d < a.nb; ++d)
            {
                const uint32_t c = blk % a.bext[d];
                blk /= a.bext[d];
                aoff += c * a.ba[d];
                boff += c * a.bb[d];
            }
            const uint32_t is = ti * a.c_i, js = tj * a.c_j;
            const uint32_t ci = (a.e_i - is) < a.c_i ? (a.e_i - is) : a.c_i;
            const uint32_t cj = (a.e_j - js) < a.c_j ? (a.e_j - js) : a.c_j;
            const uint32_t nx = a.e_c * ci, ny = a.e_c * cj; // run lengths inside the extents
            const uint32_t RV = a.e_c * a.c_i / VR, CV = a.e_c * a.c_j / VW; // vectors per nominal run
            aoff += is * a.e_c + js * a.a_j;
            boff += is * a.b_i + js * a.e_c;
            const T alpha = static_cast<T>(a.alpha);

            const uint32_t total_r = RV * cj;
            for(uint32_t u0 = 0; u0 < total_r; u0 += NT * U)
            {
                Vec<T, VR> r[U];
                uint32_t   at[U];
#pragma unroll
                for(int k = 0; k < U; ++k)
                {
                    const uint32_t v  = u0 + tid + k * NT;
                    const uint32_t y1 = __umulhi(v, a.m_rv), xv = v - y1 * RV;
                    const bool     ok = v < total_r && xv * VR < nx;
                    at[k]             = ok ? y1 * a.pitch + xv * VR : 0xFFFFFFFFu;
                    r[k] = load_stream<T, VR>(A + aoff + (ok ? xv * VR + y1 * a.a_j : 0u));
                }
#pragma unroll
                for(int k = 0; k < U; ++k)
                {
                    if(at[k] != 0xFFFFFFFFu)
                    {
#pragma unroll
                        for(int e = 0; e < VR; ++e)
                            tile[at[k] + e] = element_op(r[k].v[e], alpha, a.op_a, a.op_b);
                    }
                }
            }
            __syncthreads();
            const uint32_t total_w = CV * ci;
            for(uint32_t v = tid; v < total_w; v += NT)
            {
                const uint32_t x1 = __umulhi(v, a.m_cv), yv = v - x1 * CV;
                if(yv * VW < ny)
                {
                    const uint32_t y1 = __umulhi(yv * VW, a.m_ec), c = yv * VW - y1 * a.e_c;
                    Vec<T, VW>     o;
#pragma unroll
                    for(int e = 0; e < VW; ++e)
                        o.v[e] = tile[y1 * a.pitch + x1 * a.e_c + c + e];
                    store_stream<T, VW>(B + boff + yv * VW + x1 * a.b_i, o);
                }
            }
        }

        template <typename T, int V>
        __global__ __launch_bounds__(PERM_THREADS) void permute_copy_kernel(
            const void* Av, void* Bv, uint32_t nvec, float alphaF, int op_a, int op_b)
        {
            constexpr int U = 4;
            const auto*   A = static_cast<const Vec<T, V>*>(Av);
            auto*         B = static_cast<Vec<T, V>*>(Bv);
            const T       alpha = static_cast<T>(alphaF);
            const uint32_t base = blockIdx.x * (PERM_THREADS * U) + threadIdx.x;
            Vec<T, V>      r[U];
#pragma unroll
            for(int u = 0; u < U; ++u)
            {
                const uint32_t idx = base + u * PERM_THREADS;
                r[u]               = load_stream<T, V>(reinterpret_cast<const T*>(A + (idx < nvec ? idx : 0u)));
            }
#pragma unroll
            for(int u = 0; u < U; ++u)
            {
                const uint32_t idx = base + u * PERM_THREADS;
#pragma unroll
                for(int e = 0; e < V; ++e)
                    r[u].v[e] = element_op(r[u].v[e], alpha, op_a, op_b);
                if(idx < nvec)
                    store_stream<T, V>(reinterpret_cast<T*>(B + idx), r[u]);
            }
        }

        template <typename T>
        __global__ __launch_bounds__(PERM_THREADS) void permute_gather_kernel(GArgs g)
        {
            const uint32_t idx = blockIdx.x * PERM_THREADS + threadIdx.x;
            if(idx >= g.n)
                return;
            // index -> coordinates by multiplication: with m = floor(2^32 / e) + 1 the high word of
            // rem * m is the quotient or one more, for every 32-bit rem; one compare corrects it
            uint32_t rem = idx, aoff = 0;
            for(int d = 0; d < g.rank; ++d)
            {
                const uint32_t e = g.ext[d];
                uint32_t       q = __umulhi(rem, g.magic[d]);
                uint32_t       c = rem - q * e;
                if((int32_t)c < 0)
                {
                    q -= 1;
                    c += e;
                }
                rem = q;
                aoff += c * g.astr[d];
            }
            const T alpha               = static_cast<T>(g.alpha);
            static_cast<T*>(g.B)[idx] = element_op(static_cast<const T*>(g.A)[aoff], alpha, g.op_a, g.op_b);
        }

        // ---------------------------------------------------------------- host side

        struct TileShape
        {
            int ti, tj;
        };
        // element tiles per element size: square, long along i, long along j, and a 64 KiB tile
        // (512 threads, TILED only) whose rows and columns are twice as long as the square's
        constexpr int       NUM_TILES         = 4;
        constexpr TileShape TILES4[NUM_TILES] = {{64, 64}, {256, 16}, {16, 256}, {128, 128}};
        constexpr TileShape TILES2[NUM_TILES] = {{128, 128}, {512, 32}, {32, 512}, {256, 128}};

        template <typename T, int TI, int TJ, int VR, int VW, bool TR, bool BIG>
        int launch_tile(const PArgs& a, uint32_t grid, hipStream_t s)
        {
            if constexpr(BIG)
            {
                if constexpr(TR)
                    hipLaunchKernelGGL((permute_tile_kernel<T, TI, TJ, VR, VW, true, 512, true>), dim3(grid), dim3(512), 0, s, a);
                else
                    return -1;
            }
            else
                hipLaunchKernelGGL((permute_tile_kernel<T, TI, TJ, VR, VW, TR>), dim3(grid), dim3(PERM_THREADS), 0, s, a);
            return (int)hipGetLastError();
        }

        template <typename T, int TI, int TJ, int VMAX, bool BIG = false>
        int launch_tile_vec(bool transpose, int vr, int vw, const PArgs& a, uint32_t grid, hipStream_t s)
        {
#define HIPTK_PERM_CASE(R, W)                                                   \
    if(vr == R && vw == W)                                                      \
        return transpose ? launch_tile<T, TI, TJ, R, W, true, BIG>(a, grid, s)   \
                         : (R == W ? launch_tile<T, TI, TJ, R, R, false, BIG>(a, grid, s) : -1);
            HIPTK_PERM_CASE(1, 1)
            HIPTK_PERM_CASE(1, 2)
            HIPTK_PERM_CASE(1, VMAX)
            HIPTK_PERM_CASE(2, 1)
            HIPTK_PERM_CASE(2, 2)
            HIPTK_PERM_CASE(2, VMAX)
            HIPTK_PERM_CASE(VMAX, 1)
            HIPTK_PERM_CASE(VMAX, 2)
            HIPTK_PERM_CASE(VMAX, VMAX)
#undef HIPTK_PERM_CASE
            return -1;
        }

        template <typename T, int VMAX>
        int launch_tile_shape(int tile, bool transpose, int vr, int vw, const PArgs& a, uint32_t grid, hipStream_t s)
        {
            constexpr const TileShape* TS = sizeof(T) == 4 ? TILES4 : TILES2;
            switch(tile)
            {
            case 0: return launch_tile_vec<T, TS[0].ti, TS[0].tj, VMAX>(transpose, vr, vw, a, grid, s);
            case 1: return launch_tile_vec<T, TS[1].ti, TS[1].tj, VMAX>(transpose, vr, vw, a, grid, s);
            case 2: return launch_tile_vec<T, TS[2].ti, TS[2].tj, VMAX>(transpose, vr, vw, a, grid, s);
            case 3: return launch_tile_vec<T, TS[3].ti, TS[3].tj, VMAX, true>(transpose, vr, vw, a, grid, s);
            default: return -1;
            }
        }

        template <typename T>
        int launch_copy(int vec, const void* A, void* B, uint32_t n, float alpha, int oa, int ob, hipStream_t s)
        {
            const uint32_t nvec = n / vec;
            const uint32_t grid = (nvec + PERM_THREADS * 4 - 1) / (PERM_THREADS * 4);
#define HIPTK_COPY_CASE(V)                                                                                           \
    if(vec == V)                                                                                                     \
    {                                                                                                                \
        hipLaunchKernelGGL((permute_copy_kernel<T, V>), dim3(grid), dim3(PERM_THREADS), 0, s, A, B, nvec, alpha, oa, ob); \
        return (int)hipGetLastError();                                                                               \
    }
            HIPTK_COPY_CASE(1)
            HIPTK_COPY_CASE(2)
            HIPTK_COPY_CASE(4)
            if constexpr(sizeof(T) == 2)
            {
                HIPTK_COPY_CASE(8)
            }
#undef HIPTK_COPY_CASE
            return -1;
        }

        // Strips hold e_s rows of TL elements in LDS (about 32 KiB at most): 2 KiB rows while the
        // short mode has at most 8 elements, 512-byte rows up to 64.
        constexpr int STRIP_MAX_SHORT = 64;
        constexpr int STRIP_WIDE_MAX  = 8;

        constexpr int strip_len(int elem_bytes, int e_s)
        {
            return (e_s <= STRIP_WIDE_MAX ? 2048 : 512) / elem_bytes;
        }

        template <typename T, int VMAX, int TL>
        int launch_strip_len(bool linear_write, int vl, int vs, const SArgs& a, uint32_t grid, hipStream_t s)
        {
            const size_t lds = (size_t)a.e_s * (TL * sizeof(T) + 4);
#define HIPTK_STRIP_CASE(L, S)                                                                                      \
    if(vl == L && vs == S)                                                                                          \
    {                                                                                                               \
        if(linear_write)                                                                                            \
            hipLaunchKernelGGL((permute_strip_kernel<T, TL, L, S, true>), dim3(grid), dim3(PERM_THREADS), lds, s, a);  \
        else                                                                                                        \
            hipLaunchKernelGGL((permute_strip_kernel<T, TL, L, S, false>), dim3(grid), dim3(PERM_THREADS), lds, s, a); \
        return (int)hipGetLastError();                                                                              \
    }
            HIPTK_STRIP_CASE(1, 1)
            HIPTK_STRIP_CASE(1, 2)
            HIPTK_STRIP_CASE(1, VMAX)
            HIPTK_STRIP_CASE(2, 1)
            HIPTK_STRIP_CASE(2, 2)
            HIPTK_STRIP_CASE(2, VMAX)
            HIPTK_STRIP_CASE(VMAX, 1)
            HIPTK_STRIP_CASE(VMAX, 2)
            HIPTK_STRIP_CASE(VMAX, VMAX)
#undef HIPTK_STRIP_CASE
            return -1;
        }

        template <typename T, int VMAX>
        int launch_strip(bool linear_write, int vl, int vs, const SArgs& a, uint32_t grid, hipStream_t s)
        {
            if(a.e_s <= (uint32_t)STRIP_WIDE_MAX)
                return launch_strip_len<T, VMAX, strip_len(sizeof(T), 1)>(linear_write, vl, vs, a, grid, s);
            return launch_strip_len<T, VMAX, strip_len(sizeof(T), STRIP_MAX_SHORT)>(linear_write, vl, vs, a, grid, s);
        }

        constexpr int GROUP_MAX_FAST = 128; // longest fastest mode the grouped kernel takes
        constexpr int GROUP_MAX_LDS  = 60 * 1024;

        uint32_t magic_of(uint32_t d)
        {
            return (uint32_t)((uint64_t(1) << 32) / d) + 1u;
        }

        template <typename T, int VMAX>
        int launch_group(int vr, int vw, const QArgs& a, uint32_t grid, size_t lds, hipStream_t s)
        {
#define HIPTK_GROUP_CASE(R, W)                                                                                     \
    if(vr == R && vw == W)                                                                                         \
    {                                                                                                              \
        hipLaunchKernelGGL((permute_group_kernel<T, R, W>), dim3(grid), dim3(PERM_THREADS), lds, s, a);              \
        return (int)hipGetLastError();                                                                             \
    }
            HIPTK_GROUP_CASE(1, 1)
            HIPTK_GROUP_CASE(1, 2)
            HIPTK_GROUP_CASE(1, VMAX)
            HIPTK_GROUP_CASE(2, 1)
            HIPTK_GROUP_CASE(2, 2)
            HIPTK_GROUP_CASE(2, VMAX)
            HIPTK_GROUP_CASE(VMAX, 1)
            HIPTK_GROUP_CASE(VMAX, 2)
            HIPTK_GROUP_CASE(VMAX, VMAX)
#undef HIPTK_GROUP_CASE
            return -1;
        }

        template <typename T, int VMAX>
        int launch_shared(int v, const HArgs& a, uint32_t grid, size_t lds, hipStream_t s)
        {
#define HIPTK_SHARED_CASE(V)                                                                                  \
    if(v == V)                                                                                                \
    {                                                                                                         \
        hipLaunchKernelGGL((permute_shared_kernel<T, V, V>), dim3(grid), dim3(PERM_THREADS), lds, s, a);        \
        return (int)hipGetLastError();                                                                        \
    }
            HIPTK_SHARED_CASE(1)
            HIPTK_SHARED_CASE(2)
            HIPTK_SHARED_CASE(VMAX)
#undef HIPTK_SHARED_CASE
            return -1;
        }

        bool vec_allowed(int elem_bytes, int v)
        {
            return v == 1 || v == 2 || (elem_bytes == 4 ? v == 4 : v == 8);
        }
        bool copy_vec_allowed(int elem_bytes, int v)
        {
            return v == 1 || v == 2 || v == 4 || (elem_bytes == 2 && v == 8);
        }

        bool aligned(const void* p, int bytes)
        {
            return (reinterpret_cast<uintptr_t>(p) % (uintptr_t)bytes) == 0;
        }

        // Shape checks shared by the name query and the launcher.
        bool well_formed(const hiptk_permute_t* p, int64_t* count)
        {
            if(!p || (p->elem_bytes != 2 && p->elem_bytes != 4) || p->rank < 1 || p->rank > HIPTK_PERM_MAX_RANK)
                return false;
            if(((p->op_a | p->op_b) & ~1) && !(p->op_a == HIPTK_PERM_OP_RAW && p->op_b == 0))
                return false;
            int64_t n = 1;
            for(int d = 0; d < p->rank; ++d)
            {
                if(p->extent[d] < 1 || p->a_stride[d] < 1 || p->b_stride[d] < 1)
                    return false;
                n *= p->extent[d];
                if(n >= (int64_t(1) << 31))
                    return false;
            }
            // A is packed in the order given
            int64_t s = 1;
            for(int d = 0; d < p->rank; ++d)
            {
                if(p->a_stride[d] != s)
                    return false;
                s *= p->extent[d];
            }
            // B is packed in some order of the same modes
            int order[HIPTK_PERM_MAX_RANK];
            for(int d = 0; d < p->rank; ++d)
                order[d] = d;
            std::sort(order, order + p->rank, [p](int x, int y) {
                return p->b_stride[x] != p->b_stride[y] ? p->b_stride[x] < p->b_stride[y] : x < y;
            });
            s = 1;
            for(int d = 0; d < p->rank; ++d)
            {
                if(p->b_stride[order[d]] != s)
                    return false;
                s *= p->extent[order[d]];
            }
            *count = n;
            return true;
        }

        const char* type_tag(int elem_bytes)
        {
            return elem_bytes == 4 ? "f32" : "f16";
        }
    }
}

extern "C" const char* hiptk_permute_kernel_name(const hiptk_permute_t* p)
{
    using namespace hiptk;
    static thread_local char name[96];
    name[0]   = 0;
    int64_t n = 0;
    if(!well_formed(p, &n))
        return name;
    switch(p->kernel)
    {
    case HIPTK_PERM_COPY:
        if(p->rank == 1 && copy_vec_allowed(p->elem_bytes, p->vec_r))
            snprintf(name, sizeof(name), "permute_copy_%s_v%d", type_tag(p->elem_bytes), p->vec_r);
        break;
    case HIPTK_PERM_TILED:
    case HIPTK_PERM_ROWS:
    {
        if(p->tile < 0 || p->tile >= NUM_TILES || !vec_allowed(p->elem_bytes, p->vec_r) || !vec_allowed(p->elem_bytes, p->vec_w))
            break;
        if(p->kernel == HIPTK_PERM_ROWS && (p->vec_r != p->vec_w || p->tile == 3))
            break;
        const TileShape t = (p->elem_bytes == 4 ? TILES4 : TILES2)[p->tile];
        snprintf(name,
                 sizeof(name),
                 "permute_%s_%s_%dx%d_r%d_w%d",
                 p->kernel == HIPTK_PERM_TILED ? "tiled" : "rows",
                 type_tag(p->elem_bytes),
                 t.ti,
                 t.tj,
                 p->vec_r,
                 p->vec_w);
        break;
    }
    case HIPTK_PERM_GATHER: snprintf(name, sizeof(name), "permute_gather_%s", type_tag(p->elem_bytes)); break;
    case HIPTK_PERM_GROUPED:
        if(vec_allowed(p->elem_bytes, p->vec_r) && vec_allowed(p->elem_bytes, p->vec_w) && p->chunk_i >= 1 && p->chunk_j >= 1)
            snprintf(name,
                     sizeof(name),
                     "permute_grouped_%s_%dx%d_r%d_w%d",
                     type_tag(p->elem_bytes),
                     p->width_i * p->chunk_i,
                     p->width_j * p->chunk_j,
                     p->vec_r,
                     p->vec_w);
        break;
    case HIPTK_PERM_SHARED:
        if(vec_allowed(p->elem_bytes, p->vec_r) && p->vec_r == p->vec_w && p->chunk_i >= 1 && p->chunk_j >= 1)
            snprintf(name,
                     sizeof(name),
                     "permute_shared_%s_%dx%dx%d_v%d",
                     type_tag(p->elem_bytes),
                     p->extent[0],
                     p->chunk_i,
                     p->chunk_j,
                     p->vec_r);
        break;
    case HIPTK_PERM_STRIP:
        if((p->tile == 0 || p->tile == 1) && p->mode_j >= 1 && p->mode_j < p->rank && vec_allowed(p->elem_bytes, p->vec_r)
           && vec_allowed(p->elem_bytes, p->vec_w))
            snprintf(name,
                     sizeof(name),
                     "permute_strip_%s_%s_%d_r%d_w%d",
                     type_tag(p->elem_bytes),
                     p->tile == 0 ? "linear_write" : "linear_read",
                     strip_len(p->elem_bytes, p->extent[p->tile == 0 ? p->mode_j : 0]),
                     p->vec_r,
                     p->vec_w);
        break;
    default: break;
    }
    return name;
}

extern "C" int hiptk_permute(const hiptk_permute_t* p, const void* A, void* B, void* stream, int* hip_error)
{
    using namespace hiptk;
    if(hip_error)
        *hip_error = 0;
    int64_t n = 0;
    if(!well_formed(p, &n) || !A || !B)
        return HIPTK_ERR_ARG;
    if(!aligned(A, p->elem_bytes) || !aligned(B, p->elem_bytes))
        return HIPTK_ERR_ARG;
    hipStream_t s  = static_cast<hipStream_t>(stream);
    int         rc = -1;

    if(p->kernel == HIPTK_PERM_COPY)
    {
        const int v = p->vec_r;
        if(p->rank != 1 || !copy_vec_allowed(p->elem_bytes, v))
            return HIPTK_ERR_NO_KERNEL;
        if(n % v != 0 || !aligned(A, v * p->elem_bytes) || !aligned(B, v * p->elem_bytes))
            return HIPTK_ERR_ARG;
        rc = p->elem_bytes == 4 ? launch_copy<float>(v, A, B, (uint32_t)n, p->alpha, p->op_a, p->op_b, s)
                                : launch_copy<_Float16>(v, A, B, (uint32_t)n, p->alpha, p->op_a, p->op_b, s);
    }
    else if(p->kernel == HIPTK_PERM_GATHER)
    {
        GArgs g;
        memset(&g, 0, sizeof(g));
        g.A     = A;
        g.B     = B;
        g.n     = (uint32_t)n;
        g.rank  = p->rank;
        g.alpha = p->alpha;
        g.op_a  = p->op_a;
        g.op_b  = p->op_b;
        int order[HIPTK_PERM_MAX_RANK];
        for(int d = 0; d < p->rank; ++d)
            order[d] = d;
        std::sort(order, order + p->rank, [p](int x, int y) {
            return p->b_stride[x] != p->b_stride[y] ? p->b_stride[x] < p->b_stride[y] : x < y;
        });
        int kept = 0;
        for(int d = 0; d < p->rank; ++d)
        {
            const uint32_t e = (uint32_t)p->extent[order[d]];
            if(e == 1)
                continue; // its coordinate is always 0
            g.ext[kept]   = e;
            g.astr[kept]  = (uint32_t)p->a_stride[order[d]];
            g.magic[kept] = magic_of(e);
            ++kept;
        }
        g.rank = kept;
        const uint32_t grid = (uint32_t)((n + PERM_THREADS - 1) / PERM_THREADS);
        if(p->elem_bytes == 4)
            hipLaunchKernelGGL((permute_gather_kernel<float>), dim3(grid), dim3(PERM_THREADS), 0, s, g);
        else
            hipLaunchKernelGGL((permute_gather_kernel<_Float16>), dim3(grid), dim3(PERM_THREADS), 0, s, g);
        rc = (int)hipGetLastError();
    }
    else if(p->kernel == HIPTK_PERM_TILED || p->kernel == HIPTK_PERM_ROWS)
    {
        const bool transpose = p->kernel == HIPTK_PERM_TILED;
        const int  mi = p->mode_i, mj = p->mode_j;
        if(p->rank < 2 || mi != 0 || mj < 1 || mj >= p->rank || p->tile < 0 || p->tile >= NUM_TILES)
            return HIPTK_ERR_ARG;
        if(!vec_allowed(p->elem_bytes, p->vec_r) || !vec_allowed(p->elem_bytes, p->vec_w))
            return HIPTK_ERR_NO_KERNEL;
        if(!transpose && p->vec_r != p->vec_w)
            return HIPTK_ERR_NO_KERNEL;
        // the layout each kernel assumes
        if(transpose ? p->b_stride[mj] != 1 : p->b_stride[0] != 1)
            return HIPTK_ERR_ARG;
        // what the vector widths assume: whole vectors inside the extents, every other
        // stride and both base pointers multiples of the vector
        const int vr = p->vec_r, vw = p->vec_w;
        if(p->extent[0] % vr != 0 || !aligned(A, vr * p->elem_bytes))
            return HIPTK_ERR_ARG;
        for(int d = 1; d < p->rank; ++d)
            if(p->a_stride[d] % vr != 0)
                return HIPTK_ERR_ARG;
        const int wmode = transpose ? mj : 0; // the mode stores run along
        if(p->extent[wmode] % vw != 0 || !aligned(B, vw * p->elem_bytes))
            return HIPTK_ERR_ARG;
        for(int d = 0; d < p->rank; ++d)
            if(d != wmode && p->b_stride[d] % vw != 0)
                return HIPTK_ERR_ARG;

        const TileShape t = (p->elem_bytes == 4 ? TILES4 : TILES2)[p->tile];
        PArgs           a;
        memset(&a, 0, sizeof(a));
        a.A     = A;
        a.B     = B;
        a.e_i   = (uint32_t)p->extent[0];
        a.e_j   = (uint32_t)p->extent[mj];
        a.a_j   = (uint32_t)p->a_stride[mj];
        a.b_i   = (uint32_t)p->b_stride[0];
        a.b_j   = (uint32_t)p->b_stride[mj];
        a.nt_i  = (a.e_i + t.ti - 1) / t.ti;
        a.nt_j  = (a.e_j + t.tj - 1) / t.tj;
        a.group = p->group == 0 ? 0u : (uint32_t)std::max(1, std::min(p->group, (int32_t)a.nt_j));
        a.alpha = p->alpha;
        a.op_a  = p->op_a;
        a.op_b  = p->op_b;
        int64_t grid = (int64_t)a.nt_i * a.nt_j;
        for(int d = 1; d < p->rank; ++d)
        {
            if(d == mj)
                continue;
            a.bext[a.nb] = (uint32_t)p->extent[d];
            a.ba[a.nb]   = (uint32_t)p->a_stride[d];
            a.bb[a.nb]   = (uint32_t)p->b_stride[d];
            ++a.nb;
            grid *= p->extent[d];
        }
        if(grid >= (int64_t(1) << 31))
            return HIPTK_ERR_ARG;
        rc = p->elem_bytes == 4 ? launch_tile_shape<float, 4>(p->tile, transpose, vr, vw, a, (uint32_t)grid, s)
                                : launch_tile_shape<_Float16, 8>(p->tile, transpose, vr, vw, a, (uint32_t)grid, s);
    }
    else if(p->kernel == HIPTK_PERM_GROUPED)
    {
        const int mj = p->mode_j, mi2 = p->mode_i2, mj2 = p->mode_j2;
        if(p->rank < 2 || p->mode_i != 0 || mj < 1 || mj >= p->rank || p->b_stride[mj] != 1)
            return HIPTK_ERR_ARG;
        if(!vec_allowed(p->elem_bytes, p->vec_r) || !vec_allowed(p->elem_bytes, p->vec_w))
            return HIPTK_ERR_NO_KERNEL;
        // the second modes, where present, directly follow the first ones in memory and are
        // distinct from every other tile mode
        if(mi2 != -1 && (mi2 < 1 || mi2 >= p->rank || mi2 == mj || mi2 == mj2 || p->a_stride[mi2] != p->extent[0]))
            return HIPTK_ERR_ARG;
        if(mj2 != -1 && (mj2 < 1 || mj2 >= p->rank || mj2 == mj || p->b_stride[mj2] != p->extent[mj]))
            return HIPTK_ERR_ARG;
        const int e_i1 = mi2 == -1 ? 1 : p->extent[mi2], e_j1 = mj2 == -1 ? 1 : p->extent[mj2];
        const int w_i = p->width_i, w_j = p->width_j;
        if(w_i < 1 || w_i > p->extent[0] || w_j < 1 || w_j > p->extent[mj] || p->chunk_i < 1 || p->chunk_j < 1
           || p->chunk_i > e_i1 || p->chunk_j > e_j1)
            return HIPTK_ERR_ARG;
        // a tile takes several indices of a second mode only together with the whole first mode
        if((p->chunk_i > 1 && w_i != p->extent[0]) || (p->chunk_j > 1 && w_j != p->extent[mj]))
            return HIPTK_ERR_ARG;
        // vectors: whole vectors inside the tile widths and the fastest modes, every other stride
        // and both bases aligned
        const int vr = p->vec_r, vw = p->vec_w;
        if(p->extent[0] % vr != 0 || p->extent[mj] % vw != 0 || w_i % vr != 0 || w_j % vw != 0 || !aligned(A, vr * p->elem_bytes)
           || !aligned(B, vw * p->elem_bytes))
            return HIPTK_ERR_ARG;
        for(int d = 1; d < p->rank; ++d)
            if(p->a_stride[d] % vr != 0)
                return HIPTK_ERR_ARG;
        for(int d = 0; d < p->rank; ++d)
            if(d != mj && p->b_stride[d] % vw != 0)
                return HIPTK_ERR_ARG;

        QArgs a;
        memset(&a, 0, sizeof(a));
        a.A    = A;
        a.B    = B;
        a.e_i0 = (uint32_t)p->extent[0];
        a.e_i1 = (uint32_t)e_i1;
        a.e_j0 = (uint32_t)p->extent[mj];
        a.e_j1 = (uint32_t)e_j1;
        a.w_i  = (uint32_t)w_i;
        a.w_j  = (uint32_t)w_j;
        a.c_i  = (uint32_t)p->chunk_i;
        a.c_j  = (uint32_t)p->chunk_j;
        a.a_j0 = (uint32_t)p->a_stride[mj];
        a.a_j1 = mj2 == -1 ? 0u : (uint32_t)p->a_stride[mj2];
        a.b_i0 = (uint32_t)p->b_stride[0];
        a.b_i1 = mi2 == -1 ? 0u : (uint32_t)p->b_stride[mi2];
        a.nt_i0 = (a.e_i0 + a.w_i - 1) / a.w_i;
        a.nt_j0 = (a.e_j0 + a.w_j - 1) / a.w_j;
        a.nt_i  = (a.e_i1 + a.c_i - 1) / a.c_i;
        a.nt_j  = (a.e_j1 + a.c_j - 1) / a.c_j;
        const uint32_t TI = a.w_i * a.c_i, TJ = a.w_j * a.c_j;
        const uint32_t wordElems = 4u / (uint32_t)p->elem_bytes; // elements per 32-bit word
        uint32_t       pitchWords = (TI + wordElems - 1) / wordElems;
        pitchWords |= 1u; // odd: consecutive rows start in different banks
        a.pitch          = pitchWords * wordElems;
        const size_t lds = (size_t)TJ * a.pitch * p->elem_bytes;
        if(lds > (size_t)GROUP_MAX_LDS || TI / vr < 2 || TJ / vw < 2 || w_i < 2 || w_j < 2)
            return HIPTK_ERR_ARG; // (the reciprocals below are exact for divisors of 2 and more)
        a.m_rv = magic_of(TI / vr);
        a.m_wj = magic_of(a.w_j);
        a.m_cv = magic_of(TJ / vw);
        a.m_wi = magic_of(a.w_i);
        a.alpha = p->alpha;
        a.op_a  = p->op_a;
        a.op_b  = p->op_b;
        int64_t grid = (int64_t)a.nt_i0 * a.nt_j0 * a.nt_i * a.nt_j;
        for(int d = 1; d < p->rank; ++d)
        {
            if(d == mj || d == mi2 || d == mj2)
                continue;
            a.bext[a.nb] = (uint32_t)p->extent[d];
            a.ba[a.nb]   = (uint32_t)p->a_stride[d];
            a.bb[a.nb]   = (uint32_t)p->b_stride[d];
            ++a.nb;
            grid *= p->extent[d];
        }
        if(grid >= (int64_t(1) << 31))
            return HIPTK_ERR_ARG;
        rc = p->elem_bytes == 4 ? launch_group<float, 4>(vr, vw, a, (uint32_t)grid, lds, s)
                                : launch_group<_Float16, 8>(vr, vw, a, (uint32_t)grid, lds, s);
    }
    else if(p->kernel == HIPTK_PERM_SHARED)
    {
        const int mi = p->mode_i2, mj = p->mode_j2, v = p->vec_r;
        if(p->rank < 3 || p->mode_i != 0 || p->b_stride[0] != 1 || mi < 1 || mi >= p->rank || mj < 1 || mj >= p->rank || mi == mj)
            return HIPTK_ERR_ARG;
        if(p->a_stride[mi] != p->extent[0] || p->b_stride[mj] != p->extent[0])
            return HIPTK_ERR_ARG;
        if(!vec_allowed(p->elem_bytes, v) || p->vec_w != v)
            return HIPTK_ERR_NO_KERNEL;
        if(p->extent[0] > GROUP_MAX_FAST || p->chunk_i < 1 || p->chunk_j < 1 || p->chunk_i > p->extent[mi] || p->chunk_j > p->extent[mj])
            return HIPTK_ERR_ARG;
        if(p->extent[0] % v != 0 || !aligned(A, v * p->elem_bytes) || !aligned(B, v * p->elem_bytes))
            return HIPTK_ERR_ARG;
        for(int d = 1; d < p->rank; ++d)
            if(p->a_stride[d] % v != 0 || p->b_stride[d] % v != 0)
                return HIPTK_ERR_ARG;
        HArgs a;
        memset(&a, 0, sizeof(a));
        a.A    = A;
        a.B    = B;
        a.e_c  = (uint32_t)p->extent[0];
        a.e_i  = (uint32_t)p->extent[mi];
        a.e_j  = (uint32_t)p->extent[mj];
        a.c_i  = (uint32_t)p->chunk_i;
        a.c_j  = (uint32_t)p->chunk_j;
        a.a_j  = (uint32_t)p->a_stride[mj];
        a.b_i  = (uint32_t)p->b_stride[mi];
        a.nt_i = (a.e_i + a.c_i - 1) / a.c_i;
        a.nt_j = (a.e_j + a.c_j - 1) / a.c_j;
        const uint32_t TI = a.e_c * a.c_i, TJ = a.e_c * a.c_j;
        const uint32_t wordElems  = 4u / (uint32_t)p->elem_bytes;
        uint32_t       pitchWords = (TI + wordElems - 1) / wordElems;
        pitchWords |= 1u;
        a.pitch          = pitchWords * wordElems;
        const size_t lds = (size_t)a.c_j * a.pitch * p->elem_bytes;
        if(lds > (size_t)GROUP_MAX_LDS || TI / v < 2 || TJ / v < 2)
            return HIPTK_ERR_ARG;
        a.m_rv  = magic_of(TI / v);
        a.m_cv  = magic_of(TJ / v);
        a.m_ec  = magic_of(a.e_c);
        a.alpha = p->alpha;
        a.op_a  = p->op_a;
        a.op_b  = p->op_b;
        int64_t grid = (int64_t)a.nt_i * a.nt_j;
        for(int d = 1; d < p->rank; ++d)
        {
            if(d == mi || d == mj)
                continue;
            a.bext[a.nb] = (uint32_t)p->extent[d];
            a.ba[a.nb]   = (uint32_t)p->a_stride[d];
            a.bb[a.nb]   = (uint32_t)p->b_stride[d];
            ++a.nb;
            grid *= p->extent[d];
        }
        if(grid >= (int64_t(1) << 31))
            return HIPTK_ERR_ARG;
        rc = p->elem_bytes == 4 ? launch_shared<float, 4>(v, a, (uint32_t)grid, lds, s)
                                : launch_shared<_Float16, 8>(v, a, (uint32_t)grid, lds, s);
    }
    else if(p->kernel == HIPTK_PERM_STRIP)
    {
        // tile == 0: long mode 0 (A's fastest), short mode mode_j (B's fastest), B holds mode 0
        //            right after it; the strip is linear in B.
        // tile == 1: short mode 0 (A's fastest) with long mode mode_j right after it in A and
        //            fastest in B; the strip is linear in A.
        const int  mj           = p->mode_j;
        const bool linear_write = p->tile == 0;
        if(p->rank < 2 || p->mode_i != 0 || mj < 1 || mj >= p->rank || (p->tile != 0 && p->tile != 1))
            return HIPTK_ERR_ARG;
        if(!vec_allowed(p->elem_bytes, p->vec_r) || !vec_allowed(p->elem_bytes, p->vec_w))
            return HIPTK_ERR_NO_KERNEL;
        const int ms = linear_write ? mj : 0, ml = linear_write ? 0 : mj; // short, long
        if(p->extent[ms] > STRIP_MAX_SHORT || p->b_stride[mj] != 1)
            return HIPTK_ERR_ARG;
        if(linear_write ? p->b_stride[0] != p->extent[mj] : p->a_stride[mj] != p->extent[0])
            return HIPTK_ERR_ARG;
        // vector preconditions: the linear side needs whole vectors in every strip and aligned
        // strip starts, the row side whole vectors in every row
        const int     vr = p->vec_r, vw = p->vec_w;
        const int     vl = linear_write ? vw : vr, vs = linear_write ? vr : vw;
        const int64_t run = (int64_t)p->extent[0] * p->extent[mj];
        const int32_t* lin_stride = linear_write ? p->b_stride : p->a_stride;
        const int32_t* row_stride = linear_write ? p->a_stride : p->b_stride;
        if(run % vl != 0 || p->extent[ml] % vs != 0)
            return HIPTK_ERR_ARG;
        for(int d = 1; d < p->rank; ++d)
        {
            if(d != mj && lin_stride[d] % vl != 0)
                return HIPTK_ERR_ARG;
            if((d != mj || linear_write) && row_stride[d] % vs != 0)
                return HIPTK_ERR_ARG;
        }
        if(!linear_write && p->b_stride[0] % vs != 0)
            return HIPTK_ERR_ARG;
        if(!aligned(A, vr * p->elem_bytes) || !aligned(B, vw * p->elem_bytes))
            return HIPTK_ERR_ARG;

        const int TL = strip_len(p->elem_bytes, p->extent[ms]);
        SArgs     a;
        memset(&a, 0, sizeof(a));
        a.A          = A;
        a.B          = B;
        a.e_s        = (uint32_t)p->extent[ms];
        a.e_l        = (uint32_t)p->extent[ml];
        a.row_stride = (uint32_t)(linear_write ? p->a_stride[mj] : p->b_stride[0]);
        a.magic      = (uint32_t)((uint64_t(1) << 32) / a.e_s) + 1u;
        a.nt         = (a.e_l + TL - 1) / TL;
        a.alpha      = p->alpha;
        a.op_a       = p->op_a;
        a.op_b       = p->op_b;
        int64_t grid = a.nt;
        for(int d = 1; d < p->rank; ++d)
        {
            if(d == mj)
                continue;
            a.bext[a.nb] = (uint32_t)p->extent[d];
            a.ba[a.nb]   = (uint32_t)p->a_stride[d];
            a.bb[a.nb]   = (uint32_t)p->b_stride[d];
            ++a.nb;
            grid *= p->extent[d];
        }
        if(grid >= (int64_t(1) << 31))
            return HIPTK_ERR_ARG;
        rc = p->elem_bytes == 4 ? launch_strip<float, 4>(linear_write, vl, vs, a, (uint32_t)grid, s)
                                : launch_strip<_Float16, 8>(linear_write, vl, vs, a, (uint32_t)grid, s);
    }
    else
        return HIPTK_ERR_NO_KERNEL;

    if(rc == -1)
        return HIPTK_ERR_NO_KERNEL;
    if(hip_error)
        *hip_error = rc;
    return rc == 0 ? HIPTK_OK : HIPTK_ERR_LAUNCH;
}
