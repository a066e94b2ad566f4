// Contraction planner: turns (extents, strides, mode labels) of A, B, C, D into one
// GEMM view whose addressing is carried by eight one-dimensional offset tables.
//
// It takes the place of the reference's normalizeTensorModes
// (library/src/contraction/contraction_solution.cpp:34-160), which pads every problem
// to 6 M + 6 N + 6 K modes on each execute call and hands the 12-long arrays to
// Composable Kernel.  Here the regrouping happens once, at plan time; modes are
// additionally ordered and fused by stride so that contiguous runs are as long as
// the layout allows, and the vector width / direction of every operand's gather is
// derived from those runs.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace hipta
{
    // hipDataType / hiptensorComputeType_t values as plain ints (no HIP headers needed)
    struct TensorIn
    {
        int                  dtype = -1; // hipDataType
        std::vector<int64_t> len, stride;
        std::vector<int32_t> mode;
        uint32_t             align = 0; // bytes, as given to InitContractionDescriptor
    };

    struct ProblemIn
    {
        TensorIn A, B, C, D; // C.dtype < 0  => scale
        bool     bilinear = false;
        int      compute  = 0; // hiptensorComputeType_t
    };

    enum class PlanStatus
    {
        OK,
        INVALID, // inconsistent extents / modes
        UNSUPPORTED_TYPES, // no kernel class for (types, compute)
        UNSUPPORTED_SHAPE // batch modes, repeated labels, offsets beyond 2^31 elements, empty
    };

    struct Dim
    {
        int64_t len = 1;
        int64_t sx = 0, sy = 0, sc = 0, sd = 0; // strides in X / Y / C / D (0 where absent)
    };

    struct GemmView
    {
        int     cls = -1; // HIPTK_* element class
        bool    bilinear = false;
        bool    swapped  = false; // true: X = B, Y = A  (q runs over the M modes)
        int64_t P = 1, Q = 1, K = 1;
        std::vector<Dim> pdims, qdims, kdims; // after ordering and fusion, fastest first
        // offset tables (element units), padded as the kernel ABI requires
        std::vector<int32_t> xp, xk, yq, yk, cp, cq, dp, dq;
        int x_kfast = 1, y_kfast = 1, x_vec = 1, y_vec = 1, cd_vec = 1;
        // the K modes fused into (at most) one: k offsets are k * stride
        int     k_affine = 0;
        int64_t xk_stride = 0, yk_stride = 0;
        // P and Q each fused into (at most) one dim in C and D: offsets are index * stride
        int     cd_affine = 0;
        int64_t dp_stride = 0, dq_stride = 0, cp_stride = 0, cq_stride = 0;
        // vectors run along a row (column) index that is one contiguous run whose extent is not a
        // multiple of the vector: tiles that would overhang are moved back to end at P (Q)
        int shift_p = 0, shift_q = 0;
        // every 16-byte vector of X and Y starts a multiple of 16 bytes from its tensor's base
        int xy_aligned = 0;
        // largest element offset of X / Y that the tables address
        int64_t xp_stride = 0, yq_stride = 0; // with cd_affine: element stride of the one row mode of X / column mode of Y
        int64_t x_max_off = 0, y_max_off = 0;
        // k-contiguous operand: the vectors of consecutive rows are neighbours in memory more often than consecutive
        // vectors of one row (a hint for the kernels' LDS layout)
        int x_rows_adjacent = 0, y_rows_adjacent = 0;
        int elem_bytes = 0;
        // bytes each tensor spans in memory (1 + sum (len-1)*stride elements)
        int64_t spanA = 0, spanB = 0, spanC = 0, spanD = 0;
    };

    // Maps (data type of A/B/C/D, compute type) to a kernel class; -1 if none.
    int  kernel_class(int typeA, int typeB, int typeC, int typeD, bool bilinear, int compute);
    int  class_elem_bytes(int cls);
    int  class_max_vec(int cls);

    PlanStatus build_view(const ProblemIn& in, GemmView& out, std::string& why);

    // 1 + sum (len - 1) * stride, 0 for an empty tensor
    int64_t span_elems(const std::vector<int64_t>& len, const std::vector<int64_t>& stride);
}
