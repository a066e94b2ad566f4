/*
 * Kernel-layer C ABI: the only interface between the host-side planner (plain
 * C++) and the HIP translation units.  Everything crossing it is a plain pointer,
 * an integer or the POD below; no kernel template is visible to host code.
 *
 * It takes the place of the Composable Kernel device-operation objects that the
 * reference drives through BaseOperator / BaseArgument / BaseInvoker pointers
 * (library/src/contraction/contraction_solution.hpp:147-150) and whose Run() is
 * the device boundary (library/src/contraction/contraction_solution.cpp:258).
 *
 * A contraction arrives here already folded into one GEMM view
 *     acc[p][q] = sum_k X[xp[p] + xk[k]] * Y[yq[q] + yk[k]]
 *     D[dp[p] + dq[q]] = alpha * acc[p][q] (+ beta * C[cp[p] + cq[q]])
 * where the eight offset tables (element units, device memory) carry every mode
 * extent and stride of the original tensors.
 */
#ifndef HIPTK_KERNELS_H
#define HIPTK_KERNELS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element classes the kernels are instantiated for */
enum
{
    HIPTK_F16  = 0, /* f16 storage, f16 MFMA inputs, f32 accumulate        */
    HIPTK_BF16 = 1, /* bf16 storage, bf16 MFMA inputs, f32 accumulate      */
    HIPTK_F32  = 2, /* f32 storage, f32 MFMA                              */
    HIPTK_F64  = 3, /* f64 storage, f64 MFMA                              */
    HIPTK_C32  = 4, /* complex f32 storage, f32 MFMA on (re,im) K pairs    */
    HIPTK_C64  = 5, /* complex f64 storage, f64 MFMA on (re,im) K pairs    */
    HIPTK_F32_AS_F16  = 6, /* f32 storage, inputs rounded to f16 when staged  */
    HIPTK_F32_AS_BF16 = 7, /* f32 storage, inputs rounded to bf16 when staged */
    HIPTK_F64_AS_F32  = 8, /* f64 storage, inputs narrowed to f32 when staged */
    HIPTK_NUM_CLASSES = 9
};

enum
{
    HIPTK_OP_SCALE    = 0,
    HIPTK_OP_BILINEAR = 1
};

enum
{
    HIPTK_OK             = 0,
    HIPTK_ERR_ARG        = 1, /* malformed problem (caught on the host, nothing launched) */
    HIPTK_ERR_NO_KERNEL  = 2, /* no instantiation for (class, tile, layout, vector)       */
    HIPTK_ERR_WORKSPACE  = 3, /* split-K asked for and workspace too small                */
    HIPTK_ERR_LAUNCH     = 4  /* hipLaunchKernel reported an error                        */
};

/* One tile configuration of one element class. */
typedef struct hiptk_tile_info
{
    int32_t tile_id;
    int32_t bp, bq, bk; /* workgroup tile                                    */
    int32_t threads;    /* workgroup size                                    */
    int32_t lds_bytes;  /* static LDS                                        */
    char    name[64];
    int32_t k_multiple; /* 0: operand tiles staged through registers, any K.  Otherwise the tile loads
                           them straight into LDS: K must be a multiple of this (1: any) and at least bk,
                           and the problem xy_aligned                          */
    int32_t mfma_k;     /* 32: a 16-bit tile built on v_mfma_f32_16x16x32 (else 0)   */
} hiptk_tile_info_t;

typedef struct hiptk_problem
{
    int32_t cls;     /* HIPTK_F16 ...                                         */
    int32_t op;      /* HIPTK_OP_SCALE / HIPTK_OP_BILINEAR                    */
    int32_t tile_id; /* index into the class's tile list                      */
    int32_t split_k; /* >= 1; > 1 needs workspace                             */
    int64_t P, Q, K; /* GEMM view extents (rows, columns, reduction)          */
    /* offset tables, element units.  xp / cp / dp hold P entries followed by valid
     * offsets (e.g. 0) up to roundup(P, 256) + 256 entries, so that a tile that
     * overhangs P reads something harmless; yq / cq / dq likewise for Q; xk / yk
     * hold K entries followed by zeros up to roundup(K, 256) + 256 entries (the
     * kernels read k offsets up to three K tiles ahead).                         */
    const int32_t *xp, *xk, *yq, *yk, *cp, *cq, *dp, *dq;
    int32_t x_kfast; /* 1: X vectors run along k, 0: along p                   */
    int32_t y_kfast; /* 1: Y vectors run along k, 0: along q                   */
    int32_t x_vec;   /* contiguous elements per X vector (1 = scalar gather)   */
    int32_t y_vec;
    int32_t cd_vec;  /* contiguous elements along q shared by C and D          */
    int32_t k_affine; /* 1: xk[k] == k * xk_stride and yk[k] == k * yk_stride for all k < K;
                         a kernel that multiplies instead of reading xk / yk is used when
                         one is instantiated (the tables must still be valid)          */
    int32_t xk_stride, yk_stride;
    int32_t cd_affine; /* 1: dp[p] == p * dp_stride, dq[q] == q * dq_stride (and likewise cp / cq
                          for a bilinear problem) for all p < P, q < Q: the epilogue then computes
                          offsets instead of reading the tables (which must still be valid)      */
    int32_t dp_stride, dq_stride, cp_stride, cq_stride;
    int32_t xp_stride, yq_stride; /* with cd_affine = 1 also: xp[p] == p * xp_stride and yq[q] == q * yq_stride for p < P,
                                     q < Q (the rows of X and the columns of Y are one mode each): kernels may then
                                     compute their operands' row offsets as well (0: look them up)               */
    int32_t shift_p; /* 1: the rows are one contiguous run of P elements in every tensor that is read
                        or written in vectors along them, P need not be a multiple of the vector: a
                        tile that would overhang P is moved back to end at P (it recomputes some of
                        its neighbour's rows and stores only its own).  Needs P >= the tile's rows;
                        tiles that do not fit are reported as unavailable                          */
    int32_t shift_q; /* likewise for the columns                                                    */
    int32_t xy_aligned; /* 1: every 16-byte vector of X and Y starts a multiple of 16 bytes from its
                           tensor's base (table entries at vector starts are multiples of the vector,
                           no tile is moved back along a vector direction).  The kernels that load
                           their operand tiles straight into LDS take only such problems, and only
                           when the base addresses are 16-byte aligned too (checked at the launch,
                           which otherwise runs the class's largest register-staged tile instead)  */
    int32_t x_max_off, y_max_off; /* largest element offset xp[p] + xk[k] (yq[q] + yk[k]) over p < P, k < K:
                                     the kernels that build load addresses from table entries they have
                                     themselves moved through LDS clamp every address to it, and the
                                     direct-load kernels are offered only while the byte offset of the
                                     last vector fits 32 bits */
    int32_t x_rows_adjacent, y_rows_adjacent; /* a hint, for a k-contiguous operand only: 1 when the vectors of
                                     consecutive rows follow one another in memory more often than consecutive
                                     vectors of one row do (xp[p + 1] - xp[p] == x_vec against xk[k + x_vec] -
                                     xk[k] == x_vec).  The kernels that load operand tiles straight into LDS and
                                     read k offsets from the tables then stage the operand chunk-major, so that
                                     neighbouring lanes load neighbouring memory.  Any value gives the same results */
    /* Filled by hiptk_resolve (zero otherwise): the registry entries this problem runs, looked up once
     * when the plan is made instead of at every launch.  `kernel` is what hiptk_kernel_name names;
     * `kernel_unaligned` is what runs in its place when X or Y is not 16-byte aligned at the launch (the
     * same entry, unless `kernel` loads operand tiles straight into LDS).  Both are tied to the fields
     * above: a caller that changes any of them afterwards clears these two (or resolves again). */
    const void *kernel, *kernel_unaligned;
} hiptk_problem_t;

/* Number of tile configurations of a class, and their description. */
int hiptk_tile_count(int cls);
int hiptk_tile_info(int cls, int tile_id, hiptk_tile_info_t* out);

/* 1 when a kernel is instantiated for the problem's (class, tile, layout, vector)
 * combination; its name ("" if none). */
int         hiptk_kernel_available(const hiptk_problem_t* prob);
const char* hiptk_kernel_name(const hiptk_problem_t* prob);

/* Looks the problem's kernels up once and stores them in prob->kernel / prob->kernel_unaligned, so
 * that hiptk_contract does not search the registry at every launch.  HIPTK_ERR_NO_KERNEL if there is
 * none.  Optional: hiptk_contract searches when the two fields are null. */
int hiptk_resolve(hiptk_problem_t* prob);
/* Name of the kernel a launch with these operand addresses runs: the resolved (or looked-up) kernel,
 * or its register-staged stand-in when X or Y is not 16-byte aligned. */
const char* hiptk_kernel_name_at(const hiptk_problem_t* prob, const void* X, const void* Y);

/* Bytes of workspace the problem needs (0 when split_k == 1). */
uint64_t hiptk_workspace_bytes(const hiptk_problem_t* prob);

/* Enqueue the contraction on `stream` (a hipStream_t passed as void*).  alpha and
 * beta point to host scalars: float for the 16/32-bit real classes, double for
 * HIPTK_F64 and HIPTK_F64_AS_F32, float[2] for HIPTK_C32, double[2] for HIPTK_C64.
 * Returns a HIPTK_* code; *hip_error (optional) receives the hipError_t. */
int hiptk_contract(const hiptk_problem_t* prob,
                   const void*            alpha,
                   const void*            beta,
                   const void*            X,
                   const void*            Y,
                   const void*            C,
                   void*                  D,
                   void*                  workspace,
                   uint64_t               workspace_bytes,
                   void*                  stream,
                   int*                   hip_error);

/* Device address and size of the workspace the library itself holds on the current device: a
 * file-scope device array of HIPTK_STATIC_WORKSPACE_BYTES, present on every device from the moment
 * the library is loaded until the process ends.  The first call on a device looks the address up
 * (hipGetSymbolAddress; nothing is allocated), later calls return the stored address.  No
 * counterpart in the reference; it serves hiptensorAmdContractionNoAlloc, the entry point for
 * callers that cannot allocate.  Every user of the address on one device shares the same bytes. */
#define HIPTK_STATIC_WORKSPACE_BYTES (32u << 20)
int hiptk_static_workspace(void** ptr, uint64_t* bytes, int* hip_error);

/* Fills `bytes` (a multiple of 4) of device memory with pseudo-random finite elements of the
 * class's storage type, magnitudes in [0.5, 1) and random signs, on `stream`.  No counterpart
 * in the reference: the measured kernel selection times its candidates on such data, since
 * the clock this device sustains depends on the operand values. */
int hiptk_fill_pattern(void* dst, uint64_t bytes, int cls, void* stream);

/* ------------------------------------------------------------------------------------------
 * Tensor permutation, B[perm(index)] = opB(alpha * opA(A[index])).  Takes the place of the
 * Composable Kernel DeviceElementwise objects the reference drives for this operation
 * (library/src/permutation/permutation_solution_impl.hpp:134-152,
 * library/src/permutation/permutation_solution.cpp).  The problem arrives with modes already
 * fused: extent / a_stride / b_stride are listed in A's order, a_stride[0] == 1.
 * ------------------------------------------------------------------------------------------ */
enum
{
    HIPTK_PERM_COPY   = 0, /* one fused mode: a scaled copy                                      */
    HIPTK_PERM_TILED  = 1, /* A's fastest mode (mode_i) and B's fastest mode (mode_j) differ:
                              two-dimensional tiles of those two modes go through LDS, read along
                              mode_i and written along mode_j                                     */
    HIPTK_PERM_ROWS   = 2, /* both tensors share the fastest mode (mode_i == 0): runs of that mode
                              are copied, tiles span it and one further mode (mode_j)             */
    HIPTK_PERM_GATHER = 3, /* one thread per element of B, any layout                             */
    HIPTK_PERM_STRIP  = 4, /* TILED with one tile mode of at most 64 elements whose partner follows it
                              directly in memory on that side: a strip of the long mode times the
                              whole short mode is one contiguous run there.  tile == 0: mode_j is the
                              short one and the run lies in B; tile == 1: mode 0 is the short one and
                              the run lies in A                                                   */
    HIPTK_PERM_GROUPED = 5, /* TILED with run-time tile shapes, for short fastest modes: a tile row
                              spans width_i elements of mode 0 and, when width_i == extent[0],
                              chunk_i indices of A's next mode (mode_i2, contiguous in A); a tile
                              column width_j elements of mode_j and, when width_j == extent[mode_j],
                              chunk_j indices of B's next mode (mode_j2, contiguous in B); a second
                              mode may be absent (-1, chunk 1)                                    */
    HIPTK_PERM_SHARED = 6  /* ROWS for a short shared fastest mode (at most 128 elements, e.g. the
                              four channels of RGBA pixels): a tile is mode 0 times chunk_i indices of
                              A's next mode (mode_i2) times chunk_j indices of B's next mode (mode_j2);
                              it is read in runs of extent[0] * chunk_i and, through LDS, written in
                              runs of extent[0] * chunk_j                                        */
};

#define HIPTK_PERM_MAX_RANK 6
#define HIPTK_PERM_OP_RAW 2

typedef struct hiptk_permute
{
    int32_t elem_bytes; /* 2: f16, 4: f32                                                        */
    int32_t rank;       /* fused modes, 1..6                                                      */
    int32_t extent[HIPTK_PERM_MAX_RANK];
    int32_t a_stride[HIPTK_PERM_MAX_RANK]; /* elements                                            */
    int32_t b_stride[HIPTK_PERM_MAX_RANK];
    int32_t op_a, op_b; /* 0: identity, 1: square; op_a = HIPTK_PERM_OP_RAW (with op_b = 0): the bits
                         * are moved as they are, alpha is not applied                           */
    float   alpha;      /* multiplies in float for f32, rounded to half first for f16             */
    int32_t kernel;     /* HIPTK_PERM_*                                                           */
    int32_t mode_i, mode_j; /* TILED / ROWS: positions (in this struct's order) of the two tile modes */
    int32_t tile;       /* TILED / ROWS: 0 square, 1 long along mode_i, 2 long along mode_j;
                           TILED only: 3 a 64 KiB tile with rows and columns twice the square's;
                           STRIP: 0 / 1, see HIPTK_PERM_STRIP                                     */
    int32_t vec_r;      /* elements per global load (1, 2, 4; 8 for f16)                          */
    int32_t vec_w;      /* elements per global store                                              */
    int32_t group;      /* TILED / ROWS: workgroups walk the tile plane in bands of this many tiles
                           along mode_j, mode_j first inside a band (1: mode_i first throughout)  */
    int32_t mode_i2, mode_j2; /* GROUPED: the second row / column mode, or -1                     */
    int32_t chunk_i, chunk_j; /* GROUPED: indices of mode_i2 / mode_j2 per tile (1 when absent)   */
    int32_t width_i, width_j; /* GROUPED: elements of mode 0 / mode_j per tile                    */
} hiptk_permute_t;

/* Name of the kernel a problem selects ("" if the combination is not instantiated). */
const char* hiptk_permute_kernel_name(const hiptk_permute_t* prob);

/* Enqueue on `stream`.  The launcher checks, before anything is launched, that the problem is
 * well formed and that A, B and every stride meet the alignment vec_r / vec_w ask for;
 * the two tensors hold fewer than 2^31 elements each.  Returns a HIPTK_* code. */
int hiptk_permute(const hiptk_permute_t* prob, const void* A, void* B, void* stream, int* hip_error);

#ifdef __cplusplus
}
#endif
#endif /* HIPTK_KERNELS_H */
