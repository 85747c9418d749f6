/*
 * frisk_hip.h -- C ABI of libfrisk_hip.so: the gfx950 (MI355X) execution path
 * of the tiled GEMM that the Frisk dialect describes.
 *
 * The reference (Xiebaokang/frisk) stops at IR construction: its pybind11
 * module exposes only `init_ffi_ir` (ffi/ffi.h:12, ffi/ffi.cpp:3-7) and leaves
 * the slot for a compile/launch surface commented out (`init_ffi_passes`,
 * ffi/ffi.h:14).  The entry points below are what a binding in that slot calls:
 * one descriptor carrying the attributes of `frisk.gemm`
 * (include/Dialect/Frisk/IR/FriskOps.td:248-289: transA, transB, M, N, K,
 * clear_accum) plus what the surrounding `frisk.parallel`/`frisk.alloc_buffer`/
 * `frisk.copy` ops fix (tile shape, wave grid, element types; tmp/ir.mlir:1-17),
 * and raw device pointers.
 *
 * Rules of the boundary: plain C types only; every function returns a status
 * code and never throws; the caller owns all device buffers and the stream; a
 * launch is asynchronous on the given stream; the library never allocates or
 * synchronises behind the caller's back.
 */
#ifndef FRISK_HIP_H_
#define FRISK_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FRISK_HIP_ABI_VERSION 1

/* element types; `dtype = "fp16" | "fp32" | "e4m3fn" ...` strings of
 * create_alloc_buffer_op (ffi/ir.cpp:407-429) map onto these */
typedef enum frisk_dtype {
  FRISK_F32 = 0,
  FRISK_F16 = 1,
  FRISK_BF16 = 2,
  FRISK_I8 = 3,
  FRISK_E4M3 = 4, /* OCP e4m3fn, the reference's Float8E4M3FNType (ffi/ir.cpp:164,411) */
  FRISK_I32 = 5
} frisk_dtype;

typedef enum frisk_epilogue {
  FRISK_EPI_NONE = 0,          /* out = cast(acc)                                    */
  FRISK_EPI_ROW_COL_SCALE = 1, /* out = cast((float(acc) * scaleA[m]) * scaleB[n])   */
  FRISK_EPI_TENSOR_SCALE = 2   /* out = cast((float(acc) * scaleA[0]) * scaleB[0])   */
} frisk_epilogue;

/* GemmWarpPolicy of the dialect (include/Dialect/Frisk/IR/FriskEnums.td:16-25) */
typedef enum frisk_wave_policy { FRISK_POLICY_SQUARE = 0, FRISK_POLICY_FULL_ROW = 1, FRISK_POLICY_FULL_COL = 2 } frisk_wave_policy;

typedef enum frisk_status {
  FRISK_OK = 0,
  FRISK_ERR_NULL = 1,        /* a required pointer is null                            */
  FRISK_ERR_ABI = 2,         /* descriptor abi_version mismatch                       */
  FRISK_ERR_DTYPE = 3,       /* unsupported element-type combination                  */
  FRISK_ERR_SHAPE = 4,       /* negative extent, leading dimension too small, overflow */
  FRISK_ERR_TILE = 5,        /* requested tile / wave grid not available              */
  FRISK_ERR_LDS = 6,         /* tile needs more than the 160 KiB of LDS per CU        */
  FRISK_ERR_EPILOGUE = 7,    /* epilogue needs scales that were not given             */
  FRISK_ERR_WORKSPACE = 8,   /* workspace missing or too small                        */
  FRISK_ERR_DEVICE = 9,      /* no gfx950 device / HIP runtime error                  */
  FRISK_ERR_ALIGNMENT = 10,  /* a pointer is not aligned to its element size */
  FRISK_ERR_ARGUMENT = 11    /* an enumerated argument (reduce kind, dim) is out of range */
} frisk_status;

/*
 * One GEMM:  C[M,N] (+)= op(A)[M,K] . op(B)[K,N]
 *   transA = 0: A stored row-major [M][K], lda >= K;  transA = 1: stored [K][M], lda >= M
 *   transB = 0: B stored row-major [K][N], ldb >= N;  transB = 1: stored [N][K], ldb >= K
 *   C stored row-major [M][N], ldc >= N.  Leading dimensions are in elements.
 *   clear_accum = 1: C = A.B ;  clear_accum = 0: C = C + A.B  (frisk.gemm, FriskOps.td:262)
 * Supported (dtype_ab -> dtype_acc -> dtype_out):
 *   F32->F32->F32, F16->F32->{F16,F32}, BF16->F32->{BF16,F32},
 *   I8->I32->{I32, F16 with ROW_COL_SCALE}, E4M3->F32->{BF16,F32} (NONE or TENSOR_SCALE)
 * tile_* and waves_* = 0 let the planner choose.  With rows and pointers on 16-byte boundaries and K a multiple of
 * the K tile (64 elements of 16 bits, 128 of 8 bits, 32 of fp32) the fast kernels run, for any M and N (where those
 * are no multiples of the tile, variants of the same kernels whose stores are checked against M and N); anything
 * else (K off the K tile, odd leading dimensions, element-aligned pointers, K = 0) runs a bounds-checked kernel with
 * the same arithmetic: one that moves 16-byte chunks while rows and pointers are aligned and K is a whole number of
 * chunks, an element-wise one otherwise.
 */
typedef struct frisk_gemm_desc {
  int32_t abi_version; /* FRISK_HIP_ABI_VERSION */
  int32_t dtype_ab, dtype_acc, dtype_out;
  int64_t M, N, K;
  int64_t lda, ldb, ldc;
  uint8_t transA, transB, clear_accum;
  uint8_t split_k; /* slices of K computed by separate work-groups and summed through the workspace:
                      0 = planner's choice (splits only skinny problems, and only if a workspace is passed), 1 = never */
  int32_t epilogue;
  int32_t policy;                 /* frisk_wave_policy: only kernel variants whose wave grid is the policy's partition of their tile
                                     (frisk_hip_wave_partition) qualify; FRISK_ERR_TILE when none is compiled.  Ignored when
                                     waves_m / waves_n name a grid */
  int32_t tile_m, tile_n, tile_k; /* block tile = the M,N,K attrs of the tile-level frisk.gemm */
  int32_t waves_m, waves_n;       /* wave grid inside the work-group */
  int32_t stages;                 /* LDS stages of the global->LDS pipeline (of B when A and B differ), 0 = planner's choice */
  int32_t atom;                   /* rows of the MFMA atom: 32 (32x32xK), 16 (16x16x2K), 0 = planner's choice.  Occupies what was
                                     tail padding of the structure: its size is unchanged and zero-initialised callers keep working */
} frisk_gemm_desc;

/* XOR swizzle of an LDS tile: 16-byte chunk index c of row r is stored at
 * chunk  c ^ (((r >> row_shift) & row_mask) << chunk_shift)
 *          ^ (((r >> row_shift2) & row_mask2) << chunk_shift2)
 * (the second term is absent when row_mask2 == 0; the tiles read by transpose
 * reads for 16-row MFMA atoms use it).  This is the
 * representation of the reference's makeQuarter/Half/FullBankSwizzle layouts
 * (lib/Dialect/Frisk/IR/FriskOps.cpp:500-558), with the parameters chosen for
 * the gfx950 LDS instead of by the column-count rule of :560-618. */
typedef struct frisk_lds_layout {
  int32_t rows, row_bytes; /* tile as stored in LDS */
  int32_t k_contiguous;    /* 1: rows index M (or N), K runs along the row */
  int32_t row_shift, row_mask, chunk_shift;
  int32_t read_instr;      /* 0 ds_read_b128, 1 ds_read_b64_tr_b16, 2 ds_read_b64_tr_b8, 3 ds_read_b32 */
  float read_cycles;       /* modelled LDS cycles per wave-wide fragment read */
  float write_cycles;      /* modelled LDS cycles per KiB staged */
  int32_t row_shift2, row_mask2, chunk_shift2; /* second XOR term, all 0 when unused */
} frisk_lds_layout;

typedef struct frisk_gemm_plan {
  int32_t kernel_id;                 /* index into the compiled kernel table, -1 if none */
  int32_t tile_m, tile_n, tile_k;
  int32_t waves_m, waves_n, threads; /* result of the wave partition (reference: computeWarpPartition, FriskOps.cpp:825-888) */
  int32_t waves_k;                   /* >1: that many waves split the K steps of each tile (threads = waves_m*waves_n*waves_k*64) */
  int32_t mfma_m, mfma_n, mfma_k;    /* MFMA atom */
  int32_t stages, stages_b;          /* LDS ring depth for tiles of A and of B */
  int32_t lds_bytes;                 /* total, <= 163840 */
  int32_t grid_x, grid_y;            /* work-group grid (tiles along N, tiles along M) */
  int32_t split_k;                   /* >1: partial sums go through the workspace */
  int32_t xcd_remap;                 /* 1: work-group ids are remapped so each XCD owns a compact block of tiles */
  int32_t guarded;                   /* 1: a bounds-checked kernel runs (K off the K tile, unaligned rows or pointers) */
  frisk_lds_layout lds_a, lds_b;
  size_t workspace_bytes;
  double flops;                      /* 2.M.N.K */
  double bytes;                      /* |A| + |B| + |C| (+ scales) */
  int32_t tail_tiles, tail_split;    /* tail_split > 1: the last tail_tiles tiles (grid % 256, a partly filled last round) are
                                        computed by tail_split work-groups each, a share of the K tiles apiece, and summed
                                        through the workspace */
} frisk_gemm_plan;

int frisk_hip_abi_version(void);

/* Optional one-time set-up on the current device: everything that is not a stream operation (the kernels' dynamic
 * LDS limits).  Launches do this lazily for the kernel they pick, so the call is only needed before launches are
 * captured into a HIP graph, where such set-up is not allowed.  The reference has no counterpart (it launches nothing). */
int frisk_hip_init(void);

/* thread-local text of the last non-OK status returned on this thread */
const char* frisk_hip_last_error(void);

/* Pure host: validate the descriptor and fill the plan.  Needs no GPU. */
int frisk_hip_plan(const frisk_gemm_desc* desc, frisk_gemm_plan* plan);

/* Pure host: bytes of device workspace `frisk_hip_gemm` wants for this descriptor: split_k * M * N * 4 when the
 * plan splits K, tail_split * tail_tiles * tile_m * tile_n * 4 for a tail split, else 0.  With split_k = 0 in the
 * descriptor a launch without workspace still runs, unsplit. */
size_t frisk_hip_workspace_bytes(const frisk_gemm_desc* desc);

/* Launch on `stream` (a hipStream_t, may be NULL for the default stream).
 * A, B, C, scaleA, scaleB, workspace are device pointers.  scaleA/scaleB are
 * fp32: M and N entries for ROW_COL_SCALE, one entry each for TENSOR_SCALE. */
int frisk_hip_gemm(const frisk_gemm_desc* desc, const void* A, const void* B, void* C, const float* scaleA,
                   const float* scaleB, void* workspace, size_t workspace_bytes, void* stream);

/* frisk_hip_gemm for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc) and therefore have no workspace to pass.  No counterpart in the reference.  The
 * partial sums of a split-K or tail-split plan go to a fixed array of FRISK_HIP_STATIC_WS_BYTES that lives in the
 * library's device image (one copy per GPU, held until the process ends); neither this call nor anything it calls
 * allocates or frees.  (The HIP runtime places a device image on a GPU when it is first used there, which takes device
 * memory once: call frisk_hip_init() on each GPU beforehand and that has happened before the first launch.)  Same planner, kernels and results as frisk_hip_gemm with a large enough workspace, with two
 * exceptions for plans that need more than the array holds: an explicit split_k > 1 in the descriptor is refused with
 * FRISK_ERR_WORKSPACE, and a split the planner chose itself (split_k = 0: the tail split of a large grid can want
 * 64 MiB) is dropped, the launch running as a single pass exactly as frisk_hip_gemm does without a workspace.  All calls on one GPU share the array: calls that may overlap on that GPU (different streams,
 * different host threads) race on it and must be serialised by the caller; calls on one stream are ordered. */
#define FRISK_HIP_STATIC_WS_BYTES (32u << 20)
size_t frisk_hip_static_workspace_bytes(void);
int frisk_hip_gemm_static_ws(const frisk_gemm_desc* desc, const void* A, const void* B, void* C, const float* scaleA,
                             const float* scaleB, void* stream);

/* Pure host: modelled LDS cycles for one wave-wide access given the 64 byte
 * addresses the lanes present.  instr: 0 ds_read_b128, 1 ds_read_b64 /
 * ds_read_b64_tr_b16 / ds_read_b64_tr_b8, 3 ds_read_b32.  Replaces the bank
 * histogram of the reference's layout tool (exp/layout/gemm_layout_tool.cpp:135-208). */
float frisk_hip_lds_access_cycles(int instr, const int32_t* lane_byte_addr);

/* Pure host: exhaustive swizzle search for one operand tile.  `shape` gives rows, row_bytes and
 * k_contiguous of the tile as stored; elem_bytes / frag_bytes describe the MFMA operand (bytes per
 * element, bytes per lane per MFMA); tile_mn / tile_k the logical extents in elements; waves the
 * number of waves staging the tile.  Writes the best layout (swizzle fields, read_instr and the
 * modelled read_cycles per access) to `best`; `unswizzled_cycles` (may be NULL) receives the
 * modelled cycles per access of the same tile without a swizzle. */
int frisk_hip_lds_search(const frisk_lds_layout* shape, int elem_bytes, int frag_bytes, int tile_mn, int tile_k, int waves,
                         frisk_lds_layout* best, float* unswizzled_cycles);
/* The same for operands of MFMA atoms of `atom` rows / columns: 32 (32x32xK atoms, what frisk_hip_lds_search assumes) or
 * 16 (16x16x2K atoms: lane l serves row l % 16 and K-group l / 16 of four). */
int frisk_hip_lds_search_atom(const frisk_lds_layout* shape, int elem_bytes, int frag_bytes, int tile_mn, int tile_k, int waves, int atom,
                         frisk_lds_layout* best, float* unswizzled_cycles);

/* Pure host: byte offset inside an LDS tile of element (row, col_byte) under `layout`. */
int32_t frisk_hip_lds_offset(const frisk_lds_layout* layout, int32_t row, int32_t col_byte);

/* Pure host: wave partition for a block tile (restates computeWarpPartition for 64-wide waves
 * and 32x32 MFMA atoms). Returns FRISK_OK and writes waves_m, waves_n. */
int frisk_hip_wave_partition(int policy, int tile_m, int tile_n, int num_waves, int* waves_m, int* waves_n);

/* Number of kernels compiled into the library and a printable name for each. */
int frisk_hip_kernel_count(void);
const char* frisk_hip_kernel_name(int kernel_id);

/* ------------------------------------------------------------------------------------------------
 * The dialect's data-movement ops on rank-2 views of device memory (row-major, leading dimension in
 * elements; a rank-1 view is rows = 1).  Element types F32, F16, BF16.  All launches are asynchronous
 * on `stream`; nothing is allocated.  Index maps and indices of the ops are applied by the caller as
 * pointer offsets: a view is (pointer to its first element, rows, cols, ld).
 * ------------------------------------------------------------------------------------------------ */
typedef enum frisk_reduce_kind {
  FRISK_REDUCE_ADD = 0,
  FRISK_REDUCE_MUL = 1,
  FRISK_REDUCE_MIN = 2,
  FRISK_REDUCE_MAX = 3
} frisk_reduce_kind;

/* frisk.fill (include/Dialect/Frisk/IR/FriskOps.td:392-410; the value is a float attribute of the element
 * type, lib/Dialect/Frisk/IR/FriskOps.cpp:1686-1701): every element of the view := value rounded to dtype. */
int frisk_hip_fill(int dtype, void* dst, int64_t rows, int64_t cols, int64_t ld, double value, void* stream);

/* frisk.copy (FriskOps.td:348-389; the window is src_extents / dst_extents, by default the destination
 * shape, FriskOps.cpp:1564-1591): the rows x cols window at `src` goes to the window at `dst`.  Element
 * types may differ (the fragment -> shared f32 -> f16 casts of tmp/ir.mlir:121,129): values are converted
 * through fp32 with round-to-nearest-even.  The windows must not overlap. */
int frisk_hip_copy(int src_dtype, const void* src, int64_t src_ld, int dst_dtype, void* dst, int64_t dst_ld, int64_t rows,
                   int64_t cols, void* stream);

/* frisk.copy under frisk.parallel / frisk.for whose windows are placed by index maps (FriskOps.td:348-389; maps, index
 * operands and extents FriskOps.cpp:1551-1683): n0 x n1 tiles of tile_rows x tile_cols elements.  Tile (a, b) is read
 * at element offset a * src_step0 + b * src_step1 from `src` and written at a * dst_step0 + b * dst_step1 from `dst`;
 * inside a tile consecutive rows lie src_ld / dst_ld elements apart.  One launch for placements that a single window
 * copy cannot express, e.g. tiles placed transposed (the tile at block (a, b) of the source going to block (b, a) of the
 * destination; the elements of a tile keep their order, as frisk.copy copies a window).  Destination tiles must not
 * overlap one another or the source.  Steps are non-negative; n0 * n1 <= 2^31 - 1. */
int frisk_hip_copy_tiles(int src_dtype, const void* src, int64_t src_ld, int dst_dtype, void* dst, int64_t dst_ld, int64_t tile_rows,
                         int64_t tile_cols, int64_t n0, int64_t src_step0, int64_t dst_step0, int64_t n1, int64_t src_step1,
                         int64_t dst_step1, void* stream);

/* frisk.reduce (FriskOps.td:412-441, verifier FriskOps.cpp:1733-1767): reduces the rows x cols view along
 * `dim` (0: over rows, dst has cols entries; 1: over columns, dst has rows entries) with `kind`.  Arithmetic
 * in fp32, result rounded to dtype.  clear = 1: dst := reduction; clear = 0: dst := kind(dst, reduction).
 * min / max ignore NaN operands (maxnum / minnum).  Long reductions are split over work-groups through
 * `workspace` (frisk_hip_reduce_workspace_bytes; 0 for most shapes). */
size_t frisk_hip_reduce_workspace_bytes(int dtype, int64_t rows, int64_t cols, int dim);
int frisk_hip_reduce(int dtype, const void* src, int64_t rows, int64_t cols, int64_t ld, int dim, int kind, int clear, void* dst,
                     void* workspace, size_t workspace_bytes, void* stream);

/* Row softmax in base 2, the kernel sketched as @online_softmax in the reference's tmp/ir.mlir:21-66 (per row: copy,
 * reduce max, block exp2(x * cst - max * cst), reduce sum, running log-sum; then exp2(x * cst - lse)):
 *   dst[r][j] = 2^(scale_log2 * src[r][j]) / sum_j 2^(scale_log2 * src[r][j])
 * on rank-2 views as above (F32, F16, BF16; arithmetic in fp32, result rounded to dtype).  scale_log2 is the sketch's
 * `cst`; a natural softmax with scale s is scale_log2 = s * log2(e).  lse (may be NULL) receives, per row, the
 * base-2 logarithm of the denominator, the sketch's `lse`.  dst may be src.  Rows of -inf only give NaN, as the
 * arithmetic does.  A few very long rows (fewer than 1024 rows of at least 32 KiB) are split over several work-groups
 * each when the caller passes `workspace` (frisk_hip_softmax_workspace_bytes, pure host; 0 for other shapes); without
 * one they run unsplit, a work-group per row. */
size_t frisk_hip_softmax_workspace_bytes(int dtype, int64_t rows, int64_t cols);
int frisk_hip_softmax(int dtype, const void* src, int64_t src_ld, void* dst, int64_t dst_ld, int64_t rows, int64_t cols,
                      float scale_log2, float* lse, void* workspace, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------------------------------------
 * frisk.block (include/Dialect/Frisk/IR/FriskOps.td:143-190; built by create_block_op, ffi/ir.cpp:383-394): a body of
 * affine.load / arith / math / affine.store ops run for every point of an iteration space.  The reference defines the
 * op and lowers it nowhere.  Here a body that stores one value per point is run as ONE kernel that interprets the
 * stored expression, given as a postfix program: no code is generated at run time.
 *   out[r][c] = program(in_0[r][c], in_1[r][c], ...)   for r < rows, c < cols   (a rank-1 block is rows = 1)
 * Operand k is read at element  r * in_row_stride[k] + c * in_col_stride[k]  from inputs[k]: col stride 1 walks a row,
 * col stride 0 broadcasts one element along the row, row stride 0 the same row to every row (so a per-row scalar x[r]
 * is (1, 0), a per-column vector (0, 1), a scalar (0, 0)).  Element types F32, F16, BF16, per operand.  The program
 * is evaluated on a stack in fp32 (width casts inside a body are transparent) and the result rounded once to out_dtype:
 *   FRISK_EW_INPUT  push operand arg[i]          FRISK_EW_CONST  push imm[i]
 *   ADD SUB MUL DIV MAX MIN   pop b, pop a, push a op b   (MAX / MIN ignore a NaN operand: arith.maxnumf / minnumf)
 *   NEG EXP2 LOG2             replace the top            (math.exp2 / math.log2: base 2)
 * A program must leave exactly one value and never hold more than FRISK_EW_MAX_STACK.  out must not overlap an input
 * other than element for element (in place is allowed).  Asynchronous on `stream`; nothing is allocated.
 * ------------------------------------------------------------------------------------------------ */
#define FRISK_EW_MAX_INPUTS 8
#define FRISK_EW_MAX_OPS 48
#define FRISK_EW_MAX_STACK 6
typedef enum frisk_ew_op {
  FRISK_EW_INPUT = 0,
  FRISK_EW_CONST = 1,
  FRISK_EW_ADD = 2,
  FRISK_EW_SUB = 3,
  FRISK_EW_MUL = 4,
  FRISK_EW_DIV = 5,
  FRISK_EW_MAX = 6,
  FRISK_EW_MIN = 7,
  FRISK_EW_NEG = 8,
  FRISK_EW_EXP2 = 9,
  FRISK_EW_LOG2 = 10
} frisk_ew_op;

typedef struct frisk_elementwise_desc {
  int32_t abi_version;   /* FRISK_HIP_ABI_VERSION */
  int32_t n_inputs, n_ops;
  int32_t out_dtype;
  int64_t rows, cols, out_ld;
  int32_t in_dtype[FRISK_EW_MAX_INPUTS];
  int32_t in_col_stride[FRISK_EW_MAX_INPUTS];   /* 0 or 1 */
  int64_t in_row_stride[FRISK_EW_MAX_INPUTS];   /* >= 0, elements */
  int32_t op[FRISK_EW_MAX_OPS];                 /* frisk_ew_op */
  int32_t arg[FRISK_EW_MAX_OPS];                /* operand index of FRISK_EW_INPUT */
  float imm[FRISK_EW_MAX_OPS];                  /* value of FRISK_EW_CONST */
} frisk_elementwise_desc;

int frisk_hip_elementwise(const frisk_elementwise_desc* desc, const void* const* inputs, void* out, void* stream);

/* ------------------------------------------------------------------------------------------------
 * Fused attention forward: O = softmax(scale * Q K^T) V per (batch, head), the kernel sketched in the
 * reference's tmp/ir.mlir:87-157 (frisk.copy Q; frisk.for over key tiles { copy K; gemm; reduce max;
 * block exp2; reduce sum; block rescale; copy V; gemm }; copy O) executed as one launch with a running
 * maximum and denominator.  The sketch multiplies scores by a constant and uses exp2
 * (tmp/ir.mlir:91,114-127): that constant is scale * log2(e) here.
 * Tensors are dense: Q [batch, heads, seq_q, head_dim], V [batch, heads, seq_k, head_dim],
 * O like Q, K like V or, with k_transposed = 1, [batch, heads, head_dim, seq_k] (the layout of the sketch's
 * second argument, tmp/ir.mlir:88).  Products accumulate in fp32; the probabilities are rounded to dtype
 * before the second product.  Supported: head_dim 128, seq_q a multiple of 256, seq_k a multiple of 64,
 * 16-byte aligned pointers; anything else is FRISK_ERR_SHAPE / FRISK_ERR_ALIGNMENT.
 * ------------------------------------------------------------------------------------------------ */
typedef struct frisk_attention_desc {
  int32_t abi_version;   /* FRISK_HIP_ABI_VERSION */
  int32_t dtype;         /* FRISK_F16 or FRISK_BF16: element type of Q, K, V and O */
  int64_t batch, heads, seq_q, seq_k, head_dim;
  float scale;           /* > 0; 1/sqrt(head_dim) is the usual choice */
  uint8_t k_transposed;
  uint8_t reserved[3];
} frisk_attention_desc;

/* lse (may be NULL): [batch, heads, seq_q] floats, log(sum_k exp(scale * s_k)) of every query row, from the
 * probabilities as rounded for the second product (the denominator the output is normalised by).
 * Asynchronous on `stream`; nothing is allocated. */
int frisk_hip_attention(const frisk_attention_desc* desc, const void* Q, const void* K, const void* V, void* O, float* lse,
                        void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FRISK_HIP_H_ */
