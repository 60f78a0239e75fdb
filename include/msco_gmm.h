/*
 * msco_gmm.h -- C ABI of the MI355X (gfx950) backend for the grouped quantized matmul path.
 *
 * This is the boundary the C++ operator-registration layer calls instead of the reference's
 * closed kernel objects:
 *
 *   reference kernel-object life cycle (what the op glue calls)          this ABI
 *   ------------------------------------------------------------------  ---------------------------
 *   internal_v2::CreateGroupedMatmulOp(inputs, outputs, MatmulParam)     msco_gmm_create
 *     ops/c_api/grouped_matmul/grouped_matmul.cc:216-232,266-276
 *   InternalOp::Init / UpdateShape / GetTilingSize / Tiling /            msco_gmm_plan
 *   GetWorkspaceSize
 *     ops/framework/ms_kernels_internal/pyboost/internal_pyboost_runner.cc:34-58,99-113
 *   InternalOp::Launch(in_addrs, out_addrs, ws_addrs, stream, name)      msco_gmm_launch
 *     ops/framework/ms_kernels_internal/pyboost/internal_pyboost_runner.cc:210-231
 *   aclnnGroupedMatmulV4 GetWorkspaceSize + execute                      msco_gmm_plan + msco_gmm_launch
 *     ops/c_api/grouped_matmul_v4_cops/grouped_matmul_v4_cops.cc:94-97,359-363
 *   aclnnQuantMatmulV4  GetWorkspaceSize + execute                       msco_gmm_plan + msco_gmm_launch
 *     ops/c_api/quant_batch_matmul/quant_batch_matmul.cc:78-80,144-145
 *   INTERNAL_PRINT_TILING (tests/st/test_grouped_matmul.py:86)           msco_gmm_plan_info
 *
 * Conventions
 *   - every entry point returns an int status, 0 (MSCO_OK) on success; the C++ layer above turns a
 *     non-zero status into an exception exactly where the reference does
 *     (internal_pyboost_runner.cc:227-229);
 *   - all tensor arguments are raw device pointers to contiguous row-major buffers that the caller
 *     owns; an absent optional input is a NULL pointer (internal_pyboost_runner.h:69-78);
 *   - group_list stays on the device: nothing in plan or launch reads tensor values on the host;
 *   - launch enqueues on the given stream, never synchronises and never allocates.  A plan that
 *     needs cross-workgroup reduction state keeps a few KiB of device memory inside the handle
 *     (allocated by msco_gmm_plan, released by msco_gmm_destroy); because that state is per handle,
 *     one handle must not be launched concurrently on two streams.
 */
#ifndef MSCO_GMM_H_
#define MSCO_GMM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MSCO_GMM_ABI_VERSION 1

#if defined(MSCO_BUILDING_LIB)
#define MSCO_API __attribute__((visibility("default")))
#else
#define MSCO_API
#endif

typedef enum msco_status {
  MSCO_OK = 0,
  MSCO_ERR_INVALID_ARG = 1,   /* NULL where a pointer is required, bad enum value */
  MSCO_ERR_UNSUPPORTED = 2,   /* dtype / layout combination the backend does not implement */
  MSCO_ERR_SHAPE = 3,         /* shape rule violated (K, N, E alignment or mismatch) */
  MSCO_ERR_NOT_PLANNED = 4,   /* launch before plan */
  MSCO_ERR_WORKSPACE = 5,     /* workspace too small or NULL when the plan needs one */
  MSCO_ERR_DEVICE = 6         /* HIP runtime error (no device, launch failure) */
} msco_status;

typedef enum msco_dtype {
  MSCO_DT_NONE = 0,  /* input absent */
  MSCO_DT_I8 = 1,
  MSCO_DT_I32 = 2,
  MSCO_DT_I64 = 3,
  MSCO_DT_U64 = 4,
  MSCO_DT_F16 = 5,
  MSCO_DT_BF16 = 6,
  MSCO_DT_F32 = 7
} msco_dtype;

/* Storage of the weight tensor.  The reference keeps its weights in the device's own blocked format (FRACTAL_NZ,
 * produced once by trans_data, ops/c_api/trans_data/trans_data.cc:203-223; grouped_matmul forces it,
 * ops/c_api/grouped_matmul/grouped_matmul.cc:216-232); MSCO_WL_PACKED is this backend's counterpart: per group
 * ceil(N/16) column groups of ceil(K/64) blocks of 1024 bytes, zero outside K x N; byte 16 l + i (l = 0..63,
 * i = 0..15) of block (a, b) holds w[k = 64 b + 16 (l / 16) + i][n = 16 a + (l % 16)].  Decode shapes stream it at
 * the rate of a contiguous read. */
enum {
  MSCO_WL_ROW_MAJOR = 0,       /* [E,K,N], or [E,N,K] when transpose_b */
  MSCO_WL_PACKED = 1           /* e * msco_packed_weight_bytes(k, n) bytes written by msco_pack_weight */
};

/* Activation fused into the epilogue: the act_type argument that the reference forwards unchanged to
 * aclnnGroupedMatmulV4 (ops/c_api/grouped_matmul_v4_cops/grouped_matmul_v4_cops.cc:96,112,363; the reference defines no
 * values and holds no golden for it, so the values are those of CANN's GMMActType and the functions their textbook
 * forms).  Applied to the float32 result of the dequant epilogue (or of the weight-only matmul), before the cast to
 * bf16 / f16; not available with int32 output.
 *   RELU       max(v, 0)
 *   GELU_TANH  v * sigmoid(2 * sqrt(2 / pi) * (v + 0.044715 v^3))      (= 0.5 v (1 + tanh(...)))
 *   FAST_GELU  v * sigmoid(1.702 v)
 *   SILU       v * sigmoid(v) */
enum {
  MSCO_ACT_NONE = 0,
  MSCO_ACT_RELU = 1,
  MSCO_ACT_GELU_TANH = 2,
  MSCO_ACT_GELU_ERF = 3,       /* listed by CANN as unsupported; refused here too */
  MSCO_ACT_FAST_GELU = 4,
  MSCO_ACT_SILU = 5
};

/* Positional inputs of msco_gmm_launch.  Slots 0..6 follow the order the reference passes to its
 * kernel object (grouped_matmul.cc:201-207,301-307); slot 7 is the V4 antiquant offset
 * (grouped_matmul_v4_cops.cc:94-97). */
enum {
  MSCO_IN_X = 0,               /* [M,K] int8 (W8A8) or bf16/f16 (W8A16) */
  MSCO_IN_WEIGHT = 1,          /* [E,K,N] int8, or [E,N,K] when transpose_b, or packed (weight_layout) */
  MSCO_IN_BIAS = 2,            /* [E,N] int32, optional */
  MSCO_IN_SCALE = 3,           /* [E,N] f32 / bf16 / int64|uint64 carrying f32 bits in the low word; optional */
  MSCO_IN_GROUP_LIST = 4,      /* [E] int32 / int64; NULL = E equal groups of M/E rows (dense / batched) */
  MSCO_IN_PER_TOKEN_SCALE = 5, /* [M] f32, optional */
  MSCO_IN_ANTIQUANT_SCALE = 6, /* [E,N] in x's dtype, W8A16 only */
  MSCO_IN_ANTIQUANT_OFFSET = 7,/* [E,N] in x's dtype, W8A16 only, optional */
  MSCO_IN_COUNT = 8
};

/* Immutable description of one operator instance (dtypes, layouts, flags) -- the part the
 * reference hashes into its op key (internal_pyboost_runner.h:43-48). */
typedef struct msco_gmm_desc {
  int32_t abi_version;       /* MSCO_GMM_ABI_VERSION */
  int32_t x_dtype;           /* I8 | BF16 | F16 */
  int32_t weight_dtype;      /* I8 */
  int32_t out_dtype;         /* BF16 | F16 | I32 (raw accumulator + bias; scales are not applied) */
  int32_t group_list_dtype;  /* I32 | I64 | NONE */
  int32_t group_list_type;   /* 0 cumulative row ends, 1 per-group row counts */
  int32_t bias_dtype;        /* NONE | I32 */
  int32_t scale_dtype;       /* NONE | F32 | BF16 | I64 | U64 */
  int32_t per_token_dtype;   /* NONE | F32 */
  int32_t antiquant_dtype;   /* NONE | BF16 | F16 (scale and offset share it) */
  int32_t has_antiquant_offset;
  int32_t transpose_b;       /* 0: weight [E,K,N]; 1: weight [E,N,K] */
  int32_t scale_per_group;   /* 1: scale/bias are [E,N]; 0: one [N] (or [1]) row shared by all groups */
  int32_t scale_is_scalar;   /* 1: scale holds a single element broadcast over N */
  int32_t kernel_override;   /* 0 auto; else force a kernel family, for tests and planner checks: 1 eight-wave 256 x 256 tile,
                              * 2 128 x 128, 3 64 x 128, 4 decode (streaming) kernels, 5 generic, 6 persistent four-wave
                              * 256 x 256 (16 x 16 x 64 MFMAs), 7 128 x 256, 8 the persistent kernel's 32 x 32 x 32 MFMA form,
                              * 9 / 10 / 11 packed weights: chunks of up to 128 / 256 / 160 rows through LDS and weights
                              * straight into MFMA operands
                              * (msco_gmm_plan_info names what was planned) */
  int32_t weight_layout;     /* MSCO_WL_ROW_MAJOR: as transpose_b says; MSCO_WL_PACKED: written by msco_pack_weight */
  int32_t act_type;          /* msco_act: activation applied to the dequantised float32 value before the output cast */
  int32_t force_split_k;     /* 0 auto; else the K split across workgroups of the kernels that have one, for tests */
  int32_t reserved[2];
} msco_gmm_desc;

typedef struct msco_gmm_op *msco_gmm_handle;

/* Create an operator instance.  Replaces CreateGroupedMatmulOp + Init. */
MSCO_API int msco_gmm_create(const msco_gmm_desc *desc, msco_gmm_handle *out_handle);

/* Fix the shapes (shape-dependent work of Resize: kernel choice, grid, workspace size).
 * m = rows of x, k = reduction length, n = output columns, e = number of groups.
 * Replaces UpdateShape + Tiling + GetWorkspaceSize.  May be called again with new shapes, but only while no launch
 * of this handle is in flight on any stream: planning re-zeroes (with a synchronous hipMemset) the arrival counters
 * that a split-K launch of the handle reduces through, and may free and re-allocate them.  Callers that re-plan per
 * shape keep one handle per (shape, stream), as the operator layer's plan cache does. */
MSCO_API int msco_gmm_plan(msco_gmm_handle h, int64_t m, int64_t k, int64_t n, int64_t e, size_t *workspace_bytes);

/* Enqueue the computation.  inputs[MSCO_IN_COUNT] are device pointers (NULL = absent);
 * out is [M,N] in out_dtype; stream is a hipStream_t (NULL = default stream). */
MSCO_API int msco_gmm_launch(msco_gmm_handle h, const void *const *inputs, void *out, void *workspace,
                    size_t workspace_bytes, void *stream);

/* The same launch for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.  The split-K partial tiles that
 * msco_gmm_launch keeps in the caller's workspace go to a fixed array of MSCO_GMM_STATIC_WORKSPACE_BYTES bytes inside
 * the library instead (every GPU the library runs on holds it until the process ends); a plan whose workspace is
 * larger is refused with MSCO_ERR_WORKSPACE and a message on stderr.  Nothing is allocated or freed.  All calls on one
 * GPU share the array: two calls that overlap in time on one GPU (different streams, or different handles on
 * different streams) race; calls on one stream are ordered and safe. */
#define MSCO_GMM_STATIC_WORKSPACE_BYTES (32u << 20)
MSCO_API int msco_gmm_launch_static(msco_gmm_handle h, const void *const *inputs, void *out, void *stream);

/* Human-readable description of the current plan (kernel family, tile, grid, split) -- the
 * counterpart of the reference's INTERNAL_PRINT_TILING switch.  Returns the number of characters
 * that the full text needs (excluding the terminating NUL). */
MSCO_API int msco_gmm_plan_info(msco_gmm_handle h, char *buf, size_t buf_len);

/* Release the instance and any device state it holds. */
MSCO_API int msco_gmm_destroy(msco_gmm_handle h);

/* Batched 2-D transpose on the device: src [batch, rows, cols] -> dst [batch, cols, rows], elements of
 * elem_bytes (1, 2 or 4) bytes.  Serves transpose_x1 of quant_batch_matmul, which the reference passes
 * down to aclnnQuantMatmulV4 as a flag (ops/c_api/quant_batch_matmul/quant_batch_matmul.cc:78-80,144-145);
 * the HIP kernels read x rows K-contiguous, so the op layer materialises x1 transposed once. */
MSCO_API int msco_transpose_2d(const void *src, void *dst, int64_t batch, int64_t rows, int64_t cols,
                               int32_t elem_bytes, void *stream);

/* Grouped A8W4 matmul -- the counterpart of internal_v2::CreateGroupedMatmulW4Op behind grouped_matmul_w4
 * (ops/c_api/grouped_matmul_w4/grouped_matmul_w4.cc:50-88,186,218; golden tests/st/test_grouped_matmul_w4.py:100-113):
 *   out[m, n] = x_scale[m] * sum_g weight_scale[e, g, n] * sum_{k in K group g} x[m, k] * w[e, n, k],   e = group of row m
 * x int8 [m, k]; weight [e, n, k / 2] bytes, two signed 4-bit values per byte, k even in the low nibble
 * (i8toi4, test_grouped_matmul_w4.py:115-118); group_list int32 [e] cumulative row ends; x_scale float32 [m];
 * weight_scale float32 [e, k / group_size, n]; out float16 [m, n] (rows at or past group_list[e - 1] are not
 * written).  k a multiple of 32 and of group_size, group_size a multiple of 32, k <= 8192.  The reference op also takes
 * a float32 bias [e, n] that must hold 8 * sum_k dequantised w[e, k, n] (test :103-106): its kernel multiplies the
 * nibbles unsigned and needs the term to compensate; this one multiplies them signed, so the argument does not exist
 * here and the op layer above does not read it.  Nothing is allocated, everything is enqueued on the given stream. */
MSCO_API int msco_gmm_a8w4(const int8_t *x, const void *weight, const int32_t *group_list, const float *x_scale,
                           const float *weight_scale, void *out, int64_t m, int64_t k, int64_t n, int64_t e,
                           int64_t group_size, void *stream);

/* 4-bit weights of grouped_matmul_v4_cops widened to int8 on the device.  The reference hands its qint4x2 weight
 * [E, K, N / 2] to aclnnGroupedMatmulV4 as an int4 tensor of shape [E, K, N] (UnifyWeightShape,
 * ops/c_api/grouped_matmul_v4_cops/grouped_matmul_v4_cops.cc:56-66,274-295); this backend multiplies int8, so the op
 * layer widens the nibbles first: byte i of src holds element 2 i in its low nibble and element 2 i + 1 in its high
 * nibble (tests/st/test_grouped_matmul_v4_cops.py:458-460), each a signed 4-bit value; dst receives 2 * src_bytes
 * int8 values.  Both pointers 16-byte aligned.  Enqueued on the given stream, nothing is allocated. */
MSCO_API int msco_unpack_int4(const void *src, void *dst, int64_t src_bytes, void *stream);

/* Weight prepack, once at load time -- the counterpart of the reference's trans_data ND -> FRACTAL_NZ step
 * (ops/c_api/trans_data/trans_data.cc:203-223, shape contract ops/c_api/trans_data/trans_data.md:45-99).
 * src is [e,k,n] int8 (or [e,n,k] when src_transposed); dst receives e * msco_packed_weight_bytes(k, n) bytes in the
 * MSCO_WL_PACKED layout.  Enqueues on the stream, allocates nothing. */
MSCO_API size_t msco_packed_weight_bytes(int64_t k, int64_t n);
MSCO_API int msco_pack_weight(const void *src, void *dst, int64_t e, int64_t k, int64_t n, int32_t src_transposed,
                              void *stream);

/* Static text for a status code. */
MSCO_API const char *msco_status_string(int status);

/* ABI version the library was built with. */
MSCO_API int msco_gmm_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif  /* MSCO_GMM_H_ */
