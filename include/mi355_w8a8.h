/*
 * mi355_w8a8.h -- plain C ABI of the MI355X (gfx950) W8A8 LoRA linear forward path.
 *
 * Every entry point enqueues work on the caller's HIP stream and returns; none
 * synchronises, allocates or frees device memory, or keeps a pointer after it
 * returns.  All pointers are device pointers unless marked "host".  A stream is
 * passed as void* (a hipStream_t; NULL = the default stream).  Return value:
 * MI355_W8A8_OK or a negative mi355_w8a8_status.
 *
 * What each entry point replaces in the reference (paths relative to its root):
 *   - mi355_w8a8_quantize_rows_v1      skyrl/tx/kernels/quantized_lora.py:199-212
 *                                      (= skyrl/tx/kernels/rocm/w8a8_lora.py:179-187)
 *   - mi355_w8a8_pack_weight_v1        the load-time permutation sanctioned by
 *                                      rocm/QUANTIZED_FFI.md:71-74 of the storage format
 *                                      skyrl/tx/kernels/quantized_lora.py:20-41
 *   - mi355_w8a8_lora_linear_v1        skyrl/tx/kernels/quantized_lora.py:400-453 and
 *                                      skyrl/tx/kernels/rocm/w8a8_lora.py:827-920 (forward),
 *                                      with the per-row adapter routing of
 *                                      skyrl/tx/layers/lora.py:118-157
 *   - mi355_w8a8_rms_gateup_swiglu_v1  skyrl/tx/kernels/rocm/bf16_rms_gate_up_lora_swiglu_contiguous.py:698-712
 *                                      (forward) on W8A8 weights
 *   - mi355_w8a8_lora_residual_v1      skyrl/tx/kernels/rocm/bf16_lora_residual.py:507-522 (forward)
 *                                      on W8A8 weights
 *   - mi355_w8a8_grouped_v1            skyrl/tx/layers/lora.py:394-444 (LoRAExpert.__call__) with
 *                                      the ragged_dot of skyrl/tx/layers/util.py:8-59
 *   - mi355_w8a8_lora_linear_bwd_v1    skyrl/tx/kernels/quantized_lora.py:337-394 (the VJP)
 *   - mi355_w8a8_grouped_bwd_v1        the same rule over skyrl/tx/layers/lora.py:394-444
 *   - mi355_w8a8_swiglu_bwd_v1 / mi355_w8a8_rms_norm_bwd_v1
 *                                      skyrl/tx/kernels/rocm/bf16_rms_gate_up_lora_swiglu_contiguous.py:541-574
 *   - mi355_w8a8_qkv_split_norm_rope_v1 skyrl/tx/kernels/qwen3_5_qkv_lora.py:266-286
 *   - mi355_w8a8_qkv_split_norm_rope_bwd_v1, mi355_w8a8_delta_rms_norm_bwd_v1
 *                                       skyrl/tx/kernels/qwen3_5_qkv_lora.py:360-451
 *   - mi355_w8a8_moe_route_v1 / _moe_dispatch_v1 / _moe_combine_v1
 *                                      skyrl/tx/models/qwen3.py:172-210, skyrl/tx/layers/util.py:66-87
 *   - mi355_w8a8_gq_linear_v1          skyrl/tx/kernels/quantized_lora.py:215-304 in its general form
 *                                      (W4 / W8 codes, A4 / A8 activations, scales per K group)
 * The typed-FFI handler shape these sit behind is rocm/QUANTIZED_FFI.md:589-599 and
 * skyrl/tx/kernels/rocm/ffi/gdn_ffi_smoke.hip:43-82.
 */
#ifndef MI355_W8A8_H_
#define MI355_W8A8_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MI355_W8A8_ABI_VERSION 1

typedef enum mi355_w8a8_status {
  MI355_W8A8_OK = 0,
  MI355_W8A8_ERR_NULL = -1,        /* a required pointer is NULL */
  MI355_W8A8_ERR_SHAPE = -2,       /* a dimension is zero, too large or inconsistent */
  MI355_W8A8_ERR_ALIGN = -3,       /* a pointer is not 16-byte aligned */
  MI355_W8A8_ERR_ALIAS = -4,       /* the output overlaps an input */
  MI355_W8A8_ERR_WORKSPACE = -5,   /* workspace missing or too small */
  MI355_W8A8_ERR_LAUNCH = -6,      /* the HIP runtime refused a launch */
  MI355_W8A8_ERR_UNSUPPORTED = -7, /* valid request outside this build's geometry */
  MI355_W8A8_ERR_STRUCT = -8       /* struct_size does not match this header */
} mi355_w8a8_status;

/* Flags of mi355_w8a8_problem.flags */
#define MI355_W8A8_FLAG_SWIGLU 1u      /* out[m, j] = bf16(silu(y[m,2j]) * y[m,2j+1]); out is [M, N/2] */
#define MI355_W8A8_FLAG_FORCE_TILED 2u /* never take the skinny-M (split-K) kernel, whole or in 32-row chunks */
#define MI355_W8A8_FLAG_FORCE_SKINNY 4u/* always take the skinny-M kernel (M <= 32) */
#define MI355_W8A8_FLAG_LORA_SPLIT2 8u /* carry x@A as 2 bf16 terms instead of 3 in the LoRA-B product */
/* Stage selection for measurement: the workspace keeps the prologue's results between calls, so a
 * call with SKIP_PROLOGUE after a full call with the same arguments re-runs only the GEMM kernel. */
/* Calls of 33..128 rows that run as 32-row chunks of the skinny-M kernels (see FORCE_TILED) keep no
 * prologue results and answer these two flags with MI355_W8A8_ERR_UNSUPPORTED. */
#define MI355_W8A8_FLAG_SKIP_PROLOGUE 16u /* do not run routing / quantization / LoRA-A */
#define MI355_W8A8_FLAG_SKIP_GEMM 32u     /* run only routing / quantization / LoRA-A */
/* tile geometry of the tiled GEMM (at most one of the four; two are refused with MI355_W8A8_ERR_SHAPE);
 * default: 128 x 128 while at most 512 such tiles cover the output, else 256 x 256 (256 x 128 when k is
 * too short for that kernel's stage schedule).  TILE_256X128_PAIR is the 256 x 256 kernel's instruction
 * (16 x 16 x 64) and schedule in 256 x 128 tiles, two workgroups per CU. */
#define MI355_W8A8_FLAG_TILE_256X128 64u
#define MI355_W8A8_FLAG_TILE_256X256 128u
#define MI355_W8A8_FLAG_TILE_128X128 2048u
#define MI355_W8A8_FLAG_TILE_256X128_PAIR 4096u
/* tile rows of the grouped call (and the slots every group is padded to); default: 128 once the
 * groups average at least 96 rows, else 64.  Pass the same flags to the workspace query. */
#define MI355_W8A8_FLAG_GROUPED_TILE64 256u
#define MI355_W8A8_FLAG_GROUPED_TILE128 512u
/* The workspace still holds the LoRA A and B in operand order that an earlier call of the tiled path
 * (more than 32 rows, not run as 32-row chunks: see mi355_w8a8_forward_path) wrote there for the same
 * lora_a / lora_b contents and the same (k, n, n_adapters, rank): this call does not write them again
 * (adapters that do not change between calls, as in serving).  They sit at the start of the workspace, at
 * places that depend on (k, n, n_adapters, rank) only, so the earlier call may have had another m, other
 * adapter_indices or another tile geometry.  The caller vouches for it; calls that run as 32-row chunks
 * keep no such copies and ignore the flag. */
/* For calls of at most 16 rows (rank <= 32) the flag covers something else: the per-row regrouped copy of B
 * the decode kernels keep in the workspace.  There it vouches that the earlier call was a decode call with
 * the same m and that lora_b and adapter_indices have the contents they had then. */
/* mi355_w8a8_grouped_v1 takes the flag too: its launch that lays out the slots then leaves the transposed A
 * and the packed B of an earlier grouped call on the same workspace with the same (k, n, n_groups, rank) as
 * they are. */
#define MI355_W8A8_FLAG_LORA_PACK_VALID 1024u

/*
 * One forward call.  y = dequant(quant(n) @ W) + s[idx] * ((n @ A[idx]) @ B[idx]) (+ residual),
 * n = x or rmsnorm(x).  The float32 epilogue is cast to bf16 exactly once.
 */
typedef struct mi355_w8a8_problem {
  uint32_t struct_size;     /* sizeof(mi355_w8a8_problem) */
  uint32_t flags;
  uint32_t m;               /* rows of x */
  uint32_t k;               /* in features; multiple of 8 */
  uint32_t n;               /* out features of W (before SwiGLU halving) */
  uint32_t n_adapters;      /* leading dim of lora_a/lora_b/lora_scaling; 0 = no LoRA */
  uint32_t rank;            /* LoRA rank r (<= 64) */
  float rms_eps;            /* used when rms_gamma != NULL */
  const void* x;            /* bf16 [m, k] */
  const void* w_packed;     /* from mi355_w8a8_pack_weight_v1 for the same (k, n) */
  const float* w_scales;    /* f32 [n], one per output channel */
  const void* lora_a;       /* bf16 [n_adapters, k, rank] or NULL */
  const void* lora_b;       /* bf16 [n_adapters, rank, n] or NULL */
  const float* lora_scaling;/* f32 [n_adapters] (alpha / rank) or NULL */
  const int32_t* adapter_indices; /* int32 [m], one adapter per row; NULL = adapter 0 for every row */
  const float* rms_gamma;   /* f32 [k] multiplier of the fused RMSNorm prologue, or NULL */
  const void* residual;     /* bf16 [m, n_out] added in the f32 epilogue, or NULL */
  void* out;                /* bf16 [m, n_out]; n_out = n, or n/2 with FLAG_SWIGLU */
  void* workspace;          /* >= mi355_w8a8_workspace_bytes(...) bytes, 256-byte aligned */
  uint64_t workspace_bytes;
  /* Optional auxiliary outputs (NULL to skip); they exist for parity checks. */
  int8_t* aux_x_codes;      /* int8 [m, k] row-major activation codes */
  float* aux_x_scales;      /* f32 [m] activation scales */
  int32_t* aux_acc;         /* int32 [m, n] raw integer accumulators */
  void* aux_normalized;     /* bf16 [m, k] RMSNorm output (only with rms_gamma) */
} mi355_w8a8_problem;

/*
 * Grouped (ragged) call: rows of x are already sorted by group (expert); group g owns
 * group_sizes[g] consecutive rows, its own packed weight, scales and LoRA pair.
 */
typedef struct mi355_w8a8_grouped_problem {
  uint32_t struct_size;     /* sizeof(mi355_w8a8_grouped_problem) */
  uint32_t flags;           /* MI355_W8A8_FLAG_SWIGLU, _GROUPED_TILE64 / _GROUPED_TILE128, and for measurement
                             * _SKIP_PROLOGUE / _SKIP_GEMM (same arguments and workspace as the full call before) */
  uint32_t m;               /* total rows */
  uint32_t k;
  uint32_t n;
  uint32_t n_groups;
  uint32_t rank;            /* 0 = no LoRA */
  uint32_t groups_per_weight; /* weight / scale index = group / groups_per_weight (0 or 1: one per group) */
  const void* x;            /* bf16 [m, k] */
  const void* w_packed;     /* n_groups / groups_per_weight packed weights back to back, each
                               mi355_w8a8_packed_weight_bytes(k, n) */
  const float* w_scales;    /* f32 [n_groups / groups_per_weight, n] */
  const void* lora_a;       /* bf16 [n_groups, k, rank] or NULL */
  const void* lora_b;       /* bf16 [n_groups, rank, n] or NULL */
  const float* lora_scaling;/* f32 [n_groups] or NULL */
  const int32_t* group_sizes; /* int32 [n_groups]; rows beyond sum(group_sizes) produce zeros */
  void* out;                /* bf16 [m, n_out] */
  void* workspace;
  uint64_t workspace_bytes;
  int8_t* aux_x_codes;
  float* aux_x_scales;
  int32_t* aux_acc;         /* int32 [m, n]; rows beyond sum(group_sizes) are not written */
  /* Optional gather on the way in (NULL: row i of the call is row i of x).  With a map, row i is
   * read from x[x_row_map[i] / x_row_repeat] and x holds one row per token: passing the
   * sort_indices of mi355_w8a8_moe_dispatch_v1 and repeat = top_k lets the first expert projection
   * read the unsorted hidden states, and the dispatch can skip the row copies.  A map value outside
   * [0, x_rows * x_row_repeat) reads the nearest row of x (the last one, or row 0 for a negative value)
   * instead of memory beyond x. */
  const int32_t* x_row_map; /* int32 [m] or NULL */
  uint32_t x_row_repeat;    /* >= 1 with a map */
  uint32_t x_rows;          /* rows of x with a map; 0 = ceil(m / x_row_repeat), one row per token */
} mi355_w8a8_grouped_problem;

/*
 * Backward of the plain W8A8 LoRA linear (no RMSNorm / SwiGLU / residual stage):
 *   dx  = dy @ bf16(codes * scales).T + ((dy @ B[idx].T) * s[idx]) @ A[idx].T
 *   dA[g] = x_g.T @ ((dy_g @ B[g].T) * s[g])     dB[g] = ((x_g @ A[g]).T @ dy_g) * s[g]
 *   ds[g] = sum(dy_g * ((x_g @ A[g]) @ B[g]))    (rows of adapter g; zero for adapters without rows)
 * The activation quantizer is treated as the identity (straight-through), as the reference does.
 */
typedef struct mi355_w8a8_bwd_problem {
  uint32_t struct_size;     /* sizeof(mi355_w8a8_bwd_problem) */
  uint32_t flags;           /* 0, or MI355_W8A8_FLAG_SKIP_PROLOGUE / _SKIP_GEMM (measurement only) */
  uint32_t m;               /* rows */
  uint32_t k;               /* in features (columns of dx); multiple of 8 */
  uint32_t n;               /* out features (columns of dy); multiple of 8 */
  uint32_t n_adapters;      /* 0 = no LoRA */
  uint32_t rank;
  uint32_t reserved;
  const void* x;            /* bf16 [m, k]; needed only when a LoRA cotangent is requested */
  const void* dy;           /* bf16 [m, n] output cotangent */
  const void* w_packed;     /* the forward's packed weight */
  const float* w_scales;    /* f32 [n] */
  const void* lora_a;       /* bf16 [n_adapters, k, rank] or NULL */
  const void* lora_b;       /* bf16 [n_adapters, rank, n] or NULL */
  const float* lora_scaling;/* f32 [n_adapters] or NULL */
  const int32_t* adapter_indices; /* int32 [m] or NULL (adapter 0 for every row) */
  void* dx;                 /* bf16 [m, k] */
  void* d_lora_a;           /* bf16 [n_adapters, k, rank] or NULL (not wanted) */
  void* d_lora_b;           /* bf16 [n_adapters, rank, n] or NULL */
  float* d_lora_scaling;    /* f32 [n_adapters] or NULL */
  void* workspace;          /* >= mi355_w8a8_bwd_workspace_bytes(...) bytes, 256-byte aligned */
  uint64_t workspace_bytes;
} mi355_w8a8_bwd_problem;

/*
 * Backward of the grouped call (plain epilogue): rows of x and dy are sorted by group as in the
 * forward; group g owns group_sizes[g] consecutive rows and its own LoRA pair, groups_per_weight
 * consecutive groups share a frozen weight.  Cotangents of groups without rows are zero, dx rows
 * beyond sum(group_sizes) are zero.
 */
typedef struct mi355_w8a8_grouped_bwd_problem {
  uint32_t struct_size;     /* sizeof(mi355_w8a8_grouped_bwd_problem) */
  uint32_t flags;           /* 0 */
  uint32_t m;               /* total rows */
  uint32_t k;               /* multiple of 8 */
  uint32_t n;               /* multiple of 8 */
  uint32_t n_groups;        /* <= 1024 */
  uint32_t rank;            /* 0 = no LoRA */
  uint32_t groups_per_weight; /* 0 or 1: one weight per group */
  const void* x;            /* bf16 [m, k]; needed only when a LoRA cotangent is requested */
  const void* dy;           /* bf16 [m, n] */
  const void* w_packed;     /* n_groups / groups_per_weight packed weights back to back */
  const float* w_scales;    /* f32 [n_groups / groups_per_weight, n] */
  const void* lora_a;       /* bf16 [n_groups, k, rank] or NULL */
  const void* lora_b;       /* bf16 [n_groups, rank, n] or NULL */
  const float* lora_scaling;/* f32 [n_groups] or NULL */
  const int32_t* group_sizes; /* int32 [n_groups] */
  void* dx;                 /* bf16 [m, k] */
  void* d_lora_a;           /* bf16 [n_groups, k, rank] or NULL (not wanted) */
  void* d_lora_b;           /* bf16 [n_groups, rank, n] or NULL */
  float* d_lora_scaling;    /* f32 [n_groups] or NULL */
  void* workspace;          /* >= mi355_w8a8_grouped_bwd_workspace_bytes(...), 256-byte aligned */
  uint64_t workspace_bytes;
} mi355_w8a8_grouped_bwd_problem;

/*
 * Qwen3.5 attention input stage behind the fused QKV projection: split of the interleaved
 * projection (per kv head: queries_per_kv (q, gate) chunk pairs, then k, then v), RMSNorm with
 * (1 + weight) over every Q and K head, partial RoPE on Q and K.
 */
typedef struct mi355_w8a8_qkv_post_problem {
  uint32_t struct_size;     /* sizeof(mi355_w8a8_qkv_post_problem) */
  uint32_t flags;           /* 0 */
  uint32_t m;               /* rows (batch * sequence) */
  uint32_t num_query_heads;
  uint32_t num_kv_heads;    /* divides num_query_heads */
  uint32_t head_dim;        /* even, <= 512 */
  uint32_t rotary_dim;      /* even, <= head_dim; 0 = no RoPE */
  float rope_theta;
  float rms_eps;
  uint32_t reserved;
  const void* fused;        /* bf16 [m, num_query_heads * 2 * head_dim + 2 * num_kv_heads * head_dim] */
  const float* q_norm_weight; /* f32 [head_dim], delta form: the multiplier is 1 + weight */
  const float* k_norm_weight; /* f32 [head_dim] */
  const int32_t* positions; /* int32 [m] */
  void* q;                  /* bf16 [m, num_query_heads, head_dim] */
  void* k;                  /* bf16 [m, num_kv_heads, head_dim] */
  void* v;                  /* bf16 [m, num_kv_heads, head_dim] */
  void* gate;               /* bf16 [m, num_query_heads * head_dim] */
} mi355_w8a8_qkv_post_problem;

/*
 * Pull-back of the stage above.  fused is the raw projection the forward consumed; the four output
 * cotangents come in, the cotangent of the fused projection goes out, optionally with the
 * cotangents of the two head-norm weights.
 */
typedef struct mi355_w8a8_qkv_post_bwd_problem {
  uint32_t struct_size;     /* sizeof(mi355_w8a8_qkv_post_bwd_problem) */
  uint32_t flags;           /* 0 */
  uint32_t m;
  uint32_t num_query_heads;
  uint32_t num_kv_heads;
  uint32_t head_dim;
  uint32_t rotary_dim;
  float rope_theta;
  float rms_eps;
  uint32_t reserved;
  const void* fused;        /* bf16 [m, fused width] */
  const float* q_norm_weight; /* f32 [head_dim], delta form */
  const float* k_norm_weight; /* f32 [head_dim] */
  const int32_t* positions; /* int32 [m] */
  const void* d_q;          /* bf16 [m, num_query_heads, head_dim] */
  const void* d_k;          /* bf16 [m, num_kv_heads, head_dim] */
  const void* d_v;          /* bf16 [m, num_kv_heads, head_dim] */
  const void* d_gate;       /* bf16 [m, num_query_heads * head_dim] */
  void* d_fused;            /* bf16 [m, fused width] */
  float* d_q_norm_weight;   /* f32 [head_dim] or NULL; both or neither */
  float* d_k_norm_weight;   /* f32 [head_dim] or NULL */
  void* workspace;          /* needed with the weight cotangents only */
  uint64_t workspace_bytes; /* >= mi355_w8a8_qkv_bwd_workspace_bytes(m, head_dim) */
} mi355_w8a8_qkv_post_bwd_problem;

int mi355_w8a8_abi_version(void);
const char* mi355_w8a8_status_string(int status);

/* Bytes of the packed form of a [k, n] int8 weight (0 when k or n is 0). */
uint64_t mi355_w8a8_packed_weight_bytes(uint32_t k, uint32_t n);

/* One-time re-layout of row-major int8 codes [k, n] into the MFMA fragment order. */
int mi355_w8a8_pack_weight_v1(const int8_t* codes_kn, void* packed, uint32_t k, uint32_t n,
                              void* stream);
/* Inverse of the above (packed -> row-major [k, n]); used by tests and exporters. */
int mi355_w8a8_unpack_weight_v1(const void* packed, int8_t* codes_kn, uint32_t k, uint32_t n,
                                void* stream);

/* Per-token dynamic symmetric int8 quantization: codes int8 [m, k], scales f32 [m]. */
int mi355_w8a8_quantize_rows_v1(const void* x_bf16, int8_t* codes, float* scales, uint32_t m,
                                uint32_t k, void* stream);

/* Workspace requirement of the dense entry points below.  It depends on the dimensions only (never on
 * the flags or on which rows use which adapter) and covers every layout a call of these dimensions may
 * choose: adapters packed or each on a 32-slot boundary, any tile geometry, the decode kernels. */
uint64_t mi355_w8a8_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t n_adapters,
                                    uint32_t rank, uint32_t flags);
uint64_t mi355_w8a8_grouped_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t n_groups,
                                            uint32_t rank, uint32_t flags);

/* W8A8 linear + (multi-adapter) LoRA; rms_gamma, residual and FLAG_SWIGLU must be unset. */
int mi355_w8a8_lora_linear_v1(const mi355_w8a8_problem* problem, void* stream);
/* RMSNorm -> W8A8 gate/up + LoRA -> SwiGLU; requires rms_gamma and FLAG_SWIGLU, even n. */
int mi355_w8a8_rms_gateup_swiglu_v1(const mi355_w8a8_problem* problem, void* stream);
/* W8A8 down projection + LoRA + residual; requires residual. */
int mi355_w8a8_lora_residual_v1(const mi355_w8a8_problem* problem, void* stream);
/* Any combination of the optional stages (superset of the three above). */
int mi355_w8a8_forward_v1(const mi355_w8a8_problem* problem, void* stream);
/* Grouped / ragged per-expert variant. */
int mi355_w8a8_grouped_v1(const mi355_w8a8_grouped_problem* problem, void* stream);
/*
 * mi355_w8a8_forward_v1 on a workspace the library owns.  No counterpart in the reference: it is for
 * callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid it).  problem->workspace and problem->workspace_bytes are ignored; the call
 * uses a static device array of MI355_W8A8_STATIC_WORKSPACE_BYTES that every GPU the library runs on
 * holds until the process ends, and returns MI355_W8A8_ERR_WORKSPACE when
 * mi355_w8a8_workspace_bytes(...) of the problem exceeds that size.  Inputs and outputs are the
 * caller's as before.  All calls on one GPU share the array: calls that overlap in time on one GPU
 * (two streams, two threads) race; calls on one stream are ordered and safe.  The first call on a
 * device resolves the array's address (a host-side lookup, no allocation): make one call on a device
 * before capturing a graph there.  Because any caller's call in between may have overwritten the array,
 * MI355_W8A8_FLAG_LORA_PACK_VALID and MI355_W8A8_FLAG_SKIP_PROLOGUE are answered with
 * MI355_W8A8_ERR_UNSUPPORTED.
 */
#define MI355_W8A8_STATIC_WORKSPACE_BYTES (32u << 20)
int mi355_w8a8_forward_static_ws_v1(const mi355_w8a8_problem* problem, void* stream);

/*
 * Backward (VJP) of mi355_w8a8_lora_linear_v1: replaces the custom_vjp rule
 * _quantized_lora_linear_bwd (skyrl/tx/kernels/quantized_lora.py:337-394) with the bf16 weight
 * policy of the ROCm prototype's pull-back (skyrl/tx/kernels/rocm/w8a8_lora.py:298-339,722-821).
 */
uint64_t mi355_w8a8_bwd_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t n_adapters,
                                        uint32_t rank, uint32_t flags);
int mi355_w8a8_lora_linear_bwd_v1(const mi355_w8a8_bwd_problem* problem, void* stream);

/*
 * Backward of mi355_w8a8_grouped_v1 without FLAG_SWIGLU: the derivative of LoRAExpert.__call__
 * (skyrl/tx/layers/lora.py:394-444, ragged_dot of skyrl/tx/layers/util.py:8-59) under the rule of
 * mi355_w8a8_lora_linear_bwd_v1, in one call for all groups: every weight's rows form their own
 * 256-row pull-back tiles, the groups that share a weight take the role of its adapters.  The
 * results are bit-equal to one mi355_w8a8_lora_linear_bwd_v1 call per weight over its rows.
 */
uint64_t mi355_w8a8_grouped_bwd_workspace_bytes(uint32_t m, uint32_t k, uint32_t n, uint32_t n_groups,
                                                uint32_t rank, uint32_t groups_per_weight);
int mi355_w8a8_grouped_bwd_v1(const mi355_w8a8_grouped_bwd_problem* problem, void* stream);

/*
 * The part of qwen35_qkv_lora_rope behind the projection (skyrl/tx/kernels/qwen3_5_qkv_lora.py:
 * 266-286: _split_interleaved_qkv, the Q/gate split, _delta_rms_norm on Q and K,
 * _apply_partial_rope).  The projection with its input RMSNorm is mi355_w8a8_forward_v1 with
 * rms_gamma = 1 + input_norm_weight.
 */
int mi355_w8a8_qkv_split_norm_rope_v1(const mi355_w8a8_qkv_post_problem* problem, void* stream);

/*
 * Pull-back of qwen35_qkv_lora_rope behind and before the projection
 * (_qwen35_qkv_lora_rope_bwd, skyrl/tx/kernels/qwen3_5_qkv_lora.py:360-451).  The whole rule, with
 * fused and normalized = the projection and its normalized input (mi355_w8a8_forward_v1 with
 * rms_gamma = 1 + input_norm_weight and aux_normalized), is
 *   d_fused [, d_q_norm_weight, d_k_norm_weight] = qkv_split_norm_rope_bwd(fused, d_q, d_k, d_v, d_gate)
 *   d_normalized, d_lora_a, d_lora_b, d_lora_scaling = mi355_w8a8_lora_linear_bwd_v1(normalized, d_fused)
 *   d_hidden [, d_input_norm_weight] = delta_rms_norm_bwd(hidden, 1 + input_norm_weight, d_normalized)
 *
 * mi355_w8a8_qkv_split_norm_rope_bwd_v1 replaces :391-425: _apply_partial_rope_transpose (:148-164)
 * on d_q and d_k, _delta_rms_norm_vjp (:97-116) per Q and K head against the raw projection, and
 * _fuse_interleaved_qkv (:235-247) of the result with d_gate and d_v.
 *
 * mi355_w8a8_delta_rms_norm_bwd_v1 replaces _delta_rms_norm_vjp (:97-116) for the decoder norm: x,
 * d_normalized, d_x bf16 [m, k]; gamma f32 [k] is the multiplier 1 + weight.  d_gamma f32 [k] is
 * optional (the cotangent of the weight; 1 + weight has the same one) and then needs the workspace
 * and a d_x buffer apart from d_normalized; without it d_x may be the d_normalized buffer itself.
 */
uint64_t mi355_w8a8_qkv_bwd_workspace_bytes(uint32_t m, uint32_t head_dim);
int mi355_w8a8_qkv_split_norm_rope_bwd_v1(const mi355_w8a8_qkv_post_bwd_problem* problem, void* stream);
uint64_t mi355_w8a8_delta_rms_norm_bwd_workspace_bytes(uint32_t m, uint32_t k);
int mi355_w8a8_delta_rms_norm_bwd_v1(const void* x, const float* gamma, const void* d_normalized, void* d_x,
                                     float* d_gamma, void* workspace, uint64_t workspace_bytes, uint32_t m,
                                     uint32_t k, float eps, void* stream);

/*
 * The two stages around the projection in the pull-back of the fused RMSNorm -> gate/up + LoRA ->
 * SwiGLU call (skyrl/tx/kernels/rocm/bf16_rms_gate_up_lora_swiglu_contiguous.py:643-689).  With
 * fused = the bf16 projection (mi355_w8a8_forward_v1 with rms_gamma, without FLAG_SWIGLU, which
 * also returns the normalized activations in aux_normalized), the whole rule is
 *   d_fused = swiglu_bwd(fused, d_product)
 *   d_normalized, d_lora_a, d_lora_b, d_lora_scaling = mi355_w8a8_lora_linear_bwd_v1(normalized, d_fused)
 *   d_x = rms_norm_bwd(x, gamma, d_normalized)
 *
 * mi355_w8a8_swiglu_bwd_v1 replaces _fp32_swiglu_pullback_interleaved (:541-553): fused bf16 [m, n]
 * with columns (gate_0, up_0, gate_1, up_1, ...), d_product bf16 [m, n / 2], d_fused bf16 [m, n];
 * n % 8 == 0; d_fused may be the fused buffer itself.
 *
 * mi355_w8a8_rms_norm_bwd_v1 replaces _rms_norm_pullback (:556-574): x, d_normalized, d_x bf16
 * [m, k]; gamma f32 [k] is the multiplier itself (1 + rms_delta); the row statistics are recomputed
 * from x with the forward's rule; d_x may be the d_normalized buffer itself.  gamma gets no
 * cotangent, as in the reference.
 */
int mi355_w8a8_swiglu_bwd_v1(const void* fused, const void* d_product, void* d_fused, uint32_t m, uint32_t n,
                             void* stream);
/*
 * The SwiGLU stage on its own (_fp32_swiglu_from_interleaved, :535-538): product bf16 [m, n / 2] from the
 * bf16 projection [m, n], bit for bit what FLAG_SWIGLU produces.  A training forward that keeps the
 * projection for the pull-back (as the reference's _forward_with_residuals does, :489-532) runs the
 * projection without the flag and then this call, and its backward skips the recomputation.
 */
int mi355_w8a8_swiglu_v1(const void* fused, void* product, uint32_t m, uint32_t n, void* stream);
int mi355_w8a8_rms_norm_bwd_v1(const void* x, const float* gamma, const void* d_normalized, void* d_x, uint32_t m,
                               uint32_t k, float eps, void* stream);

/*
 * Token routing around the grouped expert GEMMs (Qwen3Experts.__call__, skyrl/tx/models/qwen3.py:
 * 172-210).  Index outputs are exact; nothing here synchronizes or allocates.
 *
 * mi355_w8a8_moe_route_v1 replaces qwen3.py:175-178: probabilities = softmax(router_logits) in
 * float32, top_k largest per token in descending order (ties: the lower expert, as lax.top_k),
 * weights divided by their sum when norm_topk_prob.  router_logits f32 [n_tokens, n_experts],
 * weights f32 and selected int32 [n_tokens, top_k]; n_experts <= 1024, top_k <= min(64, n_experts).
 */
int mi355_w8a8_moe_route_v1(const float* router_logits, uint32_t n_tokens, uint32_t n_experts, uint32_t top_k,
                            uint32_t norm_topk_prob, float* weights, int32_t* selected, void* stream);

/*
 * Pull-back of mi355_w8a8_moe_route_v1 to the logits with the selection held fixed, as lax.top_k
 * differentiates (qwen3.py:175-178): d_router_logits f32 [n_tokens, n_experts] from d_weights f32
 * [n_tokens, top_k] and the selected int32 [n_tokens, top_k] the forward returned.  d_router_logits
 * may be the router_logits buffer itself.
 */
int mi355_w8a8_moe_route_bwd_v1(const float* router_logits, const int32_t* selected, const float* d_weights,
                                uint32_t n_tokens, uint32_t n_experts, uint32_t top_k, uint32_t norm_topk_prob,
                                float* d_router_logits, void* stream);

/*
 * mi355_w8a8_moe_dispatch_v1 replaces prepare_routing (skyrl/tx/layers/util.py:66-87) together with
 * the jnp.repeat in front of it (qwen3.py:189-190): pair p = (token p / repeat, choice p % repeat)
 * belongs to group indices[p]; the pairs are sorted by group, stably, and every pair's token row is
 * copied to its sorted position.  repeat = top_k for the expert MLP, 1 for a plain prepare_routing.
 * Group indices outside [0, n_groups) are clamped into range.
 */
typedef struct mi355_w8a8_moe_dispatch_problem {
  uint32_t struct_size;     /* sizeof(mi355_w8a8_moe_dispatch_problem) */
  uint32_t flags;           /* 0 */
  uint32_t n_pairs;         /* rows to sort = tokens * repeat */
  uint32_t repeat;          /* >= 1, divides n_pairs */
  uint32_t width;           /* bf16 columns of a token row, multiple of 8 (ignored without tokens) */
  uint32_t n_groups;        /* <= 1024 */
  const void* tokens;       /* bf16 [n_pairs / repeat, width], or NULL: index outputs only */
  const int32_t* indices;   /* int32 [n_pairs] */
  const int32_t* adapter_indices; /* optional int32 [n_pairs / repeat], sorted along with the rows */
  void* sorted_tokens;      /* bf16 [n_pairs, width] (with tokens) */
  int32_t* group_sizes;     /* int32 [n_groups] */
  int32_t* sort_indices;    /* int32 [n_pairs]: the pair at every sorted position (argsort) */
  int32_t* unsort_indices;  /* int32 [n_pairs]: the sorted position of every pair (its inverse) */
  int32_t* sorted_adapters; /* int32 [n_pairs], with adapter_indices */
  void* workspace;          /* 256-byte aligned device scratch */
  uint64_t workspace_bytes; /* >= mi355_w8a8_moe_dispatch_workspace_bytes(n_pairs, n_groups) */
} mi355_w8a8_moe_dispatch_problem;

uint64_t mi355_w8a8_moe_dispatch_workspace_bytes(uint32_t n_pairs, uint32_t n_groups);
int mi355_w8a8_moe_dispatch_v1(const mi355_w8a8_moe_dispatch_problem* problem, void* stream);

/*
 * mi355_w8a8_moe_combine_v1 replaces the unsort and weighted sum of qwen3.py:205-207:
 * out[t] = bf16(sum_j f32(expert_out[unsort_indices[t * top_k + j]]) * weights[t, j]), products and
 * the sum in float32 in choice order.  expert_out bf16 [n_tokens * top_k, width] in sorted order,
 * out bf16 [n_tokens, width]; width a multiple of 8, top_k <= 64.
 */
int mi355_w8a8_moe_combine_v1(const void* expert_out, const int32_t* unsort_indices, const float* weights, void* out,
                              uint32_t n_tokens, uint32_t top_k, uint32_t width, void* stream);

/*
 * Pull-back of the combine (the derivative of qwen3.py:205-207 in its two operands): for the sorted
 * row at position pos with pair = sort_indices[pos],
 *   d_expert_out[pos] = bf16(f32(d_out[pair / top_k]) * weights[pair])
 *   d_weights[pair]   = sum_c f32(expert_out[pos, c]) * f32(d_out[pair / top_k, c])   (float32)
 * d_out bf16 [n_tokens, width]; expert_out, d_expert_out bf16 [n_tokens * top_k, width] in sorted order;
 * d_weights f32 [n_tokens, top_k] or NULL (then expert_out may be NULL too).  The cotangent of the hidden
 * rows through the gather of the dispatch is mi355_w8a8_moe_combine_v1 with unit weights.
 */
int mi355_w8a8_moe_combine_bwd_v1(const void* d_out, const void* expert_out, const int32_t* sort_indices,
                                  const float* weights, void* d_expert_out, float* d_weights, uint32_t n_tokens,
                                  uint32_t top_k, uint32_t width, void* stream);

/*
 * Group-scaled quantized linear: the general form of quantized_frozen_linear / quantized_lora_linear
 * (skyrl/tx/kernels/quantized_lora.py:215-304) -- W4 or W8 codes with one scale per (K group, output),
 * A4 or A8 activations quantized per (row, K group):
 *   out = bf16( sum_g ((f32(acc_g) * x_scale[m, g]) * w_scale[g, n])  +  s[idx] * ((x @ A[idx]) @ B[idx]) )
 * with the groups added in float32 in group order, as the reference does (the float32 base is
 * reproduced bit for bit; aux_base returns it).  group_size must be a multiple of 32 and divide
 * k_pad; k <= k_pad (the reference pads K with zeros).  The per-channel W8A8 case
 * (group_size == k) is better served by mi355_w8a8_forward_v1.
 *
 * mi355_w8a8_gq_pack_weight_v1 re-lays the reference's codes (bits 8: int8 [k_pad, n]; bits 4: uint8
 * [k_pad / 2, n] with the even k in the low nibble, quantized_lora.py:94-125) into matrix-core
 * fragments once at load time; 4-bit codes stay 4-bit (half a byte per weight in HBM).
 */
uint64_t mi355_w8a8_gq_packed_weight_bytes(uint32_t k_pad, uint32_t n, uint32_t weight_bits);
int mi355_w8a8_gq_pack_weight_v1(const void* codes, void* packed, uint32_t k_pad, uint32_t n, uint32_t weight_bits,
                                 void* stream);

/* Calls of more than 32 rows whose groups are multiples of 64 run on 128 x 128 tiles staged through the LDS;
 * this flag asks for the kernel that feeds its wave tiles straight from the L2 instead (the only one for
 * other group sizes).  Both give the same bits; the flag exists for that comparison and for measurements. */
#define MI355_W8A8_FLAG_GQ_DIRECT 1u

typedef struct mi355_w8a8_gq_problem {
  uint32_t struct_size;      /* sizeof(mi355_w8a8_gq_problem) */
  uint32_t flags;            /* 0 or MI355_W8A8_FLAG_GQ_DIRECT */
  uint32_t m, k, k_pad, n;
  uint32_t group_size;       /* multiple of 32, divides k_pad */
  uint32_t weight_bits;      /* 4 or 8 */
  uint32_t activation_bits;  /* 4 or 8 */
  uint32_t n_adapters;       /* 0 = no LoRA */
  uint32_t rank;             /* <= 64 */
  uint32_t reserved;
  const void* x;             /* bf16 [m, k] */
  const void* w_packed;      /* from mi355_w8a8_gq_pack_weight_v1 */
  const float* w_scales;     /* f32 [k_pad / group_size, n] */
  const void* lora_a;        /* bf16 [n_adapters, k, rank] or NULL */
  const void* lora_b;        /* bf16 [n_adapters, rank, n] or NULL */
  const float* lora_scaling; /* f32 [n_adapters] or NULL */
  const int32_t* adapter_indices; /* int32 [m] or NULL (adapter 0) */
  void* out;                 /* bf16 [m, n] */
  void* workspace;           /* >= mi355_w8a8_gq_workspace_bytes(...), 256-byte aligned */
  uint64_t workspace_bytes;
  /* Optional auxiliary outputs for parity checks (NULL to skip) */
  int8_t* aux_x_codes;       /* int8 [m, k_pad] */
  float* aux_x_scales;       /* f32 [m, k_pad / group_size] */
  float* aux_base;           /* f32 [m, n]: the float32 base before the LoRA term */
} mi355_w8a8_gq_problem;

uint64_t mi355_w8a8_gq_workspace_bytes(uint32_t m, uint32_t k_pad, uint32_t group_size, uint32_t n_adapters,
                                       uint32_t rank);
int mi355_w8a8_gq_linear_v1(const mi355_w8a8_gq_problem* problem, void* stream);

/*
 * Which kernels mi355_w8a8_forward_v1 and its three named forms run for these dimensions and flags
 * (no counterpart in the reference; for benchmarks and logs).  Returns an MI355_W8A8_PATH_* value or
 * a negative status.
 */
#define MI355_W8A8_PATH_SKINNY 1         /* m <= 32: row quantizer + weight-streaming kernel */
#define MI355_W8A8_PATH_SKINNY_CHUNKS 2  /* 33..128 rows: the same two kernels per chunk of 32 rows */
#define MI355_W8A8_PATH_TILED_256X128 3  /* prologue + 256 x 128 tiles, two workgroups per CU */
#define MI355_W8A8_PATH_TILED_256X256 4  /* prologue + 256 x 256 tiles, one workgroup per CU */
#define MI355_W8A8_PATH_TILED_128X128 5  /* prologue + 128 x 128 tiles, two workgroups per CU */
#define MI355_W8A8_PATH_TILED_256X128_PAIR 6  /* prologue + 256 x 128 tiles on 16 x 16 x 64 MFMAs, two workgroups per CU */
int mi355_w8a8_forward_path(uint32_t m, uint32_t k, uint32_t n, uint32_t flags);

/*
 * Calibration (no counterpart in the reference: these measure the ceilings the path is priced against,
 * for bench.py and profiles/).  mi355_w8a8_calibrate_mfma_v1 runs `iters` (at most 2^18) rounds of int8 MFMAs on
 * operands that stay in registers: shape 0 = 16 of the 32 x 32 x 32 instruction per wave and round,
 * shape 1 = 64 of the 16 x 16 x 64 one; 256 workgroups of four waves.  `operands` holds
 * mi355_w8a8_calibrate_operand_bytes() bytes of codes (zeros, random bits, realistic codes: the rate
 * the part sustains under its power limit depends on them).  One launch performs
 * mi355_w8a8_calibrate_mfma_ops(shape, iters) int8 operations.  `clocks` (2 x uint64) receives the
 * shader cycles and the 100 MHz ticks one workgroup spent in the loop; `sink` is 4 writable bytes.
 * mi355_w8a8_calibrate_read_v1 streams `bytes` (a multiple of 32768) from `src` and discards them.
 * mi355_w8a8_calibrate_copy_v1 copies `bytes` (a multiple of 16) with 16-byte loads and stores: a kernel of
 * known traffic against which hardware traffic counters are scaled.
 */
uint64_t mi355_w8a8_calibrate_operand_bytes(void);
uint64_t mi355_w8a8_calibrate_mfma_ops(uint32_t shape, uint32_t iters);
int mi355_w8a8_calibrate_mfma_v1(uint32_t shape, const void* operands, uint32_t iters, uint64_t* clocks,
                                 int32_t* sink, void* stream);
int mi355_w8a8_calibrate_read_v1(const void* src, uint64_t bytes, uint32_t* sink, void* stream);
int mi355_w8a8_calibrate_copy_v1(const void* src, void* dst, uint64_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355_W8A8_H_ */
