/*
 * llmi_hip.h -- C ABI of the gfx950 (MI355X) decode-attention backend.
 *
 * Plain pointers and sizes only. Every entry point returns LLMI_OK (0) or a
 * negative llmi_status; nothing here aborts the process. All device work is
 * enqueued on the caller's stream and borrows the caller's buffers until that
 * stream has been synchronised. Not thread-safe per pool / per stream, like
 * the engine it plugs into (one host thread, one stream).
 *
 * Reference interfaces replaced (paths relative to the reference checkout):
 *   llmi_hip_mha_decode           kernel::mha_kernel_cu
 *                                 code/source/op/kernel/cuda/mha_kernel.cu:440-529
 *                                 (registry slot kernel_interface.h:168-183,
 *                                 kernel_interface.cpp:181-190; caller
 *                                 code/source/op/mha.cpp:54-56)
 *   llmi_hip_mha_decode_append    the pair fused_qk_norm_rope_kernel_cu + mha_kernel_cu as
 *                                 the layer loop issues it, code/source/model/qwen3_fused.cpp:524-548
 *   llmi_hip_mha_decode_append_stack  that pair for every layer of the layer loop,
 *                                 code/source/model/qwen3_fused.cpp:115-127 (one resident launch)
 *   llmi_hip_mha_workspace_bytes  the KVSplitOutput buffer sizing
 *                                 code/source/model/qwen3_fused.cpp:502-503
 *   llmi_hip_mha_plan             the dispatch arithmetic inside mha_kernel_cu
 *                                 mha_kernel.cu:505-517
 *   llmi_hip_qk_norm_rope_append  kernel::fused_qk_norm_rope_kernel_cu
 *                                 code/source/op/kernel/cuda/rmsnorm_kernel.cu:248-290
 *                                 plus the K/V row placement of
 *                                 Model::slice_kv_cache code/source/model/model.cpp:90-107
 *   llmi_hip_sincos_table         kernel::sin_cos_cache_precompute_cu
 *                                 code/source/op/kernel/cuda/rope_kernel.cu:23-46
 *   llmi_hip_kv_restride          (new) converts a position-major cache
 *                                 (qwen3_fused.cpp:488-491) to the head-major layout
 *   llmi_hip_mha_workspace_side   (new) measures, once per KVSplitOutput allocation
 *                                 (qwen3_fused.cpp:502-503), which of its 8 KiB blocks lie near
 *                                 which side of the GPU package; llmi_mha_args.workspace_side
 *   llmi_hip_mha_decode_static    (new) llmi_hip_mha_decode without a caller's workspace
 *   llmi_pool_* / llmi_hip_pool_* base::CUDADeviceAllocator::allocate / release
 *                                 code/source/base/alloc_cu.cpp:7-119
 *   llmi_hip_memcpy / memset_zero base::DeviceAllocator::memcpy / memset_zero
 *                                 code/source/base/alloc.cpp:11-72
 */
#ifndef LLMI_HIP_H
#define LLMI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Bumped whenever a struct below changes size or layout, or an entry point changes meaning: a caller compiled
 * against another value must not call into this library (llmi_hip_abi_version() returns the library's).
 * 3: llmi_mha_args.workspace_side, llmi_mha_plan.workspace_side, llmi_attn_oproj_args.one_launch,
 *    llmi_hip_mha_decode_append_stack. */
#define LLMI_HIP_ABI_VERSION 3

typedef enum llmi_status {
    LLMI_OK = 0,
    LLMI_ERR_NULL_POINTER = -1,   /* a required pointer is NULL                       */
    LLMI_ERR_HEAD_DIM = -2,       /* head_dim != 128 (mha_kernel.cu:478-479)          */
    LLMI_ERR_KV_DIM = -3,         /* kv_dim not a positive multiple of head_dim / 8   */
    LLMI_ERR_ALIGNMENT = -4,      /* q/K/V/out not 16-byte aligned (mha_kernel.cu:495-498) */
    LLMI_ERR_POS_RANGE = -5,      /* pos < 0 or pos >= max_seq_len (mha_kernel.cu:473-474) */
    LLMI_ERR_WORKSPACE = -6,      /* workspace missing or too small for the split path */
    LLMI_ERR_HEAD_GROUP = -7,     /* head_num != kv_mul * (kv_dim/head_dim), or kv_mul > 16 */
    LLMI_ERR_LAYOUT = -8,         /* unknown kv_layout                                 */
    LLMI_ERR_INVALID_ARG = -9,    /* any other out-of-range scalar                     */
    LLMI_ERR_LAUNCH = -10,        /* hipGetLastError() after a launch / a HIP call failed */
    LLMI_ERR_UNKNOWN_POINTER = -11, /* pool free of a pointer the pool does not own    */
    LLMI_ERR_OUT_OF_MEMORY = -12  /* backing allocator failed                          */
} llmi_status;

/* KV-cache layouts. Both hold bf16 bit patterns (uint16_t) and head_dim = 128. */
enum {
    /* the reference's: [layer][max_seq_len][kv_head][128]  (qwen3_fused.cpp:488-491) */
    LLMI_KV_LAYOUT_POS_MAJOR = 0,
    /* re-strided:      [layer][kv_head][max_seq_len][128] -- each KV head's rows are contiguous */
    LLMI_KV_LAYOUT_HEAD_MAJOR = 1
};

/* SPLIT runs the split kernel and then a combine kernel; SPLIT_FUSED runs the
 * split kernel alone, whose last-arriving workgroup per KV head does the combine. */
enum { LLMI_PATH_AUTO = 0, LLMI_PATH_SINGLE_PASS = 1, LLMI_PATH_SPLIT = 2, LLMI_PATH_SPLIT_FUSED = 3 };

typedef struct llmi_mha_args {
    const void* query;        /* device, bf16 [head_num*head_dim]                        */
    const void* key_cache;    /* device, bf16, base of the whole cache (all layers)      */
    const void* value_cache;  /* device, bf16                                            */
    void* workspace;          /* device, fp32 split partials; may be NULL if single-pass */
    size_t workspace_bytes;   /* size of workspace                                       */
    void* output;             /* device, bf16 [head_num*head_dim]                        */
    float* output_f32;        /* optional device fp32 [head_num*head_dim] tap of the
                                 result before bf16 rounding; NULL in production         */
    int32_t layer_id;
    int32_t pos;              /* attends to positions 0..pos                             */
    int32_t kv_dim;           /* kv_heads * head_dim                                     */
    int32_t kv_mul;           /* query heads per KV head                                 */
    int32_t head_num;         /* query heads                                             */
    int32_t head_dim;         /* must be 128                                             */
    int32_t max_seq_len;      /* positions per layer in the cache                        */
    int32_t kv_layout;        /* LLMI_KV_LAYOUT_*                                        */
    int32_t force_path;       /* LLMI_PATH_*; AUTO picks by context length               */
    int32_t num_splits;       /* 0 = auto; otherwise the KV split count of the split path */
    int32_t waves_per_group;  /* 0 = auto; 1,2,4,8 wavefronts per workgroup (tuning)     */
    void* stream;             /* hipStream_t, NULL = the null stream                     */
    const int32_t* pos_device; /* optional, device int32: when non-NULL the kernels read the position
                                 from here at run time, so one captured launch serves every token
                                 up to `pos`, which then is the LARGEST position the launch may see
                                 (it sizes the grid; larger values read from the device are clamped
                                 to it). The reference bakes pos into the launch (mha.cpp:55,60-66).
                                 Not available with LLMI_PATH_SPLIT.                       */
    int32_t workspace_side;   /* 0, or what llmi_hip_mha_workspace_side reported for this workspace: the
                                 fused combine then keeps every KV head's partial results and records in
                                 the memory nearest to the XCD that head runs on. Changes the time of a call,
                                 never its result.                                          */
} llmi_mha_args;

typedef struct llmi_mha_plan {
    int32_t path;             /* LLMI_PATH_SINGLE_PASS, LLMI_PATH_SPLIT or LLMI_PATH_SPLIT_FUSED */
    int32_t num_splits;       /* 1 for single-pass                                       */
    int32_t rows_per_split;   /* most positions one split handles (multiple of 16): a head's 16-position
                                 tiles go to the splits in contiguous runs that differ by at most one tile */
    int32_t waves_per_group;
    int32_t group_pad;        /* query heads per KV head rounded up to 1,2,4,8,16        */
    int32_t workspace_side;   /* 1 if the launch lays the workspace out by package side (args->workspace_side
                                 set, fused combine, a multiple of eight KV heads, groups of at most 8 query
                                 heads at the wave count the dispatcher picks itself, room for two homes per
                                 row), else 0                                             */
    size_t workspace_needed;  /* bytes of workspace this plan uses (0 for single-pass)   */
} llmi_mha_plan;

/* Validates args and reports what llmi_hip_mha_decode would launch. Makes no
 * HIP call, so it also works on a host without a GPU. */
int llmi_hip_mha_plan(const llmi_mha_args* args, llmi_mha_plan* plan);

/* Decode attention for one layer and one new token: for every query head h,
 * out[h] = softmax(q[h].K[h/kv_mul]^T / sqrt(128)) . V[h/kv_mul] over positions
 * 0..pos, bf16 in, fp32 accumulate, bf16 out. Enqueues 1 kernel (single-pass,
 * split with fused combine) or 2 (split + combine). Allocates nothing; safe
 * under stream capture. The workspace needs no initialisation. Two calls that
 * share a workspace must not overlap in time. */
int llmi_hip_mha_decode(const llmi_mha_args* args);

/* No counterpart in the reference. For callers that cannot allocate device memory and have no workspace to
 * pass -- code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc: the same
 * computation as llmi_hip_mha_decode with the same results, but the split path's partial results and arrival
 * records go to a fixed 4 MiB array in device memory that is part of the library's code object (each GPU
 * the library runs on holds one from its first use until the process ends). `workspace` and
 * `workspace_bytes` of `args` are ignored. Calls no hipMalloc / hipFree or any other allocating routine.
 * The array bounds the split count: the automatic plan takes as many splits as fit (what
 * llmi_hip_mha_decode does with a workspace of that size: head_num * splits * 528 + 16 bytes), a forced
 * `num_splits` that needs more, or a head count so large that two splits do not fit, is rejected with
 * LLMI_ERR_WORKSPACE and llmi_hip_last_error() says so. Every call on a GPU shares that GPU's array: two
 * calls that overlap in time on one GPU (two streams, two threads) race, like two calls of
 * llmi_hip_mha_decode on one workspace. The array needs no clearing between calls (records carry a per-call
 * tag). The first call on a device looks the array's address up (which may load the code object): make it
 * outside stream capture. */
int llmi_hip_mha_decode_static(const llmi_mha_args* args);

typedef struct llmi_mha_append_args {
    llmi_mha_args mha;        /* as for llmi_hip_mha_decode, except: mha.query is the RAW query of the new
                                 token (before QK-Norm), and the caches are written at (layer_id, pos)  */
    const void* key_new;      /* device bf16 [kv_dim]: the new token's raw K row                        */
    const void* value_new;    /* device bf16 [kv_dim]: the new token's V row                            */
    const void* norm_weight;  /* device bf16 [2*128]: q_norm then k_norm                                */
    const float* sin_cache;   /* device fp32 [max_seq_len][64]                                          */
    const float* cos_cache;   /* device fp32 [max_seq_len][64]                                          */
    float eps;                /* 1e-6 in the reference                                                  */
} llmi_mha_append_args;

/* llmi_hip_qk_norm_rope_append followed by llmi_hip_mha_decode, as ONE kernel launch: the query group and
 * the new K row are normalised + rotated inside the attention kernel, the K and V rows of position `pos`
 * are stored to the cache (either layout) and used from registers. The normalised query is not written
 * back. Replaces the back-to-back pair fused_qk_norm_rope + mha of the reference's layer loop
 * (code/source/model/qwen3_fused.cpp:524-548; kernels rmsnorm_kernel.cu:248-290, mha_kernel.cu:440-529).
 * The separate-combine path (LLMI_PATH_SPLIT) is not available here. */
int llmi_hip_mha_decode_append(const llmi_mha_append_args* args);

typedef struct llmi_attn_oproj_args {
    llmi_mha_append_args attn; /* as for llmi_hip_mha_decode_append; attn.mha.output still receives the attention output */
    const void* o_weight;      /* device bf16 [hidden][head_num*128] row-major: the layer's output projection         */
    void* residual;            /* device bf16 [hidden]: residual += o_weight . attention output, rounded once          */
    int32_t hidden;
    int32_t one_launch;        /* 0 (default): two launches, attention then projection. 1: ask for the one-launch form
                                  (see below); only for a GPU the caller has to itself                                   */
} llmi_attn_oproj_args;

/* llmi_hip_mha_decode_append followed by llmi_hip_gemv in LLMI_GEMV_ADD_BF16 mode on its output: the tail of the
 * reference's attention block, mha_kernel_cu then fused_gemv_add_kernel_cu (code/source/model/qwen3_fused.cpp:548-552;
 * kernels mha_kernel.cu:440-529, matmul_kernel.cu:174-208). By default exactly those two launches (the faster form on
 * an MI355X, and one that waits for nothing). With `one_launch` = 1, and where the shape allows it, ONE launch: the
 * workgroups that have handed their partial results over fetch the projection's weight rows while the combine still
 * runs, wait (bounded, like the combine: llmi_hip_set_poll_limit) for the attention output and finish
 * residual += W x. Same results as the two calls, bit for bit. In that form workgroups wait for other workgroups of
 * the same launch, so every workgroup of the grid has to be resident at once: ask for it only on a GPU that runs
 * nothing else at the time (another stream's or process's kernel that holds compute units can keep the waited-for
 * workgroups out until the wait gives up). A wait that gives up leaves its rows of the residual as they were (no
 * NaN is stored into the in-place residual stream; the attention output is still poisoned by the combine's own
 * give-up) and is counted: check llmi_hip_poll_timeouts. The one-launch form needs: the fused split path with at
 * least two splits and a host-side position, a query group of 1, 2, 4 or 8 heads, head_num*128 <= 4096,
 * hidden <= 3 * (wavefronts of the workgroups that do not combine), a grid no larger than the device's compute unit
 * count, and head_num*4 more bytes of workspace than the plan reports. Anything else runs as the two launches.
 * llmi_hip_mha_oproj_launches tells which: 1 or 2 (or a negative status for invalid arguments). */
int llmi_hip_mha_decode_append_oproj(const llmi_attn_oproj_args* args);
int llmi_hip_mha_oproj_launches(const llmi_attn_oproj_args* args);

typedef struct llmi_mha_stack_args {
    llmi_mha_append_args first; /* the first layer's call, exactly as for llmi_hip_mha_decode_append
                                   (first.mha.layer_id = the first layer of the run)                                  */
    int32_t layer_count;        /* consecutive layers, >= 1; layer l of the run uses cache layer first.mha.layer_id + l */
    /* elements (bf16) between one layer's buffer and the next layer's; multiples of 8; 0 = every layer uses the same */
    int64_t query_stride;       /* first.mha.query      + l * query_stride       = layer l's raw query [head_num*128]  */
    int64_t key_new_stride;     /* first.key_new        + l * key_new_stride     = layer l's raw K row [kv_dim]        */
    int64_t value_new_stride;   /* first.value_new      + l * value_new_stride   = layer l's V row [kv_dim]            */
    int64_t norm_weight_stride; /* first.norm_weight    + l * norm_weight_stride = layer l's q_norm | k_norm [2*128]   */
    int64_t output_stride;      /* first.mha.output     + l * output_stride      = layer l's output [head_num*128]
                                   (and first.mha.output_f32 + l * output_stride, in floats, if that tap is set)       */
} llmi_mha_stack_args;

/* llmi_hip_mha_decode_append for `layer_count` consecutive layers at one position, in layer order: the attention part
 * of one decode step as the reference's layer loop issues it (code/source/model/qwen3_fused.cpp:115-127: per layer
 * fused_qk_norm_rope + mha, :524-548). Same results as that many calls, bit for bit, including when buffers alias
 * across layers (a layer's query may be the previous layer's output: a layer reads its query, K row and V row only
 * after the previous layer's output is complete).
 * Where the shape allows it this is ONE launch: the split path's grid stays resident and walks the layers itself, every
 * wavefront streaming its K/V tiles of all layers as one sequence (the next layer's tiles are on their way while this
 * layer's partial results are handed over and merged), and a layer's inputs are read only after every query head of
 * the layer before has published a "done" tag behind its acknowledged output. Workgroups wait for other workgroups of
 * the same launch there, so every workgroup of the grid has to be resident at once: call this only on a GPU that runs
 * nothing else at the time. Every wait is bounded (llmi_hip_set_poll_limit); one that gives up is counted
 * (llmi_hip_poll_timeouts) and turns the outputs of its layer and the following ones into NaN. The one-launch form
 * needs: the fused split path with 2..64 splits and a host-side position, a query group of at most 4 heads, a grid no
 * larger than the device's compute unit count, and a workspace sized by llmi_hip_mha_workspace_bytes (the plan's need
 * plus 4.3 KiB for the tags). Anything else runs as layer_count launches of llmi_hip_mha_decode_append.
 * llmi_hip_mha_stack_launches tells which: 1 or layer_count (or a negative status for invalid arguments). */
int llmi_hip_mha_decode_append_stack(const llmi_mha_stack_args* args);
int llmi_hip_mha_stack_launches(const llmi_mha_stack_args* args);

/* Bytes of fp32 workspace that are enough for any pos < max_seq_len. */
size_t llmi_hip_mha_workspace_bytes(int32_t head_num, int32_t head_dim, int32_t max_seq_len);

/* No counterpart in the reference. The eight XCDs of the GPU sit on two sides of the package and so does its memory:
 * which side an address belongs to changes every 8 KiB (hashed with higher address bits), and handing a value from one
 * workgroup to another takes 0.1-0.2 us longer through the far side. This call times hand-overs between two workgroups of
 * every XCD through two neighbouring 8 KiB blocks near the start of `workspace` (llmi_hip_probe_block_pingpong) and
 * derives from them which blocks are near which side, for every 2 MiB-aligned region the workspace reaches into (the
 * answer holds within such a region and differs between them): *sides gets two bits per region, counted from the region
 * the workspace starts in, 1 = XCDs 0-3 are nearest to addresses with bit 13 clear, 2 = ... set, 0 = the two did not
 * differ measurably (or the region is the 17th or later). Pass the value as llmi_mha_args.workspace_side with this
 * workspace, and size the workspace by llmi_hip_mha_workspace_bytes (the layout keeps two homes per row, one in near
 * memory for either side): 0.3-0.5 us per split-path call on a Qwen3-4B layer against the unlucky placement of the plain
 * layout, 0.1-0.25 us against the lucky one. One measurement holds for the allocation's lifetime. Overwrites the first
 * 16 KiB of every region's part of the workspace (at least 48 KiB are needed: LLMI_ERR_WORKSPACE), enqueues a small
 * kernel per region on `stream` and synchronises it: not under stream capture (LLMI_ERR_INVALID_ARG), and not while a
 * call that uses the workspace is in flight. Allocates nothing. */
int llmi_hip_mha_workspace_side(void* workspace, size_t workspace_bytes, void* stream, int32_t* sides);

typedef struct llmi_qk_norm_rope_args {
    void* query;              /* device bf16 [head_num*128]: receives the normalised+rotated query */
    const void* query_src;    /* device bf16 [head_num*128] raw query, or NULL = transform `query` in place */
    const void* key_new;      /* device bf16 [kv_dim]: this token's K row (pre-norm)      */
    const void* value_new;    /* device bf16 [kv_dim]: this token's V row, or NULL if the
                                 V row is already in the cache                            */
    void* key_cache;          /* device bf16 cache base; row (layer_id,pos) is written    */
    void* value_cache;        /* device bf16 cache base; written when value_new != NULL   */
    const void* norm_weight;  /* device bf16 [2*128]: q_norm then k_norm                  */
    const float* sin_cache;   /* device fp32 [max_seq_len][64]                            */
    const float* cos_cache;   /* device fp32 [max_seq_len][64]                            */
    int32_t layer_id;
    int32_t pos;
    int32_t kv_dim;
    int32_t head_num;
    int32_t head_dim;         /* must be 128 */
    int32_t max_seq_len;
    int32_t kv_layout;
    float eps;                /* 1e-6 in the reference (rmsnorm_kernel.cu:284)            */
    void* stream;
} llmi_qk_norm_rope_args;

/* Per-head RMSNorm * weight then half-rotation RoPE on the query (in place)
 * and on this token's K row, which is written to its cache slot for
 * (layer_id, pos) in the given layout, together with the V row. When key_new
 * points at the cache slot itself the K row is transformed in place, which is
 * what the reference does. One kernel, no allocation. */
int llmi_hip_qk_norm_rope_append(const llmi_qk_norm_rope_args* args);

/* sin/cos(pos * 1e6^(-2i/head_dim)) for pos < max_seq_len, i < head_dim/2. */
int llmi_hip_sincos_table(float* sin_cache, float* cos_cache, int32_t head_dim,
                          int32_t max_seq_len, void* stream);

/* Copies rows 0..num_pos-1 of every layer from a position-major cache into a
 * head-major one (src and dst must not overlap). */
int llmi_hip_kv_restride(const void* src_pos_major, void* dst_head_major, int32_t layer_num,
                         int32_t max_seq_len, int32_t kv_dim, int32_t head_dim, int32_t num_pos,
                         void* stream);

/* ---- pooled device allocator ------------------------------------------- */

typedef struct llmi_pool llmi_pool;
/* Backing allocator: returns 0 and sets *ptr on success. */
typedef int (*llmi_backing_alloc_fn)(void** ptr, size_t bytes, void* user);
typedef int (*llmi_backing_free_fn)(void* ptr, void* user);

typedef struct llmi_pool_stats {
    size_t backing_allocs;    /* calls that reached the backing allocator          */
    size_t reuses;            /* allocations served from a free block              */
    size_t big_busy_blocks, big_free_blocks;
    size_t small_busy_blocks, small_free_blocks;
    size_t big_busy_bytes, big_free_bytes;
    size_t small_busy_bytes, small_free_bytes;
} llmi_pool_stats;

/* A pool with the reference's policy (alloc_cu.cpp:7-119): requests above
 * 1 MiB reuse the smallest free big block that fits with less than 1 MiB of
 * slack; requests of 1 MiB or less reuse the smallest free small block that
 * fits; released blocks go back to the free sets and are never returned to
 * the backing allocator until llmi_pool_trim / llmi_pool_destroy. */
llmi_pool* llmi_pool_create(llmi_backing_alloc_fn alloc_fn, llmi_backing_free_fn free_fn,
                            void* user);
void llmi_pool_destroy(llmi_pool* pool);
/* NULL for bytes == 0 or when the backing allocator fails. */
void* llmi_pool_alloc(llmi_pool* pool, size_t bytes);
/* LLMI_OK (also for NULL), LLMI_ERR_UNKNOWN_POINTER for a pointer that is not busy in the pool. */
int llmi_pool_free(llmi_pool* pool, void* ptr);
/* Hands every free block back to the backing allocator; returns bytes released. */
size_t llmi_pool_trim(llmi_pool* pool);
int llmi_pool_get_stats(const llmi_pool* pool, llmi_pool_stats* stats);

/* The process-wide pool over hipMalloc/hipFree on the current device. */
llmi_pool* llmi_hip_default_pool(void);
void* llmi_hip_pool_alloc(size_t bytes);
int llmi_hip_pool_free(void* ptr);

/* kind: 0 host->host, 1 host->device, 2 device->host, 3 device->device
 * (base::MemcpyKind, code/include/base/alloc.h:10-15). A NULL stream copies
 * synchronously; need_sync adds a device synchronise. */
int llmi_hip_memcpy(void* dst, const void* src, size_t bytes, int32_t kind, void* stream,
                    int32_t need_sync);
int llmi_hip_memset_zero(void* ptr, size_t bytes, void* stream, int32_t need_sync);

/* ---- the GEMVs either side of the attention -------------------------------- */
/* Weights are bf16 [n][k] row-major, the input is bf16 [k], accumulation is fp32.
 * k % 8 == 0; input, weight and outputs 16-byte aligned (matmul_kernel.cu:123-128). */
enum {
    LLMI_GEMV_OUT_BF16 = 0, /* output bf16 [n]                       gemv_kernel_cu, lm_head = false  */
    LLMI_GEMV_OUT_F32 = 1,  /* output fp32 [n]                       gemv_kernel_cu, lm_head = true   */
    LLMI_GEMV_ADD_BF16 = 2  /* output bf16 [n] += W x, rounded once  fused_gemv_add_kernel_cu         */
};

typedef struct llmi_gemv_args {
    const void* input;   /* device bf16 [k]                                        */
    const void* weight;  /* device bf16 [n][k]                                     */
    void* output;        /* device [n], see the mode                               */
    int32_t n;
    int32_t k;
    int32_t mode;        /* LLMI_GEMV_*                                            */
    void* stream;        /* hipStream_t                                            */
} llmi_gemv_args;

/* Replaces gemv_kernel_cu (code/source/op/kernel/cuda/matmul_kernel.cu:100-141) and
 * fused_gemv_add_kernel_cu (:174-208): one launch, allocates nothing, capturable. */
int llmi_hip_gemv(const llmi_gemv_args* args);

typedef struct llmi_qkv_gemv_args {
    const void* input;   /* device bf16 [k]: the normalised hidden state            */
    const void* weight;  /* device bf16 [dim + 2*kv_dim][k]: wq, wk, wv stacked      */
    void* query;         /* device bf16 [dim]                                        */
    void* key;           /* device bf16 [kv_dim]                                     */
    void* value;         /* device bf16 [kv_dim]                                     */
    int32_t dim;
    int32_t kv_dim;
    int32_t k;
    void* stream;
} llmi_qkv_gemv_args;

/* Replaces fused_qkv_gemv_kernel_cu (matmul_kernel.cu:248-298). The reference points `key` and `value` at
 * the cache row of the position (model.cpp:90-107); here they are the raw rows that
 * llmi_hip_mha_decode_append (or llmi_hip_qk_norm_rope_append) normalises, rotates and files in the cache
 * of either layout, so the GEMV needs no knowledge of the cache. */
int llmi_hip_qkv_gemv(const llmi_qkv_gemv_args* args);

/* ---- misc ---------------------------------------------------------------- */
int llmi_hip_abi_version(void);
/* No counterpart in the reference (its combine is a second launch and waits for nothing). In the fused
 * split path the workgroup that merges a KV head's partial results polls device memory until every other
 * split of the head has published its record. That wait is bounded: after `polls` unsuccessful polls
 * (default 4194304, seconds of wall time, which only a fault elsewhere on the GPU can reach) it stops and
 * writes NaN to the outputs of its heads instead of hanging the device. Applies to launches enqueued
 * after the call; returns the previous limit. 0 makes every fused launch give up at once: the way to
 * exercise the failure path in a test. */
int32_t llmi_hip_set_poll_limit(int32_t polls);
/* No counterpart in the reference. How many of those bounded waits have given up on the current device since
 * the library was loaded (one count per query head and call; the NaN outputs are the other sign). Reads a
 * device counter with a synchronous copy: it waits for work already enqueued on the device and must not be
 * called while a stream is being captured. After a give-up the records that arrived late stay in the
 * workspace: clear the workspace (llmi_hip_memset_zero) before it is used again by a replay of an
 * already-captured graph, whose launches carry the same tag; fresh calls get a fresh tag and need nothing. */
int llmi_hip_poll_timeouts(uint64_t* count);
const char* llmi_hip_strerror(int status);
/* The last HIP error string seen by this library on the calling thread ("" if none). */
const char* llmi_hip_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* LLMI_HIP_H */
