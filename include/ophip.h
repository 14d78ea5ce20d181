/*
 * ophip — C ABI of the MI355X (gfx950) backend for the operators-rs operator API.
 *
 * Every entry point is the image of one item of the reference crate's Rust
 * surface (paths relative to the reference root, operators/src/...):
 *
 *   Hardware / Gpu handle ........ lib.rs:55-60, handle/cuda/mod.rs:33-72
 *   QueueAlloc ................... lib.rs:89-102, handle/cuda/alloc.rs:10-123
 *   Operator::new/scheme/launch .. lib.rs:105-144
 *   TensorLayout ................. common/tensor.rs:17-98
 *   MaybeDyn sentinels ........... common/maybe_dyn.rs:6-37
 *   SchemeError / LaunchError .... common/error.rs:1-39
 *
 * Conventions shared by all calls:
 *   - Base pointers inside *_args are DEVICE addresses; layouts are host data
 *     borrowed for the duration of the call only.  Strides are in BYTES.
 *   - A dimension, stride or f32 scalar equal to OPHIP_DYN_USIZE /
 *     OPHIP_DYN_ISIZE / +infinity means "not known yet"; scheme() tolerates
 *     them, launch() answers OPHIP_DYNAMIC_NOT_SUPPORT.
 *   - launch() only enqueues work on the queue's stream and returns; nothing
 *     synchronises.  A caller-provided workspace must outlive the enqueued work.
 *     The kernels address a workspace 16 bytes at a time: a workspace that does
 *     not start on a 16-byte boundary is used from the next boundary on, and
 *     counts as too small when what is left there is less than scheme() asked for.
 *   - Return value: OPHIP_OK, one of the nine scheme error kinds (1..9, the
 *     declaration order of SchemeErrorKind), or OPHIP_EXECUTION_FAILED.  The
 *     text of the last error raised on the calling thread is available from
 *     ophip_last_error().  Nothing aborts or throws across this boundary.
 *   - scheme() requires exclusive access to the operator (Rust &mut self);
 *     launch() may be called concurrently from several threads (&self).
 */
#ifndef OPHIP_H
#define OPHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OPHIP_API __attribute__((visibility("default")))

/* ---- status codes: common/error.rs:1-30 ---------------------------------- */
typedef enum ophip_status {
    OPHIP_OK = 0,
    OPHIP_TYPE_NOT_SUPPORT = 1,
    OPHIP_TYPE_MISMATCH = 2,
    OPHIP_RANK_NOT_SUPPORT = 3,
    OPHIP_RANK_MISMATCH = 4,
    OPHIP_SHAPE_NOT_SUPPORT = 5,
    OPHIP_SHAPE_MISMATCH = 6,
    OPHIP_STRIDES_NOT_SUPPORT = 7,
    OPHIP_ARGS_NOT_SUPPORT = 8,
    OPHIP_DYNAMIC_NOT_SUPPORT = 9,
    OPHIP_EXECUTION_FAILED = 100 /* LaunchErrorKind::ExecutionFailed */
} ophip_status;

/* Text of the last error produced on the calling thread ("" if none). */
OPHIP_API const char *ophip_last_error(void);
/* Name of a status code, e.g. "StridesNotSupport". */
OPHIP_API const char *ophip_status_name(int status);

/* ---- data types: the DigitLayout constants the hot path uses ------------- */
/* (handle/cuda/mod.rs:188-210, random_sample/kv_pair.rs:17)                  */
typedef enum ophip_dtype {
    OPHIP_DT_F16 = 1,
    OPHIP_DT_BF16 = 2,
    OPHIP_DT_F32 = 3,
    OPHIP_DT_F64 = 4,
    OPHIP_DT_U8 = 5,
    OPHIP_DT_U16 = 6,
    OPHIP_DT_U32 = 7,
    OPHIP_DT_U64 = 8,
    OPHIP_DT_I8 = 9,
    OPHIP_DT_I16 = 10,
    OPHIP_DT_I32 = 11,
    OPHIP_DT_I64 = 12,
    OPHIP_DT_BOOL = 13,
    OPHIP_DT_KVPAIR = 14 /* KVPair::LAYOUT = u(32) x 2, 8 bytes */
} ophip_dtype;

/* DigitLayout::nbytes; 0 for an unknown code. */
OPHIP_API size_t ophip_dtype_nbytes(uint64_t dt);

/* ---- MaybeDyn sentinels: common/maybe_dyn.rs:6-37 ------------------------ */
#define OPHIP_DYN_USIZE SIZE_MAX
#define OPHIP_DYN_ISIZE PTRDIFF_MAX
/* the f32 sentinel is +infinity */

/* ---- TensorLayout: common/tensor.rs:10-98 -------------------------------- */
typedef struct ophip_tensor_layout {
    uint64_t dt;              /* ophip_dtype */
    uint64_t ndim;
    const size_t *shape;      /* ndim entries, OPHIP_DYN_USIZE = dynamic */
    const ptrdiff_t *strides; /* ndim entries, bytes, OPHIP_DYN_ISIZE = dynamic */
} ophip_tensor_layout;

/* ---- Hardware handle: handle/cuda/mod.rs:33-72 (Gpu, Config) ------------- */
typedef struct ophip_device ophip_device; /* reference-counted, thread-safe */

typedef struct ophip_config { /* handle/cuda/mod.rs:40-55 */
    size_t low_diversity_cache;
    size_t medium_diversity_cache;
    size_t high_diversity_cache;
} ophip_config;

/* Gpu::new(Device::new(ordinal).context(), config); cfg == NULL => 4/16/64. */
OPHIP_API int ophip_device_create(int ordinal, const ophip_config *cfg, ophip_device **out);
OPHIP_API void ophip_device_retain(ophip_device *dev);
OPHIP_API void ophip_device_release(ophip_device *dev);
/* Number of HIP devices visible; 0 plays the role of Gpu::init() == None
 * (handle/cuda/mod.rs:74-80). */
OPHIP_API int ophip_device_count(void);

typedef struct ophip_device_info {
    char name[64];
    char arch[32];
    int compute_units;
    int wavefront_size;
    int max_threads_per_block;
    size_t lds_per_block;
    size_t total_memory;
    int clock_khz;
} ophip_device_info;
OPHIP_API int ophip_device_get_info(const ophip_device *dev, ophip_device_info *out);

/* ---- what the `cuda` driver crate gives callers: memory, streams, events - */
typedef void *ophip_stream; /* hipStream_t */
typedef void *ophip_event;  /* hipEvent_t  */

OPHIP_API int ophip_malloc(ophip_device *dev, size_t size, void **out);
OPHIP_API int ophip_free(ophip_device *dev, void *ptr);
/* Copies and fills: queued on `stream` when one is given; with a null stream the call returns
 * when the data is in place, so work queued afterwards on any stream sees it.  A fill on a stream
 * is a kernel launch (any address and size), so it can be recorded into a graph like the operators. */
OPHIP_API int ophip_memcpy_h2d(ophip_device *dev, void *dst, const void *src, size_t size,
                               ophip_stream stream);
OPHIP_API int ophip_memcpy_d2h(ophip_device *dev, void *dst, const void *src, size_t size,
                               ophip_stream stream);
OPHIP_API int ophip_memcpy_d2d(ophip_device *dev, void *dst, const void *src, size_t size,
                               ophip_stream stream);
OPHIP_API int ophip_memset(ophip_device *dev, void *dst, int value, size_t size,
                           ophip_stream stream);
OPHIP_API int ophip_stream_create(ophip_device *dev, ophip_stream *out);
OPHIP_API int ophip_stream_destroy(ophip_device *dev, ophip_stream stream);
OPHIP_API int ophip_stream_synchronize(ophip_device *dev, ophip_stream stream);
OPHIP_API int ophip_event_create(ophip_device *dev, ophip_event *out);
OPHIP_API int ophip_event_destroy(ophip_device *dev, ophip_event ev);
OPHIP_API int ophip_event_record(ophip_device *dev, ophip_event ev, ophip_stream stream);
OPHIP_API int ophip_event_synchronize(ophip_device *dev, ophip_event ev);
OPHIP_API int ophip_event_elapsed_ms(ophip_device *dev, ophip_event start, ophip_event stop,
                                     float *ms);
/* Measurement aid, no counterpart in the reference: the next kernel this thread launches on `stream` (through any
 * operator of this library) records its own begin into `start` and its own end into `stop`, so that
 * ophip_event_elapsed_ms(start, stop) is the kernel's duration on the device, without the cost of two separate event
 * records around it.  An operator that launches several kernels times its first. */
OPHIP_API int ophip_time_next_launch(ophip_device *dev, ophip_stream stream, ophip_event start, ophip_event stop);


/* Launch graphs (no counterpart in the reference's driver crate): a fixed sequence of launch()
 * calls on `stream` between begin and end is recorded instead of run, and replayed by
 * ophip_graph_launch without per-launch host cost.  Give every recorded launch a workspace of
 * its own (scheme() reports the size).  A mat_mul operator used on more than one stream has to be
 * launched once on each further stream before that stream records: its first split-K launch on a
 * stream other than the first allocates, which HIP refuses while a stream records.
 * A recorded split-K mat_mul carries the address of the arrival counters the operator keeps for the
 * stream it was recorded on.  Hence: replay a graph on the stream it was recorded on (on another stream,
 * while that one also runs split-K products of the same operator, two kernels would share one set of
 * counters and sum wrongly), and destroy a graph before the operators recorded into it (the operator
 * frees its counters) and before the stream it was recorded on (the counters a graph names go to the
 * next new stream once theirs is destroyed).  An operator keeps one 256 KiB counter buffer per stream
 * it is launched on; a stream ended with ophip_stream_destroy (which waits for the stream's work first,
 * unless the stream is still recording: then nothing is handed on) hands its buffer to the next new
 * stream, the rest is freed with the operator. */
typedef void *ophip_graph; /* hipGraphExec_t */
OPHIP_API int ophip_stream_begin_capture(ophip_device *dev, ophip_stream stream);
OPHIP_API int ophip_stream_end_capture(ophip_device *dev, ophip_stream stream, ophip_graph *out);
OPHIP_API int ophip_graph_launch(ophip_device *dev, ophip_graph graph, ophip_stream stream);
OPHIP_API int ophip_graph_destroy(ophip_device *dev, ophip_graph graph);

/* ---- QueueAlloc: lib.rs:89-102 -------------------------------------------
 * A queue (stream) plus an allocator bound to it.  `alloc`/`free` are called by
 * launch() only when the caller's workspace is too small (common/workspace.rs:
 * 14-21,45-51); `free` is called right after the work is enqueued and must be
 * stream-ordered or deferred. */
typedef struct ophip_queue_alloc {
    void *ctx;
    ophip_stream stream;
    void *(*alloc)(void *ctx, size_t size);
    void (*free)(void *ctx, void *ptr);
} ophip_queue_alloc;

/* `impl QueueAlloc for Stream` (handle/cuda/alloc.rs:103-123): stream-ordered
 * hipMallocAsync / hipFreeAsync on `stream`. */
OPHIP_API int ophip_queue_alloc_from_stream(ophip_device *dev, ophip_stream stream,
                                            ophip_queue_alloc *out);

/* StreamMemPool (handle/cuda/alloc.rs:10-90): slabs handed in with put(), carved
 * by an OffsetCalculator (common/calculator.rs:8-86: alignment-rounded best fit,
 * coalescing free list, zero-size requests get a sentinel). */
typedef struct ophip_mem_pool ophip_mem_pool;
OPHIP_API int ophip_mem_pool_create(ophip_device *dev, ophip_stream stream, ophip_mem_pool **out);
OPHIP_API int ophip_mem_pool_put(ophip_mem_pool *pool, size_t size);
OPHIP_API int ophip_mem_pool_queue_alloc(ophip_mem_pool *pool, ophip_queue_alloc *out);
OPHIP_API void ophip_mem_pool_destroy(ophip_mem_pool *pool);

/* OffsetCalculator on its own (host-only; used by the pool and unit-testable). */
typedef struct ophip_offset_calculator ophip_offset_calculator;
OPHIP_API ophip_offset_calculator *ophip_offset_calculator_create(size_t alignment);
OPHIP_API void ophip_offset_calculator_destroy(ophip_offset_calculator *c);
OPHIP_API void ophip_offset_calculator_put(ophip_offset_calculator *c, size_t start, size_t end);
/* 1 and [*start, *end) on success (zero size => SIZE_MAX..SIZE_MAX), 0 when nothing fits. */
OPHIP_API int ophip_offset_calculator_take(ophip_offset_calculator *c, size_t size, size_t *start,
                                           size_t *end);

/* ======================== operators ========================================
 * Each operator has the same four verbs:
 *   create  = Operator::new(&node)               lib.rs:113
 *   scheme  = Operator::scheme(&mut self, ..)    lib.rs:115-131  (*workspace_size <= max_workspace_size)
 *   launch  = Operator::launch(&self, ..)        lib.rs:133-143
 *   destroy = Drop
 */

/* ---- rms_norm: rms_norm/args.rs:7-15 ------------------------------------- */
typedef struct ophip_rms_norm_args {
    ophip_tensor_layout y_layout;
    void *y_base;
    ophip_tensor_layout x_layout;
    const void *x_base;
    ophip_tensor_layout w_layout;
    const void *w_base;
    float epsilon;
} ophip_rms_norm_args;
typedef struct ophip_rms_norm ophip_rms_norm;
OPHIP_API int ophip_rms_norm_create(ophip_device *dev, ophip_rms_norm **out);
OPHIP_API int ophip_rms_norm_scheme(ophip_rms_norm *op, const ophip_rms_norm_args *args,
                                    size_t max_workspace_size, size_t *workspace_size);
OPHIP_API int ophip_rms_norm_launch(const ophip_rms_norm *op, const ophip_rms_norm_args *args,
                                    void *workspace, size_t workspace_len,
                                    const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_rms_norm_destroy(ophip_rms_norm *op);

/* ---- rope: rope/args.rs:8-18, rope/mod.rs:13-58 -------------------------- */
typedef struct ophip_rope_args {
    ophip_tensor_layout t_layout;
    void *t_base;
    ophip_tensor_layout p_layout;
    const void *p_base;
    ophip_tensor_layout sin_layout; /* validated (rank 2, last dim == dh) but unused, */
    const void *sin_base;           /* exactly as the CPU and CUDA backends do        */
    ophip_tensor_layout cos_layout;
    const void *cos_base;
    float theta;
} ophip_rope_args;
typedef struct ophip_rope_seq { /* rope/mod.rs:23-26 */
    size_t pos;
    size_t len;
} ophip_rope_seq;
typedef struct ophip_rope ophip_rope;
OPHIP_API int ophip_rope_create(ophip_device *dev, ophip_rope **out);
OPHIP_API int ophip_rope_scheme(ophip_rope *op, const ophip_rope_args *args,
                                size_t max_workspace_size, size_t *workspace_size);
OPHIP_API int ophip_rope_launch(const ophip_rope *op, const ophip_rope_args *args, void *workspace,
                                size_t workspace_len, const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_rope_destroy(ophip_rope *op);
/* Rope::build_pos (rope/cuda/mod.rs:36-56): expands the sequences into nt
 * positions of type dt (U32 or U64), allocates nt*nbytes from the queue
 * allocator and uploads them on its stream.  *out is owned by the caller
 * (return it with queue_alloc->free). */
OPHIP_API int ophip_rope_build_pos(uint64_t dt, size_t nt, const ophip_rope_seq *seqs, size_t nseq,
                                   const ophip_queue_alloc *queue_alloc, void **out);
/* Rope::build_sincos (rope/cuda/mod.rs:21-34): this backend computes sin/cos
 * in-kernel, so the table is empty: *nctx = 0 and *out = alloc(0). */
OPHIP_API int ophip_rope_build_sincos(uint64_t dt, size_t nctx, size_t dh,
                                      const ophip_queue_alloc *queue_alloc, size_t *nctx_out,
                                      void **out);

/* ---- fuesd_softmax: fuesd_softmax/args.rs:5-16 --------------------------- */
typedef enum ophip_attn_mask { OPHIP_MASK_NONE = 0, OPHIP_MASK_CAUSAL = 1 } ophip_attn_mask;
typedef struct ophip_fused_softmax_args {
    uint8_t att_mask; /* ophip_attn_mask, #[repr(u8)] */
    ophip_tensor_layout att_layout;
    void *att_base;
} ophip_fused_softmax_args;
typedef struct ophip_fused_softmax ophip_fused_softmax;
OPHIP_API int ophip_fused_softmax_create(ophip_device *dev, ophip_fused_softmax **out);
OPHIP_API int ophip_fused_softmax_scheme(ophip_fused_softmax *op,
                                         const ophip_fused_softmax_args *args,
                                         size_t max_workspace_size, size_t *workspace_size);
OPHIP_API int ophip_fused_softmax_launch(const ophip_fused_softmax *op,
                                         const ophip_fused_softmax_args *args, void *workspace,
                                         size_t workspace_len,
                                         const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_fused_softmax_destroy(ophip_fused_softmax *op);

/* ---- rearrange: rearrange/args.rs:12-17 ---------------------------------- */
typedef struct ophip_rearrange_args {
    ophip_tensor_layout dst_layout;
    void *dst_base;
    ophip_tensor_layout src_layout;
    const void *src_base;
} ophip_rearrange_args;
typedef struct ophip_rearrange ophip_rearrange;
OPHIP_API int ophip_rearrange_create(ophip_device *dev, ophip_rearrange **out);
OPHIP_API int ophip_rearrange_scheme(ophip_rearrange *op, const ophip_rearrange_args *args,
                                     size_t max_workspace_size, size_t *workspace_size);
OPHIP_API int ophip_rearrange_launch(const ophip_rearrange *op, const ophip_rearrange_args *args,
                                     void *workspace, size_t workspace_len,
                                     const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_rearrange_destroy(ophip_rearrange *op);
/* The layout normaliser Scheme::new (rearrange/args.rs:35-153), host-only.
 * out receives [unit, idx_strides (ndim+1 values: count ... 1), dst_strides
 * (ndim), src_strides (ndim)] and must hold 2 + 3*args->dst_layout.ndim values;
 * *ndim_out is the merged rank. */
OPHIP_API int ophip_rearrange_plan(const ophip_rearrange_args *args, ptrdiff_t *out,
                                   size_t *ndim_out);

/* ---- swiglu: swiglu/args.rs:7-12 ----------------------------------------- */
typedef struct ophip_swiglu_args {
    ophip_tensor_layout gate_layout;
    void *gate_base;
    ophip_tensor_layout up_layout;
    const void *up_base;
} ophip_swiglu_args;
typedef struct ophip_swiglu ophip_swiglu;
OPHIP_API int ophip_swiglu_create(ophip_device *dev, ophip_swiglu **out);
OPHIP_API int ophip_swiglu_scheme(ophip_swiglu *op, const ophip_swiglu_args *args,
                                  size_t max_workspace_size, size_t *workspace_size);
OPHIP_API int ophip_swiglu_launch(const ophip_swiglu *op, const ophip_swiglu_args *args,
                                  void *workspace, size_t workspace_len,
                                  const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_swiglu_destroy(ophip_swiglu *op);

/* ---- random_sample: random_sample/args.rs:9-25, kv_pair.rs:8-32 ----------- */
typedef struct ophip_kv_pair { /* #[repr(C)] KVPair */
    uint32_t idx;
    uint32_t val; /* the value's bytes in the low bytes */
} ophip_kv_pair;
typedef struct ophip_sample_args { /* SampleArgs */
    float temperature;
    float top_p;
    size_t top_k; /* SIZE_MAX = no top-k */
} ophip_sample_args;
typedef struct ophip_random_sample_args {
    ophip_tensor_layout kv_pair; /* rank 0, dt = OPHIP_DT_KVPAIR */
    void *kv_pair_base;
    ophip_tensor_layout logits; /* [n], unit stride, f16 or f32 */
    const void *logits_base;
    ophip_tensor_layout indices; /* [n] u32; validated, not read by this backend */
    const void *indices_base;
    ophip_sample_args config;
    float seed; /* the uniform draw in [0, 1] */
} ophip_random_sample_args;
/* SampleArgs::new (args.rs:66-78): 0 ok, 1 NegativeTemperature, 2 NonPositiveTop. */
OPHIP_API int ophip_sample_args_new(float temperature, float top_p, size_t top_k,
                                    ophip_sample_args *out);
/* SampleArgs::ARG_MAX (args.rs:60-64). */
OPHIP_API ophip_sample_args ophip_sample_args_argmax(void);
typedef struct ophip_random_sample ophip_random_sample;
OPHIP_API int ophip_random_sample_create(ophip_device *dev, ophip_random_sample **out);
OPHIP_API int ophip_random_sample_scheme(ophip_random_sample *op,
                                         const ophip_random_sample_args *args,
                                         size_t max_workspace_size, size_t *workspace_size);
OPHIP_API int ophip_random_sample_launch(const ophip_random_sample *op,
                                         const ophip_random_sample_args *args, void *workspace,
                                         size_t workspace_len,
                                         const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_random_sample_destroy(ophip_random_sample *op);
/* Batched launch: no counterpart in the reference, whose operator samples one
 * row per launch (random_sample/args.rs:9-18).  `rows` independent logit rows,
 * row r starting `row_stride` bytes after row r-1, are sampled by one launch
 * with the shared config; results go to `rows` consecutive ophip_kv_pair at
 * kv_pair_base.  `seeds` is either NULL (args->seed is used for every row) or a
 * DEVICE array of `rows` draws.  Each row's result is what ophip_random_sample_launch
 * returns for that row.  The workspace need is rows times the single-row need. */
OPHIP_API int ophip_random_sample_launch_batch(const ophip_random_sample *op,
                                               const ophip_random_sample_args *args, size_t rows,
                                               ptrdiff_t row_stride, const float *seeds,
                                               void *workspace, size_t workspace_len,
                                               const ophip_queue_alloc *queue_alloc);
/* RandomSample::build_indices (random_sample/cuda/mod.rs:29-38): uploads 0..n as
 * u32.  *out is owned by the caller. */
OPHIP_API int ophip_random_sample_build_indices(size_t n, const ophip_queue_alloc *queue_alloc,
                                                void **out);

/* ---- mat_mul: mat_mul/args.rs:11-20 --------------------------------------- */
typedef struct ophip_mat_mul_args {
    ophip_tensor_layout c_layout;
    void *c_base;
    float beta;
    ophip_tensor_layout a_layout;
    const void *a_base;
    ophip_tensor_layout b_layout;
    const void *b_base;
    float alpha;
} ophip_mat_mul_args;
/* SchemeLayout (mat_mul/args.rs:22-42); strides and leading dimensions in elements. */
typedef struct ophip_mat_mul_layout {
    uint64_t dt;
    int32_t ab_swap, a_trans, b_trans, _pad;
    size_t batch, m, n, k;
    ptrdiff_t c_stride, c_ld, a_stride, a_ld, b_stride, b_ld;
} ophip_mat_mul_layout;
/* Args::layout (mat_mul/args.rs:64-121), host-only. */
OPHIP_API int ophip_mat_mul_plan(const ophip_mat_mul_args *args, ophip_mat_mul_layout *out);
typedef struct ophip_mat_mul ophip_mat_mul;
OPHIP_API int ophip_mat_mul_create(ophip_device *dev, ophip_mat_mul **out);
OPHIP_API int ophip_mat_mul_scheme(ophip_mat_mul *op, const ophip_mat_mul_args *args,
                                   size_t max_workspace_size, size_t *workspace_size);
OPHIP_API int ophip_mat_mul_launch(const ophip_mat_mul *op, const ophip_mat_mul_args *args,
                                   void *workspace, size_t workspace_len,
                                   const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_mat_mul_destroy(ophip_mat_mul *op);
/* No counterpart in the reference.  For callers that cannot allocate device memory (a stream that is
 * being recorded into a graph, a tight serving loop, a harness that forbids hipMalloc): the same product as
 * ophip_mat_mul_launch, queued on `stream`, with no workspace argument and no queue allocator.  The split-K
 * scratch (f32 partials and arrival counters) is a device array inside this library, 32 MiB + 256 KiB, held by
 * every GPU the library runs on until the process ends; nothing is allocated or freed by the call.  A product
 * whose partials need more than 32 MiB (ophip_mat_mul_scheme reports the need) is refused with
 * OPHIP_ARGS_NOT_SUPPORT.  All calls on one GPU share the array: two of them that overlap in time (on
 * different streams, or from two threads) race; calls on one stream are ordered and safe. */
OPHIP_API int ophip_mat_mul_launch_static(const ophip_mat_mul *op, const ophip_mat_mul_args *args,
                                          ophip_stream stream);
/* Diagnostics, no counterpart in the reference: writes the name of the kernel family launch()
 * would pick for these arguments on this device ("stream rows<=16 qN split_k=1 (2 on granule classes 0x22)",
 * "stream rows<=16 qN split_k=8", "skinny rows<=32 qN paired split_k=1",
 * "skinny rows<=32 qK256 split_k=2", "tile256x64 pK qN split_k=1",
 * "tile128x64 ragged pK qK split_k=1" when M or N is not in whole tiles, "tile128x32 ...", "generic") into out[0..len).
 * `op` may be null: the choice for a device of 256 compute units (needs no device; the CPU tests of the planner use it). */
OPHIP_API int ophip_mat_mul_describe(const ophip_mat_mul *op, const ophip_mat_mul_args *args, char *out, size_t len);

/* ---- attention: attention/args.rs:10-24, attention/operator.rs:31-277 ------ */
/* The composite the crate builds from mat_mul, fuesd_softmax and rearrange
 * (attention/mod.rs:8-17): att = softmax(q . k^T / sqrt(dh)) per kv-head group,
 * o = att . v.  q [nh, seq, dh], k and v [nkvh, att, dh], o [nh, seq, dh];
 * nh must be a multiple of nkvh.  As in the reference, q is overwritten (it
 * receives att . v before the copy into o) unless its layout forces a staging
 * copy, and launch() needs nh*seq*(dh + att) elements of workspace, taken from
 * the queue allocator when the caller's slice is smaller.
 * f16 / bf16 shapes that one kernel serves (prefill: many query rows per head;
 * decode: up to 64 rows per kv head with k and v of one layout) run on it instead
 * of the composite's launches: the same o within the f16 bar, q overwritten or
 * left alone exactly as the composite would, k and v untouched. */
typedef struct ophip_attention_args {
    ophip_tensor_layout q_layout;
    void *q_base;
    ophip_tensor_layout k_layout;
    const void *k_base;
    ophip_tensor_layout v_layout;
    const void *v_base;
    ophip_tensor_layout o_layout;
    void *o_base;
    uint8_t mask; /* ophip_attn_mask */
} ophip_attention_args;
typedef struct ophip_attention ophip_attention;
OPHIP_API int ophip_attention_create(ophip_device *dev, ophip_attention **out);
OPHIP_API int ophip_attention_scheme(ophip_attention *op, const ophip_attention_args *args,
                                     size_t max_workspace_size, size_t *workspace_size);
OPHIP_API int ophip_attention_launch(const ophip_attention *op, const ophip_attention_args *args,
                                     void *workspace, size_t workspace_len,
                                     const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_attention_destroy(ophip_attention *op);

/* ---- attention_kv_cached: attention_kv_cached/args.rs:8-30, operator.rs:29-183 */
/* Appends k, v [nkvh, seq, dh] to the caches [nkvh, buf, dh] at row `pos`
 * (two rearranges), then runs attention over cache rows [0, pos + seq).
 * pos + seq beyond either cache's buf is ShapeMismatch ("Out of cache
 * buffer").  As in the reference, the v-cache is addressed with the k-cache's
 * strides (operator.rs:114,156): give both caches the same layout. */
typedef struct ophip_attention_kv_cached_args {
    ophip_tensor_layout q_layout;
    void *q_base;
    ophip_tensor_layout k_layout;
    const void *k_base;
    ophip_tensor_layout v_layout;
    const void *v_base;
    ophip_tensor_layout o_layout;
    void *o_base;
    ophip_tensor_layout k_cache_layout;
    void *k_cache_base;
    ophip_tensor_layout v_cache_layout;
    void *v_cache_base;
    uint8_t mask; /* ophip_attn_mask */
    size_t pos;   /* OPHIP_DYN_USIZE = dynamic (scheme only) */
} ophip_attention_kv_cached_args;
typedef struct ophip_attention_kv_cached ophip_attention_kv_cached;
OPHIP_API int ophip_attention_kv_cached_create(ophip_device *dev, ophip_attention_kv_cached **out);
OPHIP_API int ophip_attention_kv_cached_scheme(ophip_attention_kv_cached *op,
                                               const ophip_attention_kv_cached_args *args,
                                               size_t max_workspace_size, size_t *workspace_size);
OPHIP_API int ophip_attention_kv_cached_launch(const ophip_attention_kv_cached *op,
                                               const ophip_attention_kv_cached_args *args,
                                               void *workspace, size_t workspace_len,
                                               const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_attention_kv_cached_destroy(ophip_attention_kv_cached *op);

/* ---- layer_norm: layer_norm/args.rs:7-55 ----------------------------------- */
/* y[n,d] = (x - mean) * scale / (std + epsilon) + bias, std = sqrt(mean(x^2) - mean^2)
 * (layer_norm/common_cpu/mod.rs:127-147).  (scale/bias, x/y): any pairing of f16, bf16 and f32, and (f64, f64)
 * (the CPU backend lists (f16,f16), (f32,f16), (f32,f32), (f64,f64); layer_norm/cuda/mod.rs:158-159 takes any pair of
 * named types). */
typedef struct ophip_layer_norm_args {
    ophip_tensor_layout y_layout;
    void *y_base;
    ophip_tensor_layout x_layout;
    const void *x_base;
    ophip_tensor_layout scale_layout;
    const void *scale_base;
    ophip_tensor_layout bias_layout;
    const void *bias_base;
    float epsilon;
} ophip_layer_norm_args;
typedef struct ophip_layer_norm ophip_layer_norm;
OPHIP_API int ophip_layer_norm_create(ophip_device *dev, ophip_layer_norm **out);
OPHIP_API int ophip_layer_norm_scheme(ophip_layer_norm *op, const ophip_layer_norm_args *args,
                                      size_t max_workspace_size, size_t *workspace_size);
OPHIP_API int ophip_layer_norm_launch(const ophip_layer_norm *op, const ophip_layer_norm_args *args,
                                      void *workspace, size_t workspace_len,
                                      const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_layer_norm_destroy(ophip_layer_norm *op);

/* ---- gelu: gelu/args.rs:4-36 (in place, tanh form, gelu/common_cpu/mod.rs:112-116) */
typedef struct ophip_gelu_args {
    ophip_tensor_layout layout; /* [n, d] */
    void *base;
} ophip_gelu_args;
typedef struct ophip_gelu ophip_gelu;
OPHIP_API int ophip_gelu_create(ophip_device *dev, ophip_gelu **out);
OPHIP_API int ophip_gelu_scheme(ophip_gelu *op, const ophip_gelu_args *args, size_t max_workspace_size,
                                size_t *workspace_size);
OPHIP_API int ophip_gelu_launch(const ophip_gelu *op, const ophip_gelu_args *args, void *workspace,
                                size_t workspace_len, const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_gelu_destroy(ophip_gelu *op);

/* ---- add: add/args.rs:12-19; c = a + b, equal shapes, any strides (0 = broadcast in a, b) */
typedef struct ophip_add_args {
    ophip_tensor_layout c_layout;
    void *c_base;
    ophip_tensor_layout a_layout;
    const void *a_base;
    ophip_tensor_layout b_layout;
    const void *b_base;
} ophip_add_args;
typedef struct ophip_add ophip_add;
OPHIP_API int ophip_add_create(ophip_device *dev, ophip_add **out);
OPHIP_API int ophip_add_scheme(ophip_add *op, const ophip_add_args *args, size_t max_workspace_size,
                               size_t *workspace_size);
OPHIP_API int ophip_add_launch(const ophip_add *op, const ophip_add_args *args, void *workspace,
                               size_t workspace_len, const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_add_destroy(ophip_add *op);
/* The layout normaliser Scheme::new (add/args.rs:42-167), host-only.  out receives
 * [idx_strides (ndim+1 values: count ... 1), c_strides, a_strides, b_strides (ndim each)]
 * and must hold 1 + 4*args->c_layout.ndim values; *ndim_out is the merged rank. */
OPHIP_API int ophip_add_plan(const ophip_add_args *args, ptrdiff_t *out, size_t *ndim_out);

/* ---- add_rows: add_rows/args.rs:10-17; dst[b, m, :] += src[idx[b, m], :], idx u32 or u64 */
typedef struct ophip_add_rows_args {
    ophip_tensor_layout dst_layout; /* [batch, m, n] */
    void *dst_base;
    ophip_tensor_layout src_layout; /* [k, n] */
    const void *src_base;
    ophip_tensor_layout idx_layout; /* [batch, m] */
    const void *idx_base;
} ophip_add_rows_args;
typedef struct ophip_add_rows ophip_add_rows;
OPHIP_API int ophip_add_rows_create(ophip_device *dev, ophip_add_rows **out);
OPHIP_API int ophip_add_rows_scheme(ophip_add_rows *op, const ophip_add_rows_args *args,
                                    size_t max_workspace_size, size_t *workspace_size);
OPHIP_API int ophip_add_rows_launch(const ophip_add_rows *op, const ophip_add_rows_args *args,
                                    void *workspace, size_t workspace_len,
                                    const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_add_rows_destroy(ophip_add_rows *op);

/* ---- conv: conv/args.rs:7-19, conv/im2col.rs:9-242 ------------------------- */
/* y[n, m, hy, wy] = w[m, c, hk, wk] (*) x[n, c, h, w] + b[m], the crate's im2col composite:
 * bias broadcast (rearrange), x unfolded into workspace (rearrange), one batched mat_mul
 * with beta = 1.  pads must be zero; (h - ((hk-1)*dilation+1)) must divide by the stride. */
typedef struct ophip_conv_args {
    ophip_tensor_layout y_layout;
    void *y_base;
    ophip_tensor_layout x_layout;
    const void *x_base;
    ophip_tensor_layout w_layout;
    const void *w_base;
    ophip_tensor_layout b_layout;
    const void *b_base;
    size_t strides[2];
    size_t dilations[2];
    size_t pads[4];
} ophip_conv_args;
typedef struct ophip_conv ophip_conv;
OPHIP_API int ophip_conv_create(ophip_device *dev, ophip_conv **out);
OPHIP_API int ophip_conv_scheme(ophip_conv *op, const ophip_conv_args *args, size_t max_workspace_size,
                                size_t *workspace_size);
OPHIP_API int ophip_conv_launch(const ophip_conv *op, const ophip_conv_args *args, void *workspace,
                                size_t workspace_len, const ophip_queue_alloc *queue_alloc);
OPHIP_API void ophip_conv_destroy(ophip_conv *op);

#ifdef __cplusplus
}
#endif
#endif /* OPHIP_H */
