/* fxhip.h - C ABI of the MI355X (gfx950) execution layer for FuncTs/FAIT fused
 * functionalized regions.
 *
 * This is the boundary the reference crosses when a tssa::ParallelFunctor
 * operator runs: it replaces the NVRTC code generator and launcher
 *   fait/tensorexpr/cuda_codegen_tssa.h:193-239  (class CudaCodeGenTssa)
 * and the per-operator lowering tables that define the kernel arithmetic
 *   functs/csrc/jit/tensorexpr/nnc_ext.cpp:62-392
 *   fait/fuser/custom_lowering_func.cpp:502-559
 *   fait/fuser/shape_func.cpp:274-374
 * Plain C types only: no torch types, no C++ types.  All device buffers are
 * owned by the caller.  Every function returns 0 on success or a negative
 * FX_E_* code; fx_last_error() gives the message for the calling thread.
 */
#ifndef FXHIP_H_
#define FXHIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FX_API_VERSION 1
#define FX_MAX_RANK 6 /* max rank of a region output */
#define FX_ARG_MAX_RANK 8

/* error codes */
#define FX_OK 0
#define FX_E_INVALID (-1)     /* malformed call or region (reference: malformed_input, cuda_codegen_tssa.cpp:1293-1295) */
#define FX_E_UNSUPPORTED (-2) /* op / dtype / rank outside what the kernels implement (reference aborts: graph_builder.cpp:409-414) */
#define FX_E_HIP (-3)         /* a HIP runtime call failed */
#define FX_E_LIMIT (-4)       /* a fixed capacity was exceeded (tasks x pointers, temps, nesting) */
#define FX_E_NODEVICE (-5)    /* no usable gfx950 device */

/* element types of tensors (storage) and scalars */
#define FX_DT_F32 0
#define FX_DT_I64 1
#define FX_DT_I32 2
#define FX_DT_U8 3
#define FX_DT_F16 4
#define FX_DT_BF16 5
#define FX_DT_BOOL 6 /* stored as one byte */

/* Operators a region can be built from.  Each mirrors one entry of the
 * reference's lowering tables (file:line given per group). */
enum fx_opcode {
  /* immut:: access / assign family: nnc_ext.cpp:62-392, symbol_ext.cpp:9-199 */
  FX_OP_ACCESS = 1,   /* (src) */
  FX_OP_ASSIGN,       /* (self, src) -> src                      nnc_ext.cpp:71-80 */
  FX_OP_CLONE,        /* (src)  clone / contiguous               nnc_ext.cpp:62-69 */
  FX_OP_SELECT,       /* (src, int dim, int index)               nnc_ext.cpp:166-185 */
  FX_OP_SELECT_REV,   /* (self, src, int dim, int index)         nnc_ext.cpp:187-212 */
  FX_OP_SLICE,        /* (src, int dim, int? start, int? end, int step)   custom_lowering_func.cpp:200-227 */
  FX_OP_SLICE_REV,    /* (self, src, int dim, int? start, int? end, int step)  nnc_ext.cpp:112-164 */
  FX_OP_SQUEEZE,      /* (src, int dim) */
  FX_OP_UNSQUEEZE,    /* (src, int dim)                          nnc_ext.cpp:214-229 */
  FX_OP_VIEW,         /* (src, int[] sizes)  view / reshape      nnc_ext.cpp:231-295 */
  FX_OP_PERMUTE,      /* (src, int[] dims)                       nnc_ext.cpp:320-358 */
  FX_OP_TRANSPOSE,    /* (src, int d0, int d1)                   shape_func.cpp:127-138 */
  FX_OP_EXPAND,       /* (src, int[] sizes)                      nnc_ext.cpp:360-370 */
  FX_OP_EXPAND_AS,    /* (src, other) */
  FX_OP_REPEAT,       /* (src, int[] repeats)                    nnc_ext.cpp:297-318 */
  FX_OP_INDEX,        /* (src, Tensor[] {int64 index})  dim 0    nnc_ext.cpp:372-392 */
  FX_OP_CAT,          /* (Tensor[] tensors, int dim)             custom_lowering_func.cpp:297-330 */
  FX_OP_STACK,        /* (Tensor[] tensors, int dim)             custom_lowering_func.cpp:332-350 */
  /* creation: custom_lowering_func.cpp:17-49 */
  FX_OP_FULL,         /* (int[] size | Tensor like, scalar value)  zeros / ones / full(_like); out dtype
                         required with a size list, inherited from `like` when negative */
  FX_OP_ARANGE,       /* (int start, int end)        out dtype required */
  FX_OP_SCALAR_TENSOR,/* (scalar) -> 0-dim tensor    out dtype required */
  FX_OP_TRIU,         /* (self, int diagonal) */
  /* elementwise unary: stock NNC lowerings (graph_builder.cpp:388-407) */
  FX_OP_EXP, FX_OP_LOG, FX_OP_SQRT, FX_OP_RSQRT, FX_OP_SIGMOID, FX_OP_TANH, FX_OP_RELU,
  FX_OP_NEG, FX_OP_ABS, FX_OP_FLOOR, FX_OP_CEIL, FX_OP_ROUND, FX_OP_SIN, FX_OP_COS, FX_OP_ERF,
  FX_OP_RECIPROCAL, FX_OP_LOGICAL_NOT,
  FX_OP_TO,           /* (self) dtype cast; out dtype required */
  /* elementwise binary, tensor (x) tensor|scalar with broadcasting:
   * custom_lowering_func.cpp:51-76, shape_func.cpp:23-49 */
  FX_OP_ADD,          /* (self, other, scalar alpha=1) */
  FX_OP_SUB,          /* (self, other, scalar alpha=1) */
  FX_OP_RSUB,         /* (self, other, scalar alpha=1) -> other - alpha*self */
  FX_OP_MUL, FX_OP_DIV, FX_OP_MAXIMUM, FX_OP_MINIMUM, FX_OP_POW, FX_OP_FMOD,
  FX_OP_EQ, FX_OP_NE, FX_OP_LT, FX_OP_LE, FX_OP_GT, FX_OP_GE,
  FX_OP_AND, FX_OP_OR, FX_OP_XOR,
  FX_OP_CLAMP,        /* (self, scalar? min, scalar? max)       custom_lowering_func.cpp:355-368 */
  FX_OP_WHERE,        /* (cond, self, other) */
  /* reductions over one dimension: custom_lowering_func.cpp:112-180 */
  FX_OP_MAX_DIM,      /* (self, int dim, bool keepdim) -> values */
  FX_OP_SUM_DIM,      /* (self, int dim, bool keepdim) */
  FX_OP_SOFTMAX,      /* (self, int dim) */
  /* integer scalar arithmetic on index values */
  FX_OP_INT_ADD, FX_OP_INT_SUB, FX_OP_INT_MUL, FX_OP_INT_NEG,
  FX_OP_SIZE,         /* (tensor, int dim) -> int                graph_builder.cpp:319-327 */
  /* A prim::Loop whose only carried value is a tensor read through
   * immut::select(T, dim, i) and written through immut::select_rev(T, ., dim, i),
   * collapsed to one region: (self, body, int dim, int lo, int hi) where body is
   * built with fx_region_loop_var() standing for i.  No reference counterpart:
   * the reference keeps such loops serial (parallelize_loops.cpp:17). */
  FX_OP_FORALL_SELECT_REV,
  FX_OP_TRIL,         /* (self, int diagonal)                    fusable in fait/passes/fuse_ops.cpp:57 */
  FX_OP__COUNT
};

typedef struct fx_region fx_region; /* a region under construction / compiled */
typedef struct fx_plan fx_plan;     /* a region specialised to concrete shapes */

/* One run-time argument.  Tensors may be strided; sizes/strides in elements. */
typedef struct fx_arg {
  int32_t kind; /* 0 tensor, 1 int, 2 float, 3 bool */
  int32_t dtype;
  const void* ptr; /* device pointer (tensor) */
  int32_t rank;
  int32_t reserved;
  int64_t sizes[FX_ARG_MAX_RANK];
  int64_t strides[FX_ARG_MAX_RANK];
  int64_t ival; /* int / bool scalar */
  double fval;  /* float scalar (narrowed to fp32 like graph_builder.cpp:850-854) */
} fx_arg;

const char* fx_last_error(void);
int fx_api_version(void);

/* ---- region construction (replaces GraphBuilder::compile, graph_builder.cpp:259-712) ----
 * parallel_degree / is_parallel_map have the meaning of the attributes of
 * tssa::ParallelFunctor (fait/passes/te_op.h:13-23). */
int fx_region_create(int parallel_degree, int is_parallel_map, fx_region** out);
void fx_region_destroy(fx_region*);

/* Values.  Every function returns a value id (>= 0) in *id. */
/* tensor input; per_task = the matching entry of attr::is_parallel_args (a list
 * with one tensor per task, te_op.cpp:89-98) */
int fx_region_input_tensor(fx_region*, int dtype, int rank, int per_task, int* id);
int fx_region_input_scalar(fx_region*, int kind /*1 int,2 float,3 bool*/, int per_task, int* id);
int fx_region_task_index(fx_region*, int* id); /* subgraph input 0 (te_op.cpp:192, graph_builder.cpp:269-272) */
int fx_region_loop_var(fx_region*, int* id);   /* see FX_OP_FORALL_SELECT_REV */
int fx_region_const_int(fx_region*, int64_t v, int* id);
int fx_region_const_float(fx_region*, double v, int* id);
int fx_region_const_bool(fx_region*, int v, int* id);
int fx_region_const_none(fx_region*, int* id);
/* Wherever an operator takes an int[] of sizes (view, expand, full), the id of a tensor
 * value may be passed instead and stands for that tensor's sizes (aten::size(t)). */
int fx_region_int_list(fx_region*, const int* ids, int n, int* id);
int fx_region_tensor_list(fx_region*, const int* ids, int n, int* id);
/* out_dtype < 0: infer by type promotion */
int fx_region_op(fx_region*, int opcode, const int* arg_ids, int n_args, int out_dtype, int* id);
int fx_region_output(fx_region*, int value_id);
/* Fuse an order-preserving masked row select into the region: every output x
 * becomes x[mask] (mask: bool tensor over dim 0, computed in the region).
 * Contract: ATen index/nonzero semantics, which the reference leaves to ATen
 * (convert_to_tensorssa.cpp:422-443, fuse_ops.cpp:173-200). */
int fx_region_compact_rows(fx_region*, int mask_value_id);
int fx_region_finalize(fx_region*);

/* ---- specialisation to shapes (replaces DimExprEvaluator + prepareRunArgs shape part,
 *      evaluate_dim.cpp:132-227, graph_builder.cpp:863-889) ----
 * args: for each region input in declaration order, 1 entry, or
 * parallel_degree entries if it is per-task.  The plan is owned by the region
 * and cached by shape signature. */
int fx_region_plan(fx_region*, const fx_arg* args, int n_args, const fx_plan** plan);
int fx_plan_num_outputs(const fx_plan*);
/* shape of output out_idx for task; for a compacted output sizes[0] is the upper bound */
int fx_plan_output(const fx_plan*, int out_idx, int task, int32_t* dtype, int32_t* rank, int64_t* sizes);
size_t fx_plan_scratch_bytes(const fx_plan*); /* device scratch the caller must provide to fx_region_run */
int fx_plan_launches(const fx_plan*);         /* kernel launches one fx_region_run issues */
int64_t fx_plan_algorithmic_bytes(const fx_plan*); /* compulsory input bytes + dense output bytes */
/* Row compaction in one pass (opt-in).  A compacting region with one task class whose inputs are
 * all read row by row (the prediction tensor of a detection head, its anchor tables) can run as
 * ONE kernel: persistent workgroups park their rows of the inputs in LDS with coalesced loads,
 * evaluate the mask from there, publish their kept-row count and take their write offset from
 * the counts of the earlier tiles (every wait bounded; a workgroup that waits too long counts
 * the earlier rows itself).  Results are identical to the two-pass form (count + scatter), which
 * is the default because it is the faster one on the benchmark configurations but the smallest
 * (the detection-head regions among them have a kernel of their own, below).
 * fx_plan_streaming: 1 if fx_region_run would use the one-pass form for this plan now;
 * fx_set_streaming: process-wide switch (default off; FXHIP_STREAM=1: on);
 * fx_set_stream_spin_limit: polls before a workgroup stops waiting (default 4000; 0 makes every
 * workgroup count for itself, for tests).  No reference counterpart: the reference leaves
 * x[mask] to ATen (convert_to_tensorssa.cpp:422-443). */
int fx_plan_streaming(const fx_plan*);
/* out[0..8): one-pass form available, rows per tile, tiles per task, grid, and the window input's
 * row stride, per-task offset, first and number of elements used per row (test hook) */
int fx_plan_stream_info(const fx_plan*, int64_t* out, int cap);
void fx_set_streaming(int on);
void fx_set_stream_spin_limit(uint32_t polls);
/* The decode + score filter of a YOLO-style detection head in one launch.  A compacting region
 * whose lowered programs ARE that computation (sigmoid of the centre offsets, exp of the sizes,
 * anchors [N, 4] and strides [N], objectness threshold, kept rows of boxes [K, 4], class scores
 * [K, C] and objectness [K] out of predictions [images, N, 5 + C]; the reference's flagship
 * post-processing, functs/benchmark/ai_model/yolov3/yolov3_bbox.py:12-23 and 104-130) runs through
 * a hand-written kernel instead of the generic two passes: every workgroup streams a run of
 * consecutive prediction rows through LDS, publishes its kept-row count at once and takes its
 * write offset from the counts of the earlier workgroups of its image (every wait bounded, as
 * in the one-pass form above, with the same poll limit).  The programs are compared instruction
 * by instruction (any number of rows, images and classes C with C % 4 == 0, any threshold); a
 * region that differs anywhere keeps the generic kernels.  Results are bit-identical to those.
 * A second form of the same head is recognised too: anchors folded ahead of time into box centres
 * [N, 2] and half sizes [N, 2], strides as [N, 1] (what constant propagation leaves of anchors
 * that a model generates from static feature-map sizes).
 * A call recorded under stream capture takes the generic two passes (the one-launch forms tag
 * their status words with an epoch that travels in the kernel arguments and would be frozen in
 * the graph).
 * The same for an SSD-style head (functs/benchmark/ai_model/ssd/ssd_bbox.py:163-214): a map over
 * the foreground classes whose body decodes the boxes from offsets [1, N, 4] and priors [N, 4]
 * with two variances, takes the softmax of the scores [1, N, C] and keeps, for its class, the rows
 * above a threshold as boxes [K, 4] and scores [K].  Lowered generically every task would redo
 * the decode and the softmax; a plan whose programs ARE that computation (any N, C <= 128, first
 * class, threshold, variances) runs as one launch of a kernel that computes every row once, when
 * the device holds a workgroup per 32 rows at once (up to 16 384 or 65 536 rows; more rows keep the
 * generic kernels).  Bit-identical to the generic kernels on the same computation split in a
 * dense region (decode + softmax) and a class map over its results; the generic kernels on the
 * fused region itself sum the softmax in another order (1e-6 relative).
 * fx_set_head_kernel: process-wide switch for both kernels, default on (FXHIP_HEAD=0: off; also
 * off while fx_set_specialization(0) holds).  fx_plan_head_info (test hook): out[0] = 1 (YOLO-style
 * head recognised), 2 (SSD-style head) or 0; out[1] = that kernel is in use now; out[2], out[3] = low
 * and high word of the hash of the normalised programs; then C, 5 + C, rows, images (kind 1) or
 * classes filtered, C, rows, first class (kind 2).  This is where the reference compiles the
 * subgraph of the loop body with NVRTC (fait/tensorexpr/cuda_codegen_tssa.cpp:881-1414) and leaves
 * x[mask] to ATen (convert_to_tensorssa.cpp:422-443). */
void fx_set_head_kernel(int on);
int fx_plan_head_info(const fx_plan*, int64_t* out, int cap);

/* ---- generated row-stream kernels ----
 * A compacting region whose widest input is a row-major matrix of 32-bit elements that every
 * program reads row by row (the predictions of a detection head; any mask, any outputs built
 * from elementwise operators and the access / assign family, no reductions) has a ROW-STREAM
 * form: one launch in which every workgroup streams a run of consecutive rows through LDS,
 * publishes its kept-row count at once and takes its write offset from the counts of the
 * earlier workgroups of its task (every wait bounded).  The kernel is GENERATED from the
 * region's own lowered programs: fx_plan_rowstream_source writes a HIP translation unit in which
 * each program has been executed symbolically per output column, so that predicates of the
 * select_rev / slice_rev / cat / stack chains that depend on the column are decided, and loads
 * and sub-expressions shared between columns exist once per row.  Built into the library
 * (csrc/fxhip/spec/fx_rs_<key>.hip; `python -m functs_amd.aot` writes them), it serves every
 * plan with the same key: any number of rows and tasks, any per-task offsets, any values of the
 * floating-point constants (thresholds, scale factors) as long as equal constants stay equal.
 * Results are bit-identical to the generic kernels.  A plan without a linked kernel, and a call
 * recorded under stream capture, takes the generic two passes.
 * Stands where the reference generates and compiles CUDA for every subgraph
 * (fait/tensorexpr/cuda_codegen_tssa.cpp:881-1121, :1319-1414) and leaves x[mask] to ATen
 * (functs/csrc/jit/passes/convert_to_tensorssa.cpp:422-443).
 * fx_plan_rowstream_info: out[0] = the plan has a row-stream form, out[1] = a generated kernel
 * for it is linked and enabled (fx_region_run uses it), out[2], out[3] = low and high word of its
 * key, out[4] = elements per row of the streamed input, out[5] = rows, out[6] = tasks,
 * out[7] = input buffers.  fx_plan_rowstream_why: what rules the form out (empty when out[0]).
 * The kernel's workgroups are persistent: a launch has at most as many as the device holds at
 * once, and each takes chunks of up to 256 rows in turn (a chunk looks back at the chunks before
 * it, which are done or running).  One kind of launch beyond that size keeps the generic two
 * passes (out[1] = 0): a map of several tasks that all stream the SAME rows.
 * fx_set_rowstream: process-wide switch, default 1 = on (FXHIP_ROWSTREAM=0: off; also off while
 * fx_set_specialization(0) holds); 2 = on also for that kind of launch (slower than the two passes). */
int fx_plan_rowstream_info(const fx_plan*, int64_t* out, int cap);
int fx_plan_rowstream_why(const fx_plan*, char* buf, size_t cap);               /* returns the full length */
int fx_plan_rowstream_source(const fx_plan*, const char* label, char* buf, size_t cap); /* returns the full length */
void fx_set_rowstream(int on);
/* test hook: the argument block of a generated kernel for this plan (what travels in front of the
 * marshalled block of fx_region_marshal) with the given rows per workgroup and per sub-tile, so
 * that a generated unit compiled for the CPU can be driven without a device */
int fx_plan_rowstream_launch(const fx_plan*, uint32_t chunk_rows, uint32_t sub_rows, void* out, size_t cap);
int fx_rowstream_count(void);                   /* generated row-stream kernels linked into the library */
/* debugging / test hooks: the lowered bytecode blob (like CodeGen::getCodeText) */
int fx_plan_blob(const fx_plan*, const uint32_t** words, size_t* n_words);
int fx_plan_disasm(const fx_plan*, char* buf, size_t cap);

/* ---- ahead-of-time specialised kernels ----
 * The library runs a plan's programs with a bytecode interpreter.  A plan can also be
 * compiled: fx_plan_spec_source writes a HIP translation unit holding the plan's programs as
 * compile-time constants; built into the library (csrc/fxhip/spec/), its kernels are used for
 * every plan whose programs hash to the same key.  Results are the same instruction for
 * instruction; only speed differs.  Stands where the reference compiles each subgraph at run
 * time (fait/tensorexpr/cuda_codegen_tssa.cpp:1319-1414 CompileToNVRTC). */
uint64_t fx_plan_spec_key(const fx_plan*);      /* 0: plan cannot be specialised (tasks with different programs) */
int fx_plan_specialized(const fx_plan*);        /* 1 if fx_region_run uses specialised kernels for this plan */
int fx_plan_spec_source(const fx_plan*, const char* label, char* buf, size_t cap); /* returns the full length */
void fx_set_specialization(int on);             /* process-wide switch, default on (FXHIP_SPECIALIZE=0: off) */
int fx_specialization_count(void);              /* specialised regions linked into the library */
void fx_launch_stats(uint64_t* total, uint64_t* specialised); /* region kernel launches of this process so far */
/* Dense regions of one task class with one or two outputs of 32-bit elements are run by a short
 * kernel of their own when their programs are compiled: it takes
 * what a workgroup needs in front of its first load from a small argument block and stages the
 * descriptor only if a program reads it (on a region of a few MB the start of the workgroups is
 * what a launch costs).  Same results as the general kernel, bit for bit.
 * fx_plan_dense_lean: 1 if fx_region_run uses that kernel for this plan.  fx_set_dense_lean:
 * process-wide switch, default on (FXHIP_DENSE_LEAN=0: off).  Replaces the one-element-per-thread
 * launch of fait/tensorexpr/cuda_codegen_tssa.cpp:1167-1306. */
int fx_plan_dense_lean(const fx_plan*);
void fx_set_dense_lean(int on);
int fx_spec_dump_dir(const char* dir);          /* plans without specialised kernels leave their source in dir (NULL: stop) */
int fx_spec_dump_what(int what);                /* which sources: 1 program tables (fx_spec_*), 2 row-stream units (fx_rs_*), 3 both (default), 0 none; returns the setting before */

/* ---- execution (replaces CudaCodeGenTssa::call_raw, cuda_codegen_tssa.cpp:1167-1290) ----
 * out_ptrs[out_idx * parallel_degree + task] = device buffer of that output.
 * scratch: fx_plan_scratch_bytes() of device memory (may be NULL when 0).
 * totals_host: for compacting regions, pinned host memory (device-visible) of
 *   parallel_degree uint32 that receives the kept-row count per task; it is
 *   valid after the stream has been synchronised, or after fx_region_wait_totals.
 *   NULL otherwise.
 * Asynchronous on `stream` (a hipStream_t); no hidden synchronisation. */
int fx_region_run(fx_region*, const fx_plan*, const fx_arg* args, int n_args, void* const* out_ptrs,
                  void* scratch, uint32_t* totals_host, void* stream);

/* Returns once every task's kept-row count of the last fx_region_run on `stream` with this
 * totals_host is readable.  The counts are stored early in the second pass, so this usually
 * returns while the kernels still run: the caller can size its output views and go on; the
 * outputs themselves are valid in stream order, like after any asynchronous launch.  The
 * calling thread polls the pinned words for at most fx_set_totals_spin_us microseconds (default
 * 2000; 0: not at all) and then blocks in a synchronisation of the stream, so a launch queued
 * behind long work does not keep a core busy.  Where ATen's nonzero / masked index synchronise
 * (the reference leaves x[mask] to them, convert_to_tensorssa.cpp:422-443). */
#define FX_TOTAL_PENDING 0xffffffffu
int fx_region_wait_totals(const fx_plan*, const uint32_t* totals_host, void* stream);
void fx_set_totals_spin_us(uint32_t microseconds);
/* The polling part alone: 1 as soon as every count is readable, 0 when they are not after
 * spin_us microseconds (nothing blocks, no call into the runtime), negative on error.  For a
 * caller that holds a lock it must give up before it may block (the Python interpreter's). */
int fx_region_poll_totals(const fx_plan*, const uint32_t* totals_host, uint32_t spin_us);

/* fx_region_run with a HIP event pair around every kernel on `stream`; waits for
 * the last event and returns the duration of each launch in milliseconds
 * (kernel_ms[0..*n_kernels), order of launch: [count, scatter] for compacting
 * regions, [dense] otherwise).  Measurement aid of the benchmark; the reference
 * measures with CUPTI activity records instead (fait/util/profile.cpp:29-46). */
int fx_region_run_timed(fx_region*, const fx_plan*, const fx_arg* args, int n_args, void* const* out_ptrs,
                        void* scratch, uint32_t* totals_host, void* stream, float* kernel_ms, int cap,
                        int* n_kernels);
/* The same with every kernel launched `repeat` times back to back inside its event pair
 * (1..1000; the kernels of a region are idempotent: they read the call's inputs and write its
 * outputs); kernel_ms holds the mean per launch.  An event pair around one launch adds about
 * 2 us to what it reads (an empty kernel reads 6 us that way); a batch spreads that over its
 * launches, and what is left is the duration a kernel trace reports.  Measurement aid of the
 * benchmark as well (fait/util/profile.cpp:29-46). */
int fx_region_run_timed_batched(fx_region*, const fx_plan*, const fx_arg* args, int n_args, void* const* out_ptrs,
                                void* scratch, uint32_t* totals_host, void* stream, int repeat, float* kernel_ms,
                                int cap, int* n_kernels);

/* The kernels of a call launched over n_sets argument sets of one plan in rotation (set 0,
 * 1, ..., n_sets-1, `rounds` times) inside ONE event pair on `stream`; *ms_mean is the mean
 * per launched call (which < 0: every kernel of the call, in order) or per launch of kernel
 * `which` of the call alone (0 .. fx_plan_launches-1).  Each set brings its own inputs, outputs,
 * scratch and totals; with sets that together exceed the last-level cache (256 MB) every
 * launch reads and writes cold lines, which the same buffers launched back to back do not.
 * Every set is run once untimed first.  Measurement aid of the benchmark
 * (the reference: functs/utils/evaluate.py:172-208 times whole calls on one input). */
int fx_region_run_timed_sets(fx_region*, const fx_plan*, int n_sets, const fx_arg* const* args, int n_args,
                             void* const* const* out_ptrs, void* const* scratch, uint32_t* const* totals_host,
                             void* stream, int which, int rounds, float* ms_mean);

/* The argument marshalling of fx_region_run without the launch (host only; the
 * analogue of GraphBuilder::prepareRunArgs, graph_builder.cpp:718-899).
 * dyn_out receives fx_dyn_bytes() bytes: the by-value block the kernels read. */
int fx_region_marshal(fx_region*, const fx_plan*, const fx_arg* args, int n_args, void* const* out_ptrs,
                      void* scratch, uint32_t* totals_host, void* dyn_out, size_t dyn_cap);
size_t fx_dyn_bytes(void);
/* A map of many tasks can have more pointers and scalars than that block holds (320 and 176):
 * up to 4096 of each, fx_region_run then writes the two tables to the end of the caller's scratch
 * memory (fx_plan_scratch_bytes counts them, also for a region that does not compact) with small
 * launches ahead of the kernels, which read them from there; such a plan runs the general
 * kernels or the build of its generated row-stream kernel that reads device memory (the
 * hand-written one-launch kernels and the short dense kernel read the argument block), and
 * fx_region_marshal refuses it.  The reference passes every task's buffers as kernel arguments
 * and clones the body per task (functor_parallization.cpp:12-111): its limit is the compiler's.
 * fx_plan_table_sizes: entries of the two tables, and whether the plan uploads them.
 * fx_region_marshal_tables: the tables themselves, for any plan (host only; tests). */
int fx_plan_table_sizes(const fx_plan*, size_t* n_pointers, size_t* n_scalars, int* uploaded);
int fx_region_marshal_tables(fx_region*, const fx_plan*, const fx_arg* args, int n_args, void* const* out_ptrs,
                             void* scratch, uint32_t* totals_host, uint64_t* pointers, size_t pointer_cap,
                             uint32_t* scalars, size_t scalar_cap);

/* int64 in regions.  Programs that only MOVE int64 data (select / slice / index / where / cat /
 * *_rev / row compaction ...) are exact for every value: they travel as two 32-bit words.
 * Integer ARITHMETIC is 32-bit: an int64 tensor element that enters it (a + 3, a == b, a as an
 * index) must fit 32 bits (a conversion to float uses the whole element and is exact).  The
 * loads check that; an element that does not fit sets a sticky process-wide error word, and
 * the outputs of that launch are not to be used.  Integer constants and scalar arguments outside
 * 32 bits are refused when the region is planned / run (FX_E_UNSUPPORTED / FX_E_LIMIT).  The
 * reference computes in int64 throughout (NNC kLong, functs/csrc/jit/ir/symbol_ext.cpp:17-117 for
 * the eager bodies).
 *
 * The error word is a set of bits: FX_ASYNC_INT64 from these loads, FX_ASYNC_BARRIER from a wait
 * that fx_lstm_stack gave up, FX_ASYNC_NMS_CAPACITY from fx_sort_nms (of the reports that kernels
 * make the latest one is kept).  After the stream has been synchronised the word covers every
 * launch before that.  fx_async_error returns the word and, when `clear` is non-zero, clears all
 * of it; fx_async_error_take(mask) returns and clears only the bits of `mask`, for a caller that
 * handles one kind of report and must leave the others to whoever handles those. */
#define FX_ASYNC_INT64 1
#define FX_ASYNC_BARRIER 2
#define FX_ASYNC_NMS_CAPACITY 4
int fx_async_error(int clear);
int fx_async_error_take(int mask);
/* Adds bits to the word from the host: for code built on the library that finds such an error
 * itself and reports it where its callers already look. */
void fx_async_error_report(int bits);

/* ---- stand-alone order-preserving row compaction (x[mask] for several x) ----
 * mask: n bytes (0/1); cols[i]: [n, rowlen[i]] fp32/int32 (4-byte) or int64 (8-byte) rows.
 * outs[i] must hold n * rowlen[i] elements.  Same contract as ATen
 * index(Tensor, [bool mask]) / nonzero. */
int fx_compact_rows(const uint8_t* mask, int64_t n, const void* const* cols, void* const* outs,
                    const int32_t* rowlen, const int32_t* elsize, int n_cols, void* scratch,
                    size_t scratch_bytes, uint32_t* total_host, void* stream);
size_t fx_compact_rows_scratch_bytes(int64_t n);
/* fx_compact_rows for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same arguments and results as fx_compact_rows without the scratch pair: the
 * tile counts live in a fixed 64 KiB device array of the library (one per GPU, held until
 * the process ends), and the call allocates and frees nothing.  n above
 * FX_COMPACT_ROWS_STATIC_MAX returns FX_E_LIMIT.  All calls on one GPU share the array:
 * calls that overlap on one GPU (different streams, no ordering between them) race. */
#define FX_COMPACT_ROWS_STATIC_MAX 4194304 /* rows */
int fx_compact_rows_static(const uint8_t* mask, int64_t n, const void* const* cols, void* const* outs,
                           const int32_t* rowlen, const int32_t* elsize, int n_cols, uint32_t* total_host,
                           void* stream);

/* ---- stacked LSTM recurrence as one launch ----
 * The loop nest of functs/benchmark/ai_model/lstm/lstm.py:79-133
 *   for t in [0, T): cur = x[t]
 *     for j in [0, L): gates = cur @ wih[j] + bih[j] + h[j] @ whh[j] + bhh[j]   (gate order i, f, g, o)
 *                      c[j] = sigmoid(f) * c[j] + sigmoid(i) * tanh(g); h[j] = sigmoid(o) * tanh(c[j]); cur = h[j]
 *     out[t] = cur
 * which the reference runs on the host, one fused kernel and two library GEMMs per (t, j)
 * (the loops carry state: fait/passes/parallelize_loops.cpp:17, unroll_loops.cpp:59-65), as ONE
 * persistent kernel: a workgroup per two hidden units keeps their columns of the weights in
 * registers for the whole sequence (thread k row k of them, and element k of the step's vectors);
 * the diagonals t + j follow each other without a barrier between workgroups, every h value
 * travels with the tag of the step that wrote it and readers poll for the tag they expect, with
 * bounded waits.  A wait that is given up reports FX_ASYNC_BARRIER through fx_async_error, fills
 * out / state_h / state_c with NaN and ends the kernel; its workspace stays marked, and every
 * later launch on it does no step, reports the error again and returns NaN, until the caller has
 * cleared the workspace.  A caller must therefore look at fx_async_error after synchronising and
 * before it uses the results (or test them for NaN), and clear the workspace after an error.
 * Contiguous fp32: x [T, B, H]; wih, whh [L, 4, H, H]; bih, bhh [L, 4, 1, H]; h0, c0, state_h,
 * state_c [L, B, H]; out [T, B, H]; h0 / c0 may be null (zero initial state).  H is 32, 64, ...
 * 1024 (a power of two), L <= 4, B <= 16 (FX_E_UNSUPPORTED otherwise), and H / 2 workgroups of
 * 512 threads must be resident together (FX_E_LIMIT).
 * workspace: fx_lstm_stack_workspace_bytes() of device memory, 256-byte aligned, all zero when it
 * is used for the first time.  A launch that ends without error leaves it ready for the next one,
 * so one workspace, cleared once, serves launch after launch on one stream as long as batch,
 * hidden and layers stay the same (launches that share a workspace must not overlap); after a
 * launch that reported an error the caller clears it again. */
/* 1 when fx_lstm_stack is built for these sizes, 0 otherwise: the part of its conditions that
 * needs no device, for a compiler pass that decides whether to emit the call (H a power of two in
 * 32..1024, L <= 4, B <= 16, and the weight columns of all layers fit the registers of a
 * workgroup at the occupancy that keeps all workgroups resident: L <= 2 for H = 1024). */
int fx_lstm_stack_fits(int batch, int hidden, int layers);
size_t fx_lstm_stack_workspace_bytes(int batch, int hidden, int layers);
int fx_lstm_stack(const float* x, const float* wih, const float* whh, const float* bih, const float* bhh, const float* h0,
                  const float* c0, float* out, float* state_h, float* state_c, int seq_len, int batch, int hidden,
                  int layers, void* workspace, size_t workspace_bytes, void* stream);
void fx_set_lstm_spin_limit(uint32_t polls); /* barrier polls before a wait is given up (default 1000000; tests) */

/* ---- detection tail: score threshold + sort + class-aware greedy NMS + top-k, one launch ----
 * The step behind row compaction in the reference's detection programs, which it runs as ATen /
 * torchvision kernels with host synchronisations in between:
 *   mode 1  multiclass_nms (functs/benchmark/ai_model/yolov3/yolov3_bbox.py:104-138 with batched_nms
 *           :141-171 and nms_wrapper :174-179): scores is cls [rows, n_classes] (rows scores_row_stride apart), a candidate
 *           (row, class) needs cls > score_thr, its score is cls * factors[row], its label the class;
 *   mode 0  batched_nms alone (ssd_bbox.py:175-214): scores [rows], labels [rows] (null: one class),
 *           a candidate needs score > score_thr (pass -INFINITY to take every row).
 * Per task (image): candidates in order of descending score (equal scores by ascending index),
 * a candidate is dropped when a kept one of the same class overlaps it with IoU > iou_thr
 * (classes are told apart as the reference does: boxes moved by label * (largest candidate
 * coordinate + 1)), the first max_num kept ones are returned.  IoU in float32 as torchvision's CPU
 * kernel computes it: inter / ((area_i + area_j) - inter).
 * Outputs have fixed shapes; rows from n_out[task] on are zero.  out_index is the candidate's
 * position in the input (mode 0: row, mode 1: row * n_classes + class).
 * `counts` (valid rows per task) and `n_out` may be device memory or pinned host memory: a count
 * that a compaction wrote is read by the kernel, not by the host.
 * Limits: at most FX_NMS_MAX_CANDIDATES candidates per task - `key_capacity` says how many the
 * launch is sized for (rounded up to a power of two >= 128); a task with more returns zeros, sets
 * its n_out to FX_NMS_OVERFLOW and reports FX_ASYNC_NMS_CAPACITY through fx_async_error - and
 * max_num <= FX_NMS_MAX_OUT.  boxes must be 16-byte
 * aligned, boxes_task_stride a multiple of 4.  Task strides are in elements. */
#define FX_NMS_MAX_CANDIDATES 16384
#define FX_NMS_MAX_OUT 1024
#define FX_NMS_OVERFLOW 0xffffffffu
typedef struct fx_nms_desc {
  int32_t mode;
  int32_t n_tasks;
  uint32_t rows;        /* rows per task (at most; see counts) */
  uint32_t n_classes;   /* mode 1 */
  const float* boxes;   /* [rows, 4] per task, x1 y1 x2 y2 */
  int64_t boxes_task_stride;
  const float* scores;
  int64_t scores_task_stride;
  uint32_t scores_row_stride; /* mode 1: elements from one row of scores to the next; 0: n_classes.  Larger: the row
                                 carries columns behind its class scores (the reference's padding column,
                                 yolov3_bbox.py:237-238, which multiclass_nms cuts off again, :113) that are not candidates */
  uint32_t reserved0;
  const float* factors; /* mode 1, [rows] per task; null: 1 */
  int64_t factors_task_stride;
  const int64_t* labels; /* mode 0, [rows] per task; null: one class */
  int64_t labels_task_stride;
  const uint32_t* counts; /* [n_tasks] valid rows per task; null: rows */
  float score_thr;
  float iou_thr;
  uint32_t max_num;
  uint32_t key_capacity;
  float* dets;           /* [n_tasks, max_num, 5]: x1 y1 x2 y2 score */
  int64_t* out_labels;   /* [n_tasks, max_num] */
  int64_t* out_index;    /* [n_tasks, max_num] or null */
  uint32_t* n_out;       /* [n_tasks] */
  void* workspace;       /* fx_sort_nms_workspace_bytes() of device memory, 256-byte aligned */
  size_t workspace_bytes;
} fx_nms_desc;
/* workspace: the first fx_sort_nms_workspace_clear_bytes() bytes are zero when a launch starts; every
 * launch leaves them zero, so one workspace, cleared once, serves launch after launch on one stream
 * as long as n_tasks and key_capacity stay the same (they fix where the counters lie; launches
 * that share a workspace must not overlap). */
size_t fx_sort_nms_workspace_bytes(int n_tasks, uint32_t key_capacity);
size_t fx_sort_nms_workspace_clear_bytes(int n_tasks);
int fx_sort_nms(const fx_nms_desc* desc, void* stream);

/* ---- device utilities ---- */
int fx_device_count(void);
/* plain 16-byte copy kernel of known size: counter calibration and bandwidth ceiling */
int fx_copy_bytes(const void* src, void* dst, size_t bytes, void* stream);
/* The same copy timed the way fx_region_run_timed_sets times a region's kernels: `rounds` passes
 * over n_sets (src, dst) pairs of `bytes` each, launched back to back from here between two events
 * on the stream; *ms_per_copy is the mean per launch.  (A loop in an interpreted language cannot
 * issue launches as fast as a small copy runs.) */
int fx_copy_bytes_timed_sets(const void* const* src, void* const* dst, int n_sets, size_t bytes, int rounds, void* stream,
                             float* ms_per_copy);

#ifdef __cplusplus
}
#endif
#endif /* FXHIP_H_ */
