/*
 * denox_hip.h -- C ABI of the MI355X (gfx950) execution backend for denox models.
 *
 * The reference (kistenklaus/denox) exposes this path only as C++ classes that
 * throw; each entry point below names the C++ interface it stands for.  All
 * functions return 0 on success or a DENOX_HIP_* status; the message of the
 * last failure on the calling thread is available from
 * denox_hip_last_error().  No exception crosses this boundary.  Handles are
 * opaque and not thread-safe (the reference's objects are not either); use one
 * handle from one thread at a time.
 *
 * Pointers named `host_*` are host memory, `dev_*` are device (HBM) addresses.
 * Tensors are tightly packed binary16 in the layout their descriptor states.
 */
#ifndef DENOX_HIP_H
#define DENOX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DENOX_HIP_OK 0
#define DENOX_HIP_INVALID_ARGUMENT 1
#define DENOX_HIP_INVALID_MODEL 2
#define DENOX_HIP_HIP_ERROR 3
#define DENOX_HIP_COMPILE_ERROR 4
#define DENOX_HIP_UNSUPPORTED 5
#define DENOX_HIP_IO_ERROR 6
#define DENOX_HIP_INTERNAL 7

/* dnx.fbs:82-91 TensorFormat */
#define DENOX_HIP_FORMAT_HWC 1
#define DENOX_HIP_FORMAT_CHW 2
#define DENOX_HIP_FORMAT_CHWC8 3

typedef struct denox_hip_context denox_hip_context;   /* runtime::Context   (runtime/src/denox/runtime/context.hpp:113-252) */
typedef struct denox_hip_model denox_hip_model;       /* runtime::Model     (runtime/src/denox/runtime/model.hpp:107-170)  */
typedef struct denox_hip_instance denox_hip_instance; /* runtime::Instance  (runtime/src/denox/runtime/instance.hpp:44-63) */
typedef struct denox_hip_builder denox_hip_builder;   /* compiler::Model    (compiler/src/denox/compiler/frontend/model/Model.hpp:33-62) */
typedef struct denox_hip_db denox_hip_db;             /* denox::Db          (database/src/denox/db/Db.hpp:15-69) */

const char *denox_hip_last_error(void);
const char *denox_hip_version(void);

/* Where the kernel sources (*.hip) live and where compiled code objects are
 * cached.  NULL keeps the default (next to the library).  Role of the GLSL
 * source directory + the SPIR-V cache (spirv/src/denox/glsl/GlslCompiler.hpp,
 * compiler/src/denox/compiler/compile_shaders/compile_shaders.cpp:80-83). */
int denox_hip_set_kernel_paths(const char *kernel_dir, const char *cache_dir);

/* ------------------------------------------------------------------ device_info
 * DeviceInfo (device_info/src/denox/device_info/DeviceInfo.hpp:12-20) and
 * query_driver_device_info (device_info/.../query/query_driver_device_info.hpp:9-21).
 * device < 0 returns the built-in CDNA4 table without touching a GPU. */
typedef struct denox_hip_device_info {
  char name[128];
  char arch[32];
  uint32_t subgroup_size;
  uint32_t max_workgroup_invocations;
  uint32_t max_workgroup_size[3];
  uint32_t max_workgroup_count[3];
  uint32_t max_shared_memory;
  uint32_t compute_units;
  uint32_t xcd_count;
  uint64_t hbm_bytes;
  double hbm_bytes_per_second;
  double fp16_mfma_flops;
  uint32_t matrix_shape_count;
  uint32_t matrix_shapes[4][3]; /* m, n, k; fp16 inputs, fp32 accumulation */
  int32_t from_device;
} denox_hip_device_info;
int denox_hip_query_device_info(int device, denox_hip_device_info *out);

/* ------------------------------------------------------------------ graph builder
 * compiler::Model: input / conv2d / activation / upsample / pool / concat /
 * pad / slice / output (frontend/model/Model.hpp:33-62, Model.cpp:209-259).
 * Symbolic extents are int64 handles: denox_hip_builder_sym_const / _sym_var
 * create them, _sym_op combines them (role of SymGraph,
 * common/src/denox/symbolic/SymGraph.hpp).  Tensor handles are ints >= 0. */
#define DENOX_HIP_SYM_ADD 1
#define DENOX_HIP_SYM_SUB 2
#define DENOX_HIP_SYM_MUL 3
#define DENOX_HIP_SYM_DIV 4
#define DENOX_HIP_SYM_MOD 5
#define DENOX_HIP_SYM_MIN 6
#define DENOX_HIP_SYM_MAX 7

#define DENOX_HIP_ACT_RELU 1
#define DENOX_HIP_ACT_LEAKY_RELU 2

int denox_hip_builder_create(denox_hip_builder **out);
void denox_hip_builder_destroy(denox_hip_builder *b);
int denox_hip_builder_sym_const(denox_hip_builder *b, int64_t value, int64_t *out_sym);
/* Named free variable (Model::requireValueOfName); at most 8; their values
 * are 64-bit integers supplied per Instance. */
int denox_hip_builder_sym_var(denox_hip_builder *b, const char *name, int64_t *out_sym);
int denox_hip_builder_sym_op(denox_hip_builder *b, int op, int64_t lhs, int64_t rhs, int64_t *out_sym);
int denox_hip_builder_input(denox_hip_builder *b, const char *name, int64_t width_sym, int64_t height_sym, uint32_t channels, int *out_tensor);
/* weights: binary16 [K][C][R][S] (ONNX order); bias: binary16 [K] or NULL */
int denox_hip_builder_conv2d(denox_hip_builder *b, int src, uint32_t K, uint32_t C, uint32_t R, uint32_t S,
                             const uint16_t *host_weights, const uint16_t *host_bias,
                             uint32_t stride_x, uint32_t stride_y, uint32_t pad_x, uint32_t pad_y,
                             uint32_t dil_x, uint32_t dil_y, int *out_tensor);
int denox_hip_builder_activation(denox_hip_builder *b, int src, int func, float alpha, int *out_tensor);
int denox_hip_builder_upsample(denox_hip_builder *b, int src, uint32_t scale, int *out_tensor);            /* nearest */
int denox_hip_builder_pool(denox_hip_builder *b, int src, uint32_t kx, uint32_t ky, uint32_t pad_x, uint32_t pad_y,
                           uint32_t stride_x, uint32_t stride_y, int *out_tensor);                          /* max */
/* Model::pool with PoolFunction::Avg (compiler/src/denox/compiler/frontend/model/Model.cpp:150-175,
 * common/src/denox/common/PoolFunction.hpp:7-10): the window's mean, summed in binary32 and rounded once. */
int denox_hip_builder_avg_pool(denox_hip_builder *b, int src, uint32_t kx, uint32_t ky, uint32_t pad_x, uint32_t pad_y,
                               uint32_t stride_x, uint32_t stride_y, int *out_tensor);
int denox_hip_builder_concat(denox_hip_builder *b, int src0, int src1, int *out_tensor);
int denox_hip_builder_pad(denox_hip_builder *b, int src, int64_t left_sym, int64_t right_sym, int64_t top_sym, int64_t bottom_sym, int *out_tensor); /* replicate */
/* mode: 0 replicate the border (PaddingMode::Edge of the reference), 1 zeros (PaddingMode::Zero) */
int denox_hip_builder_pad_mode(denox_hip_builder *b, int src, int64_t left_sym, int64_t right_sym, int64_t top_sym, int64_t bottom_sym, int32_t mode, int *out_tensor);
/* half-open source ranges [left, right) x [top, bottom) */
int denox_hip_builder_slice(denox_hip_builder *b, int src, int64_t left_sym, int64_t right_sym, int64_t top_sym, int64_t bottom_sym, int *out_tensor);
int denox_hip_builder_output(denox_hip_builder *b, int src, const char *name);

/* Fills an empty builder from an ONNX ModelProto held in memory: inputs (NCHW, N = 1; dynamic height / width become
 * named extents after their dim_param), layers and outputs.  Stands for denox::onnx::read
 * (compiler/src/denox/compiler/frontend/onnx/onnx.cpp:70-158), the first step of denox::compile
 * (compiler/src/denox/compiler/compile.cpp:21-61).  Operators: Conv, Relu, LeakyRelu, MaxPool, AveragePool, Resize / Upsample
 * (nearest, integer factor), Concat, Pad (edge, or constant 0), Slice, and the shape arithmetic exporters emit around them;
 * anything else reports DENOX_HIP_UNSUPPORTED with the operator's name. */
int denox_hip_builder_import_onnx(denox_hip_builder *b, const void *onnx_bytes, size_t size);
/* graph inputs / outputs of a builder, in declaration order */
int denox_hip_builder_input_count(const denox_hip_builder *b, uint32_t *out);
int denox_hip_builder_output_count(const denox_hip_builder *b, uint32_t *out);
/* name (written to `name`, at most `capacity` bytes with the terminator) and channel count of input / output i */
int denox_hip_builder_input_info(const denox_hip_builder *b, uint32_t i, char *name, size_t capacity, uint32_t *out_channels);
int denox_hip_builder_output_info(const denox_hip_builder *b, uint32_t i, char *name, size_t capacity, uint32_t *out_channels);

/* ------------------------------------------------------------------ compile
 * denox::compile(onnx, db, options) -> bytes (compiler/src/denox/compiler/compile.cpp:21-61)
 * with CompileOptions (compiler/src/denox/compiler/Options.hpp:13-72). */
typedef struct denox_hip_compile_options {
  int32_t enable_conv_relu_fusion;   /* Features::enableConvReluFusion   */
  int32_t enable_concat_conv_fusion; /* Features::enableConcatConvFusion */
  int32_t enable_upsample_fusion;    /* conv reads a half-resolution source */
  int32_t enable_pool_fusion;        /* conv stores the 2x2 max only */
  int32_t enable_pad_fusion;         /* conv reads an un-padded source through the replicate clamp */
  int32_t enable_slice_fusion;       /* conv stores only the cropped window */
  int32_t enable_alternating_traversal; /* consecutive conv dispatches walk their tiles in opposite directions (cache reuse) */
  int32_t enable_upsample_fold;      /* offer kernels that fold a fused 2x upsample into the weights: fewer multiplications, the
                                        summed weights rounded to binary16 once more (no counterpart in the reference) */
  int32_t enable_implicit_concat;    /* Features::enableImplicitConcat: a concat source whose only consumer is the concat may be
                                        written by its producer straight into the concat's output (no copy dispatch) */
  int32_t input_format;              /* DENOX_HIP_FORMAT_* of every model input  (0 = HWC) */
  int32_t output_format;             /* DENOX_HIP_FORMAT_* of every model output (0 = HWC) */
  uint32_t assumption_count;         /* extents assumed for cost estimates */
  const char *const *assumption_names;
  const int64_t *assumption_values;
  const char *force_conv_config;     /* NULL / "" = choose; else one named conv configuration */
  int32_t device;                    /* >= 0: prune configurations with that device's limits; < 0: CDNA4 table */
  /* denox_hip_db_populate only: compile every candidate kernel into the code-object cache
   * (compiler/src/denox/compiler/populate.cpp:70-99); shard index/count let several processes
   * split that work (this call compiles the kernels whose ordinal % count == index). */
  int32_t populate_compile_kernels;
  uint32_t kernel_shard_index;
  uint32_t kernel_shard_count;
  int32_t enable_conv_conv_fusion;   /* two consecutive 3x3 convolutions with at most 32 channels between them in one dispatch,
                                        the tensor between them kept on chip (no counterpart in the reference) */
  int32_t enable_blocked_layout;     /* offer every internal tensor in CHWC8 beside HWC, as two nodes of the graph the schedule is
                                        selected from (compiler/src/denox/compiler/specialization/specialization.cpp:13-16,282-306) */
  int32_t layout_preference;         /* > 0: candidates that touch a CHWC8 tensor count half their cost (to exercise or measure
                                        that path); 0: cost alone decides */
} denox_hip_compile_options;
void denox_hip_compile_options_default(denox_hip_compile_options *opt);
/* db may be NULL (roofline estimates drive the selection).  The blob is
 * malloc'ed; release it with denox_hip_free. */
int denox_hip_compile(const denox_hip_builder *b, const denox_hip_compile_options *opt, const denox_hip_db *db,
                      void **out_dnx, size_t *out_size);
/* The names `force_conv_config` accepts, separated by commas: the configuration tables of the convolution shaders, the
 * hand-listed counterpart of the configuration spaces the reference's conv shaders enumerate
 * (compiler/src/denox/compiler/implement/shaders/conv/DirectConvShaderCM.cpp:40-181).  A static string. */
const char *denox_hip_conv_config_names(void);
/* one line per selected dispatch of the most recent compile on this thread */
const char *denox_hip_last_compile_report(void);
void denox_hip_free(void *p);
/* JSON description of a compiled model with every symbolic quantity evaluated
 * at the given extents: tensors, buffers, dispatches (workgroup counts, push
 * constants, bindings, bytes and FLOPs).  Needs no GPU.  The role of reading
 * a dnx file back (runtime/src/denox/runtime/model.cpp:637-659).  Release the
 * string with denox_hip_free. */
int denox_hip_dnx_describe(const void *dnx, size_t size, const char *const *names, const int64_t *values, uint32_t n, char **out_json);

/* minimum_cost_subgraph (common/src/denox/algorithm/minimum_const_subgraph.hpp:45-49), the search
 * behind schedule selection (compiler/src/denox/compiler/selection/selection.cpp:23-266), on a
 * caller-supplied hyper-graph.  Nodes 0..node_count-1 are numbered in topological order; edge e
 * produces edge_outputs[e] from edge_inputs[edge_input_offsets[e] .. edge_input_offsets[e+1]).
 * Writes the chosen edge indices in execution order (out_chosen has room for edge_count entries).
 * *out_total >= 1e300 and zero chosen edges mean that an output cannot be produced. */
int denox_hip_min_cost_subgraph(uint32_t node_count, const uint8_t *is_input, uint32_t edge_count, const uint32_t *edge_input_offsets,
                                const int32_t *edge_inputs, const int32_t *edge_outputs, const double *edge_costs, uint32_t output_count,
                                const int32_t *outputs, uint32_t *out_chosen, uint32_t *out_chosen_count, double *out_total);

/* ------------------------------------------------------------------ database
 * Db::open / populate / bench / query / dumpcsv
 * (database/src/denox/db/Db.hpp:15-69, compiler/src/denox/compiler/populate.cpp:23-256,
 *  runtime/src/denox/runtime/db.hpp:9-37, cli/src/denox/cli/dumpcsv.cpp:15-46). */
typedef struct denox_hip_db_bench_options {
  uint32_t min_samples;        /* DbBenchOptions::minSamples, default 10 (runtime/db.hpp:9-13) */
  double max_relative_error;   /* default 0.05 */
  uint32_t max_samples;
  int32_t save_progress;
  const char *filter;          /* NULL = every row */
} denox_hip_db_bench_options;
typedef struct denox_hip_db_bench_result { uint64_t benchmarked, converged, skipped, failed; } denox_hip_db_bench_result;
int denox_hip_db_open(const char *path, denox_hip_db **out);
void denox_hip_db_close(denox_hip_db *db);
int denox_hip_db_row_count(const denox_hip_db *db, uint64_t *out);
int denox_hip_db_populate(denox_hip_db *db, const denox_hip_builder *b, const denox_hip_compile_options *opt, uint64_t *out_added);
void denox_hip_db_bench_options_default(denox_hip_db_bench_options *opt);
int denox_hip_db_bench(denox_hip_db *db, denox_hip_context *ctx, const denox_hip_db_bench_options *opt, denox_hip_db_bench_result *out);
int denox_hip_db_add_sample(denox_hip_db *db, uint64_t row, double latency_ns);   /* Db::add_dispatch_benchmark_result */
int denox_hip_db_row_stats(const denox_hip_db *db, uint64_t row, uint64_t *samples, double *mean_ns, double *std_ns);
int denox_hip_db_writeback(const denox_hip_db *db);                                /* Db::atomic_writeback */
int denox_hip_db_dump_csv(const denox_hip_db *db, char **out_csv);                 /* release with denox_hip_free */

/* ------------------------------------------------------------------ runtime
 * Context::make, Model::make(dnx, ctx), Instance::make(model, specs),
 * Instance::infer(const void**, void**), Instance::bench(), getOutputDesc
 * (runtime/src/denox/runtime/instance.hpp:44-63, instance.cpp:278-430,432-753). */
typedef struct denox_hip_tensor_desc {
  int64_t width, height, channels;
  int32_t format; /* DENOX_HIP_FORMAT_* */
  int32_t dtype;  /* dnx ScalarType, 6 = F16 */
  uint64_t byte_size;
  char name[64];
} denox_hip_tensor_desc;

typedef struct denox_hip_timing {
  char name[64];
  char input[48];
  char output[48];
  uint64_t memory_reads, memory_writes, flops;
  float latency_ms;
} denox_hip_timing;

int denox_hip_context_create(int device, denox_hip_context **out);
void denox_hip_context_destroy(denox_hip_context *ctx);
/* the stream every instance of this context launches on (a hipStream_t) */
int denox_hip_context_stream(const denox_hip_context *ctx, void **out_stream);

int denox_hip_model_create(denox_hip_context *ctx, const void *dnx, size_t size, denox_hip_model **out);
void denox_hip_model_destroy(denox_hip_model *m);
int denox_hip_model_dispatch_count(const denox_hip_model *m, uint32_t *out);

/* names/values: the dynamic extents ("H", "W", ...); unknown names are ignored,
 * a missing one is an error.  Extents that the graph cannot take (sources of a concat that differ in width or height, a
 * slice that leaves its source) are DENOX_HIP_INVALID_ARGUMENT; a tensor of 4 GiB or more is DENOX_HIP_UNSUPPORTED. */
int denox_hip_instance_create(denox_hip_model *m, const char *const *names, const int64_t *values, uint32_t n, denox_hip_instance **out);
void denox_hip_instance_destroy(denox_hip_instance *inst);
int denox_hip_instance_input_count(const denox_hip_instance *inst, uint32_t *out);
int denox_hip_instance_output_count(const denox_hip_instance *inst, uint32_t *out);
int denox_hip_instance_input_desc(const denox_hip_instance *inst, uint32_t i, denox_hip_tensor_desc *out);
int denox_hip_instance_output_desc(const denox_hip_instance *inst, uint32_t i, denox_hip_tensor_desc *out);
/* blocking; host arrays in model input / output order */
int denox_hip_instance_infer(denox_hip_instance *inst, const void *const *host_inputs, void *const *host_outputs);
/* `frames` consecutive frames, blocking; host arrays frame-major: host_inputs[f * input_count + i].  The upload of the next
 * frame, the dispatches of the current one and the download of the previous one overlap on three streams (the interface
 * tensors exist twice on the device).  The copies overlap only from / to pinned host memory (denox_hip_host_alloc); pageable
 * memory gives the same result at the speed of denox_hip_instance_infer.  No counterpart in the reference, whose
 * Instance::infer is one blocking frame (runtime/src/denox/runtime/instance.cpp:322-430): for callers that stream
 * frames from host memory. */
int denox_hip_instance_infer_many(denox_hip_instance *inst, uint32_t frames, const void *const *host_inputs, void *const *host_outputs);
/* page-locked host memory for denox_hip_instance_infer_many / _infer (hipHostMalloc); release with denox_hip_host_free */
int denox_hip_host_alloc(size_t bytes, void **out);
void denox_hip_host_free(void *p);
/* asynchronous on the context's stream; device arrays, entries (or the arrays
 * themselves) may be NULL to use the instance's own tensors.  The dispatch list is captured into a graph once per set of
 * interface addresses and the graphs of the last four sets are kept: a caller that rotates through more than four sets of
 * buffers pays a stream synchronisation and a new capture per call (keep to four, or copy into fixed buffers). */
int denox_hip_instance_infer_device(denox_hip_instance *inst, const void *const *dev_inputs, void *const *dev_outputs);
/* denox_hip_instance_infer_device for callers that cannot allocate (serving loops and harnesses that forbid hipMalloc and
 * its relatives once they are running): same arguments, same results bit for bit, and no allocation of any kind on the
 * device or through the runtime -- plain kernel launches on the context's stream (no graph is captured or instantiated;
 * the launches go to the context's own stream, so a caller that is capturing a stream of its own does not capture them),
 * with the instance's intermediate tensors kept in a static device array that the library holds on every GPU it runs on
 * (DENOX_HIP_STATIC_SCRATCH_BYTES of device memory per GPU and process from the moment the library is loaded there,
 * used or not, and not counted in denox_hip_instance_device_bytes; its address is resolved when the context is created).
 * It has no counterpart in the reference, whose Instance allocates every buffer it uses
 * (runtime/src/denox/runtime/instance.cpp:65-113).
 * Returns DENOX_HIP_UNSUPPORTED, with the size needed in the error text, when the instance's intermediate tensors need more
 * than that.  All instances on one GPU share the array and each call overwrites it; nothing in it survives from one call to
 * the next.  Calls through one context are ordered by its stream.  Calls through different contexts of one GPU are not:
 * while an earlier call through another context has not finished, the call is refused with DENOX_HIP_INVALID_ARGUMENT
 * (synchronize the other context first) rather than run into that call's tensors. */
#define DENOX_HIP_STATIC_SCRATCH_BYTES (64ull << 20)
int denox_hip_instance_infer_device_static(denox_hip_instance *inst, const void *const *dev_inputs, void *const *dev_outputs);
int denox_hip_instance_synchronize(denox_hip_instance *inst);
int denox_hip_instance_input_device_ptr(const denox_hip_instance *inst, uint32_t i, void **out);
int denox_hip_instance_output_device_ptr(const denox_hip_instance *inst, uint32_t i, void **out);
/* per-dispatch timings after `warmup` untimed passes; writes min(count, capacity) entries */
int denox_hip_instance_bench(denox_hip_instance *inst, uint32_t warmup, denox_hip_timing *out, uint32_t capacity, uint32_t *out_count);
/* Dispatch `dispatch` (an index into the timings above) timed inside `frames` whole inferences, after `warmup` untimed ones:
 * hipEvents in front of and behind that dispatch only, so that it runs with the caches, clocks and memory traffic of the
 * frame around it.  No counterpart in the reference, whose Instance::bench (runtime/src/denox/runtime/instance.cpp) times
 * every dispatch of a pass with timestamp queries; here that per-dispatch pass repeats each kernel back to back. */
int denox_hip_instance_bench_in_frame(denox_hip_instance *inst, uint32_t dispatch, uint32_t frames, uint32_t warmup, float *out_ms);
int denox_hip_instance_device_bytes(const denox_hip_instance *inst, uint64_t *out);

#ifdef __cplusplus
}
#endif
#endif /* DENOX_HIP_H */
