/* C ABI of libmononn_hip.so: a fused XLA HLO module (text) in, one monolithic gfx950 kernel out.
 *
 * Each entry point names the reference interface it stands in for (paths relative to the
 * reference checkout).  The reference exposes C++ classes to its TensorFlow fork and aborts the
 * process on error; this boundary uses opaque handles, plain pointers and sizes, integer return
 * codes (0 = success) and a thread-local error string.  A handle may be used from one thread at a
 * time; different handles are independent.
 */
#ifndef MONONN_HIP_H_
#define MONONN_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mononn_module mononn_module;

enum mononn_status {
  MONONN_OK = 0,
  MONONN_INVALID_ARGUMENT = 1,
  MONONN_PARSE_ERROR = 2,      /* malformed HLO / JSON text */
  MONONN_UNSUPPORTED = 3,      /* construct outside the accepted HLO dialect */
  MONONN_SPEC_ERROR = 4,       /* tuning specification does not fit the graph or the device */
  MONONN_COMPILE_ERROR = 5,    /* hipRTC rejected the generated source (log in the message) */
  MONONN_RUNTIME_ERROR = 6,    /* HIP runtime failure, no usable GPU */
  MONONN_RESOURCE_EXHAUSTED = 7, /* grid larger than co-resident capacity, LDS over budget */
  MONONN_NOT_FOUND = 8,
  MONONN_INTERNAL = 9
};

/* Message of the last failing call on this thread ("" when none). */
const char* mononn_last_error(void);
const char* mononn_version(void);

/* Compile from an existing tuning specification.
 * Replaces: MonoNNModule(hlo, spec, kernel_name, ...) + generate_code() + build_assembly()
 *           (mononn_engine/module/mononn_module.h:31-59, mononn_module.cc:39-193) and the worker
 *           path of CompilationThreadpool::post (mononn_engine/codegen/compilation_threadpool.cc:41-117).
 * spec_json may be NULL: a default specification is derived (tuning_space_generator.cc:312-403).
 * kernel_name may be NULL: "mononn_cluster_<id>" from the module name (README.md:186).
 * build != 0 also runs hipRTC; build == 0 stops after code generation (no GPU or compiler needed). */
int mononn_compile(const char* hlo_text, size_t hlo_len, const char* spec_json, const char* kernel_name,
                   int build, mononn_module** out);

/* Search the tuning space on `device` and return the best module.
 * Replaces: MonoNNModuleTuner::tune(const Params&) (mononn_engine/module/mononn_module_tuner.h:27-37,
 *           mononn_module_tuner.cc:620-991).  Honours TF_MONONN_DUMP_DIR (dump tree written when set or
 *           when dump_dir != NULL) and TF_MONONN_THREADPOOL_SIZE.  budget: 0 = full, 1 = faster,
 *           2 = fastest (Config::faster_tuning / fastest_tuning, mononn_engine/config/config.h:22-47). */
int mononn_tune(const char* hlo_text, size_t hlo_len, int device, const char* dump_dir, int budget,
                mononn_module** out);

/* Load what a previous tuning run dumped: <spec_dir>/<cluster_N>/best_tuning_spec.json and, unless
 * TF_MONONN_NO_USE_PTX_CACHE is true, the cached best_tuning_spec.hsaco next to it.
 * Replaces: the TF_MONONN_EXISTING_TUNING_SPEC_DIR path of the reference's TensorFlow fork
 *           (README.md:145-149, EnvVars.md:7,14).  spec_dir NULL = read that environment variable. */
int mononn_compile_from_spec_dir(const char* hlo_text, size_t hlo_len, const char* spec_dir, mononn_module** out);

void mononn_module_destroy(mononn_module* m);

/* Replaces: kernel name / get_tuning_spec() / get_cuda_program() / get_ptx()+get_cubin()
 *           (mononn_engine/module/mononn_module.h:60-74).  Returned memory belongs to the handle
 *           and stays valid until the next call that regenerates it or until destroy. */
const char* mononn_module_kernel_name(const mononn_module* m);
int mononn_module_spec_json(mononn_module* m, const char** text, size_t* len);
int mononn_module_source(const mononn_module* m, const char* file /* "main.hip" | "headers.h" */,
                         const char** text, size_t* len);
int mononn_module_code_object(const mononn_module* m, const void** data, size_t* len);
int mononn_module_summary(mononn_module* m, const char** text, size_t* len);

/* Replaces: the buffer summary the reference logs (README.md:189-196): parameter bytes in
 *           parameter order, live-out bytes in root-tuple order, temp bytes.  Pass NULL to skip. */
int mononn_module_buffer_info(const mononn_module* m, int* n_params, const int64_t** param_bytes,
                              int* n_liveouts, const int64_t** liveout_bytes, int64_t* temp_bytes);
/* grid / block / dynamic LDS of the launch (best_tuning_spec.json keys grid_dim, block_dim, smem_size;
 * README.md:199-200) and the number of grid-wide barriers in the kernel. */
/* Whether the module brings its own temp arena (the caller would then pass NULL in the temp slot of
 * mononn_launch).  Always 0 today: the caller brings the temp buffer, as in the reference's contract
 * (temp_buffer argument, mononn_engine/module/mononn_module.cc:91-143). */
int mononn_module_owns_temp(const mononn_module* m);
int mononn_module_launch_dims(const mononn_module* m, int* grid, int* block, int* smem, int* barriers);
/* How many of those barriers belong to the regional tier: barriers over the workgroups of one XCD, through its L2
 * ("mononn_hip": {"regional_synchronization": true}); the others go through the memory side and order the whole grid.
 * Replaces: the split the reference makes between global and regional synchronisation
 *           (mononn_engine/optimization/regional_synchronization_assignment_pass.cc:35-72). */
int mononn_module_regional_barriers(const mononn_module* m, int* regional);

/* Non-scalar constants of the module ("buffer_for_<node>" globals that the host fills before
 * launch: mononn_engine/codegen/graph_codegen.cc:71-86, :448-459).  needs_payload is 1 for a constant the
 * HLO text elides ("{...}") and the caller has to set, 0 for one whose literal is in the text and for one the
 * module builds itself from other constants' payloads (the column sums of a folded LayerNorm); the latter
 * cannot be set (MONONN_INVALID_ARGUMENT). */
int mononn_module_num_constants(const mononn_module* m);
int mononn_module_constant_info(const mononn_module* m, int index, const char** hlo_name, const char** role,
                                int64_t* bytes, int* needs_payload);
int mononn_module_set_constant(mononn_module* m, const char* name, const void* host_data, size_t bytes);

/* Load the code object on a GPU, size-check the grid against the co-resident capacity and upload
 * the constants given so far.  Replaces: xla::gpu::CreateKernel + FuncSetAttribute of profile_kernel
 * (mononn_engine/module/mononn_module_tuner.cc:99-131). */
int mononn_module_load(mononn_module* m, int device);

/* One forward pass = one launch of the persistent kernel.  device_ptrs: entry parameters in parameter order, then
 * live-out buffers, then the temp buffer (argument order of mononn_engine/module/mononn_module.cc:91-143).
 * The launch is an ordinary one, as in the reference; the grid was checked against the co-resident capacity at
 * load time.  Launches of such kernels must not overlap on one device (two partly resident grids would wait for
 * each other at their first grid barrier): use one stream, or build with "mononn_hip": {"cooperative_launch": true}
 * in the specification, which lets the runtime keep them apart.
 * The outputs of a launch are known to be valid once mononn_module_synchronize has returned MONONN_OK for it: a
 * caller that waits for the stream by other means (hipStreamSynchronize, an event, a framework's own stream
 * order) does not see a barrier wait that gave up, and the error word stays set until that call reads and clears it.
 * Replaces: Launch(...) of profile_kernel (mononn_module_tuner.cc:135-139); the call is asynchronous
 *           on `stream` (a hipStream_t, NULL = default stream). */
int mononn_launch(mononn_module* m, void* const* device_ptrs, size_t n_ptrs, void* stream);

/* mononn_launch for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): the temp arena is a fixed array of mononn_static_temp_bytes() bytes (64 MiB) in
 * the library's own device image instead of a buffer of the caller, and the call allocates nothing.  device_ptrs:
 * entry parameters in parameter order, then live-out buffers -- no temp slot.  A module whose temp arena is larger
 * is refused with MONONN_RESOURCE_EXHAUSTED.  Each GPU holds one such array from the first mononn_module_load on it
 * until the process ends (64 MiB of device memory per GPU for every process that loads a module, whether it uses
 * this entry point or not); every call on a GPU, from any module, shares it, so calls that overlap on one GPU race.
 * Nothing in the arena has to start at zero: every temp address is written before it is read in the same launch.
 * No counterpart in the reference. */
int mononn_launch_static_temp(mononn_module* m, void* const* device_ptrs, size_t n_ptrs, void* stream);
size_t mononn_static_temp_bytes(void);

/* Wait for `stream` and report what the kernel could not: MONONN_RUNTIME_ERROR when a grid-barrier wait of a launch
 * gave up (the grid was not resident as a whole within mononn_hip.barrier_timeout_ms of the specification, e.g. an
 * ordinary launch beside another kernel).  Every workgroup of such a launch still runs to its end, so the kernel
 * terminates; its outputs are invalid.  The barrier state is reset and the module stays usable.
 * Replaces: BlockHostUntilDone of profile_kernel (mononn_engine/module/mononn_module_tuner.cc:140-149), where a
 *           failed wait is LOG(FATAL). */
int mononn_module_synchronize(mononn_module* m, void* stream);

/* Device address and size of a module global of the loaded code object: "buffer_for_<node>" (constants,
 * mononn_engine/codegen/graph_codegen.cc:71-86), "mononn_barrier_flags", "mononn_barrier_error".
 * Replaces: the cuModuleGetGlobal lookup a host would do on the reference's PTX (README.md:179-200). */
int mononn_module_global(const mononn_module* m, const char* symbol, void** device_ptr, size_t* bytes);

/* Time `iters` launches after `warmup` with HIP events on `stream`; avg_ms receives the mean,
 * each_ms (may be NULL, else iters floats) the individual launches.  One launch checked like
 * mononn_module_synchronize comes first: a kernel whose grid-barrier waits give up is an error here, not a time.
 * Replaces: the CUPTI gpu__time_duration range of profile_in_batch
 *           (mononn_engine/module/mononn_module_tuner.cc:250-372, tuning/profiler/cupti_profiling_session.h:20-78). */
int mononn_time_kernel(mononn_module* m, void* const* device_ptrs, size_t n_ptrs, void* stream, int warmup,
                       int iters, float* avg_ms, float* each_ms);

/* Per-stage wall-clock stamps of the last launch, for kernels compiled from a specification with
 * mononn_hip.profile_stages = true: ticks[(stage * grid + workgroup) * 2 + {0: stage begin, 1: work done}].
 * "stage begin" is stamped when the workgroup's first unit of the stage may start (after its barrier wait, behind
 * which requests for constant operands may already be in flight); a workgroup without a unit in a stage leaves both
 * values at zero.  Copies at most `capacity` values; n_stages / grid / ticks_per_us describe the layout.  Stage names
 * (node names joined by '+') come from mononn_module_stage_name.
 * Replaces: the per-node report of dump_performance_report (mononn_engine/module/mononn_module_tuner.cc:422-448). */
int mononn_module_stage_clock(mononn_module* m, uint64_t* ticks, size_t capacity, int* n_stages, int* grid,
                              double* ticks_per_us);
const char* mononn_module_stage_name(mononn_module* m, int stage);

/* Write <dump_dir>/<cluster_N>/{<ctx>.json,<ctx>.hsaco,<ctx>_src/...,best_tuning_spec.{json,hsaco}}.
 * Replaces: the dump half of final_tuning (mononn_engine/module/mononn_module_tuner.cc:457-603). */
int mononn_module_dump(mononn_module* m, const char* dump_dir);

/* Device query used for the default launch shape.
 * Replaces: CUDADeviceContext::get_cuda_device_context (mononn_engine/core/context/cuda_device_context.cc:42-80). */
int mononn_device_count(void);
int mononn_device_info(int device, int* compute_units, int* wave_size, int* max_lds_per_block, char* arch,
                       size_t arch_len);

#ifdef __cplusplus
}
#endif
#endif /* MONONN_HIP_H_ */
