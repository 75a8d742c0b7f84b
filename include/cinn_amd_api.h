/*
 * C API of the front end (NetBuilder, CinnComputation) for language bindings.
 *
 * It stands where the reference has its pybind11 layer (cinn/pybind/frontend.cc:157-232, 716-761 and
 * cinn/pybind/framework.cc:146-172): a binding creates a NetBuilder, appends instructions by
 * operator name, compiles for the AMDGPU target and moves tensor data.  All functions return 0 on
 * success; on failure they return non-zero and cinn_amd_last_error() describes the problem (the
 * message belongs to the calling thread and stays valid until its next API call).
 */
#ifndef CINN_AMD_API_H_
#define CINN_AMD_API_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct cinn_amd_builder* cinn_amd_builder_t;
typedef struct cinn_amd_computation* cinn_amd_computation_t;

const char* cinn_amd_last_error(void);

/* ---- NetBuilder (cinn/frontend/net_builder.h) ---- */
int cinn_amd_builder_create(const char* name, cinn_amd_builder_t* out);
int cinn_amd_builder_destroy(cinn_amd_builder_t b);
/* NetBuilder::CreateInput; dtype is "float32", "float16", "bfloat16", "int32", ... ; the variable id is
 * written to id_out (at most id_cap bytes including the terminator). */
int cinn_amd_builder_create_input(cinn_amd_builder_t b, const char* dtype, const int32_t* shape, int32_t rank,
                                  const char* name_hint, char* id_out, size_t id_cap);
/* A NetBuilder method by its C++ name ("Add", "Softmax", "ReduceSum", "Matmul", "Conv2d", ...) or a raw
 * operator through "CustomInstr:<op_type>".  inputs: variable ids.  attrs: "key:tag=value;..." with tags
 * b i f d s vi vf vs.  The ids of the results are written to ids_out separated by ','. */
int cinn_amd_builder_call(cinn_amd_builder_t b, const char* method, const char* const* inputs, int32_t num_inputs,
                          const char* attrs, char* ids_out, size_t ids_cap);
/* shape / dtype of a variable known to the builder; rank_out receives the rank, shape_out up to 8 dims */
int cinn_amd_builder_var_info(cinn_amd_builder_t b, const char* id, int32_t* shape_out, int32_t* rank_out,
                              char* dtype_out, size_t dtype_cap);
/* Variable::set_const (cinn/frontend/syntax.h:81-87): marks an input whose data does not change between executions
 * (weights).  Operators fed by const values only run once, ahead of the first execution. */
int cinn_amd_builder_set_const(cinn_amd_builder_t b, const char* id, int32_t is_const);
int cinn_amd_builder_size(cinn_amd_builder_t b, int32_t* num_instructions);
/* textual listing of the program built so far */
int cinn_amd_builder_program_string(cinn_amd_builder_t b, char* out, size_t cap, size_t* needed);

/* ---- CinnComputation (cinn/frontend/computation.h) ---- */
/* CinnComputation::BuildAndCompile for the AMDGPU target.  outputs: ids to fetch (NULL/0: outputs of the
 * last instruction).  stream: hipStream_t or NULL.  options: "key=value;..." (keys: do_prerun,
 * fuse_conv_bn_relu, fuse_stem_pool, fuse_matmul_bias, fuse_conv_chain, fuse_shortcut_projection, conv_layout_nhwc, split_reductions,
 * merge_independent_kernels, memory_arena, reuse_intermediates, and the lowering knobs
 * reduce_cached_elems, reduce_wave_elems, elementwise_block, reduce_rows_per_block).
 * Memory: with memory_arena=1 (default) every tensor the program's instructions touch is a slice of ONE device
 * allocation (the reference allocates per tensor, cinn/hlir/framework/memory.cc:43-53, tensor.h:64-82), and with
 * reuse_intermediates=1 (default) values that are neither fed, fetched (named in `outputs`) nor const share bytes when
 * their lifetimes do not overlap; set_tensor / get_tensor on such a value fail with a message that says so. */
int cinn_amd_computation_build_and_compile(cinn_amd_builder_t b, const char* const* outputs, int32_t num_outputs,
                                           void* stream, const char* options, cinn_amd_computation_t* out);
int cinn_amd_computation_destroy(cinn_amd_computation_t c);
int cinn_amd_computation_execute(cinn_amd_computation_t c);
int cinn_amd_computation_execute_graph(cinn_amd_computation_t c);
/* Program::PreRun (cinn/hlir/framework/graph_compiler.cc:78-87): runs the pre-run instructions.  The first
 * execute does it by itself; call it again after replacing the data of a const input. */
int cinn_amd_computation_pre_run(cinn_amd_computation_t c);
/* size of the program's device allocation (0 when memory_arena=0) and the sum of its tensors' sizes without sharing */
int cinn_amd_computation_memory_info(cinn_amd_computation_t c, size_t* arena_bytes, size_t* unshared_bytes);
int cinn_amd_computation_num_instructions(cinn_amd_computation_t c, int32_t* n);
/* Stream lane of every run instruction in a graph replay (0: the computation's stream, 1: the side stream that holds
 * instructions independent of their predecessor); writes min(capacity, *count) entries. */
int cinn_amd_computation_graph_lanes(cinn_amd_computation_t c, int32_t* lanes, int32_t capacity, int32_t* count);
/* SetTensorData / GetTensorData: synchronous host <-> device copies of exactly the tensor's byte size */
int cinn_amd_computation_set_tensor(cinn_amd_computation_t c, const char* name, const void* data, size_t bytes);
int cinn_amd_computation_get_tensor(cinn_amd_computation_t c, const char* name, void* data, size_t bytes);
int cinn_amd_computation_tensor_info(cinn_amd_computation_t c, const char* name, int32_t* shape_out,
                                     int32_t* rank_out, char* dtype_out, size_t dtype_cap, void** device_ptr);
/* names separated by ','; which: 0 = inputs, 1 = outputs, 2 = all */
int cinn_amd_computation_tensor_names(cinn_amd_computation_t c, int32_t which, char* out, size_t cap, size_t* needed);
/* generated HIP source of the device module / description of the fusion groups */
int cinn_amd_computation_source_code(cinn_amd_computation_t c, char* out, size_t cap, size_t* needed);
int cinn_amd_computation_group_string(cinn_amd_computation_t c, char* out, size_t cap, size_t* needed);
/* i-th instruction: its function name and its argument names (inputs then outputs, ',' separated) */
int cinn_amd_computation_instruction_info(cinn_amd_computation_t c, int32_t index, char* fn_name, size_t fn_cap,
                                          char* args, size_t args_cap);
/* run only the i-th instruction on the computation's stream (no synchronisation) */
int cinn_amd_computation_run_instruction(cinn_amd_computation_t c, int32_t index);

/* names of all registered operators, ',' separated */
int cinn_amd_list_operators(char* out, size_t cap, size_t* needed);

/* Host stubs of single runtime-intrinsic calls, built the way a compiled program's library-call instructions are
 * (the registered extern-function prototypes of cinn/runtime/cuda/cuda_intrinsics.cc:404-733 and the host function
 * CodeGenCUDA_Host::LowerGPUKernelLauncher makes of such a call, cinn/backends/codegen_cuda_host.cc:35-168).
 * cinn_amd_extern_api_names lists the intrinsics a host function may call, ',' separated.
 * cinn_amd_host_stub_create builds the stub of `api(kernel_args, kernel_args_num, <constants>, kernel_stream)`;
 * `constants` is a ','-separated list of `i:<int>`, `f:<float>` and `b:<0|1>` items in call order.  *fn is a
 * `void (*)(void* pod_args, int32_t num_args, void* stream)` (lower_func_ptr_g) to be released with
 * cinn_amd_host_stub_release. */
int cinn_amd_extern_api_names(char* out, size_t cap, size_t* needed);
int cinn_amd_host_stub_create(const char* api, const char* constants, void** fn);
int cinn_amd_host_stub_release(void* fn);

#ifdef __cplusplus
}
#endif
#endif /* CINN_AMD_API_H_ */
