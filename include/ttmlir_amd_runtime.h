/*
 * ttmlir_amd_runtime.h -- C ABI over the C++ host runtime (libttmlir_amd_rt.so).
 *
 * The C++ API in tt-mlir_amd/runtime/runtime.h mirrors tt::runtime (tt-mlir
 * runtime/include/tt/runtime/runtime.h:31-308).  This header exposes the same calls with opaque
 * handles so that any language with a C FFI can load a `.ttnn` flatbuffer, convert inputs to the
 * program's layouts, submit and read results -- the role the nanobind module plays in the reference
 * (runtime/python/runtime/runtime.cpp:29-847).  Each function names the tt::runtime call it wraps.
 *
 * Every function returns 0 on success and 1 on failure; ttrt_last_error() holds the message of the
 * C++ exception (the reference throws std::runtime_error from LOG_FATAL).  Handles are owned by
 * the caller and released with the matching *_free / *_destroy.
 */
#ifndef TTMLIR_AMD_RUNTIME_H
#define TTMLIR_AMD_RUNTIME_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ttrt_binary ttrt_binary;
typedef struct ttrt_device ttrt_device;
typedef struct ttrt_tensor ttrt_tensor;
typedef struct ttrt_builder ttrt_builder;

/* (storage, layout, dtype) with the enum values of the flatbuffer schema
 * (StorageType: Host 0, Device 1; TensorLayout: RowMajor 0, Tile 1; DataType as in Common/types.fbs) */
typedef struct ttrt_layout {
  int storage, layout, dtype;
} ttrt_layout;

const char *ttrt_last_error(void);

/* ---- Binary: Flatbuffer::loadFromPath / loadFromMemory, getProgramInputs/Outputs (runtime/lib/binary.cpp:164-188, 422-440) */
int ttrt_binary_load_file(const char *path, ttrt_binary **out);
int ttrt_binary_load_memory(const void *data, size_t size, ttrt_binary **out);
int ttrt_binary_store(const ttrt_binary *bin, const char *path);
void ttrt_binary_free(ttrt_binary *bin);
int ttrt_binary_num_programs(const ttrt_binary *bin, uint32_t *n);
int ttrt_binary_program_name(const ttrt_binary *bin, uint32_t program, char *buf, size_t len);
int ttrt_binary_program_is_private(const ttrt_binary *bin, uint32_t program, int *is_private);
int ttrt_binary_num_inputs(const ttrt_binary *bin, uint32_t program, uint32_t *n);
int ttrt_binary_num_outputs(const ttrt_binary *bin, uint32_t program, uint32_t *n);
/* is_output 0: input `index`, 1: output `index`.  shape receives up to 8 extents. */
int ttrt_binary_tensor_desc(const ttrt_binary *bin, uint32_t program, int is_output, uint32_t index, uint32_t *shape,
                            int *rank, ttrt_layout *layout);
int ttrt_binary_ops_text(const ttrt_binary *bin, uint32_t program, char *buf, size_t len);
int ttrt_binary_info(const ttrt_binary *bin, char *identifier5, char *version, size_t version_len);
/* JSON views of one program: which = 0 inputs, 1 outputs, 2 operations (Binary::getProgram{Inputs,Outputs,Ops}AsJson,
 * runtime/lib/binary.cpp:197-224).  Returns the length needed (without the terminator) in *needed; buf may be NULL. */
int ttrt_binary_program_json(const ttrt_binary *bin, uint32_t program, int which, char *buf, size_t len, size_t *needed);
/* Embedded golden tensor of the operation at location `loc` on device 0 (Binary::getDebugInfoGolden, binary.cpp:233-253):
 * *found = 0 when there is none.  shape receives up to 8 extents; *data points into the binary. */
int ttrt_binary_golden(const ttrt_binary *bin, const char *loc, int *found, int64_t *shape, int *rank, int *dtype,
                       const uint8_t **data, size_t *size, char *name, size_t name_len);

/* ---- Device: getNumAvailableDevices / openMeshDevice / closeMeshDevice (runtime.h:151-157) */
int ttrt_num_devices(uint32_t *n);
int ttrt_device_open(ttrt_device **out);
int ttrt_device_close(ttrt_device *dev);
int ttrt_device_name(ttrt_device *dev, char *buf, size_t len);

/* ---- Tensors: createOwnedHostTensor / createBorrowedHostTensor (runtime.h:56-69); stride may be NULL
 * (contiguous) and counts elements */
int ttrt_tensor_create_host(const void *data, const uint32_t *shape, int rank, const int64_t *stride, uint32_t itemsize,
                            int dtype, int borrowed, ttrt_tensor **out);
/* createUnsafeBorrowedHostTensor (runtime.h:70-76): a borrowed tensor over the buffer of an owned row-major host tensor,
 * no copy; it must not be used after the owner's buffer is gone */
int ttrt_tensor_create_unsafe_borrowed(const ttrt_tensor *owned, ttrt_tensor **out);
/* address of a host tensor's buffer (NULL once deallocated); what the reference's tests read through getRawHostDataPtr */
int ttrt_tensor_host_data(const ttrt_tensor *t, void **data);
void ttrt_tensor_free(ttrt_tensor *t);
int ttrt_tensor_desc(const ttrt_tensor *t, uint32_t *shape, int *rank, ttrt_layout *layout, uint64_t *bytes);
int ttrt_tensor_is_allocated(const ttrt_tensor *t, int *allocated);
int ttrt_tensor_set_retain(ttrt_tensor *t, int retain);
int ttrt_tensor_get_retain(const ttrt_tensor *t, int *retain);
int ttrt_tensor_deallocate(ttrt_tensor *t, int force);                         /* deallocateTensor (runtime.h:244) */
/* createEmptyTensor (runtime.h:107-110): uninitialised tensor in the given layout; dev may be NULL for host storage */
int ttrt_tensor_create_empty(ttrt_device *dev, const ttrt_layout *layout, const uint32_t *shape, int rank, ttrt_tensor **out);
/* hasLayout (runtime.h:230); getTensorLayout (232) is the layout ttrt_tensor_desc reports */
int ttrt_tensor_has_layout(const ttrt_tensor *t, const ttrt_layout *layout, int *has);
/* getTensorVolume / getTensorLogicalVolume / getTensorElementSize / getTensorStride (runtime.h:142-146): elements in
 * storage (the tile layout's padding included), product of the shape, bytes per element (1 for block-float types) and the
 * contiguous stride in elements; stride receives up to 8 entries, any pointer may be NULL */
int ttrt_tensor_extent(const ttrt_tensor *t, uint32_t *volume, uint32_t *logical_volume, uint32_t *element_size, int64_t *stride);
/* dumpTensor / loadTensor (runtime.h:304-308): the file keeps the tensor's own layout (tile order, block-float bytes);
 * a device tensor is read back first.  load: dev NULL gives a host tensor, else the tensor is moved to that device. */
int ttrt_tensor_dump(const ttrt_tensor *t, const char *path);
int ttrt_tensor_load(const char *path, ttrt_device *dev, ttrt_tensor **out);

/* getLayout (runtime.h:234-235), toLayout (227-228; retain: -1 unset, 0, 1), toHost (221-222), wait (212-217),
 * memcpy(void*, Tensor, optional<DataType>) (237-238; target_dtype -1 = none), memcpy(Tensor, Tensor) (240) */
int ttrt_get_layout(const ttrt_binary *bin, uint32_t program, uint32_t input, ttrt_layout *layout);
int ttrt_to_layout(ttrt_tensor *t, ttrt_device *dev, const ttrt_layout *layout, int retain, ttrt_tensor **out);
int ttrt_to_host(ttrt_tensor *t, int untilize, ttrt_tensor **out);
int ttrt_wait(ttrt_tensor *t);
int ttrt_memcpy_out(void *dst, const ttrt_tensor *src, int target_dtype);
int ttrt_memcpy_tensor(ttrt_tensor *dst, const ttrt_tensor *src);

/* submit (runtime.h:299-301): outputs receives up to max_outputs new handles */
int ttrt_submit(ttrt_device *dev, const ttrt_binary *bin, uint32_t program, ttrt_tensor *const *inputs, uint32_t num_inputs,
                ttrt_tensor **outputs, uint32_t max_outputs, uint32_t *num_outputs);

/* ---- debug hooks (runtime/include/tt/runtime/debug.h:77-157): callbacks before / after every operation and before /
 * after every program (nested const-eval and func-call programs included).  hook_ctx is valid only inside the callback.
 * ttrt_hook_output: the op's first output as an untilized host tensor (NULL if none) - getOpOutputTensor, runtime.h:250.
 * ttrt_hook_input_refs / output_refs: global ids of the op's operands / results - getOpInputRefs / getOpOutputRefs,
 *   runtime.h:252-262; in a program callback both report nothing.
 * ttrt_hook_retrieve: host copy of any live tensor of the running program (NULL if not in the pool) -
 *   retrieveTensorFromPool, runtime.h:267-273.
 * ttrt_hook_update: overwrite the payload of a pool tensor from src, converting src to the pool tensor's layout -
 *   updateTensorInPool, runtime.h:275-283. */
typedef void (*ttrt_op_callback)(uint32_t op_index, const char *op_name, const char *debug_info, void *hook_ctx, void *user);
typedef void (*ttrt_program_callback)(uint32_t program_index, void *hook_ctx, void *user);
int ttrt_set_pre_op_callback(ttrt_op_callback cb, void *user);
int ttrt_set_post_op_callback(ttrt_op_callback cb, void *user);
int ttrt_set_program_callbacks(ttrt_program_callback pre, ttrt_program_callback post, void *user);
int ttrt_clear_callbacks(void);
int ttrt_hook_output(void *hook_ctx, ttrt_tensor **out);
int ttrt_hook_input_refs(void *hook_ctx, uint32_t *ids, uint32_t cap, uint32_t *count);
int ttrt_hook_output_refs(void *hook_ctx, uint32_t *ids, uint32_t cap, uint32_t *count);
int ttrt_hook_retrieve(void *hook_ctx, uint32_t global_id, int untilize, ttrt_tensor **out);
int ttrt_hook_update(void *hook_ctx, uint32_t global_id, const ttrt_tensor *src);
int ttrt_hook_program_index(void *hook_ctx, uint32_t *index);
/* location string of the operation a hook is running for (getOpLocInfo, runtime.h:248) */
int ttrt_hook_loc(void *hook_ctx, char *buf, size_t len);
/* shape and data type of one of the operation's operands or results, from the binary alone (TensorRef::get_shape /
 * get_dtype: getTensorRefShape, runtime.h:263, and getTensorRefDataType); fails if global_id is neither */
int ttrt_hook_ref_desc(void *hook_ctx, uint32_t global_id, uint32_t *shape, int *rank, int *dtype);
/* invokeCpuOp (runtime.h:285-292): the function behind the CpuOp the hook runs for, on caller-supplied host tensors that
 * match the op's declared inputs in number, shape and data type; outputs receives up to max_outputs new host tensors.
 * The function needs the program's embedded library, not its tensor pool: the call also works inside ttrt_walk_program. */
int ttrt_hook_invoke_cpu_op(void *hook_ctx, ttrt_tensor *const *inputs, uint32_t num_inputs, ttrt_tensor **outputs,
                            uint32_t max_outputs, uint32_t *num_outputs);
/* walkProgram (runtime.h:294-297): cb for every operation of the program in order; nothing runs and no device is needed.
 * Inside cb the hook context answers ttrt_hook_loc / input_refs / output_refs / ref_desc / invoke_cpu_op; there is no tensor pool, so
 * ttrt_hook_output and ttrt_hook_retrieve give NULL and ttrt_hook_update / ttrt_hook_program_index fail. */
int ttrt_walk_program(const ttrt_binary *bin, uint32_t program, ttrt_op_callback cb, void *user);
int ttrt_stat(const char *name, int64_t *value);
int ttrt_stats_clear(void);

/* ---- host dtype casts used for unsupported host dtypes (runtime/lib/common/utils.cpp:267-360) */
int ttrt_buffer_cast(const void *src, void *dst, int from_dtype, int to_dtype, int64_t n);

/* ---- program writer (no counterpart in the reference runtime: its binaries come from the compiler).
 * Tensor ids are the flatbuffer global_ids; 0 means "no tensor". */
int ttrt_pb_create(ttrt_builder **out);
void ttrt_pb_destroy(ttrt_builder *pb);
int ttrt_pb_begin_program(ttrt_builder *pb, const char *name, int is_private);
int ttrt_pb_end_program(ttrt_builder *pb, uint32_t *program_index);
int ttrt_pb_input(ttrt_builder *pb, const uint32_t *shape, int rank, const ttrt_layout *layout, uint32_t *id);
int ttrt_pb_output(ttrt_builder *pb, uint32_t id);
int ttrt_pb_finish(ttrt_builder *pb, uint8_t **data, size_t *size);              /* free with ttrt_free_bytes */
void ttrt_free_bytes(uint8_t *data);
int ttrt_pb_tensor_desc(ttrt_builder *pb, uint32_t id, uint32_t *shape, int *rank, ttrt_layout *layout);
int ttrt_pb_to_layout(ttrt_builder *pb, uint32_t in, int layout, int dtype, int storage, uint32_t *out);
int ttrt_pb_typecast(ttrt_builder *pb, uint32_t in, int dtype, uint32_t *out);
int ttrt_pb_to_device(ttrt_builder *pb, uint32_t in, uint32_t *out);
int ttrt_pb_from_device(ttrt_builder *pb, uint32_t in, uint32_t *out);
int ttrt_pb_matmul(ttrt_builder *pb, uint32_t a, uint32_t b, int transpose_a, int transpose_b, const char *activation,
                   int out_dtype, uint32_t *out);
int ttrt_pb_linear(ttrt_builder *pb, uint32_t a, uint32_t b, uint32_t bias, int transpose_a, int transpose_b,
                   const char *activation, int out_dtype, uint32_t *out);
int ttrt_pb_unary(ttrt_builder *pb, uint32_t type, uint32_t in, int has_param, float param, uint32_t *out);
int ttrt_pb_binary(ttrt_builder *pb, uint32_t type, uint32_t lhs, uint32_t rhs, uint32_t *out);
int ttrt_pb_rms_norm(ttrt_builder *pb, uint32_t in, uint32_t weight, uint32_t bias, float eps, uint32_t *out);
int ttrt_pb_softmax(ttrt_builder *pb, uint32_t in, int dim, uint32_t *out);
int ttrt_pb_reduction(ttrt_builder *pb, uint32_t type, uint32_t in, const int32_t *dims, int ndims, int keep_dim, uint32_t *out);
/* sliding_window < 0 = attribute absent; attention_sink 0 = operand absent (transformer.fbs:70-82) */
int ttrt_pb_sdpa(ttrt_builder *pb, uint32_t q, uint32_t k, uint32_t v, uint32_t mask, int is_causal, int has_scale, float scale,
                 int64_t sliding_window, uint32_t attention_sink, uint32_t *out);
/* decode path (include/ttmlir/Target/TTNN/operations/{transformer,kv_cache}.fbs); 0 = operand absent; a page table
 * selects PagedScaledDotProductAttentionDecodeOp */
int ttrt_pb_rotary_embedding(ttrt_builder *pb, uint32_t in, uint32_t cos_cache, uint32_t sin_cache, int has_token_index,
                             uint32_t token_index, uint32_t *out);
int ttrt_pb_update_cache(ttrt_builder *pb, uint32_t cache, uint32_t in, uint32_t update_index, uint32_t batch_offset);
int ttrt_pb_fill_cache(ttrt_builder *pb, uint32_t cache, uint32_t in, uint32_t batch_offset);
/* PagedUpdateCacheOp / PagedFillCacheOp (include/ttmlir/Target/TTNN/operations/kv_cache.fbs:19-32); page_table 0 = static
 * cache, batch_idx 0 = absent */
int ttrt_pb_paged_update_cache(ttrt_builder *pb, uint32_t cache, uint32_t in, uint32_t update_index, uint32_t page_table,
                               int share_cache);
int ttrt_pb_paged_fill_cache(ttrt_builder *pb, uint32_t cache, uint32_t in, uint32_t page_table, uint32_t batch_idx);
int ttrt_pb_sdpa_decode(ttrt_builder *pb, uint32_t q, uint32_t k, uint32_t v, uint32_t page_table, uint32_t mask, uint32_t cur_pos,
                        int is_causal, int has_scale, float scale, int64_t sliding_window, uint32_t attention_sink, uint32_t *out);
int ttrt_pb_reshape(ttrt_builder *pb, uint32_t in, const uint32_t *shape, int rank, uint32_t *out);
int ttrt_pb_permute(ttrt_builder *pb, uint32_t in, const int64_t *perm, int rank, uint32_t *out);
int ttrt_pb_transpose(ttrt_builder *pb, uint32_t in, int dim0, int dim1, uint32_t *out);
int ttrt_pb_concat(ttrt_builder *pb, const uint32_t *ins, int n, int dim, uint32_t *out);
int ttrt_pb_slice(ttrt_builder *pb, uint32_t in, const int64_t *begins, const int64_t *ends, const int64_t *steps, int rank,
                  uint32_t *out);
int ttrt_pb_repeat_interleave(ttrt_builder *pb, uint32_t in, uint32_t repeats, int dim, uint32_t *out);
/* RepeatOp, EltwiseBinaryCompositeOp (type = EltwiseBinaryCompositeOpType), EltwiseTernaryWhereOp, EmbeddingOp,
 * ReductionArgMaxOp (has_dim = 0: over the whole tensor), ArangeOp */
/* EltwiseUnaryCompositeOp (type = EltwiseUnaryCompositeOpType: Cbrt 0, ClampScalar 1 with bounds lo / hi written as FP or,
 * with int_bounds, as I32; Log1p 3) */
int ttrt_pb_unary_composite(ttrt_builder *pb, uint32_t type, uint32_t in, float lo, float hi, int int_bounds, uint32_t *out);
/* head merges (kind 0 ConcatenateHeadsOp, 1 NLPConcatHeadsOp, 2 NLPConcatHeadsDecodeOp with num_heads) and splits
 * (NLPCreateQKVHeadsDecodeOp, SplitQueryKeyValueAndSplitHeadsOp with kv_input 0 = fused input); the splits write the ids of
 * q, k, v to qkv_out[0..2] */
int ttrt_pb_concat_heads(ttrt_builder *pb, int kind, uint32_t in, uint32_t num_heads, uint32_t *out);
int ttrt_pb_nlp_create_qkv_heads_decode(ttrt_builder *pb, uint32_t in, uint32_t num_heads, uint32_t num_kv_heads, uint32_t *qkv_out);
int ttrt_pb_split_qkv_and_split_heads(ttrt_builder *pb, uint32_t in, uint32_t kv_input, uint32_t num_heads, uint32_t num_kv_heads,
                                      int transpose_key, uint32_t *qkv_out);
int ttrt_pb_repeat(ttrt_builder *pb, uint32_t in, const int64_t *repeats, int rank, uint32_t *out);
int ttrt_pb_binary_composite(ttrt_builder *pb, uint32_t type, uint32_t lhs, uint32_t rhs, uint32_t *out);
int ttrt_pb_where(ttrt_builder *pb, uint32_t cond, uint32_t a, uint32_t b, uint32_t *out);
int ttrt_pb_embedding(ttrt_builder *pb, uint32_t indices, uint32_t weight, uint32_t *out);
int ttrt_pb_argmax(ttrt_builder *pb, uint32_t in, int has_dim, int dim, int keep_dim, int out_dtype, uint32_t *out);
int ttrt_pb_arange(ttrt_builder *pb, float start, float end, float step, int dtype, int layout, uint32_t *out);
int ttrt_pb_constant(ttrt_builder *pb, const void *data, size_t bytes, int in_dtype, const uint32_t *shape, int rank,
                     const ttrt_layout *layout, uint32_t *out);
int ttrt_pb_full(ttrt_builder *pb, const uint32_t *shape, int rank, float value, int dtype, int layout, uint32_t *out);
int ttrt_pb_empty(ttrt_builder *pb, const uint32_t *shape, int rank, int dtype, int layout, uint32_t *out);
int ttrt_pb_copy(ttrt_builder *pb, uint32_t src, uint32_t dst);
int ttrt_pb_write_tensor(ttrt_builder *pb, uint32_t host, uint32_t device);
/* trace ops (include/ttmlir/Target/TTNN/operations/trace.fbs); the trace id is a rank-0 UInt32 host tensor */
int ttrt_pb_begin_trace_capture(ttrt_builder *pb, uint32_t *trace_id);
int ttrt_pb_end_trace_capture(ttrt_builder *pb, uint32_t trace_id);
int ttrt_pb_execute_trace(ttrt_builder *pb, uint32_t trace_id, int blocking);
int ttrt_pb_capture_or_execute_trace(ttrt_builder *pb, uint32_t capture_program, uint32_t execute_program,
                                     uint32_t allocate_slots_program, const uint32_t *ins, int n_in, const uint32_t *out_shapes,
                                     const int *out_ranks, const ttrt_layout *out_layouts, int n_out, uint32_t *outs);
int ttrt_pb_deallocate(ttrt_builder *pb, uint32_t in, int force);
/* location of the operation added last, and an expected (golden) tensor to embed for a location; data is row-major */
int ttrt_pb_last_op_loc(ttrt_builder *pb, char *buf, size_t len);
/* the next matmul / linear carries a matmul_program_config of this kind (value of the MatmulProgramConfig union,
 * include/ttmlir/Target/TTNN/operations/matmul.fbs:56-62; 0 = none) whose fused_activation is the UnaryOpType
 * `fused_activation`, absent when negative: runtime/lib/ttnn/operations/matmul/matmul.cpp:17-44 lets it replace the op's
 * own activation string */
int ttrt_pb_set_matmul_program_config(ttrt_builder *pb, int kind, int fused_activation);
/* the next tensor the builder creates is declared with this shape instead of the one its operation gives: a program that
 * lies about a result, for tests of what the executor does with one */
int ttrt_pb_declare_next_shape(ttrt_builder *pb, const uint32_t *shape, int rank);
int ttrt_pb_golden(ttrt_builder *pb, const char *loc, const char *name, const void *data, size_t bytes, const int64_t *shape,
                   int rank, int dtype);
/* out_shapes: n_out entries of 8 extents each, out_ranks / out_layouts per entry */
int ttrt_pb_load_cached(ttrt_builder *pb, uint32_t program_index, const char *callee, const uint32_t *ins, int n_in,
                        const uint32_t *out_shapes, const int *out_ranks, const ttrt_layout *out_layouts, int n_out,
                        uint32_t *outs);
int ttrt_pb_func_call(ttrt_builder *pb, uint32_t program_index, const uint32_t *ins, int n_in, const uint32_t *out_shapes,
                      const int *out_ranks, const ttrt_layout *out_layouts, int n_out, uint32_t *outs);
/* CpuOp (include/ttmlir/Target/TTNN/operations/cpu.fbs; runner runtime/lib/ttnn/operations/cpu/cpu.cpp:215-238): a call of
 * `func_name` in the dynamic library that ttrt_pb_add_dylib embedded in the open program under dylib_id
 * (Program.dylibs, include/ttmlir/Target/Common/types.fbs:157-160).  The function has the CPU-hoisting ABI of
 * runtime/include/tt/runtime/detail/common/dylib.h:35-42: WrappedTensor *f(WrappedTensor *inputs) on dense row-major host
 * tensors of 4-byte elements, outputs allocated with malloc by the callee and freed by the runtime. */
/* RotaryEmbeddingLlamaOp, ChunkedScaledDotProductAttentionOp (include/ttmlir/Target/TTNN/operations/transformer.fbs:13-22,
 * 150-160) */
int ttrt_pb_rotary_embedding_llama(ttrt_builder *pb, uint32_t in, uint32_t cos_cache, uint32_t sin_cache, uint32_t trans_mat,
                                   int decode_mode, uint32_t *out);
int ttrt_pb_chunked_sdpa(ttrt_builder *pb, uint32_t q, uint32_t k, uint32_t v, uint32_t page_table, uint32_t chunk_start,
                         int has_scale, float scale, uint32_t *out);
int ttrt_pb_add_dylib(ttrt_builder *pb, uint32_t dylib_id, const void *data, size_t size);
int ttrt_pb_cpu_op(ttrt_builder *pb, uint32_t dylib_id, const char *func_name, const uint32_t *ins, int n_in,
                   const uint32_t *out_shapes, const int *out_ranks, const ttrt_layout *out_layouts, int n_out, uint32_t *outs);

#ifdef __cplusplus
}
#endif
#endif
