// C ABI over the C++ runtime (include/ttmlir_amd_runtime.h): exception -> status translation and
// opaque handles.
#include <cstring>
#include <string>

#include "program_builder.h"
#include "runtime_impl.h"
#include "ttmlir_amd_runtime.h"

using namespace tt::runtime;
using ttmlir_amd::ProgramBuilder;

struct ttrt_binary { Binary b; };
struct ttrt_device { Device d; };
struct ttrt_tensor { Tensor t; };
struct ttrt_builder { ProgramBuilder pb; };

#define TTRT_EXPORT extern "C" __attribute__((visibility("default")))

static thread_local std::string g_err;

template <typename F>
static int guard(F &&f) {
  try {
    f();
    return 0;
  } catch (const std::exception &e) {
    g_err = e.what();
    return 1;
  } catch (...) {
    g_err = "unknown C++ exception";
    return 1;
  }
}
static void need(const void *p, const char *what) {
  if (!p) throw std::runtime_error(std::string("null argument: ") + what);
}
static Layout toLayoutStruct(const ttrt_layout &l) {
  return Layout{static_cast<StorageType>(l.storage), static_cast<TensorLayout>(l.layout), static_cast<DataType>(l.dtype)};
}
static ttrt_layout fromLayoutStruct(const Layout &l) {
  return ttrt_layout{static_cast<int>(l.storageType), static_cast<int>(l.layout), static_cast<int>(l.dataType)};
}
static void copyStr(const std::string &s, char *buf, size_t len) {
  if (!buf || !len) return;
  size_t n = std::min(len - 1, s.size());
  std::memcpy(buf, s.data(), n);
  buf[n] = 0;
}
static std::vector<std::uint32_t> shapeVec(const uint32_t *shape, int rank) {
  if (rank < 0 || rank > 8) throw std::runtime_error("rank must be 0..8");
  if (rank > 0) need(shape, "shape");
  return std::vector<std::uint32_t>(shape, shape + rank);
}
static void writeShape(const std::vector<std::uint32_t> &s, uint32_t *shape, int *rank) {
  if (s.size() > 8) throw std::runtime_error("tensor rank above 8");
  if (rank) *rank = static_cast<int>(s.size());
  if (shape) for (size_t i = 0; i < s.size(); ++i) shape[i] = s[i];
}

TTRT_EXPORT const char *ttrt_last_error(void) { return g_err.c_str(); }

// ---- binary
TTRT_EXPORT int ttrt_binary_load_file(const char *path, ttrt_binary **out) {
  return guard([&] { need(path, "path"); need(out, "out"); *out = new ttrt_binary{Binary::loadFromPath(path)}; });
}
TTRT_EXPORT int ttrt_binary_load_memory(const void *data, size_t size, ttrt_binary **out) {
  return guard([&] { need(out, "out"); *out = new ttrt_binary{Binary::loadFromMemory(data, size)}; });
}
TTRT_EXPORT int ttrt_binary_store(const ttrt_binary *bin, const char *path) {
  return guard([&] { need(bin, "binary"); need(path, "path"); bin->b.store(path); });
}
TTRT_EXPORT void ttrt_binary_free(ttrt_binary *bin) { delete bin; }
TTRT_EXPORT int ttrt_binary_num_programs(const ttrt_binary *bin, uint32_t *n) {
  return guard([&] { need(bin, "binary"); need(n, "n"); *n = bin->b.getNumPrograms(); });
}
TTRT_EXPORT int ttrt_binary_program_name(const ttrt_binary *bin, uint32_t program, char *buf, size_t len) {
  return guard([&] { need(bin, "binary"); copyStr(bin->b.getProgramName(program), buf, len); });
}
TTRT_EXPORT int ttrt_binary_program_is_private(const ttrt_binary *bin, uint32_t program, int *is_private) {
  return guard([&] { need(bin, "binary"); need(is_private, "is_private"); *is_private = bin->b.isProgramPrivate(program); });
}
TTRT_EXPORT int ttrt_binary_num_inputs(const ttrt_binary *bin, uint32_t program, uint32_t *n) {
  return guard([&] { need(bin, "binary"); need(n, "n"); *n = static_cast<uint32_t>(bin->b.getProgramInputs(program).size()); });
}
TTRT_EXPORT int ttrt_binary_num_outputs(const ttrt_binary *bin, uint32_t program, uint32_t *n) {
  return guard([&] { need(bin, "binary"); need(n, "n"); *n = static_cast<uint32_t>(bin->b.getProgramOutputs(program).size()); });
}
TTRT_EXPORT int ttrt_binary_tensor_desc(const ttrt_binary *bin, uint32_t program, int is_output, uint32_t index, uint32_t *shape,
                                        int *rank, ttrt_layout *layout) {
  return guard([&] {
    need(bin, "binary");
    auto v = is_output ? bin->b.getProgramOutputs(program) : bin->b.getProgramInputs(program);
    if (index >= v.size()) throw std::runtime_error("tensor index out of range");
    writeShape(v[index].shape, shape, rank);
    if (layout) *layout = fromLayoutStruct(v[index].layout);
  });
}
TTRT_EXPORT int ttrt_binary_ops_text(const ttrt_binary *bin, uint32_t program, char *buf, size_t len) {
  return guard([&] { need(bin, "binary"); copyStr(bin->b.getProgramOpsAsText(program), buf, len); });
}
TTRT_EXPORT int ttrt_binary_program_json(const ttrt_binary *bin, uint32_t program, int which, char *buf, size_t len, size_t *needed) {
  return guard([&] {
    need(bin, "binary");
    std::string j = which == 0 ? bin->b.getProgramInputsAsJson(program)
                  : which == 1 ? bin->b.getProgramOutputsAsJson(program)
                               : bin->b.getProgramOpsAsJson(program);
    if (needed) *needed = j.size();
    if (buf && len) copyStr(j, buf, len);
  });
}
TTRT_EXPORT int ttrt_binary_golden(const ttrt_binary *bin, const char *loc, int *found, int64_t *shape, int *rank, int *dtype,
                                   const uint8_t **data, size_t *size, char *name, size_t name_len) {
  return guard([&] {
    need(bin, "binary"); need(loc, "loc"); need(found, "found");
    auto m = bin->b.getDebugInfoGolden(loc);
    auto it = m.find(0);
    *found = it != m.end();
    if (!*found) return;
    const GoldenTensorInfo &g = it->second;
    if (g.shape.size() > 8) throw std::runtime_error("golden tensor rank above 8");
    if (rank) *rank = static_cast<int>(g.shape.size());
    if (shape) for (size_t i = 0; i < g.shape.size(); ++i) shape[i] = g.shape[i];
    if (dtype) *dtype = static_cast<int>(g.dataType);
    if (data) *data = g.data;
    if (size) *size = g.size;
    if (name && name_len) copyStr(g.name, name, name_len);
  });
}
TTRT_EXPORT int ttrt_binary_info(const ttrt_binary *bin, char *identifier5, char *version, size_t version_len) {
  return guard([&] {
    need(bin, "binary");
    copyStr(bin->b.getFileIdentifier(), identifier5, 5);
    copyStr(bin->b.getVersion(), version, version_len);
  });
}

// ---- device
TTRT_EXPORT int ttrt_num_devices(uint32_t *n) {
  return guard([&] { need(n, "n"); *n = static_cast<uint32_t>(getNumAvailableDevices()); });
}
TTRT_EXPORT int ttrt_device_open(ttrt_device **out) {
  return guard([&] { need(out, "out"); *out = new ttrt_device{openMeshDevice()}; });
}
TTRT_EXPORT int ttrt_device_close(ttrt_device *dev) {
  return guard([&] { need(dev, "device"); closeMeshDevice(dev->d); delete dev; });
}
TTRT_EXPORT int ttrt_device_name(ttrt_device *dev, char *buf, size_t len) {
  return guard([&] { need(dev, "device"); copyStr(getDeviceName(dev->d), buf, len); });
}

// ---- tensors
TTRT_EXPORT int ttrt_tensor_create_host(const void *data, const uint32_t *shape, int rank, const int64_t *stride, uint32_t itemsize,
                                        int dtype, int borrowed, ttrt_tensor **out) {
  return guard([&] {
    need(out, "out");
    auto s = shapeVec(shape, rank);
    std::vector<std::int64_t> st = stride ? std::vector<std::int64_t>(stride, stride + rank) : utils::calculateStride(s);
    DataType dt = static_cast<DataType>(dtype);
    Tensor t = borrowed ? createBorrowedHostTensor(const_cast<void *>(data), s, st, itemsize, dt) : createOwnedHostTensor(data, s, st, itemsize, dt);
    *out = new ttrt_tensor{t};
  });
}
TTRT_EXPORT int ttrt_tensor_create_unsafe_borrowed(const ttrt_tensor *owned, ttrt_tensor **out) {
  return guard([&] { need(owned, "tensor"); need(out, "out"); *out = new ttrt_tensor{createUnsafeBorrowedHostTensor(owned->t)}; });
}
TTRT_EXPORT int ttrt_tensor_host_data(const ttrt_tensor *t, void **data) {
  return guard([&] {
    need(t, "tensor"); need(data, "data");
    if (t->t.handle->storage != StorageType::Host) throw std::runtime_error("the tensor is not on the host");
    *data = t->t.handle->data.get();
  });
}
TTRT_EXPORT void ttrt_tensor_free(ttrt_tensor *t) { delete t; }
TTRT_EXPORT int ttrt_tensor_desc(const ttrt_tensor *t, uint32_t *shape, int *rank, ttrt_layout *layout, uint64_t *bytes) {
  return guard([&] {
    need(t, "tensor");
    writeShape(t->t.handle->shape, shape, rank);
    if (layout) *layout = fromLayoutStruct(getTensorLayout(t->t));
    if (bytes) *bytes = t->t.handle->bytes;
  });
}
TTRT_EXPORT int ttrt_tensor_is_allocated(const ttrt_tensor *t, int *allocated) {
  return guard([&] { need(t, "tensor"); need(allocated, "allocated"); *allocated = isTensorAllocated(t->t); });
}
TTRT_EXPORT int ttrt_tensor_set_retain(ttrt_tensor *t, int retain) {
  return guard([&] { need(t, "tensor"); setTensorRetain(t->t, retain != 0); });
}
TTRT_EXPORT int ttrt_tensor_get_retain(const ttrt_tensor *t, int *retain) {
  return guard([&] { need(t, "tensor"); need(retain, "retain"); *retain = getTensorRetain(t->t); });
}
TTRT_EXPORT int ttrt_tensor_deallocate(ttrt_tensor *t, int force) {
  return guard([&] { need(t, "tensor"); deallocateTensor(t->t, force != 0); });
}

TTRT_EXPORT int ttrt_tensor_create_empty(ttrt_device *dev, const ttrt_layout *layout, const uint32_t *shape, int rank, ttrt_tensor **out) {
  return guard([&] {
    need(layout, "layout"); need(out, "out");
    Layout l = toLayoutStruct(*layout);
    if (l.storageType == StorageType::Device) need(dev, "device");
    auto s = shapeVec(shape, rank);
    *out = new ttrt_tensor{createEmptyTensor(dev ? dev->d : Device{}, l, s, utils::calculateStride(s),
                                              utils::isBlockFormatDataType(l.dataType) ? 1 : utils::dataTypeElementSize(l.dataType))};
  });
}
TTRT_EXPORT int ttrt_tensor_has_layout(const ttrt_tensor *t, const ttrt_layout *layout, int *has) {
  return guard([&] { need(t, "tensor"); need(layout, "layout"); need(has, "has"); *has = hasLayout(t->t, toLayoutStruct(*layout)); });
}
TTRT_EXPORT int ttrt_tensor_extent(const ttrt_tensor *t, uint32_t *volume, uint32_t *logical_volume, uint32_t *element_size, int64_t *stride) {
  return guard([&] {
    need(t, "tensor");
    if (volume) *volume = getTensorVolume(t->t);
    if (logical_volume) *logical_volume = getTensorLogicalVolume(t->t);
    if (element_size) *element_size = getTensorElementSize(t->t);
    if (stride) {
      auto st = getTensorStride(t->t);
      if (st.size() > 8) throw std::runtime_error("tensor rank above 8");
      for (size_t i = 0; i < st.size(); ++i) stride[i] = st[i];
    }
  });
}
TTRT_EXPORT int ttrt_tensor_dump(const ttrt_tensor *t, const char *path) {
  return guard([&] { need(t, "tensor"); need(path, "path"); dumpTensor(t->t, path); });
}
TTRT_EXPORT int ttrt_tensor_load(const char *path, ttrt_device *dev, ttrt_tensor **out) {
  return guard([&] {
    need(path, "path"); need(out, "out");
    *out = new ttrt_tensor{loadTensor(path, dev ? std::optional<Device>(dev->d) : std::nullopt)};
  });
}

TTRT_EXPORT int ttrt_get_layout(const ttrt_binary *bin, uint32_t program, uint32_t input, ttrt_layout *layout) {
  return guard([&] { need(bin, "binary"); need(layout, "layout"); *layout = fromLayoutStruct(getLayout(bin->b, program, input)); });
}
TTRT_EXPORT int ttrt_to_layout(ttrt_tensor *t, ttrt_device *dev, const ttrt_layout *layout, int retain, ttrt_tensor **out) {
  return guard([&] {
    need(t, "tensor"); need(dev, "device"); need(layout, "layout"); need(out, "out");
    std::optional<bool> r = retain < 0 ? std::nullopt : std::optional<bool>(retain != 0);
    *out = new ttrt_tensor{toLayout(t->t, dev->d, toLayoutStruct(*layout), r)};
  });
}
TTRT_EXPORT int ttrt_to_host(ttrt_tensor *t, int untilize, ttrt_tensor **out) {
  return guard([&] { need(t, "tensor"); need(out, "out"); *out = new ttrt_tensor{toHost(t->t, untilize != 0, true).at(0)}; });
}
TTRT_EXPORT int ttrt_wait(ttrt_tensor *t) {
  return guard([&] { need(t, "tensor"); wait(t->t); });
}
TTRT_EXPORT int ttrt_memcpy_out(void *dst, const ttrt_tensor *src, int target_dtype) {
  return guard([&] {
    need(src, "tensor");
    std::optional<DataType> dt = target_dtype < 0 ? std::nullopt : std::optional<DataType>(static_cast<DataType>(target_dtype));
    tt::runtime::memcpy(dst, src->t, dt);
  });
}
TTRT_EXPORT int ttrt_memcpy_tensor(ttrt_tensor *dst, const ttrt_tensor *src) {
  return guard([&] { need(dst, "dst"); need(src, "src"); tt::runtime::memcpy(dst->t, src->t); });
}

TTRT_EXPORT int ttrt_submit(ttrt_device *dev, const ttrt_binary *bin, uint32_t program, ttrt_tensor *const *inputs, uint32_t num_inputs,
                            ttrt_tensor **outputs, uint32_t max_outputs, uint32_t *num_outputs) {
  return guard([&] {
    need(dev, "device"); need(bin, "binary"); need(num_outputs, "num_outputs");
    std::vector<Tensor> ins;
    for (uint32_t i = 0; i < num_inputs; ++i) {
      need(inputs[i], "input tensor");
      ins.push_back(inputs[i]->t);
    }
    std::vector<Tensor> outs = submit(dev->d, bin->b, program, ins);
    if (outs.size() > max_outputs) throw std::runtime_error("program returns more outputs than the caller's buffer holds");
    *num_outputs = static_cast<uint32_t>(outs.size());
    for (size_t i = 0; i < outs.size(); ++i) outputs[i] = new ttrt_tensor{outs[i]};
  });
}

// ---- hooks
struct HookCtx {
  CallbackContext cc;
  OpContext oc;
  const ttrt_binary *walked = nullptr;   // set by ttrt_walk_program: no program runs, cc is empty
  uint32_t walkedProgram = 0;
};
static debug::CallbackFn wrapOpCallback(ttrt_op_callback cb, void *user) {
  return debug::CallbackFn([cb, user](Binary, CallbackContext cc, OpContext oc) {
    HookCtx h{cc, oc};
    auto type = static_cast<ttmlir_amd::schema::OpType>(oc.op.scalar<std::uint8_t>(ttmlir_amd::schema::Operation::f_type_type, 0));
    std::string dbg = getOpDebugString(oc);
    cb(oc.index, ttmlir_amd::schema::opTypeName(type), dbg.c_str(), &h, user);
  });
}
static debug::ProgramCallbackFn wrapProgramCallback(ttrt_program_callback cb, void *user) {
  return debug::ProgramCallbackFn([cb, user](Binary, CallbackContext cc) {
    HookCtx h{cc, OpContext{}};
    cb(static_cast<uint32_t>(getProgramIndex(cc)), &h, user);
  });
}
TTRT_EXPORT int ttrt_set_post_op_callback(ttrt_op_callback cb, void *user) {
  return guard([&] {
    need(reinterpret_cast<const void *>(cb), "callback");
    debug::Hooks::get(std::nullopt, wrapOpCallback(cb, user));
  });
}
TTRT_EXPORT int ttrt_set_pre_op_callback(ttrt_op_callback cb, void *user) {
  return guard([&] {
    need(reinterpret_cast<const void *>(cb), "callback");
    debug::Hooks::get(wrapOpCallback(cb, user));
  });
}
TTRT_EXPORT int ttrt_set_program_callbacks(ttrt_program_callback pre, ttrt_program_callback post, void *user) {
  return guard([&] {
    debug::Hooks::get(std::nullopt, std::nullopt,
                      pre ? std::optional<debug::ProgramCallbackFn>(wrapProgramCallback(pre, user)) : std::nullopt,
                      post ? std::optional<debug::ProgramCallbackFn>(wrapProgramCallback(post, user)) : std::nullopt);
  });
}
static void copyRefIds(const std::vector<TensorRef> &refs, uint32_t *ids, uint32_t cap, uint32_t *count) {
  need(count, "count");
  *count = static_cast<uint32_t>(refs.size());
  if (refs.size() > cap) fatal("hook: the id array is too small for this operation's tensor references");
  for (size_t i = 0; i < refs.size(); ++i) ids[i] = getTensorRefGlobalId(refs[i]);
}
TTRT_EXPORT int ttrt_hook_input_refs(void *hook_ctx, uint32_t *ids, uint32_t cap, uint32_t *count) {
  return guard([&] {
    need(hook_ctx, "hook context");
    copyRefIds(getOpInputRefs(static_cast<HookCtx *>(hook_ctx)->oc), ids, cap, count);
  });
}
TTRT_EXPORT int ttrt_hook_output_refs(void *hook_ctx, uint32_t *ids, uint32_t cap, uint32_t *count) {
  return guard([&] {
    need(hook_ctx, "hook context");
    copyRefIds(getOpOutputRefs(static_cast<HookCtx *>(hook_ctx)->oc), ids, cap, count);
  });
}
TTRT_EXPORT int ttrt_hook_retrieve(void *hook_ctx, uint32_t global_id, int untilize, ttrt_tensor **out) {
  return guard([&] {
    need(hook_ctx, "hook context"); need(out, "out");
    auto t = retrieveTensorFromPool(static_cast<HookCtx *>(hook_ctx)->cc, global_id, untilize != 0);
    *out = t.has_value() ? new ttrt_tensor{*t} : nullptr;
  });
}
TTRT_EXPORT int ttrt_hook_update(void *hook_ctx, uint32_t global_id, const ttrt_tensor *src) {
  return guard([&] {
    need(hook_ctx, "hook context"); need(src, "source tensor");
    updateTensorInPool(static_cast<HookCtx *>(hook_ctx)->cc, global_id, src->t);
  });
}
TTRT_EXPORT int ttrt_hook_program_index(void *hook_ctx, uint32_t *index) {
  return guard([&] {
    need(hook_ctx, "hook context"); need(index, "index");
    *index = static_cast<uint32_t>(getProgramIndex(static_cast<HookCtx *>(hook_ctx)->cc));
  });
}
TTRT_EXPORT int ttrt_clear_callbacks(void) {
  return guard([&] { debug::Hooks::get().unregisterHooks(); });
}
TTRT_EXPORT int ttrt_hook_output(void *hook_ctx, ttrt_tensor **out) {
  return guard([&] {
    need(hook_ctx, "hook context"); need(out, "out");
    auto *h = static_cast<HookCtx *>(hook_ctx);
    auto m = getOpOutputTensor(h->oc, h->cc);
    *out = m.empty() ? nullptr : new ttrt_tensor{m.begin()->second};
  });
}
TTRT_EXPORT int ttrt_hook_loc(void *hook_ctx, char *buf, size_t len) {
  return guard([&] {
    need(hook_ctx, "hook context");
    copyStr(getOpLocInfo(static_cast<HookCtx *>(hook_ctx)->oc), buf, len);
  });
}
TTRT_EXPORT int ttrt_hook_ref_desc(void *hook_ctx, uint32_t global_id, uint32_t *shape, int *rank, int *dtype) {
  return guard([&] {
    need(hook_ctx, "hook context");
    const OpContext &oc = static_cast<HookCtx *>(hook_ctx)->oc;
    for (const auto &refs : {getOpInputRefs(oc), getOpOutputRefs(oc)})
      for (const TensorRef &r : refs)
        if (getTensorRefGlobalId(r) == global_id) {
          writeShape(getTensorRefShape(r), shape, rank);
          if (dtype) *dtype = static_cast<int>(getTensorRefDataType(r));
          return;
        }
    fatal("hook: tensor " + std::to_string(global_id) + " is neither an operand nor a result of this operation");
  });
}
TTRT_EXPORT int ttrt_hook_invoke_cpu_op(void *hook_ctx, ttrt_tensor *const *inputs, uint32_t num_inputs, ttrt_tensor **outputs,
                                        uint32_t max_outputs, uint32_t *num_outputs) {
  return guard([&] {
    need(hook_ctx, "hook context"); need(num_outputs, "num_outputs");
    auto *h = static_cast<HookCtx *>(hook_ctx);
    std::vector<Tensor> ins;
    for (uint32_t i = 0; i < num_inputs; ++i) {
      need(inputs[i], "input tensor");
      ins.push_back(inputs[i]->t);
    }
    std::vector<Tensor> outs = h->walked ? invokeCpuOpOf(h->walked->b, h->walkedProgram, h->oc, ins) : invokeCpuOp(h->cc, h->oc, ins);
    if (outs.size() > max_outputs) throw std::runtime_error("the CpuOp returns more outputs than the caller's buffer holds");
    *num_outputs = static_cast<uint32_t>(outs.size());
    for (size_t i = 0; i < outs.size(); ++i) outputs[i] = new ttrt_tensor{outs[i]};
  });
}
TTRT_EXPORT int ttrt_walk_program(const ttrt_binary *bin, uint32_t program, ttrt_op_callback cb, void *user) {
  return guard([&] {
    need(bin, "binary"); need(reinterpret_cast<const void *>(cb), "callback");
    walkProgram(bin->b, program, [&](OpContext oc) {
      HookCtx h{CallbackContext{}, oc, bin, program};
      auto type = static_cast<ttmlir_amd::schema::OpType>(oc.op.scalar<std::uint8_t>(ttmlir_amd::schema::Operation::f_type_type, 0));
      std::string dbg = getOpDebugString(oc);
      cb(oc.index, ttmlir_amd::schema::opTypeName(type), dbg.c_str(), &h, user);
    });
  });
}
TTRT_EXPORT int ttrt_stat(const char *name, int64_t *value) {
  return guard([&] { need(name, "name"); need(value, "value"); *value = debug::Stats::get().getStat(name); });
}
TTRT_EXPORT int ttrt_stats_clear(void) {
  return guard([&] { debug::Stats::get().clear(); });
}
TTRT_EXPORT int ttrt_buffer_cast(const void *src, void *dst, int from_dtype, int to_dtype, int64_t n) {
  return guard([&] { utils::handleBufferCast(src, dst, static_cast<DataType>(from_dtype), static_cast<DataType>(to_dtype), n); });
}

// ---- program writer
TTRT_EXPORT int ttrt_pb_create(ttrt_builder **out) {
  return guard([&] { need(out, "out"); *out = new ttrt_builder{}; });
}
TTRT_EXPORT void ttrt_pb_destroy(ttrt_builder *pb) { delete pb; }
TTRT_EXPORT int ttrt_pb_begin_program(ttrt_builder *pb, const char *name, int is_private) {
  return guard([&] { need(pb, "builder"); need(name, "name"); pb->pb.beginProgram(name, is_private != 0); });
}
TTRT_EXPORT int ttrt_pb_end_program(ttrt_builder *pb, uint32_t *program_index) {
  return guard([&] { need(pb, "builder"); uint32_t i = pb->pb.endProgram(); if (program_index) *program_index = i; });
}
static ProgramBuilder::Desc descOf(const uint32_t *shape, int rank, const ttrt_layout *l) {
  need(l, "layout");
  return ProgramBuilder::Desc{shapeVec(shape, rank), static_cast<DataType>(l->dtype), static_cast<TensorLayout>(l->layout),
                              static_cast<StorageType>(l->storage)};
}
TTRT_EXPORT int ttrt_pb_input(ttrt_builder *pb, const uint32_t *shape, int rank, const ttrt_layout *layout, uint32_t *id) {
  return guard([&] {
    need(pb, "builder"); need(id, "id");
    auto d = descOf(shape, rank, layout);
    *id = pb->pb.input(d.shape, d.dtype, d.layout, d.storage);
  });
}
TTRT_EXPORT int ttrt_pb_output(ttrt_builder *pb, uint32_t id) {
  return guard([&] { need(pb, "builder"); pb->pb.output(id); });
}
TTRT_EXPORT int ttrt_pb_finish(ttrt_builder *pb, uint8_t **data, size_t *size) {
  return guard([&] {
    need(pb, "builder"); need(data, "data"); need(size, "size");
    auto v = pb->pb.finish();
    *data = static_cast<uint8_t *>(std::malloc(v.size()));
    if (!*data) throw std::runtime_error("out of memory");
    std::memcpy(*data, v.data(), v.size());
    *size = v.size();
  });
}
TTRT_EXPORT void ttrt_free_bytes(uint8_t *data) { std::free(data); }
TTRT_EXPORT int ttrt_pb_tensor_desc(ttrt_builder *pb, uint32_t id, uint32_t *shape, int *rank, ttrt_layout *layout) {
  return guard([&] {
    need(pb, "builder");
    const auto &d = pb->pb.desc(id);
    writeShape(d.shape, shape, rank);
    if (layout) *layout = ttrt_layout{static_cast<int>(d.storage), static_cast<int>(d.layout), static_cast<int>(d.dtype)};
  });
}
#define PB_OP(call) return guard([&] { need(pb, "builder"); need(out, "out"); *out = pb->pb.call; })
TTRT_EXPORT int ttrt_pb_to_layout(ttrt_builder *pb, uint32_t in, int layout, int dtype, int storage, uint32_t *out) {
  PB_OP(toLayout(in, static_cast<TensorLayout>(layout), dtype, static_cast<StorageType>(storage)));
}
TTRT_EXPORT int ttrt_pb_typecast(ttrt_builder *pb, uint32_t in, int dtype, uint32_t *out) { PB_OP(typecast(in, static_cast<DataType>(dtype))); }
TTRT_EXPORT int ttrt_pb_to_device(ttrt_builder *pb, uint32_t in, uint32_t *out) { PB_OP(toDevice(in)); }
TTRT_EXPORT int ttrt_pb_from_device(ttrt_builder *pb, uint32_t in, uint32_t *out) { PB_OP(fromDevice(in)); }
TTRT_EXPORT int ttrt_pb_matmul(ttrt_builder *pb, uint32_t a, uint32_t b, int ta, int tb, const char *activation, int out_dtype, uint32_t *out) {
  PB_OP(matmul(a, b, ta != 0, tb != 0, activation ? activation : "", static_cast<DataType>(out_dtype)));
}
TTRT_EXPORT int ttrt_pb_linear(ttrt_builder *pb, uint32_t a, uint32_t b, uint32_t bias, int ta, int tb, const char *activation, int out_dtype,
                               uint32_t *out) {
  PB_OP(linear(a, b, bias, ta != 0, tb != 0, activation ? activation : "", static_cast<DataType>(out_dtype)));
}
TTRT_EXPORT int ttrt_pb_unary(ttrt_builder *pb, uint32_t type, uint32_t in, int has_param, float param, uint32_t *out) {
  PB_OP(unary(type, in, has_param != 0, param));
}
TTRT_EXPORT int ttrt_pb_binary(ttrt_builder *pb, uint32_t type, uint32_t lhs, uint32_t rhs, uint32_t *out) { PB_OP(binary(type, lhs, rhs)); }
TTRT_EXPORT int ttrt_pb_rms_norm(ttrt_builder *pb, uint32_t in, uint32_t weight, uint32_t bias, float eps, uint32_t *out) {
  PB_OP(rmsNorm(in, weight, bias, eps));
}
TTRT_EXPORT int ttrt_pb_softmax(ttrt_builder *pb, uint32_t in, int dim, uint32_t *out) { PB_OP(softmax(in, dim)); }
TTRT_EXPORT int ttrt_pb_reduction(ttrt_builder *pb, uint32_t type, uint32_t in, const int32_t *dims, int ndims, int keep_dim, uint32_t *out) {
  PB_OP(reduction(type, in, std::vector<int>(dims, dims + ndims), keep_dim != 0));
}
TTRT_EXPORT int ttrt_pb_sdpa(ttrt_builder *pb, uint32_t q, uint32_t k, uint32_t v, uint32_t mask, int is_causal, int has_scale, float scale,
                             int64_t sliding_window, uint32_t attention_sink, uint32_t *out) {
  PB_OP(sdpa(q, k, v, mask, is_causal != 0, has_scale != 0, scale, sliding_window, attention_sink));
}
TTRT_EXPORT int ttrt_pb_rotary_embedding(ttrt_builder *pb, uint32_t in, uint32_t cos_cache, uint32_t sin_cache, int has_token_index,
                                         uint32_t token_index, uint32_t *out) {
  PB_OP(rotaryEmbedding(in, cos_cache, sin_cache, has_token_index != 0, token_index));
}
TTRT_EXPORT int ttrt_pb_update_cache(ttrt_builder *pb, uint32_t cache, uint32_t in, uint32_t update_index, uint32_t batch_offset) {
  return guard([&] { need(pb, "builder"); pb->pb.updateCache(cache, in, update_index, batch_offset); });
}
TTRT_EXPORT int ttrt_pb_fill_cache(ttrt_builder *pb, uint32_t cache, uint32_t in, uint32_t batch_offset) {
  return guard([&] { need(pb, "builder"); pb->pb.fillCache(cache, in, batch_offset); });
}
TTRT_EXPORT int ttrt_pb_paged_update_cache(ttrt_builder *pb, uint32_t cache, uint32_t in, uint32_t update_index, uint32_t page_table,
                                           int share_cache) {
  return guard([&] { need(pb, "builder"); pb->pb.pagedUpdateCache(cache, in, update_index, page_table, share_cache != 0); });
}
TTRT_EXPORT int ttrt_pb_paged_fill_cache(ttrt_builder *pb, uint32_t cache, uint32_t in, uint32_t page_table, uint32_t batch_idx) {
  return guard([&] { need(pb, "builder"); pb->pb.pagedFillCache(cache, in, page_table, batch_idx); });
}
TTRT_EXPORT int ttrt_pb_sdpa_decode(ttrt_builder *pb, uint32_t q, uint32_t k, uint32_t v, uint32_t page_table, uint32_t mask, uint32_t cur_pos,
                                    int is_causal, int has_scale, float scale, int64_t sliding_window, uint32_t attention_sink,
                                    uint32_t *out) {
  PB_OP(sdpaDecode(q, k, v, page_table, mask, cur_pos, is_causal != 0, has_scale != 0, scale, sliding_window, attention_sink));
}
TTRT_EXPORT int ttrt_pb_reshape(ttrt_builder *pb, uint32_t in, const uint32_t *shape, int rank, uint32_t *out) { PB_OP(reshape(in, shapeVec(shape, rank))); }
TTRT_EXPORT int ttrt_pb_permute(ttrt_builder *pb, uint32_t in, const int64_t *perm, int rank, uint32_t *out) {
  PB_OP(permute(in, std::vector<std::int64_t>(perm, perm + rank)));
}
TTRT_EXPORT int ttrt_pb_transpose(ttrt_builder *pb, uint32_t in, int dim0, int dim1, uint32_t *out) { PB_OP(transpose(in, dim0, dim1)); }
TTRT_EXPORT int ttrt_pb_concat(ttrt_builder *pb, const uint32_t *ins, int n, int dim, uint32_t *out) {
  PB_OP(concat(std::vector<ProgramBuilder::Id>(ins, ins + n), dim));
}
TTRT_EXPORT int ttrt_pb_slice(ttrt_builder *pb, uint32_t in, const int64_t *begins, const int64_t *ends, const int64_t *steps, int rank,
                              uint32_t *out) {
  PB_OP(slice(in, std::vector<std::int64_t>(begins, begins + rank), std::vector<std::int64_t>(ends, ends + rank),
              std::vector<std::int64_t>(steps, steps + rank)));
}
TTRT_EXPORT int ttrt_pb_repeat_interleave(ttrt_builder *pb, uint32_t in, uint32_t repeats, int dim, uint32_t *out) {
  PB_OP(repeatInterleave(in, repeats, dim));
}
TTRT_EXPORT int ttrt_pb_unary_composite(ttrt_builder *pb, uint32_t type, uint32_t in, float lo, float hi, int int_bounds, uint32_t *out) {
  PB_OP(unaryComposite(type, in, lo, hi, int_bounds != 0));
}
TTRT_EXPORT int ttrt_pb_concat_heads(ttrt_builder *pb, int kind, uint32_t in, uint32_t num_heads, uint32_t *out) {
  PB_OP(concatHeads(kind, in, num_heads));
}
TTRT_EXPORT int ttrt_pb_nlp_create_qkv_heads_decode(ttrt_builder *pb, uint32_t in, uint32_t num_heads, uint32_t num_kv_heads, uint32_t *qkv_out) {
  return guard([&] {
    need(pb, "builder"); need(qkv_out, "out");
    auto r = pb->pb.nlpCreateQkvHeadsDecode(in, num_heads, num_kv_heads);
    for (int i = 0; i < 3; ++i) qkv_out[i] = r[i];
  });
}
TTRT_EXPORT int ttrt_pb_split_qkv_and_split_heads(ttrt_builder *pb, uint32_t in, uint32_t kv_input, uint32_t num_heads, uint32_t num_kv_heads,
                                                  int transpose_key, uint32_t *qkv_out) {
  return guard([&] {
    need(pb, "builder"); need(qkv_out, "out");
    auto r = pb->pb.splitQkvAndSplitHeads(in, kv_input, num_heads, num_kv_heads, transpose_key != 0);
    for (int i = 0; i < 3; ++i) qkv_out[i] = r[i];
  });
}
TTRT_EXPORT int ttrt_pb_repeat(ttrt_builder *pb, uint32_t in, const int64_t *repeats, int rank, uint32_t *out) {
  PB_OP(repeat(in, std::vector<std::int64_t>(repeats, repeats + rank)));
}
TTRT_EXPORT int ttrt_pb_binary_composite(ttrt_builder *pb, uint32_t type, uint32_t lhs, uint32_t rhs, uint32_t *out) {
  PB_OP(binaryComposite(type, lhs, rhs));
}
TTRT_EXPORT int ttrt_pb_where(ttrt_builder *pb, uint32_t cond, uint32_t a, uint32_t b, uint32_t *out) { PB_OP(where(cond, a, b)); }
TTRT_EXPORT int ttrt_pb_embedding(ttrt_builder *pb, uint32_t indices, uint32_t weight, uint32_t *out) { PB_OP(embedding(indices, weight)); }
TTRT_EXPORT int ttrt_pb_argmax(ttrt_builder *pb, uint32_t in, int has_dim, int dim, int keep_dim, int out_dtype, uint32_t *out) {
  PB_OP(argmax(in, has_dim != 0, dim, keep_dim != 0, static_cast<DataType>(out_dtype)));
}
TTRT_EXPORT int ttrt_pb_arange(ttrt_builder *pb, float start, float end, float step, int dtype, int layout, uint32_t *out) {
  PB_OP(arange(start, end, step, static_cast<DataType>(dtype), static_cast<TensorLayout>(layout)));
}
TTRT_EXPORT int ttrt_pb_constant(ttrt_builder *pb, const void *data, size_t bytes, int in_dtype, const uint32_t *shape, int rank,
                                 const ttrt_layout *layout, uint32_t *out) {
  return guard([&] {
    need(pb, "builder"); need(out, "out"); need(data, "data");
    auto d = descOf(shape, rank, layout);
    *out = pb->pb.constant(data, bytes, static_cast<DataType>(in_dtype), d.shape, d.dtype, d.layout, d.storage);
  });
}
TTRT_EXPORT int ttrt_pb_full(ttrt_builder *pb, const uint32_t *shape, int rank, float value, int dtype, int layout, uint32_t *out) {
  PB_OP(full(shapeVec(shape, rank), value, static_cast<DataType>(dtype), static_cast<TensorLayout>(layout)));
}
TTRT_EXPORT int ttrt_pb_empty(ttrt_builder *pb, const uint32_t *shape, int rank, int dtype, int layout, uint32_t *out) {
  PB_OP(empty(shapeVec(shape, rank), static_cast<DataType>(dtype), static_cast<TensorLayout>(layout)));
}
TTRT_EXPORT int ttrt_pb_copy(ttrt_builder *pb, uint32_t src, uint32_t dst) {
  return guard([&] { need(pb, "builder"); pb->pb.copy(src, dst); });
}
TTRT_EXPORT int ttrt_pb_write_tensor(ttrt_builder *pb, uint32_t host, uint32_t device) {
  return guard([&] { need(pb, "builder"); pb->pb.writeTensor(host, device); });
}
TTRT_EXPORT int ttrt_pb_begin_trace_capture(ttrt_builder *pb, uint32_t *out) { PB_OP(beginTraceCapture()); }
TTRT_EXPORT int ttrt_pb_end_trace_capture(ttrt_builder *pb, uint32_t trace_id) {
  return guard([&] { need(pb, "builder"); pb->pb.endTraceCapture(trace_id); });
}
TTRT_EXPORT int ttrt_pb_execute_trace(ttrt_builder *pb, uint32_t trace_id, int blocking) {
  return guard([&] { need(pb, "builder"); pb->pb.executeTrace(trace_id, blocking != 0); });
}
TTRT_EXPORT int ttrt_pb_deallocate(ttrt_builder *pb, uint32_t in, int force) {
  return guard([&] { need(pb, "builder"); pb->pb.deallocate(in, force != 0); });
}
TTRT_EXPORT int ttrt_pb_set_matmul_program_config(ttrt_builder *pb, int kind, int fused_activation) {
  return guard([&] { need(pb, "builder"); pb->pb.setMatmulProgramConfig(kind, fused_activation); });
}
TTRT_EXPORT int ttrt_pb_declare_next_shape(ttrt_builder *pb, const uint32_t *shape, int rank) {
  return guard([&] { need(pb, "builder"); pb->pb.declareNextShape(shapeVec(shape, rank)); });
}
TTRT_EXPORT int ttrt_pb_last_op_loc(ttrt_builder *pb, char *buf, size_t len) {
  return guard([&] { need(pb, "builder"); copyStr(pb->pb.lastOpLoc(), buf, len); });
}
TTRT_EXPORT int ttrt_pb_golden(ttrt_builder *pb, const char *loc, const char *name, const void *data, size_t bytes, const int64_t *shape,
                               int rank, int dtype) {
  return guard([&] {
    need(pb, "builder"); need(loc, "loc"); need(data, "data");
    pb->pb.golden(loc, name ? name : "", data, bytes, std::vector<std::int64_t>(shape, shape + rank), static_cast<DataType>(dtype));
  });
}
static std::vector<ProgramBuilder::Desc> outDescs(const uint32_t *out_shapes, const int *out_ranks, const ttrt_layout *out_layouts, int n_out) {
  std::vector<ProgramBuilder::Desc> v;
  for (int i = 0; i < n_out; ++i) v.push_back(descOf(out_shapes + 8 * i, out_ranks[i], out_layouts + i));
  return v;
}
TTRT_EXPORT int ttrt_pb_load_cached(ttrt_builder *pb, uint32_t program_index, const char *callee, const uint32_t *ins, int n_in,
                                    const uint32_t *out_shapes, const int *out_ranks, const ttrt_layout *out_layouts, int n_out, uint32_t *outs) {
  return guard([&] {
    need(pb, "builder"); need(outs, "outs");
    auto ids = pb->pb.loadCached(program_index, callee ? callee : "", std::vector<ProgramBuilder::Id>(ins, ins + n_in),
                                 outDescs(out_shapes, out_ranks, out_layouts, n_out));
    for (size_t i = 0; i < ids.size(); ++i) outs[i] = ids[i];
  });
}
TTRT_EXPORT int ttrt_pb_capture_or_execute_trace(ttrt_builder *pb, uint32_t capture_program, uint32_t execute_program,
                                                 uint32_t allocate_slots_program, const uint32_t *ins, int n_in,
                                                 const uint32_t *out_shapes, const int *out_ranks, const ttrt_layout *out_layouts,
                                                 int n_out, uint32_t *outs) {
  return guard([&] {
    need(pb, "builder"); need(outs, "outs");
    auto ids = pb->pb.captureOrExecuteTrace(capture_program, execute_program, allocate_slots_program,
                                            std::vector<ProgramBuilder::Id>(ins, ins + n_in),
                                            outDescs(out_shapes, out_ranks, out_layouts, n_out));
    for (size_t i = 0; i < ids.size(); ++i) outs[i] = ids[i];
  });
}
TTRT_EXPORT int ttrt_pb_rotary_embedding_llama(ttrt_builder *pb, uint32_t in, uint32_t cos_cache, uint32_t sin_cache, uint32_t trans_mat,
                                               int decode_mode, uint32_t *out) {
  PB_OP(rotaryEmbeddingLlama(in, cos_cache, sin_cache, trans_mat, decode_mode != 0));
}
TTRT_EXPORT int ttrt_pb_chunked_sdpa(ttrt_builder *pb, uint32_t q, uint32_t k, uint32_t v, uint32_t page_table, uint32_t chunk_start,
                                     int has_scale, float scale, uint32_t *out) {
  PB_OP(chunkedSdpa(q, k, v, page_table, chunk_start, has_scale != 0, scale));
}
TTRT_EXPORT int ttrt_pb_add_dylib(ttrt_builder *pb, uint32_t dylib_id, const void *data, size_t size) {
  return guard([&] {
    need(pb, "builder"); need(data, "data");
    pb->pb.addDylib(dylib_id, data, size);
  });
}
TTRT_EXPORT int ttrt_pb_cpu_op(ttrt_builder *pb, uint32_t dylib_id, const char *func_name, const uint32_t *ins, int n_in,
                               const uint32_t *out_shapes, const int *out_ranks, const ttrt_layout *out_layouts, int n_out, uint32_t *outs) {
  return guard([&] {
    need(pb, "builder"); need(func_name, "func_name"); need(outs, "outs");
    auto ids = pb->pb.cpuOp(dylib_id, func_name, std::vector<ProgramBuilder::Id>(ins, ins + n_in), outDescs(out_shapes, out_ranks, out_layouts, n_out));
    for (size_t i = 0; i < ids.size(); ++i) outs[i] = ids[i];
  });
}
TTRT_EXPORT int ttrt_pb_func_call(ttrt_builder *pb, uint32_t program_index, const uint32_t *ins, int n_in, const uint32_t *out_shapes,
                                  const int *out_ranks, const ttrt_layout *out_layouts, int n_out, uint32_t *outs) {
  return guard([&] {
    need(pb, "builder"); need(outs, "outs");
    auto ids = pb->pb.funcCall(program_index, std::vector<ProgramBuilder::Id>(ins, ins + n_in), outDescs(out_shapes, out_ranks, out_layouts, n_out));
    for (size_t i = 0; i < ids.size(); ++i) outs[i] = ids[i];
  });
}
