// Writer of `.ttnn` flatbuffer programs for the op subset this backend executes.  The reference
// ships no prebuilt binaries (they are produced by ttmlir-opt + ttmlir-translate, see
// test/ttmlir/Runtime/TTNN/n150/**.mlir RUN lines), so tests and benchmarks build their programs
// here; the wire format is the reference's (include/ttmlir/Target/TTNN/*.fbs).
#pragma once
#include <array>
#include <optional>
#include <string>
#include <vector>

#include "runtime.h"

namespace ttmlir_amd {

using ::tt::target::DataType;
using ::tt::target::StorageType;
using ::tt::target::TensorLayout;

class ProgramBuilder {
public:
  using Id = std::uint32_t;  // tensor global_id
  struct Desc {
    std::vector<std::uint32_t> shape;
    DataType dtype;
    TensorLayout layout;
    StorageType storage;
  };

  void beginProgram(const std::string &name, bool isPrivate = false);
  Id input(const std::vector<std::uint32_t> &shape, DataType dtype, TensorLayout layout, StorageType storage);
  void output(Id t);
  std::uint32_t endProgram();  // returns the program index

  Id toLayout(Id in, TensorLayout layout, int dtype /* -1 = keep */, StorageType storage);
  Id typecast(Id in, DataType dtype);
  Id toDevice(Id in);
  Id fromDevice(Id in);
  // The next matmul / linear carries a matmul_program_config of this kind (the MatmulProgramConfig union's value; 0 = none)
  // whose fused_activation is the given UnaryOpType, or none when negative.
  void setMatmulProgramConfig(int kind, int fusedActivation);
  Id matmul(Id a, Id b, bool transposeA, bool transposeB, const std::string &activation, DataType outDtype);
  Id linear(Id a, Id b, Id bias /* 0 = none */, bool transposeA, bool transposeB, const std::string &activation, DataType outDtype);
  Id unary(std::uint32_t type, Id in, bool hasParam, float param);
  // EltwiseUnaryCompositeOp: Cbrt, ClampScalar (bounds as FP, or as I32 when intBounds), Log1p
  Id unaryComposite(std::uint32_t type, Id in, float lo, float hi, bool intBounds);
  Id binary(std::uint32_t type, Id lhs, Id rhs);
  Id rmsNorm(Id in, Id weight, Id bias, float eps);
  Id softmax(Id in, int dim);
  Id reduction(std::uint32_t type, Id in, const std::vector<int> &dims, bool keepDim);
  Id sdpa(Id q, Id k, Id v, Id mask, bool causal, bool hasScale, float scale, std::int64_t slidingWindow = -1, Id sink = 0);
  Id reshape(Id in, const std::vector<std::uint32_t> &shape);
  Id permute(Id in, const std::vector<std::int64_t> &perm);
  Id transpose(Id in, int dim0, int dim1);
  Id concat(const std::vector<Id> &ins, int dim);
  Id slice(Id in, const std::vector<std::int64_t> &begins, const std::vector<std::int64_t> &ends, const std::vector<std::int64_t> &steps);
  Id repeatInterleave(Id in, std::uint32_t repeats, int dim);
  // the ops around a decoder layer (include/ttmlir/Target/TTNN/operations/{data_movement,eltwise,embedding,reduction,creation}.fbs)
  Id repeat(Id in, const std::vector<std::int64_t> &repeats);
  // head splits and merges (include/ttmlir/Target/TTNN/operations/transformer.fbs:7-11, 34-45, 109-132); kind 0 =
  // ConcatenateHeadsOp, 1 = NLPConcatHeadsOp, 2 = NLPConcatHeadsDecodeOp (numHeads used)
  Id concatHeads(int kind, Id in, std::uint32_t numHeads);
  std::array<Id, 3> nlpCreateQkvHeadsDecode(Id in, std::uint32_t numHeads, std::uint32_t numKvHeads);
  std::array<Id, 3> splitQkvAndSplitHeads(Id in, Id kvInput, std::uint32_t numHeads, std::uint32_t numKvHeads, bool transposeKey);
  Id binaryComposite(std::uint32_t type, Id lhs, Id rhs);
  Id where(Id cond, Id a, Id b);
  Id embedding(Id indices, Id weight);
  Id argmax(Id in, bool hasDim, int dim, bool keepDim, DataType outDtype);
  Id arange(float start, float end, float step, DataType dtype, TensorLayout layout);
  Id constant(const void *data, size_t bytes, DataType inDtype, const std::vector<std::uint32_t> &shape, DataType dtype,
              TensorLayout layout, StorageType storage);
  Id full(const std::vector<std::uint32_t> &shape, float value, DataType dtype, TensorLayout layout);
  Id rotaryEmbedding(Id in, Id cosCache, Id sinCache, bool hasTokenIndex, std::uint32_t tokenIndex);
  Id rotaryEmbeddingLlama(Id in, Id cosCache, Id sinCache, Id transMat, bool decodeMode);
  Id chunkedSdpa(Id q, Id k, Id v, Id pageTable, Id chunkStart, bool hasScale, float scale);
  void updateCache(Id cache, Id in, Id updateIndex, std::uint32_t batchOffset);
  void fillCache(Id cache, Id in, std::uint32_t batchOffset);
  void pagedUpdateCache(Id cache, Id in, Id updateIndex, Id pageTable, bool shareCache);   // pageTable 0: static cache
  void pagedFillCache(Id cache, Id in, Id pageTable, Id batchIdx);                         // batchIdx 0: row b of the table
  // pageTable = 0 writes ScaledDotProductAttentionDecodeOp, otherwise the paged op
  Id sdpaDecode(Id q, Id k, Id v, Id pageTable, Id mask, Id curPos, bool causal, bool hasScale, float scale,
                std::int64_t slidingWindow = -1, Id sink = 0);
  Id empty(const std::vector<std::uint32_t> &shape, DataType dtype, TensorLayout layout);
  void copy(Id src, Id dst);                 // ttnn.copy: dst <- src, both on device
  void writeTensor(Id host, Id device);      // ttnn.write_tensor: device <- host
  Id beginTraceCapture();                    // returns the trace id tensor (rank-0 UInt32 on host)
  void endTraceCapture(Id traceId);
  void executeTrace(Id traceId, bool blocking);
  std::vector<Id> captureOrExecuteTrace(std::uint32_t captureProgram, std::uint32_t executeProgram, std::uint32_t allocateSlotsProgram,
                                        const std::vector<Id> &ins, const std::vector<Desc> &outs);
  void deallocate(Id in, bool force);
  std::vector<Id> loadCached(std::uint32_t programIdx, const std::string &callee, const std::vector<Id> &ins, const std::vector<Desc> &outs);
  std::vector<Id> funcCall(std::uint32_t programIdx, const std::vector<Id> &ins, const std::vector<Desc> &outs);
  // CPU-hoisted function (include/ttmlir/Target/TTNN/operations/cpu.fbs): `funcName` of the dynamic library that
  // addDylib put into the open program under `dylibId`
  std::vector<Id> cpuOp(std::uint32_t dylibId, const std::string &funcName, const std::vector<Id> &ins, const std::vector<Desc> &outs);
  void addDylib(std::uint32_t dylibId, const void *data, size_t bytes);

  // Location string of the operation added last ("loc(\"<program>\"(\"op<k>\"))"); goldens are keyed by it.
  std::string lastOpLoc() const;
  // The next tensor the builder creates is declared with `shape` instead of the shape its operation gives: a program that
  // lies about a result, for tests of what the executor does with one (the compiler never writes such a program).
  void declareNextShape(const std::vector<std::uint32_t> &shape) { declaredShape_ = shape; }
  // Embeds an expected tensor for the operation at `loc` into the open program's debug info
  // (Common/debug_info.fbs: GoldenInfo.golden_map); data is row-major, contiguous.
  void golden(const std::string &loc, const std::string &name, const void *data, size_t bytes,
              const std::vector<std::int64_t> &shape, DataType dtype);

  const Desc &desc(Id t) const;
  std::vector<std::uint8_t> finish();  // size-prefixed TTNN binary

private:
  struct OpRec {
    std::uint8_t type;
    fb::Builder::Off table;
    std::string debug;
  };
  struct ProgramRec {
    std::string name;
    bool isPrivate = false;
    std::vector<Id> inputs, outputs;
    std::vector<OpRec> ops;
    std::vector<std::pair<std::string, fb::Builder::Off>> goldens;   // loc -> GoldenDeviceTensor table
    std::vector<fb::Builder::Off> dylibs;                            // DynamicLib tables
  };
  Id newTensor(const Desc &d);
  std::optional<std::vector<std::uint32_t>> declaredShape_;   // see declareNextShape
  int pendingMatmulConfig_ = 0, pendingFusedActivation_ = -1;  // see setMatmulProgramConfig
  fb::Builder::Off takeMatmulProgramConfig(std::uint8_t *kindOut);
  fb::Builder::Off tensorRef(Id t);
  fb::Builder::Off memoryConfig(StorageType storage);
  void addOp(::ttmlir_amd::schema::OpType type, fb::Builder::Off table, const std::string &debug);

  fb::Builder b_;
  std::vector<Desc> tensors_{Desc{}};  // index = id; id 0 is "none"
  std::vector<fb::Builder::Off> finishedPrograms_;
  ProgramRec cur_;
  bool open_ = false;
};

}  // namespace ttmlir_amd
