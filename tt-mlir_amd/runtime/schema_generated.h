// Field slot numbers and enum values of the TTNN flatbuffer schema (the wire-format contract
// between the tt-mlir compiler and a runtime): include/ttmlir/Target/{Common,TTNN}/**/*.fbs.
// Slots are implicit in the schema: declaration order, a union field taking two slots
// (<name>_type then <name>).  Generated from the schema text; do not edit by hand.
#pragma once
#include <cstdint>

namespace ttmlir_amd::schema {

enum class Arch : uint32_t {
  Wormhole_b0 = 0,
  Blackhole = 1,
  Quasar = 2,
};
enum class BufferType : uint16_t {
  DRAM = 0,
  L1 = 1,
  SystemMemory = 2,
  L1Small = 3,
  Trace = 4,
};
enum class CPURole : uint8_t {
  Host = 0,
  Device = 1,
};
enum class ChipCapability : uint32_t {
  HostMMIO = 0,
};
enum class Conv2dSliceType : uint16_t {
  DramHeight = 0,
  DramWidth = 1,
  L1Full = 2,
};
enum class CoreType : uint8_t {
  WORKER = 0,
  ETH = 1,
};
enum class DataMovementProcessor : uint16_t {
  RISCV_0 = 0,
  RISCV_1 = 1,
  RISCV_2 = 2,
  RISCV_3 = 3,
  RISCV_4 = 4,
  RISCV_5 = 5,
  RISCV_6 = 6,
  RISCV_7 = 7,
};
enum class DataMovementType : uint8_t {
  RISCV_0 = 0,
  RISCV_1 = 1,
};
enum class DataType : uint16_t {
  Float32 = 0,
  Float16 = 1,
  BFloat16 = 2,
  BFP_Float8 = 3,
  BFP_BFloat8 = 4,
  BFP_Float4 = 5,
  BFP_BFloat4 = 6,
  BFP_Float2 = 7,
  BFP_BFloat2 = 8,
  UInt32 = 9,
  UInt16 = 10,
  UInt8 = 11,
  Int32 = 12,
  Float64 = 13,
  Int64 = 14,
  UInt64 = 15,
  Int16 = 16,
  Int8 = 17,
  Bool = 18,
};
enum class EltwiseBinaryCompositeOpType : uint32_t {
  Maximum = 0,
  Minimum = 1,
  Remainder = 2,
  Pow = 3,
  Atan2 = 4,
  BitwiseAnd = 5,
  BitwiseOr = 6,
  BitwiseXor = 7,
  LogicalLeftShift = 8,
};
enum class EltwiseBinaryCompositeScalarOpType : uint32_t {
  PowScalar = 0,
};
enum class EltwiseBinaryOpType : uint32_t {
  Add = 0,
  Multiply = 1,
  LogicalRightShift = 2,
  Subtract = 3,
  Equal = 4,
  NotEqual = 5,
  GreaterEqual = 6,
  GreaterThan = 7,
  LessEqual = 8,
  LessThan = 9,
  Divide = 10,
  LogicalAnd = 11,
  LogicalOr = 12,
  LogicalXor = 13,
};
enum class EltwiseQuantizationOpType : uint32_t {
  Quantize = 0,
  Dequantize = 1,
  Requantize = 2,
};
enum class EltwiseUnaryCompositeOpType : uint32_t {
  Cbrt = 0,
  ClampScalar = 1,
  ClampTensor = 2,
  Log1p = 3,
};
enum class EltwiseUnaryOpType : uint32_t {
  Abs = 0,
  Ceil = 1,
  Cos = 2,
  Floor = 3,
  Gelu = 4,
  IsFinite = 5,
  LogicalNot = 6,
  Neg = 7,
  Relu = 8,
  Sqrt = 9,
  Rsqrt = 10,
  Sigmoid = 11,
  Sin = 12,
  Reciprocal = 13,
  Sign = 14,
  Tan = 15,
  Tanh = 16,
  Atan = 17,
  Exp = 18,
  Erf = 19,
  Erfc = 20,
  Log = 21,
  Expm1 = 22,
  LeakyRelu = 23,
  BitwiseNot = 24,
  Relu6 = 25,
  Silu = 26,
  Hardsigmoid = 27,
  Mish = 28,
  Acos = 29,
  Asin = 30,
  Asinh = 31,
};
enum class ExperimentalEltwiseBinaryBackwardOpType : uint32_t {
  GeluBW = 0,
};
enum class MathFidelity : uint8_t {
  LoFi = 0,
  HiFi2 = 2,
  HiFi3 = 3,
  HiFi4 = 4,
};
enum class MemorySpace : uint16_t {
  System = 0,
  SystemMMIO = 1,
  DeviceDRAM = 2,
  DeviceL1 = 3,
};
enum class MeshShardDirection : uint32_t {
  FullToShardShape = 0,
  ShardToFullShape = 1,
};
enum class MeshShardType : uint32_t {
  Replicate = 0,
  Maximal = 1,
  Devices = 2,
};
enum class MoEActivationFunction : uint16_t {
  Silu = 0,
  SwiGLU = 1,
};
enum class NamedFullOpType : uint32_t {
  Zeros = 0,
  Ones = 1,
};
enum class NocIndex : uint16_t {
  Noc0 = 0,
  Noc1 = 1,
};
enum class NocMode : uint8_t {
  DM_DEDICATED_NOC = 0,
  DM_DYNAMIC_NOC = 1,
};
enum class OOBVal : uint16_t {
  Undef = 0,
  Zero = 1,
  One = 2,
  Inf = 3,
  NegInf = 4,
};
enum class PlacementType : uint16_t {
  Replicate = 0,
  Shard = 1,
};
enum class Pool2dOpType : uint32_t {
  AvgPool2d = 0,
  MaxPool2d = 1,
};
enum class ReductionOpType : uint32_t {
  Sum = 0,
  Mean = 1,
  Max = 2,
  Min = 3,
};
enum class RoutingMode : uint16_t {
  BidirLineMesh = 0,
  UnidirRingTorus = 1,
};
enum class ScatterReduceType : uint8_t {
  Sum = 0,
  Max = 2,
  Min = 3,
  Prod = 6,
  Invalid = 7,
};
enum class ShardDistributionStrategy : uint32_t {
  RoundRobin1D = 0,
  Grid2D = 1,
};
enum class ShardOrientation : uint32_t {
  RowMajor = 0,
  ColMajor = 1,
};
enum class ShardStatus : uint32_t {
  Presharded = 0,
  Unsharded = 1,
};
enum class SliceOpType : uint32_t {
  SliceStaticOp = 0,
  SliceDynamicOp = 1,
};
enum class SourceType : uint8_t {
  FILE_PATH = 0,
  SOURCE_CODE = 1,
};
enum class StorageType : uint16_t {
  Host = 0,
  Device = 1,
};
enum class TensorLayout : uint16_t {
  RowMajor = 0,
  Tile = 1,
  Invalid = 2,
};
enum class TensorMemoryLayout : uint16_t {
  Interleaved = 0,
  HeightSharded = 1,
  WidthSharded = 2,
  BlockSharded = 3,
  NDSharded = 4,
};
enum class Topology : uint16_t {
  Ring = 0,
  Linear = 1,
  Mesh = 2,
  Torus = 3,
};
enum class UnaryOpType : uint32_t {
  Exp = 0,
  Recip = 1,
  Gelu = 2,
  Relu = 3,
  Sqrt = 4,
  Sigmoid = 5,
  Log = 6,
  Tanh = 7,
  Log2 = 8,
  Log10 = 9,
  Sin = 10,
  Cos = 11,
  Abs = 12,
  AbsInt32 = 13,
  Sign = 14,
  Square = 15,
  Eqz = 16,
  Nez = 17,
  Gtz = 18,
  Ltz = 19,
  Gez = 20,
  Lez = 21,
  ReluMax = 22,
  ReluMin = 23,
  Power = 24,
  LeakyRelu = 25,
  Elu = 26,
  Exp2 = 27,
  Heaviside = 28,
  Expm1 = 29,
  Signbit = 30,
  Asin = 31,
  Acos = 32,
  Rsqrt = 33,
  Relu6 = 34,
  Hardsigmoid = 35,
  Atan = 36,
  Erf = 37,
  Erfc = 38,
  Isinf = 39,
  Isposinf = 40,
  Isneginf = 41,
  Isnan = 42,
  LogicalNotUnary = 43,
  Isfinite = 44,
  Erfinv = 45,
  I0 = 46,
  I1 = 47,
  Tan = 48,
  Rsub = 49,
  Rdiv = 50,
  Silu = 51,
  Softplus = 52,
  Identity = 53,
  Neg = 54,
  AddUnarySfpu = 55,
  SubUnarySfpu = 56,
  MulUnarySfpu = 57,
  DivUnarySfpu = 58,
  IdentityUint32 = 59,
  UnaryNe = 60,
  UnaryGt = 61,
  UnaryLt = 62,
  TiledProd = 63,
  Typecast = 64,
  BitwiseXor = 65,
  BitwiseNot = 66,
  BitwiseAnd = 67,
  BitwiseOr = 68,
  RightShift = 69,
  Floor = 70,
  Ceil = 71,
  Round = 72,
  LeftShift = 73,
  Remainder = 74,
  Fmod = 75,
  Dropout = 76,
  Fill = 77,
  PreluSfpu = 78,
  ZeroPoint = 79,
};
enum class UnpackToDestMode : uint8_t {
  Fp32 = 0,
  Default = 1,
};
enum class ArgRef : uint8_t {
  NONE = 0,
  TensorRef = 1,
  GlobalSemaphoreRef = 2,
};
enum class EltwiseQuantizationOpParams : uint8_t {
  NONE = 0,
  QuantizeDequantizeOpParams = 1,
  RequantizeOpParams = 2,
};
enum class EltwiseUnaryCompositeOpParams : uint8_t {
  NONE = 0,
  ClampScalarOpParams = 1,
  ClampTensorOpParams = 2,
};
enum class EltwiseUnaryOpParams : uint8_t {
  NONE = 0,
  EltwiseOpWithFloatParams = 1,
};
enum class KernelArgType : uint8_t {
  NONE = 0,
  KernelArgCBBufferIndex = 1,
  KernelArgBufferAddress = 2,
  KernelArgBufferAddressOfTensor = 3,
  KernelArgSemaphoreAt = 4,
  KernelArgNamedArgument = 5,
  KernelArgGlobalSemaphore = 6,
  KernelArgScalar = 7,
  KernelArgTensorAccessorArgs = 8,
};
enum class KernelConfig : uint8_t {
  NONE = 0,
  ComputeKernelConfig = 1,
  DataMovementKernelConfig = 2,
  ReaderKernelConfig = 3,
  WriterKernelConfig = 4,
};
enum class MatmulProgramConfig : uint8_t {
  NONE = 0,
  MatmulMultiCoreReuseProgramConfig = 1,
  MatmulMultiCoreReuseMultiCastProgramConfig = 2,
  MatmulMultiCoreReuseMultiCast1DProgramConfig = 3,
  MatmulMultiCoreReuseMultiCastDRAMShardedProgramConfig = 4,
};
enum class NumberType : uint8_t {
  NONE = 0,
  FP = 1,
  I32 = 2,
};
enum class OpType : uint8_t {
  NONE = 0,
  AdamWOp = 1,
  AggregateTensorOp = 2,
  AllGatherOp = 3,
  AllReduceAsyncOp = 4,
  AllReduceOp = 5,
  AllToAllCombineOp = 6,
  AllToAllDispatchMetadataOp = 7,
  AllToAllDispatchOp = 8,
  ArangeOp = 9,
  AssignOp = 10,
  BatchNormInferenceOp = 11,
  BatchNormTrainingOp = 12,
  BitcastConvertOp = 13,
  BeginTraceCaptureOp = 14,
  CaptureOrExecuteTraceOp = 15,
  ChunkedScaledDotProductAttentionOp = 16,
  ConcatOp = 17,
  ConcatenateHeadsOp = 18,
  RotaryEmbeddingLlamaOp = 19,
  RotaryEmbeddingOp = 20,
  NLPCreateQKVHeadsDecodeOp = 21,
  NLPConcatHeadsOp = 22,
  ConstantOp = 23,
  Conv1dOp = 24,
  Conv2dOp = 25,
  ConvTranspose2dOp = 26,
  Conv3dOp = 27,
  CpuOp = 28,
  DeallocateOp = 29,
  DistributeTensorOp = 30,
  DistributedRMSNormOp = 31,
  DitRMSNormUnaryFusedOp = 32,
  DropoutOp = 33,
  EltwiseBinaryCompositeOp = 34,
  EltwiseBinaryCompositeScalarOp = 35,
  EltwiseBinaryOp = 36,
  EltwiseQuantizationOp = 37,
  EltwiseTernaryWhereOp = 38,
  EltwiseUnaryCompositeOp = 39,
  EltwiseUnaryOp = 40,
  EmbeddingBackwardOp = 41,
  EmbeddingOp = 42,
  EmptyOp = 43,
  EndTraceCaptureOp = 44,
  ExecuteTraceOp = 45,
  ExperimentalEltwiseBinaryBackwardOp = 46,
  FillCacheOp = 47,
  FromDeviceOp = 48,
  FullOp = 49,
  FuncCallOp = 50,
  GatherOp = 51,
  GenericOp = 52,
  GetDeviceOp = 53,
  GlobalAvgPool2dOp = 54,
  GroupNormOp = 55,
  IndexerScoreDsaOp = 56,
  LayerNormOp = 57,
  LayerNormPreAllGatherOp = 58,
  LayerNormPostAllGatherOp = 59,
  LinearOp = 60,
  LoadCachedOp = 61,
  MatmulOp = 62,
  SparseMatmulOp = 63,
  MaxPool2dWithIndicesOp = 64,
  MeshPartitionOp = 65,
  MoeExpertTokenRemapOp = 66,
  MoeGptOp = 67,
  PrepareMoEComputeW0W1WeightsOp = 68,
  PrepareMoEComputeW2WeightsOp = 69,
  MoeComputeOp = 70,
  CumSumOp = 71,
  CumProdOp = 72,
  NamedFullOp = 73,
  NLPConcatHeadsDecodeOp = 74,
  PadOp = 75,
  PagedFillCacheOp = 76,
  PagedFlashMultiLatentAttentionDecodeOp = 77,
  PagedScaledDotProductAttentionDecodeOp = 78,
  PagedUpdateCacheOp = 79,
  PermuteOp = 80,
  PointToPointOp = 81,
  Pool2dOp = 82,
  PrepareConv2dBiasOp = 83,
  PrepareConv2dWeightsOp = 84,
  PrepareConv3dWeightsOp = 85,
  PrepareConvTranspose2dBiasOp = 86,
  PrepareConvTranspose2dWeightsOp = 87,
  RandOp = 88,
  ReductionArgMaxOp = 89,
  ReductionOp = 90,
  ReductionProdOp = 91,
  ReduceScatterOp = 92,
  RepeatInterleaveOp = 93,
  RepeatOp = 94,
  RMSNormPreAllGatherOp = 95,
  RMSNormOp = 96,
  ReshapeOp = 97,
  SamplingOp = 98,
  ScaledDotProductAttentionOp = 99,
  ScaledDotProductAttentionDecodeOp = 100,
  FlashMlaPrefillOp = 101,
  ScatterOp = 102,
  SDPAForwardOp = 103,
  SDPABackwardOp = 104,
  SelectiveReduceCombineOp = 105,
  SliceOp = 106,
  SoftmaxOp = 107,
  SortOp = 108,
  SplitQueryKeyValueAndSplitHeadsOp = 109,
  ToDeviceOp = 110,
  ToLayoutOp = 111,
  ToMemoryConfigOp = 112,
  TransposeOp = 113,
  TypecastOp = 114,
  UpdateCacheOp = 115,
  UpsampleOp = 116,
  WriteTensorOp = 117,
  DumpTensorOp = 118,
  LoadTensorOp = 119,
  AnnotateOp = 120,
  BreakpointOp = 121,
  PrintOp = 122,
  MemorySnapshotOp = 123,
  RegionStartOp = 124,
  RegionEndOp = 125,
  TopKOp = 126,
  TopKRouterGptOp = 127,
  CreateGlobalSemaphoreOp = 128,
  ResetGlobalSemaphoreOp = 129,
  AllocateMoeComputeSemaphoreOp = 130,
  CopyOp = 131,
};
enum class Pool2dExtraParams : uint8_t {
  NONE = 0,
  AvgPool2dExtraParams = 1,
  MaxPool2dExtraParams = 2,
};
enum class ProgramType : uint8_t {
  NONE = 0,
  ProgramDescriptor = 1,
  MeshProgramDescriptor = 2,
};
enum class QuantizationScale : uint8_t {
  NONE = 0,
  PerTensorScale = 1,
  PerAxisScale = 2,
};
enum class QuantizationZeroPoint : uint8_t {
  NONE = 0,
  PerTensorZeroPoint = 1,
  PerAxisZeroPoint = 2,
};
enum class Scale2D : uint8_t {
  NONE = 0,
  UniformScale2D = 1,
  NonUniformScale2D = 2,
};
enum class SliceOpParams : uint8_t {
  NONE = 0,
  SliceStaticOpParams = 1,
  SliceDynamicOpParams = 2,
};

struct AdamWOp {
  enum : int {
    f_param = 0,
    f_grad = 1,
    f_exp_avg = 2,
    f_exp_avg_sq = 3,
    f_max_exp_avg_sq = 4,
    f_lr = 5,
    f_beta1 = 6,
    f_beta2 = 7,
    f_beta1_pow = 8,
    f_beta2_pow = 9,
    f_epsilon = 10,
    f_weight_decay = 11,
    f_stochastic_rounding = 12,
    kNumFields = 13
  };
};
struct AggregateTensorOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_composer_config = 2,
    f_device = 3,
    kNumFields = 4
  };
};
struct AllGatherOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_all_gather_dim = 2,
    f_cluster_axis = 3,
    f_sub_device_id = 4,
    f_memory_config = 5,
    f_num_links = 6,
    f_topology = 7,
    kNumFields = 8
  };
};
struct AllGatherTensor {
  enum : int {
    kNumFields = 0
  };
};
struct AllReduceAsyncOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_reduce_type = 2,
    f_cluster_axis = 3,
    f_sub_device_id = 4,
    f_memory_config = 5,
    f_num_links = 6,
    f_topology = 7,
    kNumFields = 8
  };
};
struct AllReduceOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_reduce_type = 2,
    f_cluster_axis = 3,
    f_sub_device_id = 4,
    f_memory_config = 5,
    f_num_links = 6,
    f_topology = 7,
    kNumFields = 8
  };
};
struct AllToAllCombineOp {
  enum : int {
    f_input_tensor = 0,
    f_expert_metadata = 1,
    f_expert_mapping = 2,
    f_out = 3,
    f_num_devices = 4,
    f_cluster_axis = 5,
    f_num_experts_per_tok = 6,
    f_output_shard_dim = 7,
    f_memory_config = 8,
    kNumFields = 9
  };
};
struct AllToAllDispatchMetadataOp {
  enum : int {
    f_input_tensor = 0,
    f_expert_indices = 1,
    f_expert_scores = 2,
    f_expert_mapping = 3,
    f_dispatched = 4,
    f_indices = 5,
    f_scores = 6,
    f_num_devices = 7,
    f_cluster_axis = 8,
    f_memory_config = 9,
    f_dispatched_buffer = 10,
    f_indices_buffer = 11,
    f_scores_buffer = 12,
    f_cross_device_semaphore = 13,
    kNumFields = 14
  };
};
struct AllToAllDispatchOp {
  enum : int {
    f_input_tensor = 0,
    f_expert_indices = 1,
    f_expert_mapping = 2,
    f_dispatched = 3,
    f_metadata = 4,
    f_num_devices = 5,
    f_cluster_axis = 6,
    f_memory_config = 7,
    kNumFields = 8
  };
};
struct AllocateMoeComputeSemaphoreOp {
  enum : int {
    f_core_range_set = 0,
    f_output_height_shard_dim = 1,
    f_hidden_size = 2,
    f_initial_value = 3,
    f_out = 4,
    kNumFields = 5
  };
};
struct AnnotateOp {
  enum : int {
    f_operand = 0,
    f_result = 1,
    f_annotation = 2,
    kNumFields = 3
  };
};
struct ArangeOp {
  enum : int {
    f_device = 0,
    f_start = 1,
    f_end = 2,
    f_step = 3,
    f_dtype = 4,
    f_layout = 5,
    f_memcfg = 6,
    f_out = 7,
    kNumFields = 8
  };
};
struct AssignOp {
  enum : int {
    f_input = 0,
    f_output = 1,
    f_output_memory_config = 2,
    f_output_dtype = 3,
    kNumFields = 4
  };
};
struct AvgPool2dExtraParams {
  enum : int {
    f_count_include_pad = 0,
    kNumFields = 1
  };
};
struct BatchNormInferenceOp {
  enum : int {
    f_input = 0,
    f_running_mean = 1,
    f_running_var = 2,
    f_epsilon = 3,
    f_weight = 4,
    f_bias = 5,
    f_memory_config = 6,
    f_out = 7,
    f_compute_config = 8,
    kNumFields = 9
  };
};
struct BatchNormTrainingOp {
  enum : int {
    f_input = 0,
    f_running_mean = 1,
    f_running_var = 2,
    f_epsilon = 3,
    f_momentum = 4,
    f_weight = 5,
    f_bias = 6,
    f_memory_config = 7,
    f_out = 8,
    f_compute_config = 9,
    kNumFields = 10
  };
};
struct BeginTraceCaptureOp {
  enum : int {
    f_device = 0,
    f_trace_id = 1,
    f_cq_id = 2,
    kNumFields = 3
  };
};
struct BitcastConvertOp {
  enum : int {
    f_in = 0,
    f_dtype = 1,
    f_memcfg = 2,
    f_out = 3,
    kNumFields = 4
  };
};
struct BreakpointOp {
  enum : int {
    f_operand = 0,
    kNumFields = 1
  };
};
struct CPUDesc {
  enum : int {
    f_role = 0,
    f_target_triple = 1,
    kNumFields = 2
  };
};
struct CaptureOrExecuteTraceOp {
  enum : int {
    f_device = 0,
    f_capture_program_id = 1,
    f_execute_program_id = 2,
    f_allocate_slots_program_id = 3,
    f_inputs = 4,
    f_outputs = 5,
    f_semaphore_inputs = 6,
    kNumFields = 7
  };
};
struct ChipDesc {
  enum : int {
    f_arch = 0,
    f_grid_size = 1,
    f_coord_translation_offsets = 2,
    f_l1_size = 3,
    f_num_dram_channels = 4,
    f_dram_channel_size = 5,
    f_noc_l1_address_align_bytes = 6,
    f_pcie_address_align_bytes = 7,
    f_noc_dram_address_align_bytes = 8,
    f_l1_unreserved_base = 9,
    f_erisc_l1_unreserved_base = 10,
    f_dram_unreserved_base = 11,
    f_dram_unreserved_end = 12,
    f_supported_data_types = 13,
    f_supported_tile_sizes = 14,
    f_dst_physical_size_tiles = 15,
    f_num_cbs = 16,
    f_num_compute_threads = 17,
    f_num_datamovement_threads = 18,
    f_dram_grid_size = 19,
    f_dram_bank_to_logical_worker_noc0 = 20,
    f_dram_bank_to_logical_worker_noc1 = 21,
    kNumFields = 22
  };
};
struct ChunkedScaledDotProductAttentionOp {
  enum : int {
    f_query = 0,
    f_key = 1,
    f_value = 2,
    f_page_table = 3,
    f_chunk_start_idx = 4,
    f_scale = 5,
    f_out = 6,
    f_memcfg = 7,
    f_program_config = 8,
    kNumFields = 9
  };
};
struct ClampScalarOpParams {
  enum : int {
    f_min_type = 0,
    f_min = 1,
    f_max_type = 2,
    f_max = 3,
    kNumFields = 4
  };
};
struct ClampTensorOpParams {
  enum : int {
    f_min = 0,
    f_max = 1,
    kNumFields = 2
  };
};
struct ComputeKernelConfig {
  enum : int {
    f_math_fidelity = 0,
    f_fp32_dest_acc_en = 1,
    f_dst_full_sync_en = 2,
    f_unpack_to_dest_modes = 3,
    f_bfp8_pack_precise = 4,
    f_math_approx_mode = 5,
    kNumFields = 6
  };
};
struct ConcatOp {
  enum : int {
    f_inputs = 0,
    f_out = 1,
    f_dim = 2,
    f_memory_config = 3,
    kNumFields = 4
  };
};
struct ConcatenateHeadsOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_memcfg = 2,
    kNumFields = 3
  };
};
struct ConstantOp {
  enum : int {
    f_device = 0,
    f_input = 1,
    f_input_dtype = 2,
    f_dtype = 3,
    f_layout = 4,
    f_memcfg = 5,
    f_out = 6,
    kNumFields = 7
  };
};
struct Conv1dOp {
  enum : int {
    f_input = 0,
    f_weight = 1,
    f_bias = 2,
    f_out = 3,
    f_device = 4,
    f_in_channels = 5,
    f_out_channels = 6,
    f_batch_size = 7,
    f_input_length = 8,
    f_kernel_size = 9,
    f_stride = 10,
    f_padding = 11,
    f_dilation = 12,
    f_groups = 13,
    f_output_dtype = 14,
    f_conv2d_config = 15,
    f_compute_config = 16,
    f_conv2d_slice_config = 17,
    kNumFields = 18
  };
};
struct Conv2dConfig {
  enum : int {
    f_weights_dtype = 0,
    f_activation = 1,
    f_deallocate_activation = 2,
    f_reallocate_halo_output = 3,
    f_act_block_h_override = 4,
    f_act_block_w_div = 5,
    f_reshard_if_not_optimal = 6,
    f_override_sharding_config = 7,
    f_shard_layout = 8,
    f_core_grid = 9,
    f_transpose_shards = 10,
    f_output_layout = 11,
    f_enable_act_double_buffer = 12,
    f_enable_weights_double_buffer = 13,
    f_enable_kernel_stride_folding = 14,
    f_config_tensors_in_dram = 15,
    kNumFields = 16
  };
};
struct Conv2dOp {
  enum : int {
    f_input = 0,
    f_weight = 1,
    f_bias = 2,
    f_out = 3,
    f_device = 4,
    f_in_channels = 5,
    f_out_channels = 6,
    f_batch_size = 7,
    f_input_height = 8,
    f_input_width = 9,
    f_kernel_size = 10,
    f_stride = 11,
    f_padding = 12,
    f_dilation = 13,
    f_groups = 14,
    f_output_dtype = 15,
    f_conv2d_config = 16,
    f_compute_config = 17,
    f_conv2d_slice_config = 18,
    kNumFields = 19
  };
};
struct Conv2dSliceConfig {
  enum : int {
    f_slice_type = 0,
    f_num_slices = 1,
    kNumFields = 2
  };
};
struct Conv3dConfig {
  enum : int {
    f_weights_dtype = 0,
    f_t_out_block = 1,
    f_w_out_block = 2,
    f_h_out_block = 3,
    f_c_out_block = 4,
    f_c_in_block = 5,
    f_compute_with_storage_grid_size = 6,
    kNumFields = 7
  };
};
struct Conv3dOp {
  enum : int {
    f_input = 0,
    f_weight = 1,
    f_bias = 2,
    f_out = 3,
    f_device = 4,
    f_in_channels = 5,
    f_out_channels = 6,
    f_batch_size = 7,
    f_input_depth = 8,
    f_input_height = 9,
    f_input_width = 10,
    f_kernel_size = 11,
    f_stride = 12,
    f_padding = 13,
    f_padding_mode = 14,
    f_groups = 15,
    f_output_dtype = 16,
    f_conv3d_config = 17,
    f_compute_config = 18,
    f_memory_config = 19,
    kNumFields = 20
  };
};
struct ConvTranspose2dOp {
  enum : int {
    f_input = 0,
    f_weight = 1,
    f_bias = 2,
    f_out = 3,
    f_device = 4,
    f_in_channels = 5,
    f_out_channels = 6,
    f_batch_size = 7,
    f_input_height = 8,
    f_input_width = 9,
    f_kernel_size = 10,
    f_stride = 11,
    f_padding = 12,
    f_output_padding = 13,
    f_dilation = 14,
    f_groups = 15,
    f_output_dtype = 16,
    f_conv2d_config = 17,
    f_compute_config = 18,
    f_memory_config = 19,
    f_conv2d_slice_config = 20,
    kNumFields = 21
  };
};
struct CopyOp {
  enum : int {
    f_src = 0,
    f_dst = 1,
    kNumFields = 2
  };
};
struct CoreRangeSet {
  enum : int {
    f_core_ranges = 0,
    kNumFields = 1
  };
};
struct CoreRuntimeArgs {
  enum : int {
    f_core_coord = 0,
    f_args = 1,
    kNumFields = 2
  };
};
struct CpuOp {
  enum : int {
    f_ins = 0,
    f_outs = 1,
    f_func_name = 2,
    f_dylib_id = 3,
    kNumFields = 4
  };
};
struct CreateGlobalSemaphoreOp {
  enum : int {
    f_core_range_set = 0,
    f_initial_value = 1,
    f_out = 2,
    kNumFields = 3
  };
};
struct CumProdOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_dim = 2,
    f_dtype = 3,
    f_memcfg = 4,
    kNumFields = 5
  };
};
struct CumSumOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_dim = 2,
    f_dtype = 3,
    f_memcfg = 4,
    kNumFields = 5
  };
};
struct DataMovementKernelConfig {
  enum : int {
    f_processor = 0,
    f_noc = 1,
    f_noc_mode = 2,
    kNumFields = 3
  };
};
struct DeallocateOp {
  enum : int {
    f_in = 0,
    f_force = 1,
    kNumFields = 2
  };
};
struct DebugInfo {
  enum : int {
    f_cpp = 0,
    f_mlir_stages = 1,
    f_golden_info = 2,
    kNumFields = 3
  };
};
struct DeviceComputeKernelConfig {
  enum : int {
    f_math_fidelity = 0,
    f_math_approx_mode = 1,
    f_fp32_dest_acc_en = 2,
    f_packer_l1_acc = 3,
    f_dst_full_sync_en = 4,
    kNumFields = 5
  };
};
struct DeviceRef {
  enum : int {
    f_global_id = 0,
    kNumFields = 1
  };
};
struct DistributeTensorOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_mapper_config = 2,
    f_device = 3,
    f_cq_id = 4,
    kNumFields = 5
  };
};
struct DistributedRMSNormOp {
  enum : int {
    f_input = 0,
    f_weight = 1,
    f_residual = 2,
    f_cluster_axis = 3,
    f_epsilon = 4,
    f_sub_device_id = 5,
    f_memory_config = 6,
    f_num_links = 7,
    f_topology = 8,
    f_compute_config = 9,
    f_stats = 10,
    f_program_config = 11,
    f_out = 12,
    f_semaphore = 13,
    kNumFields = 14
  };
};
struct DitRMSNormUnaryFusedOp {
  enum : int {
    f_input = 0,
    f_weight = 1,
    f_bias = 2,
    f_residual_input = 3,
    f_epsilon = 4,
    f_activation = 5,
    f_memory_config = 6,
    f_compute_config = 7,
    f_out = 8,
    kNumFields = 9
  };
};
struct DropoutOp {
  enum : int {
    f_in = 0,
    f_prob = 1,
    f_scale = 2,
    f_seed = 3,
    f_use_per_device_seed = 4,
    f_output_dtype = 5,
    f_memory_config = 6,
    f_out = 7,
    kNumFields = 8
  };
};
struct DumpTensorOp {
  enum : int {
    f_file_path = 0,
    f_in = 1,
    kNumFields = 2
  };
};
struct DynamicLib {
  enum : int {
    f_dylib_id = 0,
    f_raw_file = 1,
    kNumFields = 2
  };
};
struct EltwiseBinaryCompositeOp {
  enum : int {
    f_type = 0,
    f_lhs = 1,
    f_rhs = 2,
    f_memory_config = 3,
    f_out = 4,
    kNumFields = 5
  };
};
struct EltwiseBinaryCompositeScalarOp {
  enum : int {
    f_type = 0,
    f_lhs = 1,
    f_rhs_type = 2,
    f_rhs = 3,
    f_memory_config = 4,
    f_out = 5,
    kNumFields = 6
  };
};
struct EltwiseBinaryOp {
  enum : int {
    f_type = 0,
    f_lhs = 1,
    f_rhs = 2,
    f_output_dtype = 3,
    f_memory_config = 4,
    f_out = 5,
    kNumFields = 6
  };
};
struct EltwiseOpWithFloatParams {
  enum : int {
    f_parameter = 0,
    kNumFields = 1
  };
};
struct EltwiseQuantizationOp {
  enum : int {
    f_type = 0,
    f_in = 1,
    f_axis = 2,
    f_output_dtype = 3,
    f_memory_config = 4,
    f_out = 5,
    f_params_type = 6,
    f_params = 7,
    kNumFields = 8
  };
};
struct EltwiseTernaryWhereOp {
  enum : int {
    f_first = 0,
    f_second = 1,
    f_third = 2,
    f_memory_config = 3,
    f_out = 4,
    kNumFields = 5
  };
};
struct EltwiseUnaryCompositeOp {
  enum : int {
    f_type = 0,
    f_in = 1,
    f_memory_config = 2,
    f_out = 3,
    f_params_type = 4,
    f_params = 5,
    kNumFields = 6
  };
};
struct EltwiseUnaryOp {
  enum : int {
    f_type = 0,
    f_in = 1,
    f_memory_config = 2,
    f_out = 3,
    f_params_type = 4,
    f_params = 5,
    kNumFields = 6
  };
};
struct EmbeddingBackwardOp {
  enum : int {
    f_input = 0,
    f_weight = 1,
    f_in_grad = 2,
    f_dtype = 3,
    f_memcfg = 4,
    f_out = 5,
    kNumFields = 6
  };
};
struct EmbeddingOp {
  enum : int {
    f_input = 0,
    f_weight = 1,
    f_out = 2,
    kNumFields = 3
  };
};
struct EmptyOp {
  enum : int {
    f_device = 0,
    f_shape = 1,
    f_dtype = 2,
    f_layout = 3,
    f_memcfg = 4,
    f_out = 5,
    kNumFields = 6
  };
};
struct EndTraceCaptureOp {
  enum : int {
    f_device = 0,
    f_trace_id = 1,
    f_cq_id = 2,
    kNumFields = 3
  };
};
struct EventRef {
  enum : int {
    f_global_id = 0,
    kNumFields = 1
  };
};
struct ExecuteTraceOp {
  enum : int {
    f_device = 0,
    f_trace_id = 1,
    f_cq_id = 2,
    f_blocking = 3,
    kNumFields = 4
  };
};
struct ExperimentalEltwiseBinaryBackwardOp {
  enum : int {
    f_type = 0,
    f_grad = 1,
    f_input = 2,
    f_approximate = 3,
    f_output_dtype = 4,
    f_memory_config = 5,
    f_out = 6,
    kNumFields = 7
  };
};
struct FabricConnectionConfig {
  enum : int {
    f_noc_index = 0,
    f_topology = 1,
    f_cluster_axis = 2,
    f_routing_mode = 3,
    f_num_links = 4,
    kNumFields = 5
  };
};
struct FillCacheOp {
  enum : int {
    f_cache = 0,
    f_input = 1,
    f_batch_offset = 2,
    kNumFields = 3
  };
};
struct FlashMlaPrefillOp {
  enum : int {
    f_query = 0,
    f_key = 1,
    f_value = 2,
    f_attention_mask = 3,
    f_head_dim_v = 4,
    f_is_causal = 5,
    f_scale = 6,
    f_out = 7,
    f_memcfg = 8,
    kNumFields = 9
  };
};
struct FloatingPointType {
  enum : int {
    f_value = 0,
    kNumFields = 1
  };
};
struct FromDeviceOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    kNumFields = 2
  };
};
struct FullOp {
  enum : int {
    f_device = 0,
    f_shape = 1,
    f_fill_value_type = 2,
    f_fill_value = 3,
    f_dtype = 4,
    f_layout = 5,
    f_memcfg = 6,
    f_out = 7,
    kNumFields = 8
  };
};
struct FuncCallOp {
  enum : int {
    f_program_id = 0,
    f_inputs = 1,
    f_outputs = 2,
    f_semaphore_inputs = 3,
    kNumFields = 4
  };
};
struct GatherOp {
  enum : int {
    f_input = 0,
    f_index = 1,
    f_out = 2,
    f_dim = 3,
    f_memory_config = 4,
    kNumFields = 5
  };
};
struct GenericOp {
  enum : int {
    f_io_tensors = 0,
    f_additional_args = 1,
    f_program_type = 2,
    f_program = 3,
    kNumFields = 4
  };
};
struct GetDeviceOp {
  enum : int {
    f_mesh = 0,
    f_offset = 1,
    f_chip_ids = 2,
    f_out = 3,
    kNumFields = 4
  };
};
struct GlobalAvgPool2dOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_memory_config = 2,
    f_dtype = 3,
    kNumFields = 4
  };
};
struct GlobalSemaphoreRef {
  enum : int {
    f_global_id = 0,
    kNumFields = 1
  };
};
struct GoldenDeviceTensor {
  enum : int {
    f_device = 0,
    f_value = 1,
    kNumFields = 2
  };
};
struct GoldenInfo {
  enum : int {
    f_golden_map = 0,
    kNumFields = 1
  };
};
struct GoldenKV {
  enum : int {
    f_key = 0,
    f_value = 1,
    kNumFields = 2
  };
};
struct GoldenTensor {
  enum : int {
    f_name = 0,
    f_shape = 1,
    f_stride = 2,
    f_dtype = 3,
    f_data = 4,
    kNumFields = 5
  };
};
struct GroupNormOp {
  enum : int {
    f_input = 0,
    f_input_mask = 1,
    f_weight = 2,
    f_bias = 3,
    f_num_groups = 4,
    f_epsilon = 5,
    f_memory_config = 6,
    f_out = 7,
    kNumFields = 8
  };
};
struct IndexerScoreDsaOp {
  enum : int {
    f_query = 0,
    f_key = 1,
    f_weights = 2,
    f_chunk_start_idx = 3,
    f_out = 4,
    f_cluster_axis = 5,
    kNumFields = 6
  };
};
struct IntegralType {
  enum : int {
    f_value = 0,
    kNumFields = 1
  };
};
struct KernelArg {
  enum : int {
    f_arg_type = 0,
    f_arg = 1,
    kNumFields = 2
  };
};
struct KernelArgBufferAddress {
  enum : int {
    f_address = 0,
    kNumFields = 1
  };
};
struct KernelArgBufferAddressOfTensor {
  enum : int {
    f_operand_index = 0,
    kNumFields = 1
  };
};
struct KernelArgCBBufferIndex {
  enum : int {
    f_buffer_index = 0,
    kNumFields = 1
  };
};
struct KernelArgGlobalSemaphore {
  enum : int {
    f_operand_index = 0,
    kNumFields = 1
  };
};
struct KernelArgNamedArgument {
  enum : int {
    f_name = 0,
    f_value = 1,
    kNumFields = 2
  };
};
struct KernelArgScalar {
  enum : int {
    f_operand_index = 0,
    kNumFields = 1
  };
};
struct KernelArgSemaphoreAt {
  enum : int {
    f_semaphore_index = 0,
    kNumFields = 1
  };
};
struct KernelArgTensorAccessorArgs {
  enum : int {
    f_operand_index = 0,
    kNumFields = 1
  };
};
struct KernelCBDescriptor {
  enum : int {
    f_total_size = 0,
    f_core_range = 1,
    f_formats = 2,
    f_buffer = 3,
    kNumFields = 4
  };
};
struct KernelCBFormat {
  enum : int {
    f_buffer_index = 0,
    f_dtype = 1,
    f_page_size = 2,
    kNumFields = 3
  };
};
struct KernelCoreArgs {
  enum : int {
    f_args = 0,
    kNumFields = 1
  };
};
struct KernelDescriptor {
  enum : int {
    f_source = 0,
    f_source_type = 1,
    f_config_type = 2,
    f_config = 3,
    f_core_ranges = 4,
    f_ct_args = 5,
    f_rt_args = 6,
    f_common_rt_args = 7,
    kNumFields = 8
  };
};
struct KernelGlobalCBIndexOfTensor {
  enum : int {
    f_tensor_operand_index = 0,
    kNumFields = 1
  };
};
struct LayerNormOp {
  enum : int {
    f_input = 0,
    f_weight = 1,
    f_bias = 2,
    f_epsilon = 3,
    f_memory_config = 4,
    f_out = 5,
    kNumFields = 6
  };
};
struct LayerNormPostAllGatherOp {
  enum : int {
    f_input = 0,
    f_stats = 1,
    f_weight = 2,
    f_bias = 3,
    f_epsilon = 4,
    f_dtype = 5,
    f_memory_config = 6,
    f_compute_config = 7,
    f_program_config = 8,
    f_out = 9,
    kNumFields = 10
  };
};
struct LayerNormPreAllGatherOp {
  enum : int {
    f_input = 0,
    f_residual_input = 1,
    f_recip = 2,
    f_dtype = 3,
    f_memory_config = 4,
    f_compute_config = 5,
    f_program_config = 6,
    f_out = 7,
    kNumFields = 8
  };
};
struct LayerNormShardedMultiCoreProgramConfig {
  enum : int {
    f_compute_with_storage_grid_size = 0,
    f_subblock_w = 1,
    f_block_h = 2,
    f_block_w = 3,
    f_inplace = 4,
    kNumFields = 5
  };
};
struct LayoutDesc {
  enum : int {
    f_oob_val = 0,
    f_memory_desc = 1,
    kNumFields = 2
  };
};
struct LinearOp {
  enum : int {
    f_a = 0,
    f_b = 1,
    f_bias = 2,
    f_out = 3,
    f_transpose_a = 4,
    f_transpose_b = 5,
    f_matmul_program_config_type = 6,
    f_matmul_program_config = 7,
    f_activation = 8,
    f_compute_config = 9,
    kNumFields = 10
  };
};
struct LoadCachedOp {
  enum : int {
    f_inputs = 0,
    f_callee_name = 1,
    f_program_idx = 2,
    f_outputs = 3,
    f_program_hash = 4,
    kNumFields = 5
  };
};
struct LoadTensorOp {
  enum : int {
    f_file_path = 0,
    f_device = 1,
    f_out = 2,
    kNumFields = 3
  };
};
struct MLIR {
  enum : int {
    f_name = 0,
    f_source = 1,
    kNumFields = 2
  };
};
struct MatmulMultiCoreReuseMultiCast1DProgramConfig {
  enum : int {
    f_compute_with_storage_grid_size = 0,
    f_in0_block_w = 1,
    f_out_subblock_h = 2,
    f_out_subblock_w = 3,
    f_out_block_h = 4,
    f_out_block_w = 5,
    f_per_core_m = 6,
    f_per_core_n = 7,
    f_fuse_batch = 8,
    f_fused_activation = 9,
    f_mcast_in0 = 10,
    f_gather_in0 = 11,
    f_hop_cores = 12,
    f_num_global_cb_receivers = 13,
    f_untilize_out = 14,
    kNumFields = 15
  };
};
struct MatmulMultiCoreReuseMultiCastDRAMShardedProgramConfig {
  enum : int {
    f_in0_block_w = 0,
    f_per_core_m = 1,
    f_per_core_n = 2,
    f_fused_activation = 3,
    kNumFields = 4
  };
};
struct MatmulMultiCoreReuseMultiCastProgramConfig {
  enum : int {
    f_compute_with_storage_grid_size = 0,
    f_in0_block_w = 1,
    f_out_subblock_h = 2,
    f_out_subblock_w = 3,
    f_out_block_h = 4,
    f_out_block_w = 5,
    f_per_core_m = 6,
    f_per_core_n = 7,
    f_transpose_mcast = 8,
    f_fused_activation = 9,
    f_fuse_batch = 10,
    kNumFields = 11
  };
};
struct MatmulMultiCoreReuseProgramConfig {
  enum : int {
    f_compute_with_storage_grid_size = 0,
    f_in0_block_w = 1,
    f_out_subblock_h = 2,
    f_out_subblock_w = 3,
    f_per_core_m = 4,
    f_per_core_n = 5,
    kNumFields = 6
  };
};
struct MatmulOp {
  enum : int {
    f_a = 0,
    f_b = 1,
    f_out = 2,
    f_transpose_a = 3,
    f_transpose_b = 4,
    f_matmul_program_config_type = 5,
    f_matmul_program_config = 6,
    f_activation = 7,
    f_compute_config = 8,
    kNumFields = 9
  };
};
struct MaxPool2dExtraParams {
  enum : int {
    kNumFields = 0
  };
};
struct MaxPool2dWithIndicesOp {
  enum : int {
    f_in = 0,
    f_result = 1,
    f_result_indices = 2,
    f_batch_size = 3,
    f_input_height = 4,
    f_input_width = 5,
    f_channels = 6,
    f_kernel_size = 7,
    f_stride = 8,
    f_padding = 9,
    f_dilation = 10,
    f_memory_config = 11,
    f_applied_shard_scheme = 12,
    f_ceil_mode = 13,
    f_reallocate_halo_output = 14,
    f_config_tensors_in_dram = 15,
    kNumFields = 16
  };
};
struct MemoryConfig {
  enum : int {
    f_tensor_memory_layout = 0,
    f_buffer_type = 1,
    f_shard_spec = 2,
    f_nd_shard_spec = 3,
    kNumFields = 4
  };
};
struct MemoryDesc {
  enum : int {
    f_storage_type = 0,
    f_tile_shape = 1,
    f_data_type = 2,
    f_memory_config = 3,
    kNumFields = 4
  };
};
struct MemorySnapshotOp {
  enum : int {
    f_operand = 0,
    f_file_path = 1,
    kNumFields = 2
  };
};
struct MeshComposerConfig {
  enum : int {
    f_dims = 0,
    f_mesh_shape_override = 1,
    kNumFields = 2
  };
};
struct MeshCoord {
  enum : int {
    f_coords = 0,
    kNumFields = 1
  };
};
struct MeshCoordRange {
  enum : int {
    f_start = 0,
    f_end = 1,
    kNumFields = 2
  };
};
struct MeshMapperConfig {
  enum : int {
    f_placements = 0,
    f_mesh_shape_override = 1,
    kNumFields = 2
  };
};
struct MeshPartitionOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_dim = 2,
    f_cluster_axis = 3,
    f_memory_config = 4,
    kNumFields = 5
  };
};
struct MeshProgram {
  enum : int {
    f_device_range = 0,
    f_program = 1,
    kNumFields = 2
  };
};
struct MeshProgramDescriptor {
  enum : int {
    f_mesh_programs = 0,
    f_fabric_connection_config = 1,
    kNumFields = 2
  };
};
struct MoeComputeOp {
  enum : int {
    f_tilize_input_tensor = 0,
    f_tilize_expert_indices_tensor = 1,
    f_tilize_expert_scores_tensor = 2,
    f_tilize_expert_mapping_tensor = 3,
    f_matmul_w0_w1_tensor = 4,
    f_matmul_w2_tensor = 5,
    f_optional_output_tensor = 6,
    f_cross_device_semaphore = 7,
    f_device = 8,
    f_layer_id = 9,
    f_output_height_shard_dim = 10,
    f_intermediate_size = 11,
    f_has_bias = 12,
    f_cluster_axis = 13,
    f_activation_function = 14,
    f_num_links = 15,
    f_topology = 16,
    f_mux_core_range_set = 17,
    f_combine_output = 18,
    kNumFields = 19
  };
};
struct MoeExpertTokenRemapOp {
  enum : int {
    f_topk_tensor = 0,
    f_expert_mapping = 1,
    f_expert_metadata = 2,
    f_mapping = 3,
    f_reduced = 4,
    f_reduction_size = 5,
    f_memory_config = 6,
    kNumFields = 7
  };
};
struct MoeGptOp {
  enum : int {
    f_input_tensor = 0,
    f_expert_indices = 1,
    f_expert_scores = 2,
    f_expert_mapping = 3,
    f_w0_w1_tensor = 4,
    f_w2_tensor = 5,
    f_output_height_shard_dim = 6,
    f_output_width_shard_dim = 7,
    f_hidden_size = 8,
    f_cluster_axis = 9,
    f_token_counts = 10,
    f_activation_records = 11,
    f_token_indices = 12,
    f_tilize_out = 13,
    f_tilize_out_rm = 14,
    kNumFields = 15
  };
};
struct NDShardSpec {
  enum : int {
    f_core_range_set = 0,
    f_shape = 1,
    f_orientation = 2,
    f_distribution_strategy = 3,
    kNumFields = 4
  };
};
struct NLPConcatHeadsDecodeOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_num_heads = 2,
    f_memcfg = 3,
    kNumFields = 4
  };
};
struct NLPConcatHeadsOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_memcfg = 2,
    kNumFields = 3
  };
};
struct NLPCreateQKVHeadsDecodeOp {
  enum : int {
    f_input = 0,
    f_q_out = 1,
    f_k_out = 2,
    f_v_out = 3,
    f_num_heads = 4,
    f_num_kv_heads = 5,
    f_overlap_qk_coregrid = 6,
    f_batch_offset = 7,
    f_slice_size = 8,
    f_memcfg = 9,
    kNumFields = 10
  };
};
struct NamedFullOp {
  enum : int {
    f_type = 0,
    f_device = 1,
    f_shape = 2,
    f_dtype = 3,
    f_layout = 4,
    f_memcfg = 5,
    f_out = 6,
    kNumFields = 7
  };
};
struct NonUniformScale2D {
  enum : int {
    f_scale = 0,
    kNumFields = 1
  };
};
struct Operation {
  enum : int {
    f_type_type = 0,
    f_type = 1,
    f_debug_info = 2,
    f_loc_info = 3,
    kNumFields = 4
  };
};
struct PadOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_padding = 2,
    f_value = 3,
    f_use_multicore = 4,
    f_memcfg = 5,
    kNumFields = 6
  };
};
struct PagedFillCacheOp {
  enum : int {
    f_cache = 0,
    f_input = 1,
    f_page_table = 2,
    f_batch_idx_tensor = 3,
    kNumFields = 4
  };
};
struct PagedFlashMultiLatentAttentionDecodeOp {
  enum : int {
    f_query = 0,
    f_key = 1,
    f_value = 2,
    f_head_dim_v = 3,
    f_page_table = 4,
    f_is_causal = 5,
    f_attention_mask = 6,
    f_cur_pos_tensor = 7,
    f_attention_sink = 8,
    f_scale = 9,
    f_out = 10,
    f_memcfg = 11,
    kNumFields = 12
  };
};
struct PagedScaledDotProductAttentionDecodeOp {
  enum : int {
    f_query = 0,
    f_key = 1,
    f_value = 2,
    f_page_table = 3,
    f_is_causal = 4,
    f_attention_mask = 5,
    f_cur_pos_tensor = 6,
    f_attention_sink = 7,
    f_scale = 8,
    f_sliding_window_size = 9,
    f_out = 10,
    f_memcfg = 11,
    f_program_config = 12,
    kNumFields = 13
  };
};
struct PagedUpdateCacheOp {
  enum : int {
    f_cache = 0,
    f_input = 1,
    f_update_index = 2,
    f_share_cache = 3,
    f_page_table = 4,
    kNumFields = 5
  };
};
struct PerAxisScale {
  enum : int {
    f_scale = 0,
    kNumFields = 1
  };
};
struct PerAxisZeroPoint {
  enum : int {
    f_zero_point = 0,
    kNumFields = 1
  };
};
struct PerTensorScale {
  enum : int {
    f_scale = 0,
    kNumFields = 1
  };
};
struct PerTensorZeroPoint {
  enum : int {
    f_zero_point = 0,
    kNumFields = 1
  };
};
struct PermuteOp {
  enum : int {
    f_in = 0,
    f_permutation = 1,
    f_memory_config = 2,
    f_pad_value = 3,
    f_out = 4,
    kNumFields = 5
  };
};
struct PointToPointOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_sender_coord = 2,
    f_receiver_coord = 3,
    f_optional_output_tensor = 4,
    kNumFields = 5
  };
};
struct Pool2dOp {
  enum : int {
    f_type = 0,
    f_in = 1,
    f_out = 2,
    f_batch_size = 3,
    f_input_height = 4,
    f_input_width = 5,
    f_channels = 6,
    f_kernel_size = 7,
    f_stride = 8,
    f_padding = 9,
    f_dilation = 10,
    f_extra_params_type = 11,
    f_extra_params = 12,
    f_memory_config = 13,
    f_applied_shard_scheme = 14,
    f_ceil_mode = 15,
    f_reallocate_halo_output = 16,
    f_config_tensors_in_dram = 17,
    kNumFields = 18
  };
};
struct PrepareConv2dBiasOp {
  enum : int {
    f_bias_tensor = 0,
    f_out = 1,
    f_input_memory_config = 2,
    f_input_tensor_layout = 3,
    f_in_channels = 4,
    f_out_channels = 5,
    f_batch_size = 6,
    f_input_height = 7,
    f_input_width = 8,
    f_kernel_size = 9,
    f_stride = 10,
    f_padding = 11,
    f_dilation = 12,
    f_groups = 13,
    f_device = 14,
    f_input_dtype = 15,
    f_output_dtype = 16,
    f_conv2d_config = 17,
    f_compute_config = 18,
    f_conv2d_slice_config = 19,
    kNumFields = 20
  };
};
struct PrepareConv2dWeightsOp {
  enum : int {
    f_weight_tensor = 0,
    f_out = 1,
    f_input_memory_config = 2,
    f_input_tensor_layout = 3,
    f_weights_format = 4,
    f_in_channels = 5,
    f_out_channels = 6,
    f_batch_size = 7,
    f_input_height = 8,
    f_input_width = 9,
    f_kernel_size = 10,
    f_stride = 11,
    f_padding = 12,
    f_dilation = 13,
    f_has_bias = 14,
    f_groups = 15,
    f_device = 16,
    f_input_dtype = 17,
    f_output_dtype = 18,
    f_conv2d_config = 19,
    f_compute_config = 20,
    f_conv2d_slice_config = 21,
    kNumFields = 22
  };
};
struct PrepareConv3dWeightsOp {
  enum : int {
    f_weight_tensor = 0,
    f_out = 1,
    f_groups = 2,
    f_c_in_block = 3,
    f_alignment = 4,
    f_device = 5,
    kNumFields = 6
  };
};
struct PrepareConvTranspose2dBiasOp {
  enum : int {
    f_bias_tensor = 0,
    f_out = 1,
    f_input_memory_config = 2,
    f_input_tensor_layout = 3,
    f_in_channels = 4,
    f_out_channels = 5,
    f_batch_size = 6,
    f_input_height = 7,
    f_input_width = 8,
    f_kernel_size = 9,
    f_stride = 10,
    f_padding = 11,
    f_dilation = 12,
    f_groups = 13,
    f_device = 14,
    f_input_dtype = 15,
    f_output_dtype = 16,
    f_conv2d_config = 17,
    f_compute_config = 18,
    f_conv2d_slice_config = 19,
    kNumFields = 20
  };
};
struct PrepareConvTranspose2dWeightsOp {
  enum : int {
    f_weight_tensor = 0,
    f_out = 1,
    f_input_memory_config = 2,
    f_input_tensor_layout = 3,
    f_weights_format = 4,
    f_in_channels = 5,
    f_out_channels = 6,
    f_batch_size = 7,
    f_input_height = 8,
    f_input_width = 9,
    f_kernel_size = 10,
    f_stride = 11,
    f_padding = 12,
    f_output_padding = 13,
    f_dilation = 14,
    f_has_bias = 15,
    f_groups = 16,
    f_device = 17,
    f_input_dtype = 18,
    f_output_dtype = 19,
    f_conv2d_config = 20,
    f_compute_config = 21,
    f_conv2d_slice_config = 22,
    f_mirror_kernel = 23,
    kNumFields = 24
  };
};
struct PrepareMoEComputeW0W1WeightsOp {
  enum : int {
    f_w0 = 0,
    f_w1 = 1,
    f_bias_0 = 2,
    f_bias_1 = 3,
    f_device = 4,
    f_hidden_size = 5,
    f_intermediate_size = 6,
    f_out = 7,
    kNumFields = 8
  };
};
struct PrepareMoEComputeW2WeightsOp {
  enum : int {
    f_w2 = 0,
    f_bias_2 = 1,
    f_device = 2,
    f_hidden_size = 3,
    f_intermediate_size = 4,
    f_out = 5,
    kNumFields = 6
  };
};
struct PrintOp {
  enum : int {
    f_operand = 0,
    f_message = 1,
    kNumFields = 2
  };
};
struct Program {
  enum : int {
    f_name = 0,
    f_inputs = 1,
    f_outputs = 2,
    f_operations = 3,
    f_dylibs = 4,
    f_debug_info = 5,
    f_private = 6,
    f_mesh_shape = 7,
    f_semaphore_inputs = 8,
    kNumFields = 9
  };
};
struct ProgramDescriptor {
  enum : int {
    f_kernels = 0,
    f_semaphores = 1,
    f_cbs = 2,
    kNumFields = 3
  };
};
struct QuantizeDequantizeOpParams {
  enum : int {
    f_scale_type = 0,
    f_scale = 1,
    f_zero_point_type = 2,
    f_zero_point = 3,
    kNumFields = 4
  };
};
struct RMSNormOp {
  enum : int {
    f_input = 0,
    f_weight = 1,
    f_bias = 2,
    f_epsilon = 3,
    f_memory_config = 4,
    f_out = 5,
    f_compute_config = 6,
    kNumFields = 7
  };
};
struct RMSNormPreAllGatherOp {
  enum : int {
    f_input = 0,
    f_dtype = 1,
    f_residual = 2,
    f_memory_config = 3,
    f_compute_config = 4,
    f_program_config = 5,
    f_use_2d_core_grid = 6,
    f_out = 7,
    kNumFields = 8
  };
};
struct RandOp {
  enum : int {
    f_device = 0,
    f_size = 1,
    f_low = 2,
    f_high = 3,
    f_seed = 4,
    f_dtype = 5,
    f_layout = 6,
    f_memcfg = 7,
    f_out = 8,
    kNumFields = 9
  };
};
struct ReaderKernelConfig {
  enum : int {
    kNumFields = 0
  };
};
struct ReduceScatterOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_scatter_dim = 2,
    f_reduce_type = 3,
    f_cluster_axis = 4,
    f_sub_device_id = 5,
    f_memory_config = 6,
    f_num_links = 7,
    f_topology = 8,
    f_compute_config = 9,
    kNumFields = 10
  };
};
struct ReductionArgMaxOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_dim = 2,
    f_keep_dim = 3,
    f_memcfg = 4,
    kNumFields = 5
  };
};
struct ReductionOp {
  enum : int {
    f_type = 0,
    f_in = 1,
    f_out = 2,
    f_dim_arg = 3,
    f_keep_dim = 4,
    f_compute_config = 5,
    kNumFields = 6
  };
};
struct ReductionProdOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_dim_arg = 2,
    f_keep_dim = 3,
    f_memcfg = 4,
    kNumFields = 5
  };
};
struct RegionEndOp {
  enum : int {
    f_operand = 0,
    f_result = 1,
    f_region_id = 2,
    kNumFields = 3
  };
};
struct RegionStartOp {
  enum : int {
    f_operand = 0,
    f_result = 1,
    f_region_id = 2,
    kNumFields = 3
  };
};
struct RepeatInterleaveOp {
  enum : int {
    f_input = 0,
    f_out = 1,
    f_repeats = 2,
    f_dim = 3,
    f_memory_config = 4,
    kNumFields = 5
  };
};
struct RepeatOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_repeat_dims = 2,
    f_memcfg = 3,
    kNumFields = 4
  };
};
struct ReplicateTensor {
  enum : int {
    f_replication_factor = 0,
    kNumFields = 1
  };
};
struct RequantizeOpParams {
  enum : int {
    f_in_scale_type = 0,
    f_in_scale = 1,
    f_in_zero_point_type = 2,
    f_in_zero_point = 3,
    f_out_scale_type = 4,
    f_out_scale = 5,
    f_out_zero_point_type = 6,
    f_out_zero_point = 7,
    kNumFields = 8
  };
};
struct ResetGlobalSemaphoreOp {
  enum : int {
    f_semaphore = 0,
    f_value = 1,
    kNumFields = 2
  };
};
struct ReshapeOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_shape = 2,
    f_memory_config = 3,
    kNumFields = 4
  };
};
struct RotaryEmbeddingLlamaOp {
  enum : int {
    f_input = 0,
    f_cos_cache = 1,
    f_sin_cache = 2,
    f_trans_mat = 3,
    f_is_decode_mode = 4,
    f_out = 5,
    f_memcfg = 6,
    f_compute_config = 7,
    kNumFields = 8
  };
};
struct RotaryEmbeddingOp {
  enum : int {
    f_input = 0,
    f_cos_cache = 1,
    f_sin_cache = 2,
    f_token_index = 3,
    f_out = 4,
    f_memcfg = 5,
    f_compute_config = 6,
    kNumFields = 7
  };
};
struct SDPABackwardOp {
  enum : int {
    f_grad_output = 0,
    f_attn_output = 1,
    f_query = 2,
    f_key = 3,
    f_value = 4,
    f_intermediates = 5,
    f_attention_mask = 6,
    f_mask_type = 7,
    f_dropout_probability = 8,
    f_grad_query = 9,
    f_grad_key = 10,
    f_grad_value = 11,
    kNumFields = 12
  };
};
struct SDPAConfig {
  enum : int {
    f_compute_with_storage_grid_size = 0,
    f_sub_core_grids = 1,
    f_q_chunk_size = 2,
    f_k_chunk_size = 3,
    f_exp_approx_mode = 4,
    f_max_cores_per_head_batch = 5,
    kNumFields = 6
  };
};
struct SDPAForwardOp {
  enum : int {
    f_query = 0,
    f_key = 1,
    f_value = 2,
    f_attention_mask = 3,
    f_mask_type = 4,
    f_dropout_probability = 5,
    f_return_intermediates = 6,
    f_out = 7,
    f_intermediates = 8,
    kNumFields = 9
  };
};
struct SamplingOp {
  enum : int {
    f_input_values = 0,
    f_input_indices = 1,
    f_k = 2,
    f_p = 3,
    f_temp = 4,
    f_seed = 5,
    f_out = 6,
    kNumFields = 7
  };
};
struct ScaledDotProductAttentionDecodeOp {
  enum : int {
    f_query = 0,
    f_key = 1,
    f_value = 2,
    f_is_causal = 3,
    f_attention_mask = 4,
    f_cur_pos_tensor = 5,
    f_attention_sink = 6,
    f_scale = 7,
    f_sliding_window_size = 8,
    f_out = 9,
    f_memcfg = 10,
    f_program_config = 11,
    kNumFields = 12
  };
};
struct ScaledDotProductAttentionOp {
  enum : int {
    f_query = 0,
    f_key = 1,
    f_value = 2,
    f_is_causal = 3,
    f_attention_mask = 4,
    f_scale = 5,
    f_sliding_window_size = 6,
    f_attention_sink = 7,
    f_out = 8,
    f_memcfg = 9,
    kNumFields = 10
  };
};
struct ScatterOp {
  enum : int {
    f_input = 0,
    f_out = 1,
    f_index = 2,
    f_source = 3,
    f_dim = 4,
    f_memory_config = 5,
    f_scatter_reduce_type = 6,
    kNumFields = 7
  };
};
struct SelectiveReduceCombineOp {
  enum : int {
    f_dense_input_tensor = 0,
    f_dense_activations_tensor = 1,
    f_dense_token_maps_tensor = 2,
    f_dense_token_counts_tensor = 3,
    f_out = 4,
    f_hidden_size = 5,
    f_batch_size = 6,
    f_seq_size = 7,
    f_select_experts_k = 8,
    f_experts = 9,
    kNumFields = 10
  };
};
struct SemaphoreDescriptor {
  enum : int {
    f_id = 0,
    f_core_type = 1,
    f_core_ranges = 2,
    f_initial_value = 3,
    kNumFields = 4
  };
};
struct ShardSpec {
  enum : int {
    f_core_range_set = 0,
    f_shape = 1,
    f_orientation = 2,
    kNumFields = 3
  };
};
struct ShardTensor {
  enum : int {
    f_shard_dim = 0,
    kNumFields = 1
  };
};
struct ShardTensor2D {
  enum : int {
    f_shard_mesh = 0,
    kNumFields = 1
  };
};
struct SliceDynamicOpParams {
  enum : int {
    f_begins = 0,
    f_ends = 1,
    kNumFields = 2
  };
};
struct SliceOp {
  enum : int {
    f_type = 0,
    f_in = 1,
    f_out = 2,
    f_step = 3,
    f_params_type = 4,
    f_params = 5,
    kNumFields = 6
  };
};
struct SliceStaticOpParams {
  enum : int {
    f_begins = 0,
    f_ends = 1,
    kNumFields = 2
  };
};
struct SoftmaxOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_dimension = 2,
    f_numeric_stable = 3,
    f_compute_config = 4,
    kNumFields = 5
  };
};
struct SortOp {
  enum : int {
    f_in = 0,
    f_dim = 1,
    f_descending = 2,
    f_stable = 3,
    f_memcfg = 4,
    f_outputs = 5,
    kNumFields = 6
  };
};
struct SparseMatmulOp {
  enum : int {
    f_a = 0,
    f_b = 1,
    f_sparsity = 2,
    f_out = 3,
    f_is_input_a_sparse = 4,
    f_is_input_b_sparse = 5,
    f_nnz = 6,
    f_program_config = 7,
    f_memory_config = 8,
    f_dtype = 9,
    f_compute_config = 10,
    kNumFields = 11
  };
};
struct SplitQueryKeyValueAndSplitHeadsOp {
  enum : int {
    f_in = 0,
    f_kv_input = 1,
    f_q_out = 2,
    f_k_out = 3,
    f_v_out = 4,
    f_num_heads = 5,
    f_num_kv_heads = 6,
    f_transpose_key = 7,
    f_memcfg = 8,
    kNumFields = 9
  };
};
struct SystemDesc {
  enum : int {
    f_cpu_descs = 0,
    f_chip_descs = 1,
    f_chip_desc_indices = 2,
    f_chip_capabilities = 3,
    f_chip_coords = 4,
    f_chip_channels = 5,
    kNumFields = 6
  };
};
struct TTNNBinary {
  enum : int {
    f_version = 0,
    f_schema_hash = 1,
    f_ttmlir_git_hash = 2,
    f_system_desc = 3,
    f_mlir = 4,
    f_programs = 5,
    kNumFields = 6
  };
};
struct TensorDesc {
  enum : int {
    f_shape = 0,
    f_mesh_shape = 1,
    f_layout = 2,
    f_shard_status = 3,
    f_local_shape = 4,
    kNumFields = 5
  };
};
struct TensorRef {
  enum : int {
    f_global_id = 0,
    f_desc = 1,
    kNumFields = 2
  };
};
struct ToDeviceOp {
  enum : int {
    f_in = 0,
    f_device = 1,
    f_memcfg = 2,
    f_out = 3,
    kNumFields = 4
  };
};
struct ToLayoutOp {
  enum : int {
    f_in = 0,
    f_layout = 1,
    f_dtype = 2,
    f_memcfg = 3,
    f_out = 4,
    kNumFields = 5
  };
};
struct ToMemoryConfigOp {
  enum : int {
    f_in0 = 0,
    f_memcfg = 1,
    f_out = 2,
    kNumFields = 3
  };
};
struct TopKOp {
  enum : int {
    f_input_tensor = 0,
    f_k = 1,
    f_dim = 2,
    f_largest = 3,
    f_sorted = 4,
    f_memcfg = 5,
    f_outputs = 6,
    kNumFields = 7
  };
};
struct TopKRouterGptOp {
  enum : int {
    f_input = 0,
    f_weight = 1,
    f_bias = 2,
    f_k = 3,
    f_num_experts = 4,
    f_expert_indices = 5,
    f_expert_weights = 6,
    kNumFields = 7
  };
};
struct TransposeOp {
  enum : int {
    f_in = 0,
    f_out = 1,
    f_dim0 = 2,
    f_dim1 = 3,
    kNumFields = 4
  };
};
struct TypecastOp {
  enum : int {
    f_in = 0,
    f_dtype = 1,
    f_memcfg = 2,
    f_out = 3,
    kNumFields = 4
  };
};
struct UnaryWithParam {
  enum : int {
    f_op_type = 0,
    f_params = 1,
    kNumFields = 2
  };
};
struct UniformScale2D {
  enum : int {
    f_scale = 0,
    kNumFields = 1
  };
};
struct UpdateCacheOp {
  enum : int {
    f_cache = 0,
    f_input = 1,
    f_update_index = 2,
    f_batch_offset = 3,
    kNumFields = 4
  };
};
struct UpsampleOp {
  enum : int {
    f_in = 0,
    f_scale_factor_type = 1,
    f_scale_factor = 2,
    f_mode = 3,
    f_memory_config = 4,
    f_out = 5,
    kNumFields = 6
  };
};
struct WriteTensorOp {
  enum : int {
    f_host_tensor = 0,
    f_device_tensor = 1,
    f_blocking = 2,
    f_cq_id = 3,
    kNumFields = 4
  };
};
struct WriterKernelConfig {
  enum : int {
    kNumFields = 0
  };
};

const char *opTypeName(OpType t);
}  // namespace ttmlir_amd::schema
