// cut_hip_ops.hpp -- header-only C++17 host side over the C ABI of cut_hip.h.
//
// Mirrors the operator interface of the reference for this path so that a
// HIP backend can construct the same nodes its Dispatcher encodes today:
//   DequantOpNode      operators/impl/dequant/DequantOp.h:18-43, DequantOp.cpp:7-67
//   MatMulOpNode       operators/impl/matmul/MatMulOp.h:16-70,  MatMulOp.cpp:271-383
//   variant tables     operators/impl/matmul/MatMulQ4Variants.generated.h:13-62
// Same conventions: a node validates its shapes and allocates its own output
// at construction (MatMulOp.cpp:381-382), errors are std::runtime_error (the
// reference's logErr, core/api/src/ComputeCommon.cpp:48-52), callers are
// single-threaded.  The weights stay in GGUF file layout (row n = K/blk
// consecutive blocks), so the quantized matmul takes (A, W blocks, format)
// where the reference takes (A, packedB, scalesB).
#pragma once

#include <cstdint>
#include <cstring>
#include <optional>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "cut_hip.h"

namespace cut {
namespace hip {

inline void check(int status, const char *what) {
  if (status != CUTHIP_OK) throw std::runtime_error(std::string(what) + ": " + cuthip_last_error());
}

// DequantFormat of the reference (DequantOp.h:8-13) lists BF16/Q4_K/Q5_K/Q6_K;
// this backend covers the four block formats of the GGUF reader instead.
enum class GgufFormat : int { Q8_0 = CUTHIP_Q8_0, Q4_0 = CUTHIP_Q4_0, Q4_K = CUTHIP_Q4_K, Q6_K = CUTHIP_Q6_K };
enum class DataType : int { Float32 = CUTHIP_F32, Float16 = CUTHIP_F16 };
enum class MatMulFusion : int { None = CUTHIP_EPI_NONE, Unary = CUTHIP_EPI_UNARY, Binary = CUTHIP_EPI_BINARY };

inline uint32_t blockElems(GgufFormat f) { return (f == GgufFormat::Q8_0 || f == GgufFormat::Q4_0) ? 32u : 256u; }
inline uint32_t blockBytes(GgufFormat f) {
  switch (f) {
  case GgufFormat::Q8_0: return 34;
  case GgufFormat::Q4_0: return 18;
  case GgufFormat::Q4_K: return 144;
  default: return 210;
  }
}
inline size_t dtypeBytes(DataType t) { return t == DataType::Float32 ? 4 : 2; }
inline size_t ggufBytes(GgufFormat f, uint64_t elems) { return (size_t)(elems / blockElems(f)) * blockBytes(f); }

// Selects the device once; throws if it is not a gfx950.
inline void init(int device = 0) { check(cuthip_init(device), "cuthip_init"); }

// A stream of the backend (the reference keeps 16 of them, core/backends/cuda/CudaStructs.h:20).
class Stream {
public:
  Stream() { check(cuthip_stream_create(&s_), "cuthip_stream_create"); }
  ~Stream() {
    if (s_) cuthip_stream_destroy(s_);
  }
  Stream(const Stream &) = delete;
  Stream &operator=(const Stream &) = delete;
  void *get() const { return s_; }
  void sync() const { check(cuthip_stream_sync(s_), "cuthip_stream_sync"); }

private:
  void *s_ = nullptr;
};

// The reusable command buffer of the reference on its CUDA backend (CommandBuffer begin / encode / end / resubmit,
// core/backends/cuda/CudaCommandBuffer.cpp:261-285): the dispatches between begin() and end() are captured once and
// replay() launches them again with one call.  Buffers the kernels read on the device (activations, runtime
// parameters) may be rewritten between replays.
class CommandGraph {
public:
  CommandGraph() = default;
  ~CommandGraph() {
    if (graph_) cuthip_graph_destroy(graph_);
  }
  CommandGraph(const CommandGraph &) = delete;
  CommandGraph &operator=(const CommandGraph &) = delete;
  void begin(const Stream &s) { check(cuthip_graph_begin_capture(s.get()), "cuthip_graph_begin_capture"); }
  void end(const Stream &s) {
    if (graph_) {
      cuthip_graph_destroy(graph_);
      graph_ = nullptr;
    }
    check(cuthip_graph_end_capture(s.get(), &graph_), "cuthip_graph_end_capture");
  }
  void replay(const Stream &s) const {
    if (!graph_) throw std::runtime_error("CommandGraph::replay: nothing captured");
    check(cuthip_graph_launch(graph_, s.get()), "cuthip_graph_launch");
  }

private:
  void *graph_ = nullptr;
};

// Owning device allocation (the role of a ref-counted ComputeHandle buffer,
// core/backends/cuda/CudaContainers.cpp:354-384, without the pooling).
class DeviceBuffer {
public:
  DeviceBuffer() = default;
  explicit DeviceBuffer(size_t bytes) : bytes_(bytes) {
    if (bytes) check(cuthip_malloc(&ptr_, bytes), "cuthip_malloc");
  }
  DeviceBuffer(const void *host, size_t bytes) : DeviceBuffer(bytes) { upload(host, bytes); }
  DeviceBuffer(const DeviceBuffer &) = delete;
  DeviceBuffer &operator=(const DeviceBuffer &) = delete;
  DeviceBuffer(DeviceBuffer &&o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_) { o.ptr_ = nullptr; o.bytes_ = 0; }
  DeviceBuffer &operator=(DeviceBuffer &&o) noexcept {
    if (this != &o) {
      release();
      ptr_ = o.ptr_;
      bytes_ = o.bytes_;
      o.ptr_ = nullptr;
      o.bytes_ = 0;
    }
    return *this;
  }
  ~DeviceBuffer() { release(); }

  void upload(const void *host, size_t bytes, void *stream = nullptr) {
    if (bytes > bytes_) throw std::runtime_error("DeviceBuffer::upload: larger than the allocation");
    check(cuthip_memcpy_h2d(ptr_, host, bytes, stream), "cuthip_memcpy_h2d");
  }
  void download(void *host, size_t bytes, void *stream = nullptr) const {
    if (bytes > bytes_) throw std::runtime_error("DeviceBuffer::download: larger than the allocation");
    check(cuthip_memcpy_d2h(host, ptr_, bytes, stream), "cuthip_memcpy_d2h");
  }
  void *data() const { return ptr_; }
  size_t bytes() const { return bytes_; }

private:
  void release() {
    if (ptr_) cuthip_free(ptr_);
    ptr_ = nullptr;
  }
  void *ptr_ = nullptr;
  size_t bytes_ = 0;
};

// A device tensor: buffer + shape + dtype (Tensor/TensorStore of the reference reduced to what the path needs).
struct Tensor {
  DeviceBuffer *buffer = nullptr;
  std::vector<uint32_t> shape;
  DataType dtype = DataType::Float32;
  uint32_t rowStride = 0;   // elements between rows; 0 = shape.back()
  uint32_t stride() const { return rowStride ? rowStride : (shape.empty() ? 0u : shape.back()); }
  void *data() const { return buffer ? buffer->data() : nullptr; }
};

// ---- variant tables (k<Op>VariantCount / k<Op>DefaultVariant / get<Op>VariantName) ----
struct VariantInfo {
  std::string name;
  uint32_t wgX, wgY, effTileM, effTileN;
  std::string description;
};
inline uint32_t variantCount(cuthip_op op) { return (uint32_t)cuthip_variant_count(op); }
inline uint32_t defaultVariant(cuthip_op op) {
  int v = cuthip_variant_default(op);
  check(v < 0 ? v : CUTHIP_OK, "cuthip_variant_default");
  return (uint32_t)v;
}
inline VariantInfo variantInfo(cuthip_op op, uint32_t index) {
  cuthip_variant_info_t i;
  check(cuthip_variant_info(op, (int)index, &i), "cuthip_variant_info");
  return VariantInfo{i.name, i.wgX, i.wgY, i.effTileM, i.effTileN, i.description};
}
inline uint32_t lookupVariant(cuthip_op op, const std::string &name) {
  int v = cuthip_variant_lookup(op, name.c_str());
  check(v < 0 ? v : CUTHIP_OK, "cuthip_variant_lookup");
  return (uint32_t)v;
}
inline std::string getMatMulGgufVariantName(uint32_t index) { return variantInfo(CUTHIP_OP_MATMUL_GGUF, index).name; }

// ---- DequantOpNode ----------------------------------------------------------------------
// Input: raw GGUF block bytes of a [rows, cols] tensor.  Output: [rows, cols]
// Float32 (the reference's only output type) or Float16, row stride
// (cols+3)&~3 as in DequantOp.cpp:15.
class DequantOpNode {
public:
  DequantOpNode(const Tensor &rawData, GgufFormat format, uint32_t rows, uint32_t cols,
                DataType outDtype = DataType::Float32, std::optional<uint32_t> spec = {})
      : raw_(rawData), format_(format), rows_(rows), cols_(cols), outDtype_(outDtype) {
    if (rows == 0 || cols == 0 || cols % blockElems(format) != 0)
      throw std::runtime_error("DequantOpNode: cols must be a positive multiple of the block size");
    size_t need = ggufBytes(format, (uint64_t)rows * cols);
    if (!rawData.buffer || rawData.buffer->bytes() < need)
      throw std::runtime_error("DequantOpNode: raw tensor holds fewer bytes than rows x cols blocks");
    spec_ = spec ? *spec : defaultVariant(CUTHIP_OP_DEQUANT);
    if (spec_ >= variantCount(CUTHIP_OP_DEQUANT)) throw std::runtime_error("DequantOpNode: unknown variant index");
    outputStride_ = (cols_ + 3) & ~3u;
    storage_ = DeviceBuffer((size_t)rows_ * outputStride_ * dtypeBytes(outDtype_));
    output_ = Tensor{&storage_, {rows_, cols_}, outDtype_, outputStride_};
  }
  DequantOpNode(DequantOpNode &&) = delete;   // output() points into this node
  DataType outputDtype() const { return outDtype_; }
  std::vector<uint32_t> outputShape() const { return {rows_, cols_}; }
  uint32_t outputStride() const { return outputStride_; }
  std::string displayName() const { return "Dequantize"; }
  const Tensor &output() const { return output_; }
  // What Dispatcher::encode does for this node: one launch on `stream`.
  void dispatch(void *stream = nullptr) const {
    check(cuthip_dequant((int)format_, raw_.data(), output_.data(), (int)outDtype_, rows_, cols_, outputStride_, stream),
          "cuthip_dequant");
  }

private:
  Tensor raw_;
  GgufFormat format_;
  uint32_t rows_, cols_, outputStride_ = 0, spec_ = 0;
  DataType outDtype_;
  DeviceBuffer storage_;
  Tensor output_;
};

// ---- MatMulGgufOpNode --------------------------------------------------------------------
// C[M,N] = A[M,K] . dequant(W)[N,K]^T with W as GGUF blocks.  A is rank 1 ([K],
// M = 1) or rank 2 ([M,K]) as in MatMulOp.cpp:283-300; K is inferred from A and
// must be a multiple of the block size; N is given (the block tensor is 1-D
// bytes).  Variant: explicit `spec` or chosen by shape, as the reference's
// autoSpec_ (MatMulOp.cpp:336-374).
class MatMulGgufOpNode {
public:
  MatMulGgufOpNode(const Tensor &a, const Tensor &wBlocks, GgufFormat format, uint32_t N,
                   DataType outDtype = DataType::Float32, std::optional<uint32_t> spec = {})
      : a_(a), w_(wBlocks), format_(format), N_(N), outDtype_(outDtype) {
    if (a.shape.empty() || a.shape.size() > 2) throw std::runtime_error("MatMulGgufOpNode: A must have rank 1 or 2");
    M_ = a.shape.size() == 2 ? a.shape[0] : 1u;
    K_ = a.shape.back();
    if (M_ == 0 || K_ == 0 || N_ == 0) throw std::runtime_error("MatMulGgufOpNode: empty dimension");
    if (K_ % blockElems(format) != 0) throw std::runtime_error("MatMulGgufOpNode: K must be a multiple of the block size");
    if (!wBlocks.buffer || wBlocks.buffer->bytes() < ggufBytes(format, (uint64_t)N_ * K_))
      throw std::runtime_error("MatMulGgufOpNode: weight tensor holds fewer bytes than N x K blocks");
    if (spec) {
      if (*spec >= variantCount(CUTHIP_OP_MATMUL_GGUF)) throw std::runtime_error("MatMulGgufOpNode: unknown variant index");
      spec_ = (int)*spec;
    }
    storage_ = DeviceBuffer((size_t)M_ * N_ * dtypeBytes(outDtype_));
    output_ = Tensor{&storage_, a.shape.size() == 2 ? std::vector<uint32_t>{M_, N_} : std::vector<uint32_t>{N_}, outDtype_, N_};
  }
  MatMulGgufOpNode(MatMulGgufOpNode &&) = delete;   // output() points into this node
  // Called by the fusion passes of the reference (MatMulOp.h:39-41): `d` is the
  // [M,N] second operand of a Binary epilogue and must have the output's dtype.
  void setFusion(MatMulFusion fusion, int fusionOp = 0, const Tensor &d = {}) {
    if (fusion == MatMulFusion::Binary) {
      if (!d.buffer) throw std::runtime_error("MatMulGgufOpNode::setFusion: Binary fusion needs the tensor d");
      if (d.dtype != outDtype_ || d.stride() != N_) throw std::runtime_error("MatMulGgufOpNode::setFusion: d must match the output");
    }
    fusion_ = fusion;
    fusionOp_ = fusionOp;
    d_ = d;
  }
  MatMulFusion fusion() const { return fusion_; }
  GgufFormat format() const { return format_; }
  DataType outputDtype() const { return outDtype_; }
  std::vector<uint32_t> outputShape() const { return output_.shape; }
  std::string displayName() const { return "MatMulGguf"; }
  const Tensor &output() const { return output_; }
  // Scratch for the two-pass prefill variant (MatMulGgufDequantGemm): the weights are dequantized into it once
  // per dispatch.  With a workspace set, large M takes that variant automatically; the buffer may be shared by
  // every node of a prefill graph (dispatches on one stream run in order).
  size_t workspaceBytes() const { return cuthip_matmul_gguf_workspace_bytes((int)format_, M_, K_, N_, (int)a_.dtype); }
  void setWorkspace(DeviceBuffer *workspace) {
    if (workspace && workspace->bytes() < workspaceBytes())
      throw std::runtime_error("MatMulGgufOpNode::setWorkspace: buffer smaller than workspaceBytes()");
    workspace_ = workspace;
  }
  void dispatch(void *stream = nullptr) const {
    if (workspace_) {
      check(cuthip_matmul_gguf_ws((int)format_, w_.data(), a_.data(), (int)a_.dtype, output_.data(), (int)outDtype_, M_, K_, N_,
                                  a_.stride(), N_, (int)fusion_, fusionOp_, d_.data(), spec_, workspace_->data(),
                                  workspace_->bytes(), stream),
            "cuthip_matmul_gguf_ws");
      return;
    }
    check(cuthip_matmul_gguf((int)format_, w_.data(), a_.data(), (int)a_.dtype, output_.data(), (int)outDtype_, M_, K_, N_,
                             a_.stride(), N_, (int)fusion_, fusionOp_, d_.data(), spec_, stream),
          "cuthip_matmul_gguf");
  }

private:
  Tensor a_, w_, d_;
  GgufFormat format_;
  uint32_t M_ = 0, K_ = 0, N_ = 0;
  DataType outDtype_;
  int spec_ = -1;   // -1: chosen by shape at dispatch
  MatMulFusion fusion_ = MatMulFusion::None;
  int fusionOp_ = 0;
  DeviceBuffer *workspace_ = nullptr;
  DeviceBuffer storage_;
  Tensor output_;
};

// ---- MatMulOpNode: the reference's 3-input quantized matmul ------------------------------------
// operators/impl/matmul/MatMulOp.h:16-70, MatMulOp.cpp:271-383 on the loader's separated tensors: A fp32 [K] or
// [M, K]; packedB [K, N] int8 (Q8) or [K, N/2] nibble bytes (Q4); scalesB fp16 [K/32, N], or [2K/32, N] when the
// lower half holds the per-block minima (affine Q4).  The format is inferred from the shapes, the variant from the
// shape unless `spec` names one, exactly as the reference does it; the messages of the errors are the reference's.
enum class QuantFormat : int { None = 0, Q8 = 1, Q4 = 2 };
// What the constructor reads of store.caps() (core/api/include/ComputeCommon.h:92-97); gfx950 always has matrix cores.
struct DeviceCaps {
  bool cooperativeMatrix = true;
  // the matrix-core route of this backend (dequantize to fp16, dense MFMA GEMM) takes K in multiples of 128; where the
  // reference's K % 16 == 0 holds but this does not, the automatic choice stays with the tiled variant
  uint32_t cooperativeMatrixK = 128;
};
// Sizes of the reference's variant tables and their defaults (MatMulQ8Variants.generated.h:20-21,
// MatMulQ4Variants.generated.h:20-21); the library's CUTHIP_OP_MATMUL_Q8 / _Q4 tables hold the same numbers.
constexpr uint32_t kMatMulQ8VariantCount = 8, kMatMulQ8DefaultVariant = 2, kMatMulQ4VariantCount = 5, kMatMulQ4DefaultVariant = 0;

// Everything the constructor derives from the shapes, without touching the device (MatMulOp.cpp:283-374).
struct QuantMatMulPlan {
  QuantFormat format = QuantFormat::None;
  uint32_t M = 0, K = 0, N = 0;
  bool q4Affine = false;            // scales carry the minima in their lower half
  bool autoSpec = false;            // no explicit spec from the caller
  uint32_t spec = 0;                // index into the Q8 / Q4 variant table
  uint32_t fusionFallbackSpec = 0;  // the fusion-capable variant of the same shape class
  // push constants (MatMulOp.cpp:514-541): rows are padded to four elements
  uint32_t strideA = 0, strideB = 0, strideC = 0, scaleStride = 0;
};
inline QuantMatMulPlan planQuantMatMul(const std::vector<uint32_t> &shapeA, const std::vector<uint32_t> &shapePB,
                                       const std::vector<uint32_t> &shapeSB, DataType scalesDtype,
                                       std::optional<uint32_t> spec = {}, DeviceCaps caps = {}) {
  QuantMatMulPlan p;
  if (shapePB.size() != 2 || shapeSB.size() != 2) throw std::runtime_error("matmul requires 2D B and scales matrices");
  if (shapeA.size() == 1) {   // [K] is [1, K]: the optimizer may have removed the reshape
    p.M = 1;
    p.K = shapeA[0];
  } else if (shapeA.size() == 2) {
    p.M = shapeA[0];
    p.K = shapeA[1];
  } else {
    throw std::runtime_error("matmul: A must be 1D or 2D");
  }
  if (shapePB[0] != p.K)
    throw std::runtime_error("matmul: B rows (" + std::to_string(shapePB[0]) + ") must match A cols (" + std::to_string(p.K) + ")");
  const uint32_t bCols = shapePB[1], sCols = shapeSB[1];
  if (bCols == sCols) {
    p.format = QuantFormat::Q8;
    p.N = bCols;
  } else if (bCols * 2 == sCols) {
    p.format = QuantFormat::Q4;
    p.N = sCols;
    p.q4Affine = shapeSB[0] == 2u * ((p.K + 31u) / 32u);
  } else {
    throw std::runtime_error("matmul: cannot determine quant format from B cols (" + std::to_string(bCols) +
                             ") and scales cols (" + std::to_string(sCols) + ")");
  }
  p.autoSpec = !spec.has_value();
  if (p.format == QuantFormat::Q8)
    p.fusionFallbackSpec = p.M == 1 ? (p.N >= 8 ? 4u : 3u) : kMatMulQ8DefaultVariant;   // GemvKPar8 / GemvKPar / VecT16R4x4
  else
    p.fusionFallbackSpec = p.M == 1 ? (p.N >= 8 ? 3u : 2u) : kMatMulQ4DefaultVariant;   // Q4GemvKPar8 / Q4GemvKPar / tiled
  const bool coop = p.M > 1 && caps.cooperativeMatrix && scalesDtype == DataType::Float16 && p.K % 16 == 0 && p.N % 32 == 0 &&
                    p.K % (caps.cooperativeMatrixK ? caps.cooperativeMatrixK : 1u) == 0;
  if (spec.has_value()) p.spec = *spec;
  else if (p.format == QuantFormat::Q8 && coop) p.spec = kMatMulQ8VariantCount - 1;   // MatMulQ8CoopMatTiled
  else if (p.format == QuantFormat::Q4 && coop) p.spec = 4;                          // MatMulQ4CoopMatTiled
  else p.spec = p.fusionFallbackSpec;
  p.strideA = (p.K + 3) & ~3u;
  p.strideB = ((p.format == QuantFormat::Q4 ? p.N / 2 : p.N) + 3) & ~3u;
  p.strideC = p.scaleStride = (p.N + 3) & ~3u;
  return p;
}

class MatMulOpNode {
public:
  MatMulOpNode(const Tensor &a, const Tensor &packedB, const Tensor &scalesB, std::optional<uint32_t> spec = {}, DeviceCaps caps = {})
      : a_(a), b_(packedB), s_(scalesB), plan_(planQuantMatMul(a.shape, packedB.shape, scalesB.shape, scalesB.dtype, spec, caps)) {
    const QuantMatMulPlan &p = plan_;
    if (p.M == 0 || p.K == 0 || p.N == 0) throw std::runtime_error("matmul: empty dimension");
    if (p.K % 32 != 0) throw std::runtime_error("matmul: K must be a multiple of the 32-element quantization block");
    if (p.spec >= (p.format == QuantFormat::Q8 ? kMatMulQ8VariantCount : kMatMulQ4VariantCount))
      throw std::runtime_error("matmul: variant index " + std::to_string(p.spec) + " is outside the table");
    if (a.dtype != DataType::Float32) throw std::runtime_error("matmul: the quantized matmul takes Float32 activations");
    if (scalesB.dtype != DataType::Float16) throw std::runtime_error("matmul: scales must be Float16");
    // the reference's tensors are rows padded to four elements; a tensor that states another stride is refused
    if ((a.rowStride && a.rowStride != p.strideA) || (packedB.rowStride && packedB.rowStride != p.strideB) ||
        (scalesB.rowStride && scalesB.rowStride != p.scaleStride))
      throw std::runtime_error("matmul: row strides must be the dimensions padded to four elements");
    const size_t scaleRows = (size_t)(p.q4Affine ? 2u : 1u) * (p.K / 32);
    if (!a.buffer || a.buffer->bytes() < ((size_t)(p.M - 1) * p.strideA + p.K) * 4 || !packedB.buffer ||
        packedB.buffer->bytes() < (size_t)(p.K - 1) * p.strideB + (p.format == QuantFormat::Q4 ? p.N / 2 : p.N) ||
        !scalesB.buffer || scalesB.buffer->bytes() < ((scaleRows - 1) * p.scaleStride + p.N) * 2)
      throw std::runtime_error("matmul: a tensor holds fewer bytes than its shape and padded stride need");
    if (shapeRows(scalesB) < scaleRows) throw std::runtime_error("matmul: scales must have K/32 rows");
    storage_ = DeviceBuffer((size_t)p.M * p.strideC * 4);
    output_ = Tensor{&storage_, {p.M, p.N}, DataType::Float32, p.strideC};
    scratch_ = DeviceBuffer(cuthip_matmul_sep_workspace_bytes_for(op(), (int)p.spec, p.M, p.K, p.N));
  }
  MatMulOpNode(MatMulOpNode &&) = delete;   // output() points into this node
  // MatMulOp.cpp:389-419: the quantized cooperative-matrix variants have a fusion epilogue, so nothing falls back
  void setFusion(MatMulFusion fusion, int fusionOp = 0, const Tensor &d = {}) {
    if (fusion == MatMulFusion::Binary) {
      if (!d.buffer) throw std::runtime_error("matmul: Binary fusion needs the tensor d");
      if (d.dtype != DataType::Float32 || d.stride() != plan_.strideC) throw std::runtime_error("matmul: d must match the output");
    }
    fusion_ = fusion;
    fusionOp_ = fusionOp;
    d_ = d;
  }
  QuantFormat format() const { return plan_.format; }
  MatMulFusion fusion() const { return fusion_; }
  const QuantMatMulPlan &plan() const { return plan_; }
  DataType outputDtype() const { return DataType::Float32; }   // MatMulOp.cpp:436-438: always Float32
  std::vector<uint32_t> outputShape() const { return {plan_.M, plan_.N}; }
  std::string displayName() const {   // MatMulOp.cpp:572-603
    std::string name = plan_.format == QuantFormat::Q8 ? "MatMulQ8" : "MatMulQ4";
    if (fusion_ == MatMulFusion::Unary) name += "Unary";
    if (fusion_ == MatMulFusion::Binary) name += "Binary";
    return name;
  }
  std::string variantName() const { return variantInfo(op(), plan_.spec).name; }
  const Tensor &output() const { return output_; }
  void dispatch(void *stream = nullptr) const {
    const QuantMatMulPlan &p = plan_;
    const float *A = static_cast<const float *>(a_.data()), *D = static_cast<const float *>(d_.data());
    float *C = static_cast<float *>(output_.data());
    const uint16_t *S = static_cast<const uint16_t *>(s_.data());
    if (p.format == QuantFormat::Q8)
      check(cuthip_matmul_q8_sep(A, static_cast<const int8_t *>(b_.data()), S, D, C, p.M, p.K, p.N, p.strideA, p.strideB,
                                 p.strideC, p.scaleStride, (int)fusion_, fusionOp_, (int)p.spec, scratch_.data(),
                                 scratch_.bytes(), stream),
            "cuthip_matmul_q8_sep");
    else
      check(cuthip_matmul_q4_sep(A, static_cast<const uint8_t *>(b_.data()), S, D, C, p.M, p.K, p.N, p.strideA, p.strideB,
                                 p.strideC, p.scaleStride, (int)fusion_, fusionOp_, p.q4Affine ? 1 : 0, (int)p.spec,
                                 scratch_.data(), scratch_.bytes(), stream),
            "cuthip_matmul_q4_sep");
  }

private:
  static size_t shapeRows(const Tensor &t) { return t.shape.empty() ? 0 : t.shape[0]; }
  cuthip_op op() const { return plan_.format == QuantFormat::Q8 ? CUTHIP_OP_MATMUL_Q8 : CUTHIP_OP_MATMUL_Q4; }
  Tensor a_, b_, s_, d_;
  QuantMatMulPlan plan_;
  MatMulFusion fusion_ = MatMulFusion::None;
  int fusionOp_ = 0;
  DeviceBuffer storage_, scratch_;
  Tensor output_;
};

// ---- MatMulDenseF16OpNode ----------------------------------------------------------------
// Prefill matmul on weights kept dequantized: w16 is the fp16 [N, K] output of a DequantOpNode (DataType::Float16,
// row stride K); the float-path matmul of the reference's runner on its fp16 weight tensors (llama.cpp:800-815).
// The node owns its output and its scratch.
class MatMulDenseF16OpNode {
public:
  MatMulDenseF16OpNode(const Tensor &a, const Tensor &w16, DataType outDtype = DataType::Float16)
      : a_(a), w_(w16), outDtype_(outDtype) {
    if (a.shape.empty() || a.shape.size() > 2) throw std::runtime_error("MatMulDenseF16OpNode: A must have rank 1 or 2");
    if (w16.shape.size() != 2 || w16.dtype != DataType::Float16 || w16.stride() != w16.shape[1])
      throw std::runtime_error("MatMulDenseF16OpNode: weights must be a dense Float16 [N, K] tensor");
    M_ = a.shape.size() == 2 ? a.shape[0] : 1u;
    K_ = a.shape.back();
    N_ = w16.shape[0];
    if (M_ == 0 || K_ == 0 || N_ == 0 || w16.shape[1] != K_) throw std::runtime_error("MatMulDenseF16OpNode: A cols must match weight cols");
    if (K_ % 128 != 0) throw std::runtime_error("MatMulDenseF16OpNode: K must be a multiple of 128");
    if (!w16.buffer || w16.buffer->bytes() < (size_t)N_ * K_ * 2)
      throw std::runtime_error("MatMulDenseF16OpNode: weight tensor holds fewer bytes than N x K halfs");
    storage_ = DeviceBuffer((size_t)M_ * N_ * dtypeBytes(outDtype_));
    scratch_ = DeviceBuffer(cuthip_matmul_dense_f16_workspace_bytes(M_, K_, N_, (int)a_.dtype));
    output_ = Tensor{&storage_, a.shape.size() == 2 ? std::vector<uint32_t>{M_, N_} : std::vector<uint32_t>{N_}, outDtype_, N_};
  }
  MatMulDenseF16OpNode(MatMulDenseF16OpNode &&) = delete;
  std::vector<uint32_t> outputShape() const { return output_.shape; }
  std::string displayName() const { return "MatMulDenseF16"; }
  const Tensor &output() const { return output_; }
  void dispatch(void *stream = nullptr) const {
    check(cuthip_matmul_dense_f16(w_.data(), a_.data(), (int)a_.dtype, output_.data(), (int)outDtype_, M_, K_, N_, a_.stride(), N_,
                                  CUTHIP_EPI_NONE, 0, nullptr, scratch_.data(), scratch_.bytes(), stream),
          "cuthip_matmul_dense_f16");
  }

private:
  Tensor a_, w_;
  uint32_t M_ = 0, K_ = 0, N_ = 0;
  DataType outDtype_;
  DeviceBuffer storage_, scratch_;
  Tensor output_;
};

// ---- TransposeQ4NibbleOpNode --------------------------------------------------------------
// operators/impl/q4transpose/TransposeQ4NibbleOp.cpp:7-23: packed GGML-order nibbles [N, K/2] ->
// [K, N/2] with the even source row in the low nibble; same checks, messages and padded strides.
class TransposeQ4NibbleOpNode {
public:
  TransposeQ4NibbleOpNode(const Tensor &packedInput, uint32_t N, uint32_t K) : in_(packedInput), N_(N), K_(K) {
    if (N_ % 2 != 0) throw std::runtime_error("TransposeQ4: N must be even");
    if (K_ % 32 != 0) throw std::runtime_error("TransposeQ4: K must be a multiple of 32");
    strideInHalf_ = (K_ / 2 + 3) & ~3u;
    strideOutHalf_ = (N_ / 2 + 3) & ~3u;
    if (!packedInput.buffer || packedInput.buffer->bytes() < (size_t)N_ * strideInHalf_)
      throw std::runtime_error("TransposeQ4: input holds fewer bytes than N rows of the padded stride");
    storage_ = DeviceBuffer((size_t)K_ * strideOutHalf_);
    output_ = Tensor{&storage_, {K_, N_ / 2}, DataType::Float16 /* unused: bytes */, strideOutHalf_};
  }
  TransposeQ4NibbleOpNode(TransposeQ4NibbleOpNode &&) = delete;
  std::vector<uint32_t> outputShape() const { return {K_, N_ / 2}; }
  std::string displayName() const { return "TransposeQ4"; }
  const Tensor &output() const { return output_; }
  void dispatch(void *stream = nullptr) const {
    check(cuthip_transpose_q4_nibble(in_.data(), output_.data(), N_, K_, strideInHalf_, strideOutHalf_, stream),
          "cuthip_transpose_q4_nibble");
  }

private:
  Tensor in_;
  uint32_t N_, K_, strideInHalf_ = 0, strideOutHalf_ = 0;
  DeviceBuffer storage_;
  Tensor output_;
};

// ---- separated weights from GGUF blocks -----------------------------------------------------
// What LlamaModel::uploadQ4 / uploadQ8 build per tensor (interface/runner/llama/llama.cpp:940-1000):
// values [K, N] (int8) or [K, N/2] (nibbles) and fp16 scales [K/32, N] ([2K/32, N] for the affine
// re-encoding of Q4_K), with the reference's padded strides, produced on the device from the raw blocks.
struct SeparatedWeights {
  DeviceBuffer values, scales;
  uint32_t N = 0, K = 0, strideB = 0, scaleStride = 0;
  bool q4 = false, affine = false;
};
inline void prepareSeparated(SeparatedWeights &out, const Tensor &rawBlocks, GgufFormat format, uint32_t N, uint32_t K,
                             void *stream = nullptr) {
  if (format == GgufFormat::Q6_K) throw std::runtime_error("prepareSeparated: Q6_K has no separated layout");
  if (K == 0 || K % blockElems(format) != 0) throw std::runtime_error("prepareSeparated: K must be a multiple of the block size");
  out.q4 = format != GgufFormat::Q8_0;
  out.affine = format == GgufFormat::Q4_K;
  if (out.q4 && N % 2 != 0) throw std::runtime_error("prepareSeparated: N must be even for packed nibbles");
  if (!rawBlocks.buffer || rawBlocks.buffer->bytes() < ggufBytes(format, (uint64_t)N * K))
    throw std::runtime_error("prepareSeparated: raw tensor holds fewer bytes than N x K blocks");
  out.N = N;
  out.K = K;
  out.strideB = ((out.q4 ? N / 2 : N) + 3) & ~3u;
  out.scaleStride = (N + 3) & ~3u;
  const uint32_t scaleRows = (out.affine ? 2u : 1u) * (K / 32);
  out.values = DeviceBuffer((size_t)K * out.strideB);
  out.scales = DeviceBuffer((size_t)scaleRows * out.scaleStride * 2);
  check(cuthip_prepare_sep((int)format, rawBlocks.data(), N, K, out.values.data(), out.strideB,
                           reinterpret_cast<uint16_t *>(out.scales.data()), out.scaleStride, stream),
        "cuthip_prepare_sep");
}

}  // namespace hip
}  // namespace cut
