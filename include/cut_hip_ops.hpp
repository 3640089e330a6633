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

#include <cmath>
#include <cstdint>
#include <cstring>
#include <initializer_list>
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


// ==== the operators of one decode step =================================================================
// What LlamaModel::runLayer chains per token around the quantized matmuls (interface/runner/llama/llama.cpp:
// RMSNorm -> q / k / v projections -> FusedRoPEKVWrite -> Attention -> wo + residual -> RMSNorm -> gate + up ->
// SiLU * up -> w_down + residual; then the output norm, the head and the sampling).  The first three nodes mirror the
// reference's operators one to one; the Carry / Pair / Argmax nodes below are this backend's fused forms of the same
// chain (six launches per layer).  Every node may be given the tensor it writes (preallocOutput, as the reference's
// AttentionOpNode takes one): the residual stream and the normed activations are shared between the nodes of a layer.
namespace detail {
inline size_t tensorBytes(const Tensor &t) {
  if (t.shape.empty()) return 0;
  size_t rows = 1;
  for (size_t i = 0; i + 1 < t.shape.size(); ++i) rows *= t.shape[i];
  return ((rows - 1) * (size_t)t.stride() + t.shape.back()) * dtypeBytes(t.dtype);
}
inline void requireBytes(const Tensor &t, size_t bytes, const char *what) {
  if (!t.buffer || t.buffer->bytes() < bytes) throw std::runtime_error(std::string(what) + ": tensor holds fewer bytes than its shape");
}
inline void requireTensor(const Tensor &t, const char *what) { requireBytes(t, tensorBytes(t), what); }
}  // namespace detail

// ---- RMSNormOpNode: operators/impl/rmsnorm/RMSNormOp.h:22-44, RMSNormOp.cpp:9-47 ---------------------
// x [dim] or [rows, dim], weight [dim]; output of x's shape.  The reference asks for a weight of x's dtype and
// returns that dtype; here the weight is Float32 whatever x is and the output dtype may be chosen (the decode chain
// norms an fp32 residual stream into fp16 matmul inputs).
class RMSNormOpNode {
public:
  RMSNormOpNode(const Tensor &x, const Tensor &weight, float eps = 1e-5f, std::optional<DataType> outDtype = {},
                const Tensor &preallocOutput = {})
      : x_(x), weight_(weight), eps_(eps) {
    if (x.shape.empty() || x.shape.size() > 2 || weight.shape.size() != 1)
      throw std::runtime_error("RMSNorm requires 1D or 2D input, 1D weight");
    rows_ = x.shape.size() == 2 ? x.shape[0] : 1u;
    dim_ = x.shape.back();
    if (weight.shape[0] != dim_) throw std::runtime_error("RMSNorm: weight dimension must match input");
    if (weight.dtype != DataType::Float32) throw std::runtime_error("RMSNorm: weight must be Float32");
    if (rows_ == 0 || dim_ == 0) throw std::runtime_error("RMSNorm: empty input");
    detail::requireTensor(x, "RMSNorm");
    detail::requireTensor(weight, "RMSNorm");
    outDtype_ = outDtype.value_or(x.dtype);
    if (preallocOutput.buffer) {
      if (preallocOutput.dtype != outDtype_ || preallocOutput.shape != x.shape || preallocOutput.stride() != x.stride())
        throw std::runtime_error("RMSNorm: preallocated output must have the input's shape and row stride");
      detail::requireTensor(preallocOutput, "RMSNorm");
      output_ = preallocOutput;
    } else {
      storage_ = DeviceBuffer((size_t)rows_ * x.stride() * dtypeBytes(outDtype_));
      output_ = Tensor{&storage_, x.shape, outDtype_, x.stride()};
    }
  }
  RMSNormOpNode(RMSNormOpNode &&) = delete;
  DataType outputDtype() const { return outDtype_; }
  std::vector<uint32_t> outputShape() const { return output_.shape; }
  std::string displayName() const { return "RMSNorm"; }
  const Tensor &output() const { return output_; }
  void dispatch(void *stream = nullptr) const {
    check(cuthip_rmsnorm(x_.data(), (int)x_.dtype, static_cast<const float *>(weight_.data()), output_.data(), (int)outDtype_, rows_,
                         dim_, x_.stride(), eps_, stream),
          "cuthip_rmsnorm");
  }

private:
  Tensor x_, weight_;
  float eps_;
  uint32_t rows_ = 0, dim_ = 0;
  DataType outDtype_ = DataType::Float32;
  DeviceBuffer storage_;
  Tensor output_;
};

// The runtimeParams buffer of the reference's runner: device uint32[2] = {position, sequence length}, read by the
// kernels so that a captured graph serves the next token after an 8-byte upload.
class RuntimeParams {
public:
  RuntimeParams() : buf_(8) { set(0, 1); }
  // With a stream the copy is ordered on it (the source is a member: it stays valid until the copy has run; do not
  // call set() again before that).
  void set(uint32_t position, uint32_t seqLen, void *stream = nullptr) {
    host_[0] = position;
    host_[1] = seqLen;
    buf_.upload(host_, sizeof(host_), stream);
  }
  const uint32_t *data() const { return static_cast<const uint32_t *>(buf_.data()); }

private:
  DeviceBuffer buf_;
  uint32_t host_[2] = {0, 1};
};

// ---- FusedRoPEKVWriteOpNode: operators/impl/attention/AttentionOp.h:156-184, AttentionOp.cpp:553-612 -------
// q [qDim], k [kvDim], v [kvDim] of one dtype; tables Float32 [positions, headDim / 2]; caches Float16
// [positions, alignedKvDim].  Output: the rotated q, Float32 [qDim] (AttentionOp.cpp:576).  A position at or beyond
// the rows of the caches or tables writes nothing (the reference would write past the cache).
class FusedRoPEKVWriteOpNode {
public:
  FusedRoPEKVWriteOpNode(const Tensor &q, const Tensor &k, const Tensor &v, const RuntimeParams &runtimeParams,
                         const Tensor &cosTable, const Tensor &sinTable, const Tensor &kCache, const Tensor &vCache,
                         uint32_t headDim, const Tensor &preallocOutput = {})
      : q_(q), k_(k), v_(v), cos_(cosTable), sin_(sinTable), kc_(kCache), vc_(vCache), params_(&runtimeParams), headDim_(headDim) {
    if (q.shape.size() != 1 || k.shape.size() != 1 || v.shape.size() != 1) throw std::runtime_error("FusedRoPEKVWrite: q, k, v must be 1D");
    qDim_ = q.shape[0];
    kvDim_ = k.shape[0];
    if (v.shape[0] != kvDim_ || q.dtype != k.dtype || q.dtype != v.dtype)
      throw std::runtime_error("FusedRoPEKVWrite: k and v must have one size, q, k and v one dtype");
    if (headDim_ == 0 || headDim_ % 2 != 0 || qDim_ % headDim_ != 0 || kvDim_ % headDim_ != 0)
      throw std::runtime_error("FusedRoPEKVWrite: qDim and kvDim must be multiples of an even headDim");
    if (cosTable.shape.size() != 2 || sinTable.shape != cosTable.shape || cosTable.shape[1] != headDim_ / 2 ||
        cosTable.dtype != DataType::Float32 || sinTable.dtype != DataType::Float32)
      throw std::runtime_error("FusedRoPEKVWrite: tables must be Float32 [positions, headDim / 2]");
    if (kCache.shape.size() != 2 || vCache.shape != kCache.shape || kCache.shape[1] != kvDim_ || kCache.dtype != DataType::Float16 ||
        vCache.dtype != DataType::Float16 || kCache.stride() != vCache.stride())
      throw std::runtime_error("FusedRoPEKVWrite: caches must be Float16 [positions, kvDim] with one row stride");
    alignedKvDim_ = kCache.stride();   // the reference pads cache rows to four elements (AttentionOp.cpp:570)
    maxPositions_ = kCache.shape[0] < cosTable.shape[0] ? kCache.shape[0] : cosTable.shape[0];
    for (const Tensor *t : {&q, &k, &v, &cosTable, &sinTable, &kCache, &vCache}) detail::requireTensor(*t, "FusedRoPEKVWrite");
    if (preallocOutput.buffer) {
      if (preallocOutput.shape != std::vector<uint32_t>{qDim_}) throw std::runtime_error("FusedRoPEKVWrite: preallocated output must be [qDim]");
      detail::requireTensor(preallocOutput, "FusedRoPEKVWrite");
      output_ = preallocOutput;
    } else {
      storage_ = DeviceBuffer((size_t)qDim_ * 4);
      output_ = Tensor{&storage_, {qDim_}, DataType::Float32, qDim_};
    }
  }
  FusedRoPEKVWriteOpNode(FusedRoPEKVWriteOpNode &&) = delete;
  DataType outputDtype() const { return output_.dtype; }
  std::vector<uint32_t> outputShape() const { return {qDim_}; }
  std::string displayName() const { return "FusedRoPEKVWrite"; }
  const Tensor &output() const { return output_; }
  void dispatch(void *stream = nullptr) const {
    check(cuthip_rope_kv_write(q_.data(), k_.data(), v_.data(), (int)q_.dtype, params_->data(), static_cast<const float *>(cos_.data()),
                               static_cast<const float *>(sin_.data()), kc_.data(), vc_.data(), output_.data(), (int)output_.dtype,
                               qDim_, kvDim_, headDim_, alignedKvDim_, maxPositions_, stream),
          "cuthip_rope_kv_write");
  }

private:
  Tensor q_, k_, v_, cos_, sin_, kc_, vc_;
  const RuntimeParams *params_;
  uint32_t headDim_, qDim_ = 0, kvDim_ = 0, alignedKvDim_ = 0, maxPositions_ = 0;
  DeviceBuffer storage_;
  Tensor output_;
};

// ---- AttentionOpNode: operators/impl/attention/AttentionOp.h:33-66, AttentionOp.cpp:57-86 ---------------
// q [nHeads * headDim]; caches Float16 [maxSeqLen, kvDim]; output [nHeads * headDim] of q's dtype unless another is
// asked for; scale = 1 / sqrt(headDim) (AttentionOp.cpp:77).  maxSeqLen bounds the launch: the capacity of the cache
// unless the caller knows a tighter bound on the sequence length (the kernel reads that many positions).  The node
// owns the scratch of the context splits.
class AttentionOpNode {
public:
  AttentionOpNode(const Tensor &q, const Tensor &kCache, const Tensor &vCache, const RuntimeParams &runtimeParams, uint32_t nHeads,
                  uint32_t nKvHeads, uint32_t headDim, const Tensor &preallocOutput = {}, std::optional<DataType> outDtype = {},
                  std::optional<uint32_t> maxSeqLen = {})
      : q_(q), kc_(kCache), vc_(vCache), params_(&runtimeParams), nHeads_(nHeads), nKvHeads_(nKvHeads), headDim_(headDim) {
    if (nHeads == 0 || nKvHeads == 0 || headDim == 0 || nHeads % nKvHeads != 0)
      throw std::runtime_error("Attention: nHeads must be a positive multiple of nKvHeads");
    if (headDim > 128) throw std::runtime_error("Attention: headDim above 128 is not supported");   // Attention.cu:35-106
    if (q.shape.size() != 1 || q.shape[0] != nHeads * headDim) throw std::runtime_error("Attention: q must be [nHeads * headDim]");
    if (kCache.shape.size() != 2 || vCache.shape != kCache.shape || kCache.shape[1] != nKvHeads * headDim ||
        kCache.dtype != DataType::Float16 || vCache.dtype != DataType::Float16 || kCache.stride() != vCache.stride())
      throw std::runtime_error("Attention: caches must be Float16 [maxSeqLen, nKvHeads * headDim] with one row stride");
    maxSeqLen_ = maxSeqLen.value_or(kCache.shape[0]);
    if (maxSeqLen_ == 0 || maxSeqLen_ > kCache.shape[0]) throw std::runtime_error("Attention: maxSeqLen must lie within the cache");
    for (const Tensor *t : {&q, &kCache, &vCache}) detail::requireTensor(*t, "Attention");
    scale_ = 1.0f / std::sqrt((float)headDim);
    const DataType odt = outDtype.value_or(q.dtype);
    if (preallocOutput.buffer) {
      if (preallocOutput.shape != q.shape || preallocOutput.dtype != odt) throw std::runtime_error("Attention: preallocated output must match q's shape and the output dtype");
      detail::requireTensor(preallocOutput, "Attention");
      output_ = preallocOutput;
    } else {
      storage_ = DeviceBuffer((size_t)q.shape[0] * dtypeBytes(odt));
      output_ = Tensor{&storage_, q.shape, odt, q.shape[0]};
    }
    scratch_ = DeviceBuffer(cuthip_attn_decode_workspace_bytes(nHeads, headDim, maxSeqLen_));
  }
  AttentionOpNode(AttentionOpNode &&) = delete;
  DataType outputDtype() const { return output_.dtype; }
  std::vector<uint32_t> outputShape() const { return output_.shape; }
  std::string displayName() const { return "Attention"; }
  const Tensor &output() const { return output_; }
  void dispatch(void *stream = nullptr) const {
    check(cuthip_attn_decode(q_.data(), (int)q_.dtype, kc_.data(), vc_.data(), params_->data(), output_.data(), (int)output_.dtype,
                             nHeads_, nKvHeads_, headDim_, kc_.stride(), scale_, maxSeqLen_, scratch_.data(), scratch_.bytes(), stream),
          "cuthip_attn_decode");
  }

private:
  Tensor q_, kc_, vc_;
  const RuntimeParams *params_;
  uint32_t nHeads_, nKvHeads_, headDim_, maxSeqLen_ = 0;
  float scale_ = 0.0f;
  DeviceBuffer storage_, scratch_;
  Tensor output_;
};

// ---- load-time row permutations of the fused decode chain (whole block rows move; done once per tensor) ----
// [gate rows | up rows] -> gate_0, up_0, gate_1, up_1, ...: the layout the SiLU(gate) * up epilogue reads.
inline std::vector<uint8_t> interleaveGateUp(const std::vector<uint8_t> &blocks, uint32_t ffn) {
  if (ffn == 0 || blocks.size() % (2 * (size_t)ffn) != 0) throw std::runtime_error("interleaveGateUp: bytes are not 2 * ffn whole rows");
  const size_t rb = blocks.size() / (2 * (size_t)ffn);
  std::vector<uint8_t> out(blocks.size());
  for (uint32_t i = 0; i < ffn; ++i) {
    std::memcpy(&out[(2 * (size_t)i) * rb], &blocks[(size_t)i * rb], rb);
    std::memcpy(&out[(2 * (size_t)i + 1) * rb], &blocks[((size_t)ffn + i) * rb], rb);
  }
  return out;
}
// Rows of [heads * headDim, K] re-ordered inside every head to d = 0, headDim / 2, 1, headDim / 2 + 1, ...: the two
// partners of the half-split rotation become neighbouring rows, which is what the RoPE epilogue of the pair launch reads.
inline std::vector<uint8_t> interleaveRopeRows(const std::vector<uint8_t> &blocks, uint32_t nRows, uint32_t headDim) {
  if (nRows == 0 || headDim == 0 || headDim % 2 != 0 || nRows % headDim != 0 || blocks.size() % nRows != 0)
    throw std::runtime_error("interleaveRopeRows: rows must be whole heads of an even headDim");
  const size_t rb = blocks.size() / nRows;
  const uint32_t half = headDim / 2;
  std::vector<uint8_t> out(blocks.size());
  for (uint32_t h = 0; h < nRows / headDim; ++h)
    for (uint32_t j = 0; j < half; ++j)
      for (uint32_t t = 0; t < 2; ++t)
        std::memcpy(&out[((size_t)h * headDim + 2 * j + t) * rb], &blocks[((size_t)h * headDim + t * half + j) * rb], rb);
  return out;
}

// The two sides of an RMSNorm carried across batch-1 matmuls (cuthip_norm_carry_t): the matmul that forms the
// residual stream (producer) also stores x * weight of the norm that follows as fp16 and the sum of x^2 over each
// group of 8 outputs; the matmul that reads those activations (consumer) scales its result by
// rsqrt(sum / K + eps).  The reference fuses RMSNorm into its consumers (runtime/graph/GraphOptimizer.cpp:46-70).
struct NormCarry {
  const Tensor *sumsqParts = nullptr;       // consumer: Float32 [ceil(K / 8)]
  float eps = 0.0f;
  const Tensor *nextNormWeight = nullptr;   // producer: Float32 [N]
  const Tensor *nextX16 = nullptr;          // producer: Float16 [N], written
  const Tensor *nextSumsqParts = nullptr;   // producer: Float32 [ceil(N / 8)], written
  static NormCarry consumer(const Tensor &sumsqParts, float eps) {
    NormCarry c;
    c.sumsqParts = &sumsqParts;
    c.eps = eps;
    return c;
  }
  static NormCarry producer(const Tensor &nextNormWeight, const Tensor &nextX16, const Tensor &nextSumsqParts) {
    NormCarry c;
    c.nextNormWeight = &nextNormWeight;
    c.nextX16 = &nextX16;
    c.nextSumsqParts = &nextSumsqParts;
    return c;
  }
  // K: length of the activations (consumer side); N: outputs (producer side)
  cuthip_norm_carry_t lower(uint32_t K, uint32_t N) const {
    cuthip_norm_carry_t c{};
    if (sumsqParts) {
      if (sumsqParts->dtype != DataType::Float32) throw std::runtime_error("NormCarry: partial sums must be Float32");
      detail::requireBytes(*sumsqParts, (size_t)((K + 7) / 8) * 4, "NormCarry");
      c.sumsq_parts = static_cast<const float *>(sumsqParts->data());
      c.eps = eps;
    }
    if (nextNormWeight || nextX16 || nextSumsqParts) {
      if (!nextNormWeight || !nextX16 || !nextSumsqParts) throw std::runtime_error("NormCarry: the producer side needs all three tensors");
      if (nextNormWeight->dtype != DataType::Float32 || nextX16->dtype != DataType::Float16 || nextSumsqParts->dtype != DataType::Float32)
        throw std::runtime_error("NormCarry: producer tensors are Float32 weight, Float16 activations, Float32 partial sums");
      detail::requireBytes(*nextNormWeight, (size_t)N * 4, "NormCarry");
      detail::requireBytes(*nextX16, (size_t)N * 2, "NormCarry");
      detail::requireBytes(*nextSumsqParts, (size_t)((N + 7) / 8) * 4, "NormCarry");
      c.next_norm_weight = static_cast<const float *>(nextNormWeight->data());
      c.next_x16 = nextX16->data();
      c.next_sumsq_parts = static_cast<float *>(nextSumsqParts->data());
    }
    return c;
  }
  bool any() const { return sumsqParts || nextNormWeight || nextX16 || nextSumsqParts; }
};

// ---- MatMulGgufCarryOpNode: a batch-1 MatMulGgufOpNode taking part in a carried RMSNorm -----------------
// a [K]; output [N], or [N / 2] with the SiLU(gate) * up epilogue over interleaved rows (setSwigluPairs).  With
// preallocOutput == the tensor d of a Binary add the node updates the residual stream in place.
class MatMulGgufCarryOpNode {
public:
  MatMulGgufCarryOpNode(const Tensor &a, const Tensor &wBlocks, GgufFormat format, uint32_t N, const NormCarry &carry,
                        DataType outDtype = DataType::Float32, const Tensor &preallocOutput = {}, bool swigluPairs = false)
      : a_(a), w_(wBlocks), format_(format), N_(N), swiglu_(swigluPairs) {
    if (a.shape.size() != 1) throw std::runtime_error("MatMulGgufCarryOpNode: A must be a vector (batch 1)");
    K_ = a.shape[0];
    if (K_ == 0 || N_ == 0 || K_ % blockElems(format) != 0) throw std::runtime_error("MatMulGgufCarryOpNode: K must be a positive multiple of the block size");
    if (swiglu_ && N_ % 2 != 0) throw std::runtime_error("MatMulGgufCarryOpNode: row pairs need an even N");
    detail::requireTensor(a, "MatMulGgufCarryOpNode");
    detail::requireBytes(wBlocks, ggufBytes(format, (uint64_t)N_ * K_), "MatMulGgufCarryOpNode");
    const uint32_t outN = swiglu_ ? N_ / 2 : N_;
    carry_ = carry.lower(K_, outN);
    if (preallocOutput.buffer) {
      if (preallocOutput.shape != std::vector<uint32_t>{outN}) throw std::runtime_error("MatMulGgufCarryOpNode: preallocated output of the wrong size");
      detail::requireTensor(preallocOutput, "MatMulGgufCarryOpNode");
      output_ = preallocOutput;
    } else {
      storage_ = DeviceBuffer((size_t)outN * dtypeBytes(outDtype));
      output_ = Tensor{&storage_, {outN}, outDtype, outN};
    }
  }
  MatMulGgufCarryOpNode(MatMulGgufCarryOpNode &&) = delete;
  void setFusion(MatMulFusion fusion, int fusionOp = 0, const Tensor &d = {}) {
    if (swiglu_ && fusion != MatMulFusion::None) throw std::runtime_error("MatMulGgufCarryOpNode::setFusion: the row-pair epilogue takes no further fusion");
    if (fusion == MatMulFusion::Binary) {
      if (!d.buffer) throw std::runtime_error("MatMulGgufCarryOpNode::setFusion: Binary fusion needs the tensor d");
      if (d.dtype != output_.dtype || d.shape != output_.shape) throw std::runtime_error("MatMulGgufCarryOpNode::setFusion: d must match the output");
    }
    fusion_ = fusion;
    fusionOp_ = fusionOp;
    d_ = d;
  }
  DataType outputDtype() const { return output_.dtype; }
  std::vector<uint32_t> outputShape() const { return output_.shape; }
  std::string displayName() const { return "MatMulGgufCarry"; }
  const Tensor &output() const { return output_; }
  void dispatch(void *stream = nullptr) const {
    check(cuthip_matmul_gguf_carry((int)format_, w_.data(), a_.data(), (int)a_.dtype, output_.data(), (int)output_.dtype, K_, N_,
                                   swiglu_ ? (int)CUTHIP_EPI_SWIGLU_PAIRS : (int)fusion_, fusionOp_, d_.data(), &carry_, stream),
          "cuthip_matmul_gguf_carry");
  }

private:
  Tensor a_, w_, d_;
  GgufFormat format_;
  uint32_t K_ = 0, N_ = 0;
  bool swiglu_ = false;
  cuthip_norm_carry_t carry_{};
  MatMulFusion fusion_ = MatMulFusion::None;
  int fusionOp_ = 0;
  DeviceBuffer storage_;
  Tensor output_;
};

// ---- MatMulGgufPairOpNode: two batch-1 matmuls on one activation vector in one launch -------------------
// The q | k and v projections of a decode step, whose weights differ in format in the common GGUF mixes (the
// reference fuses wqkv only when its loader could concatenate them, interface/runner/llama/llama.cpp:1710-1756).
// Plain form: outputs [Na] and [Nb].  With setRopeAppend the launch is the projections plus FusedRoPEKVWriteOpNode:
// tensor A holds the rows [q heads | k heads] in interleaveRopeRows order, tensor B the v rows; the rotated q is the
// node's output, rotated k and v go to the cache row of the position, and the plain outputs are not written.
class MatMulGgufPairOpNode {
public:
  MatMulGgufPairOpNode(const Tensor &a, const Tensor &wa, GgufFormat formatA, uint32_t Na, const Tensor &wb, GgufFormat formatB,
                       uint32_t Nb, const NormCarry &carry = {}, DataType outDtype = DataType::Float32)
      : a_(a), wa_(wa), wb_(wb), fa_(formatA), fb_(formatB), Na_(Na), Nb_(Nb), outDtype_(outDtype) {
    if (a.shape.size() != 1) throw std::runtime_error("MatMulGgufPairOpNode: A must be a vector (batch 1)");
    K_ = a.shape[0];
    if (K_ == 0 || Na == 0 || Nb == 0 || K_ % blockElems(formatA) != 0 || K_ % blockElems(formatB) != 0)
      throw std::runtime_error("MatMulGgufPairOpNode: K must be a positive multiple of both block sizes");
    detail::requireTensor(a, "MatMulGgufPairOpNode");
    detail::requireBytes(wa, ggufBytes(formatA, (uint64_t)Na * K_), "MatMulGgufPairOpNode");
    detail::requireBytes(wb, ggufBytes(formatB, (uint64_t)Nb * K_), "MatMulGgufPairOpNode");
    if (carry.nextNormWeight || carry.nextX16 || carry.nextSumsqParts)
      throw std::runtime_error("MatMulGgufPairOpNode: only the consumer side of a carried norm applies");
    hasCarry_ = carry.any();
    carry_ = carry.lower(K_, 0);
    storageA_ = DeviceBuffer((size_t)Na * dtypeBytes(outDtype));
    storageB_ = DeviceBuffer((size_t)Nb * dtypeBytes(outDtype));
    outputA_ = Tensor{&storageA_, {Na}, outDtype, Na};
    outputB_ = Tensor{&storageB_, {Nb}, outDtype, Nb};
  }
  MatMulGgufPairOpNode(MatMulGgufPairOpNode &&) = delete;
  void setRopeAppend(const RuntimeParams &runtimeParams, const Tensor &cosTable, const Tensor &sinTable, const Tensor &kCache,
                     const Tensor &vCache, uint32_t qDim, uint32_t headDim, const Tensor &preallocQ = {}) {
    if (headDim == 0 || headDim % 2 != 0 || qDim == 0 || qDim % headDim != 0 || qDim >= Na_ || (Na_ - qDim) % headDim != 0 || Nb_ != Na_ - qDim)
      throw std::runtime_error("MatMulGgufPairOpNode::setRopeAppend: tensor A is [qDim + kvDim] rows, tensor B kvDim rows, whole heads");
    if (cosTable.shape.size() != 2 || sinTable.shape != cosTable.shape || cosTable.shape[1] != headDim / 2 ||
        cosTable.dtype != DataType::Float32 || sinTable.dtype != DataType::Float32)
      throw std::runtime_error("MatMulGgufPairOpNode::setRopeAppend: tables must be Float32 [positions, headDim / 2]");
    if (kCache.shape.size() != 2 || vCache.shape != kCache.shape || kCache.shape[1] != Nb_ || kCache.dtype != DataType::Float16 ||
        vCache.dtype != DataType::Float16 || kCache.stride() != vCache.stride())
      throw std::runtime_error("MatMulGgufPairOpNode::setRopeAppend: caches must be Float16 [positions, kvDim] with one row stride");
    for (const Tensor *t : {&cosTable, &sinTable, &kCache, &vCache}) detail::requireTensor(*t, "MatMulGgufPairOpNode::setRopeAppend");
    if (preallocQ.buffer) {
      if (preallocQ.shape != std::vector<uint32_t>{qDim}) throw std::runtime_error("MatMulGgufPairOpNode::setRopeAppend: preallocated q must be [qDim]");
      detail::requireTensor(preallocQ, "MatMulGgufPairOpNode::setRopeAppend");
      qOut_ = preallocQ;
    } else {
      storageQ_ = DeviceBuffer((size_t)qDim * 4);
      qOut_ = Tensor{&storageQ_, {qDim}, DataType::Float32, qDim};
    }
    rope_ = cuthip_rope_append_t{};
    rope_.runtime_params = runtimeParams.data();
    rope_.cos_table = static_cast<const float *>(cosTable.data());
    rope_.sin_table = static_cast<const float *>(sinTable.data());
    rope_.q_out = qOut_.data();
    rope_.q_out_dtype = (int)qOut_.dtype;
    rope_.k_cache = kCache.data();
    rope_.v_cache = vCache.data();
    rope_.q_dim = qDim;
    rope_.head_dim = headDim;
    rope_.aligned_kv_dim = kCache.stride();
    rope_.max_positions = kCache.shape[0] < cosTable.shape[0] ? kCache.shape[0] : cosTable.shape[0];
    hasRope_ = true;
  }
  std::string displayName() const { return hasRope_ ? "MatMulGgufPairRoPEKVWrite" : "MatMulGgufPair"; }
  const Tensor &outputA() const { return outputA_; }
  const Tensor &outputB() const { return outputB_; }
  const Tensor &output() const {   // the rotated q once setRopeAppend was called
    if (!hasRope_) throw std::runtime_error("MatMulGgufPairOpNode::output: no RoPE epilogue set; use outputA() / outputB()");
    return qOut_;
  }
  void dispatch(void *stream = nullptr) const {
    check(cuthip_matmul_gguf_pair((int)fa_, wa_.data(), Na_, hasRope_ ? nullptr : outputA_.data(), (int)fb_, wb_.data(), Nb_,
                                  hasRope_ ? nullptr : outputB_.data(), a_.data(), (int)a_.dtype, (int)outDtype_, K_,
                                  hasCarry_ ? &carry_ : nullptr, hasRope_ ? &rope_ : nullptr, stream),
          "cuthip_matmul_gguf_pair");
  }

private:
  Tensor a_, wa_, wb_;
  GgufFormat fa_, fb_;
  uint32_t Na_, Nb_, K_ = 0;
  DataType outDtype_;
  bool hasCarry_ = false, hasRope_ = false;
  cuthip_norm_carry_t carry_{};
  cuthip_rope_append_t rope_{};
  DeviceBuffer storageA_, storageB_, storageQ_;
  Tensor outputA_, outputB_, qOut_;
};

// ---- MatMulGgufArgmaxOpNode: the output head with the sampling folded in -----------------------------------
// logits [N] = a [K] . dequant(W)^T, the repetition penalty on the listed tokens, the index of the first maximum
// (the reference runs LM head, RepetitionPenaltyOpNode and ReduceArgmax as three dispatches,
// interface/runner/llama/llama.cpp:2145-2152).  The penalty list lives on the device (setPenalties uploads it); its
// length is fixed at construction so that a captured graph can be replayed with new entries (unused ones: token -1).
class MatMulGgufArgmaxOpNode {
public:
  MatMulGgufArgmaxOpNode(const Tensor &a, const Tensor &wBlocks, GgufFormat format, uint32_t N, const NormCarry &carry = {},
                         uint32_t penaltyWindow = 0, DataType logitsDtype = DataType::Float32)
      : a_(a), w_(wBlocks), format_(format), N_(N), window_(penaltyWindow) {
    if (a.shape.size() != 1) throw std::runtime_error("MatMulGgufArgmaxOpNode: A must be a vector (batch 1)");
    K_ = a.shape[0];
    if (K_ == 0 || N_ == 0 || K_ % blockElems(format) != 0) throw std::runtime_error("MatMulGgufArgmaxOpNode: K must be a positive multiple of the block size");
    if (penaltyWindow > 1024) throw std::runtime_error("MatMulGgufArgmaxOpNode: at most 1024 penalised tokens");
    detail::requireTensor(a, "MatMulGgufArgmaxOpNode");
    detail::requireBytes(wBlocks, ggufBytes(format, (uint64_t)N_ * K_), "MatMulGgufArgmaxOpNode");
    if (carry.nextNormWeight || carry.nextX16 || carry.nextSumsqParts)
      throw std::runtime_error("MatMulGgufArgmaxOpNode: only the consumer side of a carried norm applies");
    hasCarry_ = carry.any();
    carry_ = carry.lower(K_, 0);
    logitsStorage_ = DeviceBuffer((size_t)N_ * dtypeBytes(logitsDtype));
    logits_ = Tensor{&logitsStorage_, {N_}, logitsDtype, N_};
    token_ = DeviceBuffer(4);
    scratch_ = DeviceBuffer(cuthip_matmul_gguf_argmax_workspace_bytes(N_));
    if (window_) {
      penTokens_ = DeviceBuffer((size_t)window_ * 4);
      penFactors_ = DeviceBuffer((size_t)window_ * 4);
      setPenalties({}, {});
    }
  }
  MatMulGgufArgmaxOpNode(MatMulGgufArgmaxOpNode &&) = delete;
  // The entries of the runner's factor vector that are not 1 (llama.cpp:2566-2592); the most recent ones are kept
  // when there are more than the window holds.
  void setPenalties(const std::vector<int32_t> &tokens, const std::vector<float> &factors, void *stream = nullptr) {
    if (tokens.size() != factors.size()) throw std::runtime_error("MatMulGgufArgmaxOpNode::setPenalties: one factor per token");
    if (!window_) {
      if (!tokens.empty()) throw std::runtime_error("MatMulGgufArgmaxOpNode::setPenalties: the node was built without a penalty window");
      return;
    }
    std::vector<int32_t> t(window_, -1);
    std::vector<float> f(window_, 1.0f);
    const size_t n = tokens.size() < window_ ? tokens.size() : window_, skip = tokens.size() - n;
    for (size_t i = 0; i < n; ++i) {
      t[i] = tokens[skip + i];
      f[i] = factors[skip + i];
    }
    penTokens_.upload(t.data(), t.size() * 4, stream);
    penFactors_.upload(f.data(), f.size() * 4, stream);
  }
  std::string displayName() const { return "MatMulGgufArgmax"; }
  const Tensor &output() const { return logits_; }         // the (penalised) logits
  const DeviceBuffer &token() const { return token_; }     // device uint32: the sampled token
  uint32_t readToken(void *stream = nullptr) const {
    uint32_t t = 0;
    token_.download(&t, 4, stream);
    return t;
  }
  void dispatch(void *stream = nullptr) const {
    check(cuthip_matmul_gguf_argmax((int)format_, w_.data(), a_.data(), (int)a_.dtype, logits_.data(), (int)logits_.dtype, K_, N_,
                                    hasCarry_ ? &carry_ : nullptr, static_cast<const int32_t *>(penTokens_.data()),
                                    static_cast<const float *>(penFactors_.data()), window_, scratch_.data(), scratch_.bytes(),
                                    static_cast<uint32_t *>(token_.data()), stream),
          "cuthip_matmul_gguf_argmax");
  }

private:
  Tensor a_, w_;
  GgufFormat format_;
  uint32_t N_, K_ = 0, window_;
  bool hasCarry_ = false;
  cuthip_norm_carry_t carry_{};
  DeviceBuffer logitsStorage_, token_, scratch_, penTokens_, penFactors_;
  Tensor logits_;
};

}  // namespace hip
}  // namespace cut
