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
