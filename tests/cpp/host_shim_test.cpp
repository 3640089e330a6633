// Exercises include/cut_hip_ops.hpp the way the reference's operator tests do
// (tests/harness/OpRegistry.h:1929-2086): construct nodes, dispatch, compare
// with a CPU reference.  "--cpu": variant tables and constructor validation
// only (no device call).  "--gpu": known-answer and seeded cases on device 0,
// checked against the C oracle.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <random>
#include <string>
#include <vector>

#include "cut_hip_ops.hpp"
extern "C" {
#include "cut_oracle.h"
}

using namespace cut::hip;

static int g_fail = 0;
#define EXPECT(cond)                                                     \
  do {                                                                   \
    if (!(cond)) {                                                       \
      std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);        \
      ++g_fail;                                                          \
    }                                                                    \
  } while (0)

template <class F> static bool throws(F f) {
  try {
    f();
  } catch (const std::runtime_error &) {
    return true;
  }
  return false;
}

template <class F> static std::string message_of(F f) {
  try {
    f();
  } catch (const std::runtime_error &e) {
    return e.what();
  }
  return "";
}

static void test_tables() {
  EXPECT(variantCount(CUTHIP_OP_DEQUANT) >= 1);
  uint32_t n = variantCount(CUTHIP_OP_MATMUL_GGUF);
  EXPECT(n >= 4);
  // indices are ABI: these names must stay at these positions
  EXPECT(getMatMulGgufVariantName(0) == "MatMulGgufGemvMfma");
  EXPECT(getMatMulGgufVariantName(1) == "MatMulGgufSkinnyMfma");
  EXPECT(getMatMulGgufVariantName(2) == "MatMulGgufGemmLds");
  EXPECT(getMatMulGgufVariantName(3) == "MatMulGgufGemvRows8");
  EXPECT(getMatMulGgufVariantName(4) == "MatMulGgufDequantGemm");
  for (uint32_t i = 0; i < n; ++i) EXPECT(lookupVariant(CUTHIP_OP_MATMUL_GGUF, variantInfo(CUTHIP_OP_MATMUL_GGUF, i).name) == i);
  EXPECT(throws([] { lookupVariant(CUTHIP_OP_MATMUL_GGUF, "NoSuchVariant"); }));
  EXPECT(throws([&] { variantInfo(CUTHIP_OP_MATMUL_GGUF, n); }));
}

static void test_validation() {
  DeviceBuffer none;   // empty: constructors must reject before touching the device
  Tensor raw{&none, {0}, DataType::Float32, 0};
  EXPECT(throws([&] { DequantOpNode n(raw, GgufFormat::Q4_K, 4, 100); }));    // cols not a multiple of 256
  EXPECT(throws([&] { DequantOpNode n(raw, GgufFormat::Q4_K, 4, 256); }));    // raw too small
  Tensor a{&none, {1, 2, 3}, DataType::Float16, 0};
  EXPECT(throws([&] { MatMulGgufOpNode n(a, raw, GgufFormat::Q8_0, 8); }));   // rank 3
  Tensor a2{&none, {2, 48}, DataType::Float16, 0};
  EXPECT(throws([&] { MatMulGgufOpNode n(a2, raw, GgufFormat::Q8_0, 8); }));  // K not a multiple of 32
  Tensor a3{&none, {2, 64}, DataType::Float16, 0};
  EXPECT(throws([&] { MatMulGgufOpNode n(a3, raw, GgufFormat::Q8_0, 8); }));  // weights too small
  EXPECT(throws([&] { TransposeQ4NibbleOpNode n(raw, 3, 64); }));             // odd N (TransposeQ4NibbleOp.cpp:13-15)
  EXPECT(throws([&] { TransposeQ4NibbleOpNode n(raw, 4, 48); }));             // K not a multiple of 32
  EXPECT(throws([&] { TransposeQ4NibbleOpNode n(raw, 4, 64); }));             // input too small
  Tensor w16bad{&none, {8, 200}, DataType::Float16, 0};
  Tensor a200{&none, {2, 200}, DataType::Float16, 0};
  EXPECT(throws([&] { MatMulDenseF16OpNode n(a200, w16bad); }));                // K not a multiple of 128
  Tensor w16{&none, {8, 256}, DataType::Float16, 0};
  EXPECT(throws([&] { MatMulDenseF16OpNode n(a200, w16); }));                   // A cols != weight cols
  Tensor a256{&none, {2, 256}, DataType::Float16, 0};
  EXPECT(throws([&] { MatMulDenseF16OpNode n(a256, w16); }));                   // weights too small
  // the operators of a decode step: shapes are checked before any device call
  Tensor x2{&none, {2, 64}, DataType::Float32, 64}, w64{&none, {64}, DataType::Float32, 0}, w32{&none, {32}, DataType::Float32, 0};
  Tensor x3{&none, {1, 2, 64}, DataType::Float32, 64};
  EXPECT(message_of([&] { RMSNormOpNode n(x3, w64); }) == "RMSNorm requires 1D or 2D input, 1D weight");   // RMSNormOp.cpp:20-22
  EXPECT(message_of([&] { RMSNormOpNode n(x2, x2); }) == "RMSNorm requires 1D or 2D input, 1D weight");
  EXPECT(message_of([&] { RMSNormOpNode n(x2, w32); }) == "RMSNorm: weight dimension must match input");     // RMSNormOp.cpp:34-36
  EXPECT(throws([&] { RMSNormOpNode n(x2, w64); }));                                                          // empty buffers
  Tensor q1{&none, {512}, DataType::Float32, 0};
  EXPECT(throws([&] { MatMulGgufCarryOpNode n(x2, raw, GgufFormat::Q4_K, 8, NormCarry{}); }));       // batch above 1
  EXPECT(throws([&] { MatMulGgufCarryOpNode n(q1, raw, GgufFormat::Q4_K, 7, NormCarry{}, DataType::Float32, {}, true); }));   // odd N with row pairs
  EXPECT(throws([&] { MatMulGgufPairOpNode n(x2, raw, GgufFormat::Q4_K, 8, raw, GgufFormat::Q6_K, 8); }));
  EXPECT(throws([&] { MatMulGgufArgmaxOpNode n(q1, raw, GgufFormat::Q6_K, 8, NormCarry{}, 2000); }));  // window above 1024
  {
    std::vector<uint8_t> rows(8 * 3);
    for (size_t i = 0; i < rows.size(); ++i) rows[i] = (uint8_t)(i / 3);           // row r holds the byte r
    const std::vector<uint8_t> gu = interleaveGateUp(rows, 4);                     // gate 0-3 | up 4-7 -> 0 4 1 5 2 6 3 7
    const uint8_t want_gu[8] = {0, 4, 1, 5, 2, 6, 3, 7};
    for (int r = 0; r < 8; ++r) EXPECT(gu[3 * r] == want_gu[r] && gu[3 * r + 2] == want_gu[r]);
    const std::vector<uint8_t> rr = interleaveRopeRows(rows, 8, 4);                // two heads of 4: d = 0 2 1 3 inside each
    const uint8_t want_rr[8] = {0, 2, 1, 3, 4, 6, 5, 7};
    for (int r = 0; r < 8; ++r) EXPECT(rr[3 * r] == want_rr[r]);
    EXPECT(throws([&] { interleaveGateUp(rows, 5); }));
    EXPECT(throws([&] { interleaveRopeRows(rows, 8, 3); }));
  }
  SeparatedWeights sw;
  EXPECT(throws([&] { prepareSeparated(sw, raw, GgufFormat::Q6_K, 4, 256); }));
  EXPECT(throws([&] { prepareSeparated(sw, raw, GgufFormat::Q4_0, 3, 64); }));
  EXPECT(throws([&] { prepareSeparated(sw, raw, GgufFormat::Q8_0, 4, 64); }));  // raw too small
}

// Every branch of the 3-input MatMulOpNode constructor (MatMulOp.cpp:283-374): format inference from the shapes, the
// reference's error texts, the variant it would pick, the padded strides of its push constants.
static void test_matmul_plan() {
  using V = std::vector<uint32_t>;
  const DataType f16 = DataType::Float16;
  // Q8: B.cols == scales.cols
  QuantMatMulPlan p = planQuantMatMul(V{4096}, V{4096, 14336}, V{128, 14336}, f16);
  EXPECT(p.format == QuantFormat::Q8 && p.M == 1 && p.K == 4096 && p.N == 14336 && !p.q4Affine && p.autoSpec);
  EXPECT(p.spec == 4 && p.fusionFallbackSpec == 4);                       // M == 1: MatMulQ8GemvKPar8
  EXPECT(variantInfo(CUTHIP_OP_MATMUL_Q8, p.spec).name == "MatMulQ8GemvKPar8");
  p = planQuantMatMul(V{1, 64}, V{64, 6}, V{2, 6}, f16);
  EXPECT(p.spec == 3 && p.strideA == 64 && p.strideB == 8 && p.strideC == 8 && p.scaleStride == 8);   // N < 8: GemvKPar
  p = planQuantMatMul(V{33, 4096}, V{4096, 4096}, V{128, 4096}, f16);
  EXPECT(p.M == 33 && p.spec == kMatMulQ8VariantCount - 1 && p.fusionFallbackSpec == kMatMulQ8DefaultVariant);   // CoopMatTiled
  p = planQuantMatMul(V{33, 4096}, V{4096, 4100}, V{128, 4100}, f16);
  EXPECT(p.spec == kMatMulQ8DefaultVariant);                               // N % 32 != 0: tiled
  p = planQuantMatMul(V{33, 4096}, V{4096, 4096}, V{128, 4096}, DataType::Float32);
  EXPECT(p.spec == kMatMulQ8DefaultVariant);                               // scales not Float16: tiled
  DeviceCaps nocoop;
  nocoop.cooperativeMatrix = false;
  p = planQuantMatMul(V{33, 4096}, V{4096, 4096}, V{128, 4096}, f16, {}, nocoop);
  EXPECT(p.spec == kMatMulQ8DefaultVariant);
  p = planQuantMatMul(V{33, 4112}, V{4112, 4096}, V{129, 4096}, f16);
  EXPECT(p.spec == kMatMulQ8DefaultVariant);                               // K % 16 == 0 but not a multiple of 128: tiled here
  DeviceCaps refcaps;
  refcaps.cooperativeMatrixK = 16;
  p = planQuantMatMul(V{33, 4112}, V{4112, 4096}, V{129, 4096}, f16, {}, refcaps);
  EXPECT(p.spec == kMatMulQ8VariantCount - 1);                             // the reference's own condition
  p = planQuantMatMul(V{33, 4096}, V{4096, 4096}, V{128, 4096}, f16, 5u);
  EXPECT(p.spec == 5 && !p.autoSpec);                                      // explicit spec is kept
  // Q4: 2 * B.cols == scales.cols; affine when the scales have twice the rows
  p = planQuantMatMul(V{4096}, V{4096, 7168}, V{128, 14336}, f16);
  EXPECT(p.format == QuantFormat::Q4 && p.N == 14336 && !p.q4Affine && p.spec == 3 && p.strideB == 7168);   // Q4GemvKPar8
  p = planQuantMatMul(V{4096}, V{4096, 7168}, V{256, 14336}, f16);
  EXPECT(p.q4Affine && p.spec == 3);
  p = planQuantMatMul(V{1, 64}, V{64, 3}, V{2, 6}, f16);
  EXPECT(p.spec == 2 && p.strideB == 4 && p.scaleStride == 8);             // N < 8: Q4GemvKPar
  p = planQuantMatMul(V{512, 4096}, V{4096, 7168}, V{256, 14336}, f16);
  EXPECT(p.spec == 4 && p.fusionFallbackSpec == kMatMulQ4DefaultVariant && p.q4Affine);   // MatMulQ4CoopMatTiled
  p = planQuantMatMul(V{512, 4096}, V{4096, 7170}, V{128, 14340}, f16);
  EXPECT(p.spec == kMatMulQ4DefaultVariant);
  // the reference's messages
  EXPECT(message_of([&] { planQuantMatMul(V{64}, V{64}, V{2, 6}, f16); }) == "matmul requires 2D B and scales matrices");
  EXPECT(message_of([&] { planQuantMatMul(V{64}, V{64, 6}, V{12}, f16); }) == "matmul requires 2D B and scales matrices");
  EXPECT(message_of([&] { planQuantMatMul(V{1, 2, 64}, V{64, 6}, V{2, 6}, f16); }) == "matmul: A must be 1D or 2D");
  EXPECT(message_of([&] { planQuantMatMul(V{96}, V{64, 6}, V{2, 6}, f16); }) == "matmul: B rows (64) must match A cols (96)");
  EXPECT(message_of([&] { planQuantMatMul(V{64}, V{64, 5}, V{2, 6}, f16); }) ==
         "matmul: cannot determine quant format from B cols (5) and scales cols (6)");
  // the node validates before it touches the device
  DeviceBuffer none;
  Tensor a{&none, {64}, DataType::Float32, 0}, b{&none, {64, 8}, DataType::Float32, 0}, sc{&none, {2, 8}, DataType::Float16, 0};
  EXPECT(throws([&] { MatMulOpNode n(a, b, sc); }));                         // buffers too small
  EXPECT(message_of([&] { MatMulOpNode n(a, b, sc, 8u); }).find("outside the table") != std::string::npos);
  Tensor a16{&none, {64}, DataType::Float16, 0};
  EXPECT(message_of([&] { MatMulOpNode n(a16, b, sc); }).find("Float32 activations") != std::string::npos);
  Tensor a48{&none, {48}, DataType::Float32, 0}, b48{&none, {48, 8}, DataType::Float32, 0};
  EXPECT(message_of([&] { MatMulOpNode n(a48, b48, sc); }).find("multiple of the 32-element") != std::string::npos);
  Tensor as{&none, {2, 64}, DataType::Float32, 70};
  EXPECT(message_of([&] { MatMulOpNode n(as, b, sc); }).find("padded to four") != std::string::npos);
}

static double normwise(const std::vector<float> &got, const std::vector<double> &want) {
  double num = 0, den = 0;
  for (size_t i = 0; i < got.size(); ++i) {
    num += (got[i] - want[i]) * (got[i] - want[i]);
    den += want[i] * want[i];
  }
  return std::sqrt(num / (den > 0 ? den : 1));
}

static void test_gpu() {
  init(0);
  std::mt19937 rng(7);
  std::normal_distribution<float> gw(0.0f, 0.02f), ga(0.0f, 1.0f);
  const GgufFormat fmts[4] = {GgufFormat::Q8_0, GgufFormat::Q4_0, GgufFormat::Q4_K, GgufFormat::Q6_K};
  for (GgufFormat f : fmts) {
    const uint32_t N = 72, K = 512;
    std::vector<float> w((size_t)N * K);
    for (auto &v : w) v = gw(rng);
    std::vector<uint8_t> blocks(ggufBytes(f, (uint64_t)N * K));
    EXPECT(orc_quantize((int)f, w.data(), (size_t)N * K, blocks.data()) == 0);
    DeviceBuffer wdev(blocks.data(), blocks.size());
    Tensor wt{&wdev, {(uint32_t)blocks.size()}, DataType::Float32, 0};

    // dequant: bit-exact against the oracle, fp32 with the reference's padded stride
    DequantOpNode dq(wt, f, N, K);
    dq.dispatch();
    std::vector<float> got((size_t)N * dq.outputStride()), want((size_t)N * K);
    dq.output().buffer->download(got.data(), got.size() * 4);
    EXPECT(orc_dequant((int)f, blocks.data(), want.data(), (size_t)N * K) == 0);
    bool same = true;
    for (uint32_t r = 0; r < N && same; ++r)
      same = std::memcmp(&got[(size_t)r * dq.outputStride()], &want[(size_t)r * K], K * 4) == 0;
    EXPECT(same);

    // separated [K, N] tensors made on the device, bit for bit against the oracle's host split + transpose
    if (f == GgufFormat::Q8_0) {
      SeparatedWeights sw;
      prepareSeparated(sw, wt, f, N, K);
      std::vector<int8_t> vals((size_t)K * sw.strideB), v_nk((size_t)N * K);
      std::vector<uint16_t> sc((size_t)(K / 32) * sw.scaleStride), s_nk((size_t)N * (K / 32));
      sw.values.download(vals.data(), vals.size());
      sw.scales.download(sc.data(), sc.size() * 2);
      orc_split_q8_0(blocks.data(), N, K, v_nk.data(), s_nk.data());
      bool eq = true;
      for (uint32_t k = 0; k < K && eq; ++k)
        for (uint32_t n = 0; n < N && eq; ++n)
          eq = vals[(size_t)k * sw.strideB + n] == v_nk[(size_t)n * K + k] &&
               sc[(size_t)(k / 32) * sw.scaleStride + n] == s_nk[(size_t)n * (K / 32) + k / 32];
      EXPECT(eq);
    }

    // matmul at M = 1 (rank-1 A), 3 and 40 (GEMV, batched GEMV, tiled GEMM), fp32 in / fp32 out
    for (uint32_t M : {1u, 3u, 40u}) {
      std::vector<float> a((size_t)M * K);
      for (auto &v : a) v = ga(rng);
      DeviceBuffer adev(a.data(), a.size() * 4);
      Tensor at{&adev, M == 1 ? std::vector<uint32_t>{K} : std::vector<uint32_t>{M, K}, DataType::Float32, 0};
      MatMulGgufOpNode mm(at, wt, f, N);
      mm.dispatch();
      std::vector<float> c((size_t)M * N);
      mm.output().buffer->download(c.data(), c.size() * 4);
      std::vector<double> ref((size_t)M * N);
      EXPECT(orc_matmul_gguf_f64((int)f, blocks.data(), a.data(), M, K, N, ref.data()) == 0);
      double err = normwise(c, ref);
      if (!(err < 1e-3)) std::printf("fmt %d M %u err %g\n", (int)f, M, err);
      EXPECT(err < 1e-3);

      // fused residual add: C = A.W^T + D
      std::vector<float> d((size_t)M * N, 0.5f);
      DeviceBuffer ddev(d.data(), d.size() * 4);
      Tensor dt{&ddev, {M, N}, DataType::Float32, N};
      MatMulGgufOpNode mf(at, wt, f, N);
      mf.setFusion(MatMulFusion::Binary, CUTHIP_BINARY_ADD, dt);
      mf.dispatch();
      std::vector<float> cf((size_t)M * N);
      mf.output().buffer->download(cf.data(), cf.size() * 4);
      bool ok = true;
      for (size_t i = 0; i < cf.size() && ok; ++i) ok = std::fabs(cf[i] - (c[i] + 0.5f)) <= 1e-5f * (1.0f + std::fabs(c[i]));
      EXPECT(ok);
    }
  }
  // prefill with a workspace: M = 1100 takes the two-pass variant (dequantize once, dense GEMM); variant 4 without a
  // workspace is refused
  {
    const GgufFormat f = GgufFormat::Q4_K;
    const uint32_t M = 1100, N = 136, K = 512;
    std::vector<float> w((size_t)N * K), a((size_t)M * K);
    for (auto &v : w) v = gw(rng);
    for (auto &v : a) v = ga(rng);
    std::vector<uint8_t> blocks(ggufBytes(f, (uint64_t)N * K));
    EXPECT(orc_quantize((int)f, w.data(), (size_t)N * K, blocks.data()) == 0);
    DeviceBuffer wdev(blocks.data(), blocks.size()), adev(a.data(), a.size() * 4);
    Tensor wt{&wdev, {(uint32_t)blocks.size()}, DataType::Float32, 0}, at{&adev, {M, K}, DataType::Float32, 0};
    MatMulGgufOpNode mm(at, wt, f, N);
    EXPECT(mm.workspaceBytes() >= (size_t)N * K * 2 + (size_t)M * K * 2);
    DeviceBuffer small(1024), ws(mm.workspaceBytes());
    EXPECT(throws([&] { mm.setWorkspace(&small); }));
    mm.setWorkspace(&ws);
    mm.dispatch();
    std::vector<float> c((size_t)M * N);
    mm.output().buffer->download(c.data(), c.size() * 4);
    std::vector<double> ref((size_t)M * N);
    EXPECT(orc_matmul_gguf_f64((int)f, blocks.data(), a.data(), M, K, N, ref.data()) == 0);
    EXPECT(normwise(c, ref) < 1e-3);
    MatMulGgufOpNode m4(at, wt, f, N, DataType::Float32, lookupVariant(CUTHIP_OP_MATMUL_GGUF, "MatMulGgufDequantGemm"));
    EXPECT(throws([&] { m4.dispatch(); }));
    m4.setWorkspace(&ws);
    m4.dispatch();
    std::vector<float> c4((size_t)M * N);
    m4.output().buffer->download(c4.data(), c4.size() * 4);
    // the automatic choice may hand the dense GEMM to hipBLASLt (variant 5) where that library is present: same
    // dequantized weights, fp32 accumulation in another order
    std::vector<double> c4d(c4.begin(), c4.end());
    EXPECT(normwise(c, c4d) < 1e-5);
    EXPECT(normwise(c4, ref) < 1e-3);
    // the same product on weights kept dequantized in fp16 (DequantOpNode with a Float16 output feeds the node)
    if (K % 128 == 0 && ((K + 3) & ~3u) == K) {
      DequantOpNode dq16(wt, f, N, K, DataType::Float16);
      dq16.dispatch();
      MatMulDenseF16OpNode md(at, dq16.output(), DataType::Float32);
      md.dispatch();
      std::vector<float> c16((size_t)M * N);
      md.output().buffer->download(c16.data(), c16.size() * 4);
      EXPECT(normwise(c16, ref) < 1e-3);
      EXPECT(normwise(c16, c4d) < 1e-5);
    }
  }
  // a chain of two matmuls (up projection with SiLU, then down projection with a residual add) captured once and
  // replayed on new activations: what a cached decode segment of the reference's runner does per token
  {
    const uint32_t K = 512, H = 768;
    std::mt19937 rng(7);
    std::normal_distribution<float> gw(0.0f, 0.05f), ga(0.0f, 1.0f);
    std::vector<float> w1((size_t)H * K), w2((size_t)K * H);
    for (auto &v : w1) v = gw(rng);
    for (auto &v : w2) v = gw(rng);
    std::vector<uint8_t> b1(ggufBytes(GgufFormat::Q4_K, (uint64_t)H * K)), b2(ggufBytes(GgufFormat::Q6_K, (uint64_t)K * H));
    EXPECT(orc_quantize(CUTHIP_Q4_K, w1.data(), w1.size(), b1.data()) == 0);
    EXPECT(orc_quantize(CUTHIP_Q6_K, w2.data(), w2.size(), b2.data()) == 0);
    DeviceBuffer w1dev(b1.data(), b1.size()), w2dev(b2.data(), b2.size());
    Tensor w1t{&w1dev, {(uint32_t)b1.size()}, DataType::Float32, 0}, w2t{&w2dev, {(uint32_t)b2.size()}, DataType::Float32, 0};
    std::vector<float> x(K);
    DeviceBuffer xdev(x.data(), x.size() * 4);
    Tensor xt{&xdev, {K}, DataType::Float32, 0};
    MatMulGgufOpNode up(xt, w1t, GgufFormat::Q4_K, H);
    up.setFusion(MatMulFusion::Unary, CUTHIP_UNARY_SILU);
    MatMulGgufOpNode down(up.output(), w2t, GgufFormat::Q6_K, K);
    Tensor res{&xdev, {1, K}, DataType::Float32, K};
    down.setFusion(MatMulFusion::Binary, CUTHIP_BINARY_ADD, res);
    Stream stream;
    CommandGraph graph;
    up.dispatch(stream.get());      // one eager pass first (nothing of it is needed later)
    down.dispatch(stream.get());
    stream.sync();
    graph.begin(stream);
    up.dispatch(stream.get());
    down.dispatch(stream.get());
    graph.end(stream);
    for (int rep = 0; rep < 3; ++rep) {
      for (auto &v : x) v = ga(rng);
      xdev.upload(x.data(), x.size() * 4);
      graph.replay(stream);
      stream.sync();
      std::vector<float> got(K);
      down.output().buffer->download(got.data(), got.size() * 4);
      // the same chain on the CPU: fp64 products, SiLU in between, residual at the end
      std::vector<double> h(H), y(K);
      EXPECT(orc_matmul_gguf_f64(CUTHIP_Q4_K, b1.data(), x.data(), 1, K, H, h.data()) == 0);
      std::vector<float> hf(H);
      for (uint32_t i = 0; i < H; ++i) hf[i] = (float)(h[i] / (1.0 + std::exp(-h[i])));
      EXPECT(orc_matmul_gguf_f64(CUTHIP_Q6_K, b2.data(), hf.data(), 1, H, K, y.data()) == 0);
      for (uint32_t i = 0; i < K; ++i) y[i] += x[i];
      double err = normwise(got, y);
      if (!(err < 1e-3)) std::printf("graph replay %d err %g\n", rep, err);
      EXPECT(err < 1e-3);
    }
  }
  // The 3-input MatMulOpNode on the reference's known answers (tests/harness/OpRegistry.h:1995-2086): format and
  // variant inferred from the shapes, rows padded to four elements as the reference's tensors are.
  {
    auto run = [&](uint32_t M, uint32_t K, uint32_t N, bool q4, const std::vector<uint8_t> &bvals, const std::vector<float> &scales,
                   uint32_t scaleRows, std::optional<uint32_t> spec) {
      const uint32_t cols = q4 ? N / 2 : N, sB = (cols + 3) & ~3u, sS = (N + 3) & ~3u, sA = (K + 3) & ~3u;
      std::vector<float> a((size_t)M * sA, 1.0f);
      std::vector<uint8_t> b((size_t)K * sB, 0);
      for (uint32_t k = 0; k < K; ++k)
        for (uint32_t c = 0; c < cols; ++c) b[(size_t)k * sB + c] = bvals[(size_t)k * cols + c];
      std::vector<uint16_t> s((size_t)scaleRows * sS, 0);
      for (uint32_t r = 0; r < scaleRows; ++r)
        for (uint32_t n = 0; n < N; ++n) s[(size_t)r * sS + n] = orc_f32_to_f16(scales[(size_t)r * N + n]);
      DeviceBuffer adev(a.data(), a.size() * 4), bdev(b.data(), b.size()), sdev(s.data(), s.size() * 2);
      Tensor at{&adev, M == 1 ? std::vector<uint32_t>{K} : std::vector<uint32_t>{M, K}, DataType::Float32, 0};
      Tensor bt{&bdev, {K, cols}, DataType::Float32, 0}, st{&sdev, {scaleRows, N}, DataType::Float16, 0};
      MatMulOpNode mm(at, bt, st, spec);
      EXPECT(mm.format() == (q4 ? QuantFormat::Q4 : QuantFormat::Q8));
      mm.dispatch();
      std::vector<float> c((size_t)M * mm.plan().strideC);
      mm.output().buffer->download(c.data(), c.size() * 4);
      return c;
    };
    // q8_simple: A = 1, B[k, 0] = 1, B[k, 1] = 2, scales 1 -> [32, 64]
    std::vector<uint8_t> b8(32 * 2);
    for (uint32_t k = 0; k < 32; ++k) { b8[2 * k] = 1; b8[2 * k + 1] = 2; }
    auto c = run(1, 32, 2, false, b8, {1.0f, 1.0f}, 1, {});
    EXPECT(std::fabs(c[0] - 32.0f) < 1e-3f && std::fabs(c[1] - 64.0f) < 1e-3f);
    // q8_withscales: K = 64, B = 4, scales {0.5, 2} / {1, 0.25} -> [192, 288]
    c = run(1, 64, 2, false, std::vector<uint8_t>(64 * 2, 4), {0.5f, 2.0f, 1.0f, 0.25f}, 2, {});
    EXPECT(std::fabs(c[0] - 192.0f) < 1.0f && std::fabs(c[1] - 288.0f) < 1.0f);
    // q4: nibbles 9 / 10 (values 1 / 2) -> [32, 64]; nibble 12 with the scales above -> [192, 288]
    c = run(1, 32, 2, true, std::vector<uint8_t>(32, 9 | (10 << 4)), {1.0f, 1.0f}, 1, {});
    EXPECT(std::fabs(c[0] - 32.0f) < 1e-3f && std::fabs(c[1] - 64.0f) < 1e-3f);
    c = run(1, 64, 2, true, std::vector<uint8_t>(64, 12 | (12 << 4)), {0.5f, 2.0f, 1.0f, 0.25f}, 2, {});
    EXPECT(std::fabs(c[0] - 192.0f) < 1.0f && std::fabs(c[1] - 288.0f) < 1.0f);
    // every variant index of both tables on the same case, and at M = 3 (the reference's q8/q4AllVariantsVerify)
    for (uint32_t spec = 0; spec < kMatMulQ8VariantCount; ++spec)
      for (uint32_t M : {1u, 3u}) {
        if (spec == kMatMulQ8VariantCount - 1) continue;   // the matrix-core variant needs K % 128 == 0: below
        c = run(M, 64, 2, false, std::vector<uint8_t>(64 * 2, 4), {0.5f, 2.0f, 1.0f, 0.25f}, 2, spec);
        EXPECT(std::fabs(c[0] - 192.0f) < 1.0f && std::fabs(c[1] - 288.0f) < 1.0f);
      }
    for (uint32_t spec = 0; spec + 1 < kMatMulQ4VariantCount; ++spec)
      for (uint32_t M : {1u, 3u}) {
        c = run(M, 64, 2, true, std::vector<uint8_t>(64, 12 | (12 << 4)), {0.5f, 2.0f, 1.0f, 0.25f}, 2, spec);
        EXPECT(std::fabs(c[0] - 192.0f) < 1.0f && std::fabs(c[1] - 288.0f) < 1.0f);
      }
    // M > 1 on a shape the matrix-core variants take (chosen automatically): q = 1, scales 0.5 -> K / 2 everywhere;
    // affine Q4 with nibble 9 (value 1), scale 0.5, minimum 0.25 -> K * 0.75
    {
      const uint32_t M = 40, K = 256, N = 64;
      c = run(M, K, N, false, std::vector<uint8_t>((size_t)K * N, 1), std::vector<float>((size_t)(K / 32) * N, 0.5f), K / 32, {});
      bool ok = true;
      for (uint32_t m = 0; m < M && ok; ++m)
        for (uint32_t n = 0; n < N && ok; ++n) ok = std::fabs(c[(size_t)m * N + n] - K * 0.5f) < 1e-2f;
      EXPECT(ok);
      std::vector<float> sm((size_t)(2 * K / 32) * N, 0.5f);
      for (size_t i = (size_t)(K / 32) * N; i < sm.size(); ++i) sm[i] = 0.25f;
      c = run(M, K, N, true, std::vector<uint8_t>((size_t)K * N / 2, 9 | (9 << 4)), sm, 2 * K / 32, {});
      ok = true;
      for (uint32_t m = 0; m < M && ok; ++m)
        for (uint32_t n = 0; n < N && ok; ++n) ok = std::fabs(c[(size_t)m * N + n] - K * 0.75f) < 1e-2f;
      EXPECT(ok);
    }
  }
  // an explicit variant that cannot take the shape is an error, not a silent fallback
  {
    std::vector<uint8_t> blocks(ggufBytes(GgufFormat::Q8_0, 64 * 64), 0);
    DeviceBuffer wdev(blocks.data(), blocks.size());
    Tensor wt{&wdev, {(uint32_t)blocks.size()}, DataType::Float32, 0};
    std::vector<float> a(16 * 64, 1.0f);
    DeviceBuffer adev(a.data(), a.size() * 4);
    Tensor at{&adev, {16, 64}, DataType::Float32, 0};
    MatMulGgufOpNode mm(at, wt, GgufFormat::Q8_0, 64, DataType::Float32, 3u);   // variant 3 (8-row GEMV) handles M <= 8
    EXPECT(throws([&] { mm.dispatch(); }));
    // the table's default entry (0) takes every M: beyond 8 rows it is the library's choice by shape
    MatMulGgufOpNode md(at, wt, GgufFormat::Q8_0, 64, DataType::Float32, 0u);
    EXPECT(!throws([&] { md.dispatch(); }));
  }
}

// Two layers and the output head of a decode step through the nodes of the shim, in the fused form the Python
// DecodeStep runs (six launches per layer: q | k | v with RoPE and the cache append, attention and its merge, wo +
// residual, gate + up with SiLU * up, w_down + residual; RMSNorm carried across the matmuls; the arg-max in the
// epilogue of the head), captured once and replayed for the next position, against the same chain from oracle calls.
struct ChainConfig {
  uint32_t hidden = 512, layers = 2, heads = 8, kvHeads = 2, headDim = 64, ffn = 1024, vocab = 2048, maxCtx = 64;
  float eps = 1e-5f, theta = 500000.0f;
  uint32_t qDim() const { return heads * headDim; }
  uint32_t kvDim() const { return kvHeads * headDim; }
};
struct LayerHost {
  std::vector<uint8_t> qk, v, o, gateUp, down;   // GGUF blocks, natural row order
  std::vector<float> attnNorm, ffnNorm;
};
static std::vector<float> round_f16(const std::vector<float> &x) {
  std::vector<float> r(x.size());
  for (size_t i = 0; i < x.size(); ++i) r[i] = orc_f16_to_f32(orc_f32_to_f16(x[i]));
  return r;
}
static std::vector<float> cpu_matmul(int fmt, const std::vector<uint8_t> &blocks, const std::vector<float> &a, uint32_t N) {
  std::vector<double> c(N);
  EXPECT(orc_matmul_gguf_f64(fmt, blocks.data(), a.data(), 1, (uint32_t)a.size(), N, c.data()) == 0);
  return std::vector<float>(c.begin(), c.end());
}
// activations rounded to fp16 wherever the device chain stores fp16
static std::vector<float> cpu_chain_step(const ChainConfig &c, const std::vector<LayerHost> &L, const std::vector<float> &outNorm,
                                         const std::vector<uint8_t> &head, std::vector<float> x, uint32_t pos,
                                         std::vector<std::vector<uint16_t>> &kc, std::vector<std::vector<uint16_t>> &vc,
                                         const std::vector<float> &cosT, const std::vector<float> &sinT) {
  std::vector<float> xn(c.hidden), qRot(c.qDim()), attn(c.qDim()), act(c.ffn);
  for (uint32_t i = 0; i < c.layers; ++i) {
    orc_rmsnorm(x.data(), L[i].attnNorm.data(), 1, c.hidden, c.eps, xn.data());
    xn = round_f16(xn);
    const std::vector<float> qk = cpu_matmul(CUTHIP_Q4_K, L[i].qk, xn, c.qDim() + c.kvDim());
    const std::vector<float> v = cpu_matmul(CUTHIP_Q6_K, L[i].v, xn, c.kvDim());
    orc_rope_kv_write(qk.data(), qk.data() + c.qDim(), v.data(), pos, cosT.data(), sinT.data(), c.qDim(), c.kvDim(), c.headDim,
                      c.kvDim(), qRot.data(), kc[i].data(), vc[i].data());
    orc_attention_decode(qRot.data(), kc[i].data(), vc[i].data(), pos + 1, c.heads, c.kvHeads, c.headDim, c.kvDim(),
                         1.0f / std::sqrt((float)c.headDim), attn.data());
    const std::vector<float> o = cpu_matmul(CUTHIP_Q4_K, L[i].o, round_f16(attn), c.hidden);
    for (uint32_t j = 0; j < c.hidden; ++j) x[j] += o[j];
    orc_rmsnorm(x.data(), L[i].ffnNorm.data(), 1, c.hidden, c.eps, xn.data());
    const std::vector<float> gu = round_f16(cpu_matmul(CUTHIP_Q4_K, L[i].gateUp, round_f16(xn), 2 * c.ffn));
    orc_silu_mul(gu.data(), c.ffn, act.data());
    const std::vector<float> d = cpu_matmul(CUTHIP_Q4_K, L[i].down, round_f16(act), c.hidden);
    for (uint32_t j = 0; j < c.hidden; ++j) x[j] += d[j];
  }
  orc_rmsnorm(x.data(), outNorm.data(), 1, c.hidden, c.eps, xn.data());
  return cpu_matmul(CUTHIP_Q6_K, head, round_f16(xn), c.vocab);
}

static void test_gpu_decode_chain() {
  const ChainConfig c;
  std::mt19937 rng(11);
  std::normal_distribution<float> gw(0.0f, 0.05f), ga(0.0f, 1.0f);
  std::uniform_real_distribution<float> un(0.5f, 1.5f);
  auto qw = [&](int fmt, uint32_t n, uint32_t k) {
    std::vector<float> w((size_t)n * k);
    for (auto &v : w) v = gw(rng);
    std::vector<uint8_t> b(ggufBytes((GgufFormat)fmt, (uint64_t)n * k));
    EXPECT(orc_quantize(fmt, w.data(), w.size(), b.data()) == 0);
    return b;
  };
  auto uni = [&](uint32_t n) {
    std::vector<float> w(n);
    for (auto &v : w) v = un(rng);
    return w;
  };
  std::vector<LayerHost> L(c.layers);
  for (auto &l : L) {
    l.qk = qw(CUTHIP_Q4_K, c.qDim() + c.kvDim(), c.hidden);
    l.v = qw(CUTHIP_Q6_K, c.kvDim(), c.hidden);
    l.o = qw(CUTHIP_Q4_K, c.hidden, c.qDim());
    l.gateUp = qw(CUTHIP_Q4_K, 2 * c.ffn, c.hidden);
    l.down = qw(CUTHIP_Q4_K, c.hidden, c.ffn);
    l.attnNorm = uni(c.hidden);
    l.ffnNorm = uni(c.hidden);
  }
  const std::vector<float> outNorm = uni(c.hidden);
  const std::vector<uint8_t> head = qw(CUTHIP_Q6_K, c.vocab, c.hidden);
  // RoPE tables [position][headDim / 2]
  const uint32_t half = c.headDim / 2;
  std::vector<float> cosT((size_t)c.maxCtx * half), sinT((size_t)c.maxCtx * half);
  for (uint32_t p = 0; p < c.maxCtx; ++p)
    for (uint32_t j = 0; j < half; ++j) {
      const double ang = p / std::pow((double)c.theta, 2.0 * j / c.headDim);
      cosT[(size_t)p * half + j] = (float)std::cos(ang);
      sinT[(size_t)p * half + j] = (float)std::sin(ang);
    }
  // nine earlier tokens already in the caches, the same bits on both sides
  uint32_t pos = 9;
  std::vector<std::vector<uint16_t>> kc(c.layers, std::vector<uint16_t>((size_t)c.maxCtx * c.kvDim(), 0)), vc = kc;
  for (uint32_t i = 0; i < c.layers; ++i)
    for (size_t e = 0; e < (size_t)pos * c.kvDim(); ++e) {
      kc[i][e] = orc_f32_to_f16(0.5f * ga(rng));
      vc[i][e] = orc_f32_to_f16(ga(rng));
    }

  // ---- device side: shared tensors, then the nodes of the chain ----
  struct LayerDev {
    DeviceBuffer qk, v, o, gateUp, down, attnNorm, ffnNorm, kCache, vCache;
  };
  std::vector<LayerDev> D(c.layers);
  auto bytesTensor = [](DeviceBuffer &b) { return Tensor{&b, {(uint32_t)b.bytes()}, DataType::Float32, 0}; };
  for (uint32_t i = 0; i < c.layers; ++i) {
    const std::vector<uint8_t> qkI = interleaveRopeRows(L[i].qk, c.qDim() + c.kvDim(), c.headDim);
    const std::vector<uint8_t> guI = interleaveGateUp(L[i].gateUp, c.ffn);
    D[i].qk = DeviceBuffer(qkI.data(), qkI.size());
    D[i].v = DeviceBuffer(L[i].v.data(), L[i].v.size());
    D[i].o = DeviceBuffer(L[i].o.data(), L[i].o.size());
    D[i].gateUp = DeviceBuffer(guI.data(), guI.size());
    D[i].down = DeviceBuffer(L[i].down.data(), L[i].down.size());
    D[i].attnNorm = DeviceBuffer(L[i].attnNorm.data(), c.hidden * 4);
    D[i].ffnNorm = DeviceBuffer(L[i].ffnNorm.data(), c.hidden * 4);
    D[i].kCache = DeviceBuffer(kc[i].data(), kc[i].size() * 2);
    D[i].vCache = DeviceBuffer(vc[i].data(), vc[i].size() * 2);
  }
  DeviceBuffer outNormDev(outNorm.data(), c.hidden * 4), headDev(head.data(), head.size());
  DeviceBuffer cosDev(cosT.data(), cosT.size() * 4), sinDev(sinT.data(), sinT.size() * 4);
  DeviceBuffer xDev((size_t)c.hidden * 4), xnDev((size_t)c.hidden * 2), partsDev((size_t)(c.hidden / 8) * 4);
  DeviceBuffer qRotDev((size_t)c.qDim() * 4), attnDev((size_t)c.qDim() * 2), actDev((size_t)c.ffn * 2);
  const Tensor x{&xDev, {c.hidden}, DataType::Float32, 0}, xn{&xnDev, {c.hidden}, DataType::Float16, 0};
  const Tensor parts{&partsDev, {c.hidden / 8}, DataType::Float32, 0};
  const Tensor qRot{&qRotDev, {c.qDim()}, DataType::Float32, 0}, attn{&attnDev, {c.qDim()}, DataType::Float16, 0};
  const Tensor act{&actDev, {c.ffn}, DataType::Float16, 0};
  const Tensor cosTt{&cosDev, {c.maxCtx, half}, DataType::Float32, 0}, sinTt{&sinDev, {c.maxCtx, half}, DataType::Float32, 0};
  const Tensor outNormT{&outNormDev, {c.hidden}, DataType::Float32, 0};
  RuntimeParams params;
  const NormCarry consume = NormCarry::consumer(parts, c.eps);

  std::vector<Tensor> normA(c.layers), normF(c.layers), kcT(c.layers), vcT(c.layers);
  for (uint32_t i = 0; i < c.layers; ++i) {
    normA[i] = Tensor{&D[i].attnNorm, {c.hidden}, DataType::Float32, 0};
    normF[i] = Tensor{&D[i].ffnNorm, {c.hidden}, DataType::Float32, 0};
    kcT[i] = Tensor{&D[i].kCache, {c.maxCtx, c.kvDim()}, DataType::Float16, 0};
    vcT[i] = Tensor{&D[i].vCache, {c.maxCtx, c.kvDim()}, DataType::Float16, 0};
  }
  RMSNormOpNode firstNorm(x, normA[0], c.eps, DataType::Float16, xn);
  std::vector<std::unique_ptr<MatMulGgufPairOpNode>> qkv;
  std::vector<std::unique_ptr<AttentionOpNode>> att;
  std::vector<std::unique_ptr<MatMulGgufCarryOpNode>> wo, gateUp, down;
  for (uint32_t i = 0; i < c.layers; ++i) {
    // layer 0 reads the output of the RMSNorm node (already scaled); the others the carried form
    qkv.emplace_back(new MatMulGgufPairOpNode(xn, bytesTensor(D[i].qk), GgufFormat::Q4_K, c.qDim() + c.kvDim(), bytesTensor(D[i].v),
                                              GgufFormat::Q6_K, c.kvDim(), i > 0 ? consume : NormCarry{}));
    qkv.back()->setRopeAppend(params, cosTt, sinTt, kcT[i], vcT[i], c.qDim(), c.headDim, qRot);
    att.emplace_back(new AttentionOpNode(qRot, kcT[i], vcT[i], params, c.heads, c.kvHeads, c.headDim, attn, DataType::Float16));
    wo.emplace_back(new MatMulGgufCarryOpNode(attn, bytesTensor(D[i].o), GgufFormat::Q4_K, c.hidden,
                                              NormCarry::producer(normF[i], xn, parts), DataType::Float32, x));
    wo.back()->setFusion(MatMulFusion::Binary, CUTHIP_BINARY_ADD, x);
    gateUp.emplace_back(new MatMulGgufCarryOpNode(xn, bytesTensor(D[i].gateUp), GgufFormat::Q4_K, 2 * c.ffn, consume,
                                                  DataType::Float16, act, true));
    const Tensor &nextNorm = i + 1 < c.layers ? normA[i + 1] : outNormT;
    down.emplace_back(new MatMulGgufCarryOpNode(act, bytesTensor(D[i].down), GgufFormat::Q4_K, c.hidden,
                                                NormCarry::producer(nextNorm, xn, parts), DataType::Float32, x));
    down.back()->setFusion(MatMulFusion::Binary, CUTHIP_BINARY_ADD, x);
  }
  MatMulGgufArgmaxOpNode headNode(xn, bytesTensor(headDev), GgufFormat::Q6_K, c.vocab, consume);
  EXPECT(qkv[0]->displayName() == "MatMulGgufPairRoPEKVWrite" && wo[0]->displayName() == "MatMulGgufCarry");
  EXPECT(headNode.output().shape == std::vector<uint32_t>{c.vocab});

  Stream stream;   // the host's updates of x and of the runtime parameters go through the same stream as the launches
  auto encode = [&] {   // what Dispatcher::encode does for the nodes of the step, in graph order
    firstNorm.dispatch(stream.get());
    for (uint32_t i = 0; i < c.layers; ++i) {
      qkv[i]->dispatch(stream.get());
      att[i]->dispatch(stream.get());
      wo[i]->dispatch(stream.get());
      gateUp[i]->dispatch(stream.get());
      down[i]->dispatch(stream.get());
    }
    headNode.dispatch(stream.get());
  };
  auto check_step = [&](const std::vector<float> &xHost, const char *what) {
    const std::vector<float> want = cpu_chain_step(c, L, outNorm, head, xHost, pos, kc, vc, cosT, sinT);
    std::vector<float> got(c.vocab);
    headNode.output().buffer->download(got.data(), got.size() * 4);
    const double err = normwise(got, std::vector<double>(want.begin(), want.end()));
    if (!(err < 1e-3)) std::printf("decode chain (%s) err %g\n", what, err);
    EXPECT(err < 1e-3);
    uint32_t best = 0;
    for (uint32_t i = 1; i < c.vocab; ++i)
      if (got[i] > got[best]) best = i;
    EXPECT(headNode.readToken() == best);
    // the caches of both sides hold the same row for this position (fp16 bits, up to one unit in the last place)
    std::vector<uint16_t> row(c.kvDim());
    for (uint32_t i = 0; i < c.layers; ++i) {
      std::vector<uint16_t> all((size_t)c.maxCtx * c.kvDim());
      D[i].vCache.download(all.data(), all.size() * 2);
      double num = 0, den = 0;
      for (uint32_t e = 0; e < c.kvDim(); ++e) {
        const double g = orc_f16_to_f32(all[(size_t)pos * c.kvDim() + e]), w = orc_f16_to_f32(vc[i][(size_t)pos * c.kvDim() + e]);
        num += (g - w) * (g - w);
        den += w * w;
      }
      EXPECT(std::sqrt(num / den) < 2e-3);
    }
    return got;
  };

  std::vector<float> xHost(c.hidden);
  for (auto &v : xHost) v = ga(rng);
  xDev.upload(xHost.data(), xHost.size() * 4, stream.get());
  params.set(pos, pos + 1, stream.get());
  encode();   // eager
  stream.sync();
  const std::vector<float> eager = check_step(xHost, "eager");

  CommandGraph graph;
  graph.begin(stream);
  encode();
  graph.end(stream);
  // replay on the same input: the eager logits bit for bit (the cache row of the position is rewritten with the same values)
  xDev.upload(xHost.data(), xHost.size() * 4, stream.get());
  graph.replay(stream);
  stream.sync();
  {
    std::vector<float> again(c.vocab);
    headNode.output().buffer->download(again.data(), again.size() * 4);
    if (std::memcmp(again.data(), eager.data(), again.size() * 4) != 0) {
      size_t ndiff = 0, first = 0;
      double worst = 0;
      for (size_t i = 0; i < again.size(); ++i)
        if (again[i] != eager[i]) {
          if (!ndiff) first = i;
          ++ndiff;
          worst = std::max(worst, (double)std::fabs(again[i] - eager[i]));
        }
      std::printf("replay differs from the eager pass: %zu of %zu logits, first %zu, largest difference %g\n", ndiff, again.size(),
                  first, worst);
    }
    EXPECT(std::memcmp(again.data(), eager.data(), again.size() * 4) == 0);
  }
  // the next two positions through the same graph: only the 8 bytes of the runtime parameters and x change
  for (int rep = 0; rep < 2; ++rep) {
    ++pos;
    for (auto &v : xHost) v = ga(rng);
    xDev.upload(xHost.data(), xHost.size() * 4, stream.get());
    params.set(pos, pos + 1, stream.get());
    graph.replay(stream);
    stream.sync();
    check_step(xHost, rep ? "replay, position 11" : "replay, position 10");
  }

  // the unfused operators of the same layer-0 front: RMSNorm, the two projections, FusedRoPEKVWrite, Attention as the
  // reference's own nodes chain them, against the fused launch (same cache row, same rotated q up to rounding)
  {
    const uint32_t p2 = pos + 1;
    params.set(p2, p2 + 1, stream.get());
    for (auto &v : xHost) v = ga(rng);
    xDev.upload(xHost.data(), xHost.size() * 4, stream.get());
    RMSNormOpNode norm(x, normA[0], c.eps, DataType::Float16);
    DeviceBuffer qkNat(L[0].qk.data(), L[0].qk.size());
    MatMulGgufPairOpNode proj(norm.output(), bytesTensor(qkNat), GgufFormat::Q4_K, c.qDim() + c.kvDim(), bytesTensor(D[0].v),
                              GgufFormat::Q6_K, c.kvDim());
    DeviceBuffer kc2((size_t)c.maxCtx * c.kvDim() * 2), vc2((size_t)c.maxCtx * c.kvDim() * 2);
    std::vector<uint16_t> kcHost((size_t)c.maxCtx * c.kvDim()), vcHost(kcHost.size());
    D[0].kCache.download(kcHost.data(), kcHost.size() * 2);
    D[0].vCache.download(vcHost.data(), vcHost.size() * 2);
    kc2.upload(kcHost.data(), kcHost.size() * 2);
    vc2.upload(vcHost.data(), vcHost.size() * 2);
    const Tensor kc2T{&kc2, {c.maxCtx, c.kvDim()}, DataType::Float16, 0}, vc2T{&vc2, {c.maxCtx, c.kvDim()}, DataType::Float16, 0};
    // q and k are the two halves of the pair's first output
    DeviceBuffer qBuf((size_t)c.qDim() * 4), kBuf((size_t)c.kvDim() * 4);
    const Tensor qT{&qBuf, {c.qDim()}, DataType::Float32, 0}, kT{&kBuf, {c.kvDim()}, DataType::Float32, 0};
    FusedRoPEKVWriteOpNode rope(qT, kT, proj.outputB(), params, cosTt, sinTt, kc2T, vc2T, c.headDim);
    AttentionOpNode attention(rope.output(), kc2T, vc2T, params, c.heads, c.kvHeads, c.headDim);
    norm.dispatch(stream.get());
    proj.dispatch(stream.get());
    check(cuthip_memcpy_d2d(qBuf.data(), proj.outputA().data(), (size_t)c.qDim() * 4, stream.get()), "cuthip_memcpy_d2d");
    check(cuthip_memcpy_d2d(kBuf.data(), static_cast<const uint8_t *>(proj.outputA().data()) + (size_t)c.qDim() * 4,
                            (size_t)c.kvDim() * 4, stream.get()),
          "cuthip_memcpy_d2d");
    rope.dispatch(stream.get());
    attention.dispatch(stream.get());
    // the fused form on the same input
    firstNorm.dispatch(stream.get());
    qkv[0]->dispatch(stream.get());
    att[0]->dispatch(stream.get());
    stream.sync();
    std::vector<float> unfused(c.qDim());
    attention.output().buffer->download(unfused.data(), unfused.size() * 4);
    std::vector<uint16_t> fusedBits(c.qDim());
    attnDev.download(fusedBits.data(), fusedBits.size() * 2);
    std::vector<double> fused(c.qDim());
    for (uint32_t i = 0; i < c.qDim(); ++i) fused[i] = orc_f16_to_f32(fusedBits[i]);
    const double err = normwise(unfused, fused);
    if (!(err < 2e-3)) std::printf("unfused against fused attention front err %g\n", err);
    EXPECT(err < 2e-3);
    // and against the oracle's operators on the same inputs
    std::vector<float> xnH(c.hidden), qRotH(c.qDim()), attnH(c.qDim());
    orc_rmsnorm(xHost.data(), L[0].attnNorm.data(), 1, c.hidden, c.eps, xnH.data());
    xnH = round_f16(xnH);
    const std::vector<float> qkH = cpu_matmul(CUTHIP_Q4_K, L[0].qk, xnH, c.qDim() + c.kvDim());
    const std::vector<float> vH = cpu_matmul(CUTHIP_Q6_K, L[0].v, xnH, c.kvDim());
    orc_rope_kv_write(qkH.data(), qkH.data() + c.qDim(), vH.data(), p2, cosT.data(), sinT.data(), c.qDim(), c.kvDim(), c.headDim, c.kvDim(),
                      qRotH.data(), kcHost.data(), vcHost.data());
    orc_attention_decode(qRotH.data(), kcHost.data(), vcHost.data(), p2 + 1, c.heads, c.kvHeads, c.headDim, c.kvDim(),
                         1.0f / std::sqrt((float)c.headDim), attnH.data());
    const double err2 = normwise(unfused, std::vector<double>(attnH.begin(), attnH.end()));
    if (!(err2 < 1e-3)) std::printf("unfused attention front against the oracle err %g\n", err2);
    EXPECT(err2 < 1e-3);
  }
}

int main(int argc, char **argv) {
  std::string mode = argc > 1 ? argv[1] : "--cpu";
  test_tables();
  test_validation();
  test_matmul_plan();
  if (mode == "--gpu") {
    test_gpu();
    test_gpu_decode_chain();
  }
  std::printf("%s: %d failure(s)\n", mode.c_str(), g_fail);
  return g_fail ? 1 : 0;
}
