// Exercises include/cut_hip_ops.hpp the way the reference's operator tests do
// (tests/harness/OpRegistry.h:1929-2086): construct nodes, dispatch, compare
// with a CPU reference.  "--cpu": variant tables and constructor validation
// only (no device call).  "--gpu": known-answer and seeded cases on device 0,
// checked against the C oracle.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
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
  SeparatedWeights sw;
  EXPECT(throws([&] { prepareSeparated(sw, raw, GgufFormat::Q6_K, 4, 256); }));
  EXPECT(throws([&] { prepareSeparated(sw, raw, GgufFormat::Q4_0, 3, 64); }));
  EXPECT(throws([&] { prepareSeparated(sw, raw, GgufFormat::Q8_0, 4, 64); }));  // raw too small
}

template <class F> static std::string message_of(F f) {
  try {
    f();
  } catch (const std::runtime_error &e) {
    return e.what();
  }
  return "";
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

int main(int argc, char **argv) {
  std::string mode = argc > 1 ? argv[1] : "--cpu";
  test_tables();
  test_validation();
  test_matmul_plan();
  if (mode == "--gpu") test_gpu();
  std::printf("%s: %d failure(s)\n", mode.c_str(), g_fail);
  return g_fail ? 1 : 0;
}
