// C++ tests of the delegator adapter (include/mace_hip_delegator.h).
//   test_delegator.bin registry   -- registry keys and fallback rule; needs no GPU
//   test_delegator.bin compute    -- ops through the registry on the GPU, checked against the
//                                    reference's golden vectors and the CPU oracle
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "mace_hip_delegator.h"
#include "../../oracle/mace_oracle.h"

using namespace mace_hip;

static int g_fail = 0;
#define EXPECT(cond)                                                              \
  do {                                                                            \
    if (!(cond)) { printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); ++g_fail; } \
  } while (0)

struct DummyGemv : public delegator::Gemv {
  explicit DummyGemv(const DelegatorParam &p) : delegator::Gemv(p) {}
  MaceStatus Compute(const OpContext *, const Tensor *, const Tensor *, const Tensor *,
                     const index_t, const index_t, const index_t, const bool, const bool,
                     Tensor *) override { return MaceStatus::MACE_UNSUPPORTED; }
};

static int test_registry() {
  OpDelegatorRegistry reg;
  // key string: name_dtype_runtime_impl_tag (op_delegator_registry.cc:39-44)
  EXPECT(MACE_HIP_DELEGATOR_KEY(Gemm, RT_CPU, float, REF).ToString() == "Gemm_1_0_0_general");
  EXPECT(MACE_HIP_DELEGATOR_KEY_EX(Conv2d, RT_CPU, float, NEON, K1x1).ToString() ==
         "Conv2d_1_0_1_K1x1");
  EXPECT(hip::RegisterAllHipDelegators(&reg) == MaceStatus::MACE_SUCCESS);
  // duplicate keys are rejected (a CHECK failure in the reference, :52-58)
  EXPECT(hip::RegisterAllHipDelegators(&reg) == MaceStatus::MACE_INVALID_ARGS);
  EXPECT((bool)reg.GetCreator(MACE_HIP_DELEGATOR_KEY(Gemm, RT_CPU, float, kCpuImplType)));
  EXPECT((bool)reg.GetCreator(MACE_HIP_DELEGATOR_KEY(Gemv, RT_CPU, uint8_t, kCpuImplType)));
  // fallback: NEON + tag -> NEON general -> REF + tag -> REF general (:64-103)
  EXPECT((bool)reg.GetCreator(MACE_HIP_DELEGATOR_KEY(Gemv, RT_CPU, float, NEON)));
  EXPECT((bool)reg.GetCreator(MACE_HIP_DELEGATOR_KEY_EX(Gemv, RT_CPU, float, NEON, K3x3)));
  EXPECT((bool)reg.GetCreator(MACE_HIP_DELEGATOR_KEY_EX(Conv2d, RT_CPU, float, NEON, K1x1)));
  // a tagged-only registration does not serve the general key
  EXPECT(!reg.GetCreator(MACE_HIP_DELEGATOR_KEY(Conv2d, RT_CPU, float, REF)));
  EXPECT(!reg.GetCreator(MACE_HIP_DELEGATOR_KEY(Gemm, RT_OPENCL, float, REF)));
  // an exact NEON registration wins over the REF fallback
  EXPECT(MACE_HIP_REGISTER_DELEGATOR(&reg, DummyGemv, DelegatorParam,
                                     MACE_HIP_DELEGATOR_KEY(Gemv, RT_CPU, float, NEON)) ==
         MaceStatus::MACE_SUCCESS);
  auto c = reg.GetCreator(MACE_HIP_DELEGATOR_KEY_EX(Gemv, RT_CPU, float, NEON, K3x3));
  std::unique_ptr<OpDelegator> d = c(DelegatorParam());
  EXPECT(dynamic_cast<DummyGemv *>(d.get()) != nullptr);
  // MatMul shape derivation (matmul.cc:55-83, 117-154)
  ops::MatMulShape s;
  Tensor a(nullptr, DT_FLOAT, {2, 3, 31, 61}), b(nullptr, DT_FLOAT, {61, 67});
  EXPECT(ops::MatMulInferShape(&a, &b, false, false, &s) == MaceStatus::MACE_SUCCESS);
  EXPECT(s.batch == 6 && s.rows == 31 && s.cols == 67 && s.depth == 61 && s.lhs_batched &&
         !s.rhs_batched && s.output_shape == (std::vector<index_t>{2, 3, 31, 67}));
  Tensor a3(nullptr, DT_FLOAT, {2, 3, 4}), b3(nullptr, DT_FLOAT, {3, 4, 5});
  EXPECT(ops::MatMulInferShape(&a3, &b3, false, false, &s) == MaceStatus::MACE_INVALID_ARGS);
  Tensor a1(nullptr, DT_FLOAT, {3}), b2(nullptr, DT_FLOAT, {3, 2});
  EXPECT(ops::MatMulInferShape(&a1, &b2, false, false, &s) == MaceStatus::MACE_INVALID_ARGS);
  Tensor a2(nullptr, DT_FLOAT, {3, 4}), b4(nullptr, DT_FLOAT, {5, 6});
  EXPECT(ops::MatMulInferShape(&a2, &b4, false, false, &s) == MaceStatus::MACE_INVALID_ARGS);
  EXPECT(ops::MatMulInferShape(&a2, &b4, true, false, &s) == MaceStatus::MACE_INVALID_ARGS);
  Tensor b5(nullptr, DT_FLOAT, {6, 4});
  EXPECT(ops::MatMulInferShape(&a2, &b5, false, true, &s) == MaceStatus::MACE_SUCCESS);
  EXPECT(s.rows == 3 && s.cols == 6 && s.depth == 4 && s.batch == 1);
  return g_fail;
}

static bool near(const std::vector<float> &got, const std::vector<float> &want) {
  if (got.size() != want.size()) return false;
  for (size_t i = 0; i < got.size(); ++i)
    if (std::fabs(got[i] - want[i]) > 1e-5 * std::fabs(want[i]) + 1e-8 + 1e-5) return false;
  return true;
}

static int test_compute() {
  mace_hip_ctx *hctx = nullptr;
  if (mace_hip_ctx_create(0, &hctx) != MACE_HIP_SUCCESS) { printf("FAIL: no context\n"); return 1; }
  OpContext context(hctx);
  OpDelegatorRegistry reg;
  EXPECT(hip::RegisterAllHipDelegators(&reg) == MaceStatus::MACE_SUCCESS);

  {  // matmul_test.cc:56-58 SimpleCPU
    std::vector<float> a = {1, 2, 3, 4, 5, 6}, b = {1, 2, 3, 4, 5, 6}, c(4);
    Tensor A(a.data(), DT_FLOAT, {1, 2, 3}), B(b.data(), DT_FLOAT, {1, 3, 2}), C(c.data(), DT_FLOAT, {});
    ops::MatMulOpFloat op(&reg, false, false);
    EXPECT(op.Run(&context, &A, &B, nullptr, &C) == MaceStatus::MACE_SUCCESS);
    EXPECT(C.shape() == (std::vector<index_t>{1, 2, 2}));
    EXPECT(near(c, {22, 28, 49, 64}));
    // rows == 1 && transpose_b -> Gemv branch with bias as initial value (matmul.cc:158-168)
    std::vector<float> x = {1, 2, 3}, w = {1, 0, 1, 2, 2, 2}, bias = {10, 20}, y(2);
    Tensor X(x.data(), DT_FLOAT, {1, 3}), W(w.data(), DT_FLOAT, {2, 3}), Bi(bias.data(), DT_FLOAT, {2}),
        Y(y.data(), DT_FLOAT, {});
    ops::MatMulOpFloat opv(&reg, false, true);
    EXPECT(opv.Run(&context, &X, &W, &Bi, &Y) == MaceStatus::MACE_SUCCESS);
    EXPECT(near(y, {14, 32}));
    // Gemm branch with per-column bias (matmul.cc:195-211)
    std::vector<float> bias2 = {0.5f, -1.f}, c2(4);
    Tensor Bi2(bias2.data(), DT_FLOAT, {2}), C2(c2.data(), DT_FLOAT, {});
    EXPECT(op.Run(&context, &A, &B, &Bi2, &C2) == MaceStatus::MACE_SUCCESS);
    EXPECT(near(c2, {22.5f, 27, 49.5f, 63}));
  }
  {  // fully_connected_test.cc:78-81 SimpleCPU (second case) and :89-93 WithBatch
    std::vector<float> x = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10};
    std::vector<float> w = {1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 10, 20, 30, 40, 50, 60, 70, 80, 90, 100};
    std::vector<float> bias = {2, 3}, y(2);
    Tensor X(x.data(), DT_FLOAT, {1, 1, 2, 5}), W(w.data(), DT_FLOAT, {2, 1, 2, 5}, 0, 0, true),
        Bi(bias.data(), DT_FLOAT, {2}), Y(y.data(), DT_FLOAT, {});
    ops::FullyConnectedOp<float> fc(&reg);
    EXPECT(fc.Run(&context, &X, &W, &Bi, &Y) == MaceStatus::MACE_SUCCESS);
    EXPECT(Y.shape() == (std::vector<index_t>{1, 2, 1, 1}));
    EXPECT(near(y, {387, 3853}));
    Tensor Wbad(w.data(), DT_FLOAT, {2, 1, 5, 2});
    EXPECT(fc.Run(&context, &X, &Wbad, &Bi, &Y) == MaceStatus::MACE_INVALID_ARGS);
  }
  {  // conv_2d_test.cc:1240-1275: the quantized known answer 230, as a 1x1 conv over 18 channels
    std::vector<uint8_t> f = {102, 150, 123, 135, 1, 216, 137, 47, 53, 75, 145, 130, 171, 62, 255, 122, 72, 211};
    std::vector<uint8_t> in = {1, 75, 117, 161, 127, 119, 94, 151, 203, 151, 84, 61, 55, 142, 113, 139, 3, 255};
    std::vector<int32_t> bias = {2};
    std::vector<uint8_t> out(1);
    Tensor F(f.data(), DT_UINT8, {1, 1, 1, 18}, 0.0226f, 127, true), I(in.data(), DT_UINT8, {1, 1, 1, 18}, 0.0204f, 93),
        Bi(bias.data(), DT_INT32, {1}, 0.00046104f, 0, true), O(out.data(), DT_UINT8, {}, 0.000711f, 1);
    ops::Conv2dK1x1OpQuant conv;
    EXPECT(conv.Run(&context, &I, &F, &Bi, &O) == MaceStatus::MACE_SUCCESS);
    EXPECT(out[0] == 230);
    Tensor F3(f.data(), DT_UINT8, {1, 3, 3, 2}, 0.0226f, 127, true);
    EXPECT(conv.Run(&context, &I, &F3, &Bi, &O) == MaceStatus::MACE_UNSUPPORTED);
    // the same test as the reference runs it: a 3x3 VALID convolution over a 3x3x2 input
    Tensor I3(in.data(), DT_UINT8, {1, 3, 3, 2}, 0.0204f, 93);
    ops::Conv2dOpQuant conv3({1, 1}, ops::VALID);
    out[0] = 0;
    EXPECT(conv3.Run(&context, &I3, &F3, &Bi, &O) == MaceStatus::MACE_SUCCESS);
    EXPECT(out[0] == 230 && O.shape() == (std::vector<index_t>{1, 1, 1, 1}));
    ops::Conv2dOpQuant dilated({1, 1}, ops::SAME, {}, {2, 2});
    EXPECT(dilated.Run(&context, &I3, &F3, &Bi, &O) == MaceStatus::MACE_INVALID_ARGS);
  }
  {  // 3x3 SAME stride 2 against the oracle (conv_2d_test.cc:1387 shape, smaller)
    std::mt19937 rng(11);
    const index_t n = 2, h = 9, w = 11, cin = 16, cout = 24;
    std::vector<uint8_t> x(n * h * w * cin), f(cout * 9 * cin);
    std::vector<int32_t> bias(cout);
    for (auto &v : x) v = rng() & 255;
    for (auto &v : f) v = rng() & 255;
    for (auto &v : bias) v = (int32_t)(rng() % 65536) - 32768;
    int64_t oh, ow; int ph, pw;
    EXPECT(orc_calc_padding_and_output_size(h, w, 3, 3, 1, 1, 2, 2, 1, &oh, &ow, &ph, &pw) == 0);
    std::vector<uint8_t> y(n * oh * ow * cout), want(y.size());
    Tensor X(x.data(), DT_UINT8, {n, h, w, cin}, 0.02f, 120), F(f.data(), DT_UINT8, {cout, 3, 3, cin}, 0.01f, 130, true),
        Bi(bias.data(), DT_INT32, {cout}, 0.0002f, 0, true), Y(y.data(), DT_UINT8, {}, 0.5f, 100);
    ops::Conv2dOpQuant conv({2, 2}, ops::SAME, {}, {1, 1}, 100, 200);   // fused ReLUx as a clamp
    EXPECT(conv.Run(&context, &X, &F, &Bi, &Y) == MaceStatus::MACE_SUCCESS);
    EXPECT(Y.shape() == (std::vector<index_t>{n, oh, ow, cout}));
    EXPECT(orc_conv2d_q8_nhwc(x.data(), f.data(), bias.data(), n, h, w, cin, cout, 3, 3, 2, 2, ph, pw, 0.02f,
                              120, 0.01f, 130, 0.0002f, 0.5f, 100, 100, 200, want.data(), 4) == 0);
    EXPECT(y == want);
  }
  {  // quantized MatMul and FullyConnected vs the oracle, seeded
    std::mt19937 rng(7);
    const index_t batch = 3, rows = 31, depth = 61, cols = 67;
    std::vector<uint8_t> a(batch * depth * rows), b(cols * depth);
    for (auto &v : a) v = rng() & 255;
    for (auto &v : b) v = rng() & 255;
    // transpose_a = transpose_b = true, rhs not batched (matmul_test.cc:425)
    Tensor A(a.data(), DT_UINT8, {batch, depth, rows}, 0.02f, 77), B(b.data(), DT_UINT8, {cols, depth}, 0.015f, 201);
    std::vector<int32_t> c32(batch * rows * cols), want32(c32.size());
    Tensor C32(c32.data(), DT_INT32, {});
    ops::MatMulOpQuant op32(true, true, DT_INT32);
    EXPECT(op32.Run(&context, &A, &B, &C32) == MaceStatus::MACE_SUCCESS);
    EXPECT(C32.zero_point() == 0 && C32.scale() == 0.02f * 0.015f);
    orc_q8_gemm_i32(a.data(), b.data(), batch, rows, cols, depth, ORC_COL_MAJOR, ORC_COL_MAJOR,
                    ORC_ROW_MAJOR, 1, 0, -77, -201, want32.data(), 4);
    EXPECT(c32 == want32);
    std::vector<uint8_t> c8(c32.size()), want8(c32.size());
    Tensor C8(c8.data(), DT_UINT8, {}, 40.f, 128);
    ops::MatMulOpQuant op8(true, true, DT_UINT8);
    EXPECT(op8.Run(&context, &A, &B, &C8) == MaceStatus::MACE_SUCCESS);
    int32_t mult; int shift;
    EXPECT(orc_get_output_multiplier_and_shift(0.02f, 0.015f, 40.f, &mult, &shift) == 0);
    orc_q8_gemm_u8(a.data(), b.data(), batch, rows, cols, depth, ORC_COL_MAJOR, ORC_COL_MAJOR,
                   ORC_ROW_MAJOR, 1, 0, -77, -201, nullptr, mult, shift, 128, 0, 255, want8.data(), 4);
    EXPECT(c8 == want8);
    Tensor Cbad(c8.data(), DT_UINT8, {}, 1e-6f, 128);   // multiplier >= 1: the reference CHECKs
    EXPECT(op8.Run(&context, &A, &B, &Cbad) == MaceStatus::MACE_INVALID_ARGS);

    // The same MatMul on device-resident tensors with B flagged as a constant weight: the op
    // registers it once (matmul.cc:101-108 passes is_weight() as should_cache_pack_), the second
    // Run() reuses its panel and sums, the result stays bit-exact.
    {
      mace_hip_ctx *h = context.hip();
      void *da = nullptr, *db = nullptr, *dc = nullptr;
      EXPECT(mace_hip_malloc(h, a.size(), &da) == MACE_HIP_SUCCESS);
      EXPECT(mace_hip_malloc(h, b.size(), &db) == MACE_HIP_SUCCESS);
      EXPECT(mace_hip_malloc(h, c8.size(), &dc) == MACE_HIP_SUCCESS);
      EXPECT(mace_hip_memcpy_h2d(h, da, a.data(), a.size()) == MACE_HIP_SUCCESS);
      EXPECT(mace_hip_memcpy_h2d(h, db, b.data(), b.size()) == MACE_HIP_SUCCESS);
      Tensor dA(da, DT_UINT8, {batch, depth, rows}, 0.02f, 77, false, true);
      Tensor dB(db, DT_UINT8, {cols, depth}, 0.015f, 201, /*is_weight=*/true, /*on_device=*/true);
      Tensor dC(dc, DT_UINT8, {}, 40.f, 128, false, true);
      ops::MatMulOpQuant dev_op(true, true, DT_UINT8);
      int64_t builds0 = 0, hits0 = 0, builds1 = 0, hits1 = 0;
      EXPECT(mace_hip_weight_cache_stats(h, &builds0, &hits0) == MACE_HIP_SUCCESS);
      for (int run = 0; run < 3; ++run) {
        EXPECT(dev_op.Run(&context, &dA, &dB, &dC) == MaceStatus::MACE_SUCCESS);
        std::vector<uint8_t> got(c8.size());
        EXPECT(mace_hip_memcpy_d2h(h, got.data(), dc, got.size()) == MACE_HIP_SUCCESS);
        EXPECT(got == want8);
      }
      EXPECT(mace_hip_weight_cache_stats(h, &builds1, &hits1) == MACE_HIP_SUCCESS);
      EXPECT(builds1 - builds0 == 1 && hits1 - hits0 == 2);
      EXPECT(mace_hip_weight_unregister(h, db) == MACE_HIP_SUCCESS);
      mace_hip_free(h, da); mace_hip_free(h, db); mace_hip_free(h, dc);
    }

    const index_t n = 2, o = 40, isz = 7 * 7 * 32;
    std::vector<uint8_t> x(n * isz), w(o * isz), y(n * o), wanty(n * o);
    std::vector<int32_t> bias(o);
    for (auto &v : x) v = rng() & 255;
    for (auto &v : w) v = rng() & 255;
    for (auto &v : bias) v = (int32_t)(rng() % 65536) - 32768;
    Tensor X(x.data(), DT_UINT8, {n, 7, 7, 32}, 0.02f, 128), W(w.data(), DT_UINT8, {o, 7, 7, 32}, 0.01f, 127, true),
        Bi(bias.data(), DT_INT32, {o}, 0.0002f, 0, true), Y(y.data(), DT_UINT8, {}, 0.9f, 30);
    ops::FullyConnectedOp<uint8_t> fc(&reg);
    EXPECT(fc.Run(&context, &X, &W, &Bi, &Y) == MaceStatus::MACE_SUCCESS);
    EXPECT(Y.shape() == (std::vector<index_t>{n, 1, 1, o}));
    orc_q8_gemv_u8(w.data(), x.data(), bias.data(), n, o, isz, 0, 1, 127, 128, 0.01f, 0.02f, 0.9f, 30,
                   ORC_REQUANT_NEON, wanty.data(), 4);
    EXPECT(y == wanty);
  }
  {
    // Quantize -> Dequantize as in the reference's test (quantize_test.cc:24-76): round trip
    // within 0.1, every quantized value > 0 when non_zero is set; bit-exact against the oracle
    const std::vector<std::vector<float>> inputs = {
        {-2, -1, 0, 1, 2, 3, 4}, {0, 1, 2, 3, 4}, {2, 3, 4, 5, 6}, {2, 4, 6, 8}, {-2, -4, -6, -8}};
    for (const auto &in : inputs)
      for (int non_zero = 0; non_zero < 2; ++non_zero) {
        const index_t n = (index_t)in.size();
        std::vector<float> x = in, back(n), wantback(n);
        std::vector<uint8_t> q(n), wantq(n);
        Tensor X(x.data(), DT_FLOAT, {n}), Q(q.data(), DT_UINT8, {}), Y(back.data(), DT_FLOAT, {});
        ops::QuantizeOp quantize(non_zero != 0);
        EXPECT(quantize.Run(&context, &X, &Q) == MaceStatus::MACE_SUCCESS);
        float ws; int32_t wz;
        orc_quantize_dynamic_u8(x.data(), n, non_zero, wantq.data(), &ws, &wz);
        EXPECT(q == wantq && Q.scale() == ws && Q.zero_point() == wz);
        if (non_zero) for (auto v : q) EXPECT(v > 0);
        ops::DequantizeOp<uint8_t> dequantize;
        EXPECT(dequantize.Run(&context, &Q, &Y) == MaceStatus::MACE_SUCCESS);
        orc_dequantize_u8(q.data(), n, ws, wz, wantback.data());
        EXPECT(back == wantback && Y.shape() == X.shape());
        for (index_t i = 0; i < n; ++i) EXPECT(std::fabs(back[i] - x[i]) <= 0.1f);
        // an output that already carries a scale is quantized with it
        Tensor Q2(q.data(), DT_UINT8, {}, 0.05f, 100);
        EXPECT(quantize.Run(&context, &X, &Q2) == MaceStatus::MACE_SUCCESS);
        orc_quantize_with_scale_u8(x.data(), n, 0.05f, 100, wantq.data());
        EXPECT(q == wantq && Q2.scale() == 0.05f && Q2.zero_point() == 100);
      }
  }
  mace_hip_ctx_destroy(hctx);
  return g_fail;
}

// Per-call cost of small ops from a C++ caller (what MACE's engine thread would see): device
// tensors, back-to-back calls, HIP events on the context's stream.  Prints, checks nothing.
static int time_small_calls() {
  mace_hip_ctx *h = nullptr;
  if (mace_hip_ctx_create(0, &h) != MACE_HIP_SUCCESS) return 1;
  struct Case { const char *name; int64_t m, k, n; int b_order; };
  const Case cases[] = {{"uint8 MatMul 128x256 . 256x128 (B row-major)", 128, 256, 128, MACE_HIP_ROW_MAJOR},
                        {"uint8 MatMul 256x256 . 256x256 (B k-contiguous)", 256, 256, 256, MACE_HIP_COL_MAJOR},
                        {"uint8 MatMul 1024x512 . 512x1024 (B row-major)", 1024, 512, 1024, MACE_HIP_ROW_MAJOR}};
  int32_t mult = 0; int shift = 0;
  mace_hip_get_output_multiplier_and_shift(0.02f, 0.015f, 0.05f, &mult, &shift);
  for (const Case &c : cases) {
    void *a = nullptr, *b = nullptr, *o = nullptr;
    mace_hip_malloc(h, (size_t)(c.m * c.k), &a);
    mace_hip_malloc(h, (size_t)(c.k * c.n), &b);
    mace_hip_malloc(h, (size_t)(c.m * c.n), &o);
    std::vector<uint8_t> init((size_t)std::max(c.m * c.k, c.k * c.n), 77);
    mace_hip_memcpy_h2d(h, a, init.data(), (size_t)(c.m * c.k));
    mace_hip_memcpy_h2d(h, b, init.data(), (size_t)(c.k * c.n));
    auto call = [&]() {
      return mace_hip_gemm_q8_u8(h, (const uint8_t *)a, MACE_HIP_ROW_MAJOR, (const uint8_t *)b, c.b_order,
                                 (uint8_t *)o, MACE_HIP_ROW_MAJOR, 1, c.m, c.k, c.n, 1, 1, -128, -128,
                                 nullptr, mult, shift, 128, 0, 255);
    };
    for (int i = 0; i < 20; ++i) call();
    mace_hip_sync(h);
    const int reps = 2000;
    float ms = 0.f;
    mace_hip_timer_start(h);
    for (int i = 0; i < reps; ++i) call();
    mace_hip_timer_stop(h, &ms);
    printf("%-52s %6.2f us per call\n", c.name, ms * 1e3 / reps);
    mace_hip_free(h, a); mace_hip_free(h, b); mace_hip_free(h, o);
  }
  {  // the floor: a kernel with next to nothing to do (Quantize of 256 floats)
    void *x = nullptr, *q = nullptr;
    mace_hip_malloc(h, 1024, &x);
    mace_hip_malloc(h, 256, &q);
    std::vector<float> init(256, 1.5f);
    mace_hip_memcpy_h2d(h, x, init.data(), 1024);
    for (int i = 0; i < 20; ++i) mace_hip_quantize_tensor_u8(h, (const float *)x, 256, 0.03f, 128, (uint8_t *)q);
    mace_hip_sync(h);
    const int reps = 2000;
    float ms = 0.f;
    mace_hip_timer_start(h);
    for (int i = 0; i < reps; ++i) mace_hip_quantize_tensor_u8(h, (const float *)x, 256, 0.03f, 128, (uint8_t *)q);
    mace_hip_timer_stop(h, &ms);
    printf("%-52s %6.2f us per call\n", "Quantize of 256 floats (launch floor)", ms * 1e3 / reps);
    mace_hip_free(h, x); mace_hip_free(h, q);
  }
  mace_hip_ctx_destroy(h);
  return 0;
}

int main(int argc, char **argv) {
  const char *mode = argc > 1 ? argv[1] : "registry";
  if (strcmp(mode, "time") == 0) return time_small_calls();
  int fails = strcmp(mode, "compute") == 0 ? test_compute() : test_registry();
  printf("%s: %s (%d failures)\n", mode, fails ? "FAILED" : "ok", fails);
  return fails ? 1 : 0;
}
