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

// Every operand of a call has to live where the output does: a device output with a host weight
// or bias (or the other way round) is refused before anything reaches the library -- the context
// here is null, so any call that got through would fail differently.
static void test_placement(OpDelegatorRegistry *reg) {
  OpContext context(nullptr);
  const MaceStatus bad = MaceStatus::MACE_INVALID_ARGS;
  float f[64] = {0};
  uint8_t q[64] = {0};
  int32_t i32[8] = {0};
  auto T = [&](void *p, DataType dt, std::vector<index_t> shape, bool dev, bool weight = false) {
    return Tensor(p, dt, std::move(shape), 0.5f, 3, weight, dev);
  };
  for (int mix = 0; mix < 3; ++mix) {     // which operand sits on the other side
    const bool out_dev = mix != 2;
    Tensor out_f = T(f, DT_FLOAT, {}, out_dev), out_q = T(q, DT_UINT8, {}, out_dev),
           out_i = T(i32, DT_INT32, {}, out_dev);
    Tensor lhs_f = T(f, DT_FLOAT, {4, 4}, mix == 0 ? !out_dev : out_dev, true);
    Tensor rhs_f = T(f, DT_FLOAT, {4, 4}, mix == 1 ? !out_dev : out_dev);
    Tensor bias_f = T(f, DT_FLOAT, {4}, mix == 2 ? !out_dev : out_dev, true);
    hip::Gemm<float> gemm((delegator::GemmParam(true)));
    if (mix < 2) {
      EXPECT(gemm.Compute(&context, &lhs_f, &rhs_f, 1, 4, 4, 4, RowMajor, RowMajor, RowMajor, true, true,
                          &out_f) == bad);
      EXPECT(gemm.Compute(&context, &lhs_f, &rhs_f, 1, 4, 4, 4, 4, false, false, false, true, true,
                          &out_f) == bad);
    }
    hip::Gemv<float> gemv((DelegatorParam()));
    EXPECT(gemv.Compute(&context, &lhs_f, &rhs_f, &bias_f, 1, 4, 4, false, true, &out_f) == bad);
    Tensor lhs_q = T(q, DT_UINT8, {4, 4}, mix == 0 ? !out_dev : out_dev, true);
    Tensor rhs_q = T(q, DT_UINT8, {1, 4}, mix == 1 ? !out_dev : out_dev);
    Tensor bias_i = T(i32, DT_INT32, {4}, mix == 2 ? !out_dev : out_dev, true);
    hip::Gemv<uint8_t> gemv_q((DelegatorParam()));
    hip::Gemv<int32_t> gemv_i((DelegatorParam()));
    EXPECT(gemv_q.Compute(&context, &lhs_q, &rhs_q, &bias_i, 1, 4, 4, false, true, &out_q) == bad);
    EXPECT(gemv_i.Compute(&context, &lhs_q, &rhs_q, &bias_i, 1, 4, 4, false, true, &out_i) == bad);
    // ops
    Tensor in4 = T(f, DT_FLOAT, {1, 4, 1, 1}, rhs_f.on_device());
    Tensor w4 = T(f, DT_FLOAT, {4, 4, 1, 1}, lhs_f.on_device(), true);
    ops::FullyConnectedOp<float> fc(reg, RELU);
    EXPECT(fc.Run(&context, &in4, &w4, &bias_f, &out_f) == bad);
    Tensor in4q = T(q, DT_UINT8, {1, 4, 1, 1}, rhs_q.on_device());
    Tensor w4q = T(q, DT_UINT8, {4, 4, 1, 1}, lhs_q.on_device(), true);
    ops::FullyConnectedOp<uint8_t> fcq(reg);
    EXPECT(fcq.Run(&context, &in4q, &w4q, &bias_i, &out_q) == bad);
    ops::Conv2dOpFloat conv(reg, {1, 1}, VALID);
    Tensor img = T(f, DT_FLOAT, {1, 4, 2, 2}, rhs_f.on_device());
    EXPECT(conv.Run(&context, &img, &w4, &bias_f, &out_f) == bad);
    ops::Conv2dOpQuant convq({1, 1}, VALID);
    Tensor imgq = T(q, DT_UINT8, {1, 2, 2, 4}, rhs_q.on_device());
    Tensor filtq = T(q, DT_UINT8, {4, 1, 1, 4}, lhs_q.on_device(), true);
    EXPECT(convq.Run(&context, &imgq, &filtq, &bias_i, &out_q) == bad);
    if (mix < 2) {
      ops::MatMulOpQuant mm(false, false, DT_UINT8), mm32(false, false, DT_INT32);
      Tensor bq = T(q, DT_UINT8, {4, 4}, rhs_q.on_device());
      EXPECT(mm.Run(&context, &lhs_q, &bq, &out_q) == bad);
      EXPECT(mm32.Run(&context, &lhs_q, &bq, &out_i) == bad);
      ops::MatMulOpFloat mmf(reg, false, false);
      Tensor bias_ok = T(f, DT_FLOAT, {4}, out_dev);
      EXPECT(mmf.Run(&context, &lhs_f, &rhs_f, &bias_ok, &out_f) == bad);
      EXPECT(mmf.Run(&context, &lhs_f, &rhs_f, nullptr, &out_f) == bad);
      ops::QuantizeOp qop;
      Tensor qout = T(q, DT_UINT8, {}, out_dev), qin = T(f, DT_FLOAT, {16}, !out_dev);
      EXPECT(qop.Run(&context, &qin, &qout) == bad);
      ops::DequantizeOp<uint8_t> dq;
      Tensor dqin = T(q, DT_UINT8, {16}, !out_dev);
      EXPECT(dq.Run(&context, &dqin, &out_f) == bad);
    }
  }
  // the float FullyConnected names an activation it does not apply instead of dropping it
  float w[16] = {0}, x[4] = {0}, y[4];
  Tensor W(w, DT_FLOAT, {4, 4, 1, 1}), X(x, DT_FLOAT, {1, 4, 1, 1}), Y(y, DT_FLOAT, {});
  ops::FullyConnectedOp<float> tanh_fc(reg, TANH);
  EXPECT(tanh_fc.Run(&context, &X, &W, nullptr, &Y) == MaceStatus::MACE_UNSUPPORTED);
  ActivationType t = NOOP;
  EXPECT(StringToActivationType("RELUX", &t) && t == RELUX);
  EXPECT(StringToActivationType("HARDSIGMOID", &t) && t == HARDSIGMOID);
  EXPECT(!StringToActivationType("relu", &t));
}

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
  // the float Conv2d delegator answers the general key (what Conv2dOp asks for on a host
  // without NEON, conv_2d.cc:88-91) and the K1x1 tag of a NEON build
  EXPECT((bool)reg.GetCreator(MACE_HIP_DELEGATOR_KEY(Conv2d, RT_CPU, float, REF)));
  EXPECT((bool)reg.GetCreator(MACE_HIP_DELEGATOR_KEY_EX(Conv2d, RT_CPU, float, REF, K1x1)));
  EXPECT(!reg.GetCreator(MACE_HIP_DELEGATOR_KEY(Conv2d, RT_CPU, uint8_t, REF)));
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
  test_placement(&reg);
  return g_fail;
}

// delegator::Gemv served by the CPU oracle: the yardstick the GPU-backed ops are compared with
struct OracleGemv : public delegator::Gemv {
  explicit OracleGemv(const DelegatorParam &p) : delegator::Gemv(p) {}
  MaceStatus Compute(const OpContext *, const Tensor *lhs, const Tensor *rhs, const Tensor *bias,
                     const index_t batch, const index_t h, const index_t w, const bool lb,
                     const bool rb, Tensor *out) override {
    orc_gemv_f32(lhs->data<float>(), rhs->data<float>(), bias ? bias->data<float>() : nullptr,
                 batch, h, w, lb, rb, out->mutable_data<float>(), 1);
    return MaceStatus::MACE_SUCCESS;
  }
};

// reference tolerance of the float comparisons (matmul_test.cc:142-143)
static bool close_enough(const std::vector<float> &got, const std::vector<float> &want) {
  if (got.size() != want.size()) return false;
  for (size_t i = 0; i < got.size(); ++i)
    if (!(std::fabs(got[i] - want[i]) <= 1e-2 + 1e-4 * std::fabs(want[i]))) return false;
  return true;
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
  {  // float FullyConnected with its activation (fully_connected.cc:62-75,121): NOOP / RELU / RELUX
     // against the oracle's Gemv followed by the oracle's activation, host and device tensors,
     // batch 1 (one vector per pass) and batch 5 (shared weights, four vectors per pass), a width
     // that is not a multiple of 4 (the general kernel)
    std::mt19937 rng(99);
    std::normal_distribution<float> nd(0.f, 1.f);
    mace_hip_ctx *hc = context.hip();
    for (index_t in_size : {256, 203}) {
      for (index_t batch : {1, 5}) {
        const index_t out_size = 77;
        std::vector<float> x(batch * in_size), w(out_size * in_size), bias(out_size);
        for (auto &v : x) v = nd(rng);
        for (auto &v : w) v = nd(rng);
        for (auto &v : bias) v = nd(rng);
        for (int act = 0; act < 3; ++act) {
          const float limit = 1.5f;
          std::vector<float> want(batch * out_size), y(want.size(), -99.f);
          orc_gemv_f32(w.data(), x.data(), bias.data(), batch, out_size, in_size, 0, 1, want.data(), 1);
          orc_activation_f32(want.data(), (int64_t)want.size(), act, limit);
          Tensor X(x.data(), DT_FLOAT, {batch, in_size, 1, 1}), W(w.data(), DT_FLOAT, {out_size, in_size, 1, 1}, 0, 0, true),
              Bi(bias.data(), DT_FLOAT, {out_size}, 0, 0, true), Y(y.data(), DT_FLOAT, {});
          ops::FullyConnectedOp<float> fc(&reg, (ActivationType)act, limit);
          EXPECT(fc.Run(&context, &X, &W, &Bi, &Y) == MaceStatus::MACE_SUCCESS);
          EXPECT(Y.shape() == (std::vector<index_t>{batch, out_size, 1, 1}));
          EXPECT(close_enough(y, want));
          if (act == 1) { float lo = 0.f; for (float v : y) lo = std::min(lo, v); EXPECT(lo == 0.f); }
          if (act == 2) { float hi = 0.f; for (float v : y) hi = std::max(hi, v); EXPECT(hi == limit); }
          // device tensors
          void *dx = nullptr, *dw = nullptr, *db = nullptr, *dy = nullptr;
          mace_hip_malloc(hc, x.size() * 4, &dx); mace_hip_malloc(hc, w.size() * 4, &dw);
          mace_hip_malloc(hc, bias.size() * 4, &db); mace_hip_malloc(hc, y.size() * 4, &dy);
          mace_hip_memcpy_h2d(hc, dx, x.data(), x.size() * 4);
          mace_hip_memcpy_h2d(hc, dw, w.data(), w.size() * 4);
          mace_hip_memcpy_h2d(hc, db, bias.data(), bias.size() * 4);
          Tensor dX(dx, DT_FLOAT, {batch, in_size, 1, 1}, 0, 0, false, true), dW(dw, DT_FLOAT, {out_size, in_size, 1, 1}, 0, 0, true, true),
              dB(db, DT_FLOAT, {out_size}, 0, 0, true, true), dY(dy, DT_FLOAT, {}, 0, 0, false, true);
          {
            ops::FullyConnectedOp<float> dfc(&reg, (ActivationType)act, limit);
            EXPECT(dfc.Run(&context, &dX, &dW, &dB, &dY) == MaceStatus::MACE_SUCCESS);
            std::vector<float> got(y.size());
            mace_hip_memcpy_d2h(hc, got.data(), dy, got.size() * 4);
            EXPECT(close_enough(got, want));
          }
          mace_hip_free(hc, dx); mace_hip_free(hc, dw); mace_hip_free(hc, db); mace_hip_free(hc, dy);
        }
      }
    }
    // the C entry point names an activation it does not apply
    float one = 1.f, out1 = 0.f;
    EXPECT(mace_hip_gemv_f32_act_host(hc, &one, &one, nullptr, 1, 1, 1, 0, 1, 4 /* TANH */, 0.f, &out1) ==
           MACE_HIP_UNSUPPORTED);
  }
  {  // Constant operands in host memory stay on the GPU between calls (the counterpart of the
     // reference's pack cache, gemm.h:28-33, arm/base/gemm.cc:560-576): a uint8 FullyConnected on
     // host tensors uploads its weight matrix and bias once per op instance, later Run() calls move
     // the input and the output only; results stay bit-exact.  A weight changed in place is stale
     // until it is registered again; the registration ends with the op.
    std::mt19937 rng(123);
    mace_hip_ctx *hc = context.hip();
    const index_t out_size = 200, in_size = 1024, batch = 3;
    std::vector<uint8_t> w(out_size * in_size), x(batch * in_size), y(batch * out_size), want(y.size());
    std::vector<int32_t> bias(out_size);
    for (auto &v : w) v = rng() & 255;
    for (auto &v : bias) v = (int32_t)(rng() % 65536) - 32768;
    Tensor W(w.data(), DT_UINT8, {out_size, in_size, 1, 1}, 0.01f, 127, true), Bi(bias.data(), DT_INT32, {out_size}, 0.0002f, 0, true),
        Y(y.data(), DT_UINT8, {}, 1.0f, 128);
    int64_t up0 = 0, hit0 = 0, up1 = 0, hit1 = 0;
    EXPECT(mace_hip_host_weight_stats(hc, &up0, &hit0) == MACE_HIP_SUCCESS);
    {
      ops::FullyConnectedOp<uint8_t> fc(&reg);
      for (int round = 0; round < 4; ++round) {
        for (auto &v : x) v = rng() & 255;
        Tensor X(x.data(), DT_UINT8, {batch, in_size, 1, 1}, 0.02f, 128);
        EXPECT(fc.Run(&context, &X, &W, &Bi, &Y) == MaceStatus::MACE_SUCCESS);
        orc_q8_gemv_u8(w.data(), x.data(), bias.data(), batch, out_size, in_size, 0, 1, 127, 128, 0.01f, 0.02f,
                       1.0f, 128, ORC_REQUANT_NEON, want.data(), 2);
        EXPECT(y == want);
      }
      EXPECT(mace_hip_host_weight_stats(hc, &up1, &hit1) == MACE_HIP_SUCCESS);
      EXPECT(up1 - up0 == 2);            // the weight matrix and the bias, once each
      EXPECT(hit1 - hit0 == 8);          // ... and found resident by every one of the four calls
      // a weight changed in place: the resident copy is what the calls keep using ...
      std::vector<uint8_t> stale = want;
      for (auto &v : w) v = rng() & 255;
      Tensor X(x.data(), DT_UINT8, {batch, in_size, 1, 1}, 0.02f, 128);
      EXPECT(fc.Run(&context, &X, &W, &Bi, &Y) == MaceStatus::MACE_SUCCESS);
      EXPECT(y == stale);
      // ... until it is registered again
      EXPECT(mace_hip_host_weight_register(hc, w.data(), w.size()) == MACE_HIP_SUCCESS);
      EXPECT(fc.Run(&context, &X, &W, &Bi, &Y) == MaceStatus::MACE_SUCCESS);
      orc_q8_gemv_u8(w.data(), x.data(), bias.data(), batch, out_size, in_size, 0, 1, 127, 128, 0.01f, 0.02f,
                     1.0f, 128, ORC_REQUANT_NEON, want.data(), 2);
      EXPECT(y == want && y != stale);
    }
    // the op is gone: so are its registrations (unregistering again is an error), and the same
    // address now holds other values that a fresh op must see
    EXPECT(mace_hip_host_weight_unregister(hc, w.data()) == MACE_HIP_INVALID_ARGS);
    for (auto &v : w) v = rng() & 255;
    ops::FullyConnectedOp<uint8_t> fresh(&reg);
    Tensor X(x.data(), DT_UINT8, {batch, in_size, 1, 1}, 0.02f, 128);
    EXPECT(fresh.Run(&context, &X, &W, &Bi, &Y) == MaceStatus::MACE_SUCCESS);
    orc_q8_gemv_u8(w.data(), x.data(), bias.data(), batch, out_size, in_size, 0, 1, 127, 128, 0.01f, 0.02f,
                   1.0f, 128, ORC_REQUANT_NEON, want.data(), 2);
    EXPECT(y == want);
    // a uint8 MatMul with a constant host right-hand matrix: uploaded once, repacked once
    const index_t rows = 300, depth = 512, cols = 260;
    std::vector<uint8_t> a(rows * depth), b(depth * cols), c(rows * cols), cw(c.size());
    for (auto &v : b) v = rng() & 255;
    Tensor B(b.data(), DT_UINT8, {depth, cols}, 0.015f, 120, true), Cc(c.data(), DT_UINT8, {}, 40.f, 128);
    int32_t mult; int shift;
    EXPECT(orc_get_output_multiplier_and_shift(0.02f, 0.015f, 40.f, &mult, &shift) == 0);
    int64_t builds0 = 0, builds1 = 0, h0 = 0, h1 = 0;
    EXPECT(mace_hip_ctx_set_kernel_mask(hc, 1 | 2 | 4) == MACE_HIP_SUCCESS);   // the path that repacks
    EXPECT(mace_hip_weight_cache_stats(hc, &builds0, &h0) == MACE_HIP_SUCCESS);
    {
      ops::MatMulOpQuant mm(false, false, DT_UINT8);
      for (int round = 0; round < 3; ++round) {
        for (auto &v : a) v = rng() & 255;
        Tensor A(a.data(), DT_UINT8, {rows, depth}, 0.02f, 131);
        EXPECT(mm.Run(&context, &A, &B, &Cc) == MaceStatus::MACE_SUCCESS);
        orc_q8_gemm_u8(a.data(), b.data(), 1, rows, cols, depth, ORC_ROW_MAJOR, ORC_ROW_MAJOR, ORC_ROW_MAJOR, 1, 1,
                       -131, -120, nullptr, mult, shift, 128, 0, 255, cw.data(), 4);
        EXPECT(c == cw);
      }
    }
    EXPECT(mace_hip_weight_cache_stats(hc, &builds1, &h1) == MACE_HIP_SUCCESS);
    EXPECT(builds1 - builds0 == 1 && h1 - h0 == 2);
    EXPECT(mace_hip_ctx_set_kernel_mask(hc, 0) == MACE_HIP_SUCCESS);
    // float Gemm delegator created with should_cache_pack_: the constant side is uploaded once
    std::normal_distribution<float> nd(0.f, 1.f);
    std::vector<float> fl(64 * 48), fr(48 * 80), fo(64 * 80), fw(fo.size());
    for (auto &v : fl) v = nd(rng);
    Tensor FL(fl.data(), DT_FLOAT, {64, 48}, 0, 0, true), FO(fo.data(), DT_FLOAT, {});
    EXPECT(mace_hip_host_weight_stats(hc, &up0, &hit0) == MACE_HIP_SUCCESS);
    {
      auto creator = reg.GetCreator(MACE_HIP_DELEGATOR_KEY(Gemm, RT_CPU, float, kCpuImplType));
      std::unique_ptr<OpDelegator> d = creator(delegator::GemmParam(true));
      auto *gemm = static_cast<delegator::Gemm *>(d.get());
      for (int round = 0; round < 3; ++round) {
        for (auto &v : fr) v = nd(rng);
        Tensor FR(fr.data(), DT_FLOAT, {48, 80});
        EXPECT(gemm->Compute(&context, &FL, &FR, 1, 64, 80, 48, RowMajor, RowMajor, RowMajor, true, true, &FO) ==
               MaceStatus::MACE_SUCCESS);
        orc_gemm_f32(fl.data(), fr.data(), 1, 64, 80, 48, ORC_ROW_MAJOR, ORC_ROW_MAJOR, ORC_ROW_MAJOR, 1, 1, fw.data(), 2);
        EXPECT(close_enough(fo, fw));
      }
    }
    EXPECT(mace_hip_host_weight_stats(hc, &up1, &hit1) == MACE_HIP_SUCCESS);
    EXPECT(up1 - up0 == 1 && hit1 - hit0 == 3);
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
      mace_hip_free(h, da); mace_hip_free(h, db); mace_hip_free(h, dc);
    }
    // The registration ends with the op: once the op is gone the address is no longer a weight,
    // and a tensor that reuses it (the allocator may hand a freed filter's address to an
    // activation) is summed afresh.
    {
      mace_hip_ctx *h = context.hip();
      void *da = nullptr, *db = nullptr, *dc = nullptr;
      mace_hip_malloc(h, a.size(), &da); mace_hip_malloc(h, b.size(), &db); mace_hip_malloc(h, c8.size(), &dc);
      mace_hip_memcpy_h2d(h, da, a.data(), a.size());
      mace_hip_memcpy_h2d(h, db, b.data(), b.size());
      Tensor dA(da, DT_UINT8, {batch, depth, rows}, 0.02f, 77, false, true);
      Tensor dC(dc, DT_UINT8, {}, 40.f, 128, false, true);
      {
        Tensor dB(db, DT_UINT8, {cols, depth}, 0.015f, 201, true, true);
        ops::MatMulOpQuant op(true, true, DT_UINT8);
        EXPECT(op.Run(&context, &dA, &dB, &dC) == MaceStatus::MACE_SUCCESS);
      }
      // the op is gone; the same address now holds other bytes and is an activation
      EXPECT(mace_hip_weight_unregister(h, db) == MACE_HIP_INVALID_ARGS);   // already released
      std::vector<uint8_t> b2(b.size());
      for (auto &v : b2) v = rng() & 255;
      mace_hip_memcpy_h2d(h, db, b2.data(), b2.size());
      Tensor dB2(db, DT_UINT8, {cols, depth}, 0.015f, 201, false, true);
      ops::MatMulOpQuant op2(true, true, DT_UINT8);
      EXPECT(op2.Run(&context, &dA, &dB2, &dC) == MaceStatus::MACE_SUCCESS);
      std::vector<uint8_t> got(c8.size()), want2(c8.size());
      mace_hip_memcpy_d2h(h, got.data(), dc, got.size());
      orc_q8_gemm_u8(a.data(), b2.data(), batch, rows, cols, depth, ORC_COL_MAJOR, ORC_COL_MAJOR,
                     ORC_ROW_MAJOR, 1, 0, -77, -201, nullptr, mult, shift, 128, 0, 255, want2.data(), 4);
      EXPECT(got == want2);
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
  {  // float Conv2D through the registry's general key (what an x86 host asks for): 1x1 with
     // bias + ReLUx fused, host and device tensors, a padded 1x1, and the geometry it forwards
    std::mt19937 rng(21);
    std::normal_distribution<float> nd(0.f, 1.f);
    const index_t n = 3, cin = 40, h = 9, w = 7, cout = 24;
    std::vector<float> x(n * cin * h * w), f(cout * cin), bias(cout);
    for (auto &v : x) v = nd(rng);
    for (auto &v : f) v = nd(rng);
    for (auto &v : bias) v = nd(rng);
    Tensor X(x.data(), DT_FLOAT, {n, cin, h, w}), F(f.data(), DT_FLOAT, {cout, cin, 1, 1}, 0, 0, true),
        Bi(bias.data(), DT_FLOAT, {cout});
    std::vector<float> y(n * cout * h * w), want(y.size());
    Tensor Y(y.data(), DT_FLOAT, {});
    ops::Conv2dOpFloat conv(&reg, {1, 1}, ops::SAME, {}, {1, 1}, RELUX, 1.5f);
    EXPECT(conv.Run(&context, &X, &F, &Bi, &Y) == MaceStatus::MACE_SUCCESS);
    EXPECT(Y.shape() == (std::vector<index_t>{n, cout, h, w}));
    orc_conv1x1_f32_nchw(x.data(), f.data(), bias.data(), n, cin, h * w, cout, ORC_ACT_RELUX, 1.5f,
                         want.data(), 2);
    EXPECT(close_enough(y, want));
    // the delegator alone (no bias, no activation), created through the NEON K1x1 tag as well
    auto creator = reg.GetCreator(MACE_HIP_DELEGATOR_KEY_EX(Conv2d, RT_CPU, float, NEON, K1x1));
    EXPECT((bool)creator);
    std::unique_ptr<OpDelegator> d = creator(delegator::Conv2dParam({1, 1}, {1, 1}, {}, ops::VALID));
    EXPECT(static_cast<delegator::Conv2d *>(d.get())->Compute(&context, &X, &F, &Y) == MaceStatus::MACE_SUCCESS);
    orc_conv1x1_f32_nchw(x.data(), f.data(), nullptr, n, cin, h * w, cout, ORC_ACT_NOOP, 0.f, want.data(), 2);
    EXPECT(close_enough(y, want));
    // explicit paddings {2, 3}: the reference pads the input with zeros (1 row on top, 1 column
    // on the left, conv_2d_1x1.cc:37-60) and the result has (h + 2) x (w + 3) pixels
    {
      const index_t ph = h + 2, pw = w + 3;
      std::vector<float> xp(n * cin * ph * pw, 0.f), yp(n * cout * ph * pw), wantp(yp.size());
      for (index_t i = 0; i < n * cin; ++i)
        for (index_t r = 0; r < h; ++r)
          for (index_t c = 0; c < w; ++c) xp[(i * ph + r + 1) * pw + c + 1] = x[(i * h + r) * w + c];
      orc_conv1x1_f32_nchw(xp.data(), f.data(), bias.data(), n, cin, ph * pw, cout, ORC_ACT_RELU, 0.f,
                           wantp.data(), 2);
      Tensor Yp(yp.data(), DT_FLOAT, {});
      ops::Conv2dOpFloat padded(&reg, {1, 1}, ops::VALID, {2, 3}, {1, 1}, RELU, 0.f);
      EXPECT(padded.Run(&context, &X, &F, &Bi, &Yp) == MaceStatus::MACE_SUCCESS);
      EXPECT(Yp.shape() == (std::vector<index_t>{n, cout, ph, pw}));
      EXPECT(close_enough(yp, wantp));
      // the same on device tensors
      mace_hip_ctx *hc = context.hip();
      void *dx = nullptr, *df = nullptr, *dbias = nullptr, *dy = nullptr;
      mace_hip_malloc(hc, x.size() * 4, &dx); mace_hip_malloc(hc, f.size() * 4, &df);
      mace_hip_malloc(hc, bias.size() * 4, &dbias); mace_hip_malloc(hc, yp.size() * 4, &dy);
      mace_hip_memcpy_h2d(hc, dx, x.data(), x.size() * 4);
      mace_hip_memcpy_h2d(hc, df, f.data(), f.size() * 4);
      mace_hip_memcpy_h2d(hc, dbias, bias.data(), bias.size() * 4);
      Tensor dX(dx, DT_FLOAT, {n, cin, h, w}, 0, 0, false, true), dF(df, DT_FLOAT, {cout, cin, 1, 1}, 0, 0, true, true),
          dB(dbias, DT_FLOAT, {cout}, 0, 0, true, true), dY(dy, DT_FLOAT, {}, 0, 0, false, true);
      EXPECT(padded.Run(&context, &dX, &dF, &dB, &dY) == MaceStatus::MACE_SUCCESS);
      std::vector<float> got(yp.size());
      mace_hip_memcpy_d2h(hc, got.data(), dy, got.size() * 4);
      EXPECT(close_enough(got, wantp));
      mace_hip_free(hc, dx); mace_hip_free(hc, df); mace_hip_free(hc, dbias); mace_hip_free(hc, dy);
    }
    // a 3x3 filter, a stride or a dilation is not this delegator's: it forwards (UNSUPPORTED,
    // nothing written)
    std::vector<float> f3(cout * cin * 9, 1.f);
    Tensor F3(f3.data(), DT_FLOAT, {cout, cin, 3, 3});
    y.assign(y.size(), -7.f);
    EXPECT(conv.Run(&context, &X, &F3, &Bi, &Y) == MaceStatus::MACE_UNSUPPORTED);
    EXPECT(y[0] == -7.f && y.back() == -7.f);
    ops::Conv2dOpFloat strided(&reg, {2, 2}, ops::SAME);
    EXPECT(strided.Run(&context, &X, &F, &Bi, &Y) == MaceStatus::MACE_UNSUPPORTED);
    Tensor Fbad(f.data(), DT_FLOAT, {cout, cin + 1, 1, 1});
    EXPECT(conv.Run(&context, &X, &Fbad, &Bi, &Y) == MaceStatus::MACE_INVALID_ARGS);
  }
  {  // float MatMul with the per-column bias on device tensors (matmul.cc:195-211), all transposes
    std::mt19937 rng(31);
    std::normal_distribution<float> nd(0.f, 1.f);
    const index_t batch = 3, rows = 70, depth = 48, cols = 52;
    std::vector<float> a(batch * rows * depth), b(batch * depth * cols), bias(cols);
    for (auto &v : a) v = nd(rng);
    for (auto &v : b) v = nd(rng);
    for (auto &v : bias) v = nd(rng);
    mace_hip_ctx *hc = context.hip();
    void *da = nullptr, *db = nullptr, *dbias = nullptr, *dc = nullptr;
    mace_hip_malloc(hc, a.size() * 4, &da); mace_hip_malloc(hc, b.size() * 4, &db);
    mace_hip_malloc(hc, bias.size() * 4, &dbias); mace_hip_malloc(hc, batch * rows * cols * 4, &dc);
    mace_hip_memcpy_h2d(hc, da, a.data(), a.size() * 4);
    mace_hip_memcpy_h2d(hc, db, b.data(), b.size() * 4);
    mace_hip_memcpy_h2d(hc, dbias, bias.data(), bias.size() * 4);
    for (int ta = 0; ta < 2; ++ta)
      for (int tb = 0; tb < 2; ++tb) {
        Tensor A(da, DT_FLOAT, ta ? std::vector<index_t>{batch, depth, rows} : std::vector<index_t>{batch, rows, depth}, 0, 0, false, true);
        Tensor B(db, DT_FLOAT, tb ? std::vector<index_t>{batch, cols, depth} : std::vector<index_t>{batch, depth, cols}, 0, 0, false, true);
        Tensor Bi(dbias, DT_FLOAT, {cols}, 0, 0, false, true), Cc(dc, DT_FLOAT, {}, 0, 0, false, true);
        ops::MatMulOpFloat op(&reg, ta != 0, tb != 0);
        EXPECT(op.Run(&context, &A, &B, &Bi, &Cc) == MaceStatus::MACE_SUCCESS);
        std::vector<float> got(batch * rows * cols), want(got.size());
        mace_hip_memcpy_d2h(hc, got.data(), dc, got.size() * 4);
        orc_gemm_f32(a.data(), b.data(), batch, rows, cols, depth, ta ? ORC_COL_MAJOR : ORC_ROW_MAJOR,
                     tb ? ORC_COL_MAJOR : ORC_ROW_MAJOR, ORC_ROW_MAJOR, 1, 1, want.data(), 2);
        for (index_t i = 0; i < batch * rows; ++i)
          for (index_t w2 = 0; w2 < cols; ++w2) want[i * cols + w2] += bias[w2];
        EXPECT(close_enough(got, want));
        Tensor BadBias(dbias, DT_FLOAT, {cols - 1}, 0, 0, false, true);
        EXPECT(op.Run(&context, &A, &B, &BadBias, &Cc) == MaceStatus::MACE_INVALID_ARGS);
      }
    mace_hip_free(hc, da); mace_hip_free(hc, db); mace_hip_free(hc, dbias); mace_hip_free(hc, dc);
  }
  {  // the Winograd caller of Gemm (conv_2d_3x3_winograd.cc): 2x2 tiles on a small image, 6x6
     // tiles on a larger one, against the textbook 3x3 convolution sum
    std::mt19937 rng(41);
    std::uniform_real_distribution<float> ud(-1.f, 1.f);
    struct Geo { index_t n, cin, h, w, cout; ops::Padding pad; };
    for (const Geo &g : {Geo{2, 5, 11, 13, 7, ops::SAME}, Geo{1, 8, 12, 9, 16, ops::VALID},
                         Geo{2, 6, 23, 19, 9, ops::SAME}, Geo{1, 16, 30, 30, 8, ops::VALID}}) {
      std::vector<float> x(g.n * g.cin * g.h * g.w), f(g.cout * g.cin * 9);
      for (auto &v : x) v = ud(rng);
      for (auto &v : f) v = ud(rng);
      const index_t oh = g.pad == ops::SAME ? g.h : g.h - 2, ow = g.pad == ops::SAME ? g.w : g.w - 2;
      const int top = g.pad == ops::SAME ? 1 : 0;
      std::vector<float> y(g.n * g.cout * oh * ow), want(y.size());
      for (index_t b = 0; b < g.n; ++b)
        for (index_t oc = 0; oc < g.cout; ++oc)
          for (index_t r = 0; r < oh; ++r)
            for (index_t c = 0; c < ow; ++c) {
              double s = 0;
              for (index_t ic = 0; ic < g.cin; ++ic)
                for (int kh = 0; kh < 3; ++kh)
                  for (int kw = 0; kw < 3; ++kw) {
                    const index_t iy = r + kh - top, ix = c + kw - top;
                    if (iy >= 0 && iy < g.h && ix >= 0 && ix < g.w)
                      s += (double)x[((b * g.cin + ic) * g.h + iy) * g.w + ix] * f[((oc * g.cin + ic) * 3 + kh) * 3 + kw];
                  }
              want[((b * g.cout + oc) * oh + r) * ow + c] = (float)s;
            }
      Tensor X(x.data(), DT_FLOAT, {g.n, g.cin, g.h, g.w}), F(f.data(), DT_FLOAT, {g.cout, g.cin, 3, 3}, 0, 0, true),
          Y(y.data(), DT_FLOAT, {});
      ops::Conv2dK3x3WinogradOp wino(&reg, g.pad);
      EXPECT(wino.Run(&context, &X, &F, &Y) == MaceStatus::MACE_SUCCESS);
      EXPECT(Y.shape() == (std::vector<index_t>{g.n, g.cout, oh, ow}));
      // the reference compares its Winograd with the direct convolution at 1e-3 / 1e-5
      // (conv_2d_test.cc: ExpectTensorNear); the 6x6 transform loses a few more bits
      bool ok = true;
      for (size_t i = 0; i < y.size(); ++i) ok = ok && std::fabs(y[i] - want[i]) <= 2e-3 + 1e-3 * std::fabs(want[i]);
      EXPECT(ok);
    }
  }
  {  // DynamicLSTM (dynamic_lstm.cc:160-372): the op with the GPU Gemv against the same op with a
     // Gemv served by the CPU oracle; with zero weights the step has a closed form
    std::mt19937 rng(51);
    std::normal_distribution<float> nd(0.f, 0.3f);
    OpDelegatorRegistry cpu_reg;
    EXPECT(MACE_HIP_REGISTER_DELEGATOR(&cpu_reg, OracleGemv, DelegatorParam,
                                       MACE_HIP_DELEGATOR_KEY(Gemv, RT_CPU, float, kCpuImplType)) ==
           MaceStatus::MACE_SUCCESS);
    ops::DynamicLSTMArgs args;
    const index_t batch = 2, chunk = 7, input_dim = 40, cell = 64, out_dim = 48;
    args.prev_out_delay = -3; args.prev_cell_delay = -3; args.prev_out_offset = 8; args.prev_out_dim = 24;
    args.prev_cell_dim = cell; args.subsample_factor = 3; args.scale = 0.9f;
    args.forward_indexes = {0, 1, 2, 4, 6};
    args.out_cache_indexes = {4}; args.cell_cache_indexes = {4};
    const index_t a_in = input_dim + args.prev_out_dim, a_out = 4 * cell;
    std::vector<float> x(batch * chunk * input_dim), po(batch * 1 * args.prev_out_dim), pc(batch * 1 * cell),
        wa(a_out * a_in), params(3 * cell), wb(out_dim * cell), ba(a_out), bb(out_dim);
    for (auto *v : {&x, &po, &pc, &wa, &params, &wb, &ba, &bb}) for (auto &e : *v) e = nd(rng);
    Tensor X(x.data(), DT_FLOAT, {batch, chunk, input_dim}), PO(po.data(), DT_FLOAT, {batch, 1, args.prev_out_dim}),
        PC(pc.data(), DT_FLOAT, {batch, 1, cell}), WA(wa.data(), DT_FLOAT, {a_out, a_in}, 0, 0, true),
        P(params.data(), DT_FLOAT, {3, cell}), WB(wb.data(), DT_FLOAT, {out_dim, cell}, 0, 0, true),
        BA(ba.data(), DT_FLOAT, {a_out}), BB(bb.data(), DT_FLOAT, {out_dim});
    std::vector<float> y[2], oc[2], cc[2];
    for (int which = 0; which < 2; ++which) {
      y[which].assign(batch * chunk * out_dim, 0.f);
      oc[which].assign(batch * args.prev_out_dim, 0.f);
      cc[which].assign(batch * cell, 0.f);
      Tensor Y(y[which].data(), DT_FLOAT, {}), OC(oc[which].data(), DT_FLOAT, {}), CC(cc[which].data(), DT_FLOAT, {});
      ops::DynamicLSTMOp op(which == 0 ? &reg : &cpu_reg, args);
      EXPECT(op.Run(&context, &X, &PO, &PC, &WA, &P, &WB, &BA, &BB, &Y, &OC, &CC) == MaceStatus::MACE_SUCCESS);
      EXPECT(Y.shape() == (std::vector<index_t>{batch, chunk, out_dim}));
      EXPECT(OC.shape() == (std::vector<index_t>{batch, 1, args.prev_out_dim}));
      EXPECT(CC.shape() == (std::vector<index_t>{batch, 1, cell}));
    }
    EXPECT(close_enough(y[0], y[1]) && close_enough(oc[0], oc[1]) && close_enough(cc[0], cc[1]));
    float energy = 0.f;
    for (float v : y[0]) energy += v * v;
    EXPECT(energy > 1.f);
    // closed form: zero weights, biases and peepholes, first frame, c_prev given:
    // i = f = o = sigmoid(0) = 1/2, c = c_prev / 2 + tanh(0) / 2, m = tanh(c) / 2, out = 0 (+ bias_b)
    std::vector<float> zwa(wa.size(), 0.f), zwb(wb.size(), 0.f), zp(params.size(), 0.f), y0(batch * chunk * out_dim),
        oc0(batch * args.prev_out_dim), cc0(batch * cell);
    Tensor ZWA(zwa.data(), DT_FLOAT, {a_out, a_in}), ZWB(zwb.data(), DT_FLOAT, {out_dim, cell}), ZP(zp.data(), DT_FLOAT, {3, cell}),
        Y0(y0.data(), DT_FLOAT, {}), OC0(oc0.data(), DT_FLOAT, {}), CC0(cc0.data(), DT_FLOAT, {});
    ops::DynamicLSTMArgs one = args;
    one.forward_indexes = {0}; one.out_cache_indexes = {0}; one.cell_cache_indexes = {0}; one.scale = 1.0f;
    ops::DynamicLSTMOp op1(&reg, one);
    EXPECT(op1.Run(&context, &X, &PO, &PC, &ZWA, &ZP, &ZWB, nullptr, &BB, &Y0, &OC0, &CC0) == MaceStatus::MACE_SUCCESS);
    bool ok = true;
    for (index_t b = 0; b < batch; ++b) {
      for (index_t c = 0; c < cell; ++c) ok = ok && std::fabs(cc0[b * cell + c] - 0.5f * pc[b * cell + c]) < 1e-6f;
      for (index_t k = 0; k < out_dim; ++k) ok = ok && std::fabs(y0[b * out_dim + k] - bb[k]) < 1e-6f;
    }
    EXPECT(ok);
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
