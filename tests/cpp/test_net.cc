// C++ tests of the NetDef loader and serial runner (include/mace_hip_net.h).
//   test_net.bin wire   -- protobuf wire format: round trip, packed and unpacked repeated fields,
//                          unknown fields, truncated input; needs no GPU
//   test_net.bin run    -- a quantized net (Quantize, three Conv2D, FullyConnected, Dequantize,
//                          Squeeze) loaded from its serialized form and run on the GPU, eagerly and
//                          as a HIP graph, against the CPU oracle's ops chained by hand
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

#include "mace_hip_net.h"
#include "../../oracle/mace_oracle.h"

using namespace mace_hip;
using namespace mace_hip::net;

static int g_fail = 0;
#define EXPECT(cond)                                                              \
  do {                                                                            \
    if (!(cond)) { printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond); ++g_fail; } \
  } while (0)

static Argument IntArg(const char *name, int64_t v) { Argument a; a.name = name; a.i = v; a.has_i = true; return a; }
static Argument IntsArg(const char *name, std::vector<int64_t> v) { Argument a; a.name = name; a.ints = std::move(v); return a; }

struct Model {
  NetDef net;
  std::vector<uint8_t> data;   // the weights buffer
  // what the oracle needs
  index_t n = 2, h = 14, w = 14, c0 = 64, c1 = 128, c2 = 128, c3 = 256, classes = 10;
  float s_in = 0.05f; int32_t z_in = 119;
  float s_f[4] = {0.01f, 0.012f, 0.009f, 0.011f}; int32_t z_f[4] = {127, 131, 120, 125};
  float s_act[4] = {0.5f, 3.0f, 12.0f, 600.f}; int32_t z_act[4] = {0, 0, 0, 60};
};

static void AddTensor(Model *m, const char *name, std::vector<int64_t> dims, int dt, const void *bytes,
                      size_t nbytes, float scale, int32_t zp) {
  ConstTensor c;
  c.name = name; c.dims = std::move(dims); c.data_type = dt; c.scale = scale; c.zero_point = zp;
  while (m->data.size() % 16) m->data.push_back(0);
  c.offset = (int64_t)m->data.size();
  c.data_size = (int64_t)(nbytes / (dt == DT_UINT8 ? 1 : 4));
  m->data.insert(m->data.end(), (const uint8_t *)bytes, (const uint8_t *)bytes + nbytes);
  m->net.tensors.push_back(c);
}

struct Weights {
  std::vector<uint8_t> f0, f1, f2, fc;
  std::vector<int32_t> b0, b1, b2, bfc;
};

static Model BuildModel(Weights *wt) {
  Model m;
  std::mt19937 rng(99);
  auto u8 = [&](size_t n) { std::vector<uint8_t> v(n); for (auto &e : v) e = (uint8_t)(rng() % 255 + 1); return v; };
  auto i32 = [&](size_t n) { std::vector<int32_t> v(n); for (auto &e : v) e = (int32_t)(rng() % 8192) - 4096; return v; };
  wt->f0 = u8(m.c1 * 9 * m.c0); wt->f1 = u8(m.c2 * m.c1); wt->f2 = u8(m.c3 * m.c2);
  wt->fc = u8(m.classes * 7 * 7 * m.c3);
  wt->b0 = i32(m.c1); wt->b1 = i32(m.c2); wt->b2 = i32(m.c3); wt->bfc = i32(m.classes);
  m.net.name = "toy_quantized_net";
  AddTensor(&m, "conv0/filter", {m.c1, 3, 3, m.c0}, DT_UINT8, wt->f0.data(), wt->f0.size(), m.s_f[0], m.z_f[0]);
  AddTensor(&m, "conv0/bias", {m.c1}, DT_INT32, wt->b0.data(), wt->b0.size() * 4, m.s_in * m.s_f[0], 0);
  AddTensor(&m, "conv1/filter", {m.c2, 1, 1, m.c1}, DT_UINT8, wt->f1.data(), wt->f1.size(), m.s_f[1], m.z_f[1]);
  AddTensor(&m, "conv1/bias", {m.c2}, DT_INT32, wt->b1.data(), wt->b1.size() * 4, m.s_act[0] * m.s_f[1], 0);
  AddTensor(&m, "conv2/filter", {m.c3, 1, 1, m.c2}, DT_UINT8, wt->f2.data(), wt->f2.size(), m.s_f[2], m.z_f[2]);
  AddTensor(&m, "conv2/bias", {m.c3}, DT_INT32, wt->b2.data(), wt->b2.size() * 4, m.s_act[1] * m.s_f[2], 0);
  AddTensor(&m, "fc/weight", {m.classes, 7, 7, m.c3}, DT_UINT8, wt->fc.data(), wt->fc.size(), m.s_f[3], m.z_f[3]);
  AddTensor(&m, "fc/bias", {m.classes}, DT_INT32, wt->bfc.data(), wt->bfc.size() * 4, m.s_act[2] * m.s_f[3], 0);

  InputOutputInfo in; in.name = "data"; in.dims = {m.n, m.h, m.w, m.c0}; in.data_type = DT_FLOAT;
  m.net.input_info.push_back(in);
  InputOutputInfo out; out.name = "prob"; out.dims = {m.n, m.classes}; out.data_type = DT_FLOAT;
  m.net.output_info.push_back(out);

  auto op = [&](const char *type, const char *name, std::vector<std::string> ins, const char *o,
                std::vector<int64_t> shape, int dt, float scale, int32_t zp, std::vector<Argument> args) {
    OperatorDef d;
    d.type = type; d.name = name; d.input = std::move(ins); d.output = {o};
    d.output_shape = {std::move(shape)}; d.output_type = {dt};
    if (scale > 0.f) { QuantizeActivationInfo q; q.scale = scale; q.zero_point = zp; d.quantize_info = {q}; }
    d.arg = std::move(args);
    m.net.op.push_back(d);
  };
  op("Quantize", "quantize", {"data"}, "data_q", {m.n, m.h, m.w, m.c0}, DT_UINT8, m.s_in, m.z_in, {IntArg("T", DT_UINT8)});
  op("Conv2D", "conv0", {"data_q", "conv0/filter", "conv0/bias"}, "act0", {m.n, 7, 7, m.c1}, DT_UINT8, m.s_act[0],
     m.z_act[0], {IntArg("T", DT_UINT8), IntsArg("strides", {2, 2}), IntArg("padding", SAME), IntsArg("dilations", {1, 1})});
  op("Conv2D", "conv1", {"act0", "conv1/filter", "conv1/bias"}, "act1", {m.n, 7, 7, m.c2}, DT_UINT8, m.s_act[1],
     m.z_act[1], {IntArg("T", DT_UINT8), IntsArg("strides", {1, 1}), IntArg("padding", VALID)});
  op("Conv2D", "conv2", {"act1", "conv2/filter", "conv2/bias"}, "act2", {m.n, 7, 7, m.c3}, DT_UINT8, m.s_act[2],
     m.z_act[2], {IntArg("T", DT_UINT8), IntsArg("strides", {1, 1}), IntArg("padding", SAME)});
  op("FullyConnected", "fc", {"act2", "fc/weight", "fc/bias"}, "logits_q", {m.n, 1, 1, m.classes}, DT_UINT8,
     m.s_act[3], m.z_act[3], {IntArg("T", DT_UINT8)});
  op("Dequantize", "dequantize", {"logits_q"}, "logits", {m.n, 1, 1, m.classes}, DT_FLOAT, 0.f, 0, {IntArg("T", DT_UINT8)});
  op("Squeeze", "squeeze", {"logits"}, "prob", {m.n, m.classes}, DT_FLOAT, 0.f, 0, {IntsArg("axis", {1, 2})});
  return m;
}

// the same net with the CPU oracle's ops chained by hand
static std::vector<float> OracleRun(const Model &m, const Weights &wt, const std::vector<float> &x) {
  std::vector<uint8_t> q(x.size()), a0(m.n * 49 * m.c1), a1(m.n * 49 * m.c2), a2(m.n * 49 * m.c3), lq(m.n * m.classes);
  orc_quantize_with_scale_u8(x.data(), (int64_t)x.size(), m.s_in, m.z_in, q.data());
  int64_t oh, ow; int ph, pw;
  orc_calc_padding_and_output_size(m.h, m.w, 3, 3, 1, 1, 2, 2, 1, &oh, &ow, &ph, &pw);
  orc_conv2d_q8_nhwc(q.data(), wt.f0.data(), wt.b0.data(), m.n, m.h, m.w, m.c0, m.c1, 3, 3, 2, 2, ph, pw, m.s_in,
                     m.z_in, m.s_f[0], m.z_f[0], m.s_in * m.s_f[0], m.s_act[0], m.z_act[0], 0, 255, a0.data(), 4);
  orc_conv2d_q8_nhwc(a0.data(), wt.f1.data(), wt.b1.data(), m.n, 7, 7, m.c1, m.c2, 1, 1, 1, 1, 0, 0, m.s_act[0],
                     m.z_act[0], m.s_f[1], m.z_f[1], m.s_act[0] * m.s_f[1], m.s_act[1], m.z_act[1], 0, 255, a1.data(), 4);
  orc_conv2d_q8_nhwc(a1.data(), wt.f2.data(), wt.b2.data(), m.n, 7, 7, m.c2, m.c3, 1, 1, 1, 1, 0, 0, m.s_act[1],
                     m.z_act[1], m.s_f[2], m.z_f[2], m.s_act[1] * m.s_f[2], m.s_act[2], m.z_act[2], 0, 255, a2.data(), 4);
  orc_q8_gemv_u8(wt.fc.data(), a2.data(), wt.bfc.data(), m.n, m.classes, 49 * m.c3, 0, 1, m.z_f[3], m.z_act[2],
                 m.s_f[3], m.s_act[2], m.s_act[3], m.z_act[3], ORC_REQUANT_NEON, lq.data(), 4);
  std::vector<float> out(lq.size());
  orc_dequantize_u8(lq.data(), (int64_t)lq.size(), m.s_act[3], m.z_act[3], out.data());
  return out;
}

static int test_wire() {
  Weights wt;
  Model m = BuildModel(&wt);
  const std::string bytes = SerializeNetDef(m.net);
  NetDef back;
  EXPECT(ParseNetDef(bytes.data(), bytes.size(), &back));
  EXPECT(back.name == "toy_quantized_net" && back.op.size() == 7 && back.tensors.size() == 8);
  EXPECT(back.op[1].type == "Conv2D" && back.op[1].input.size() == 3 && back.op[1].input[2] == "conv0/bias");
  EXPECT(GetIntsArg(back.op[1], "strides") == (std::vector<int>{2, 2}) && GetIntArg(back.op[1], "padding", -1) == SAME);
  EXPECT(GetIntArg(back.op[1], "T", DT_FLOAT) == DT_UINT8 && GetIntArg(back.op[1], "absent", 42) == 42);
  EXPECT(back.op[1].output_shape[0] == (std::vector<int64_t>{2, 7, 7, 128}) && back.op[1].output_type[0] == DT_UINT8);
  EXPECT(back.op[1].quantize_info.size() == 1 && back.op[1].quantize_info[0].scale == 0.5f);
  EXPECT(back.op[4].quantize_info[0].zero_point == 60);
  EXPECT(back.tensors[6].name == "fc/weight" && back.tensors[6].dims == (std::vector<int64_t>{10, 7, 7, 256}) &&
         back.tensors[6].data_type == DT_UINT8 && back.tensors[6].zero_point == 125 &&
         back.tensors[6].data_size == 10 * 49 * 256 && back.tensors[6].offset == m.net.tensors[6].offset);
  EXPECT(back.input_info.size() == 1 && back.input_info[0].dims == (std::vector<int64_t>{2, 14, 14, 64}));
  EXPECT(back.output_info[0].name == "prob");
  EXPECT(SerializeNetDef(back) == bytes);
  // hand-made bytes: op { type: "X"; an unknown varint field 55; output_type packed [2, 4];
  // arg { name: "k"; ints unpacked 7, 9; floats packed [1.5] } }, then an unknown 64-bit field
  {
    wire::Writer arg; arg.bytes(1, "k"); arg.i64(6, 7); arg.i64(6, 9);
    { wire::Writer p; const float f = 1.5f; uint32_t u; memcpy(&u, &f, 4); p.out.append((const char *)&u, 4); arg.bytes(5, p.out); }
    wire::Writer op; op.bytes(4, "X"); op.i64(55, 123456789);
    { wire::Writer p; p.varint(2); p.varint(4); op.bytes(8, p.out); }
    op.bytes(6, arg.out);
    wire::Writer net; net.bytes(1, op.out); net.tag(77, 1); net.out.append("\1\2\3\4\5\6\7\10", 8);
    NetDef n2;
    EXPECT(ParseNetDef(net.out.data(), net.out.size(), &n2));
    EXPECT(n2.op.size() == 1 && n2.op[0].type == "X" && n2.op[0].output_type == (std::vector<int>{2, 4}));
    EXPECT(n2.op[0].arg.size() == 1 && n2.op[0].arg[0].ints == (std::vector<int64_t>{7, 9}) &&
           n2.op[0].arg[0].floats == (std::vector<float>{1.5f}));
    // negative int64 (ten-byte varint) survives
    wire::Writer a2; a2.bytes(1, "neg"); a2.i64(3, -5);
    Argument parsed;
    EXPECT(wire::Parse(wire::Reader((const uint8_t *)a2.out.data(), a2.out.size()), &parsed) && parsed.i == -5);
    // truncated input is refused, at every length that cuts a field
    int refused = 0;
    for (size_t cut = 1; cut < net.out.size(); ++cut) {
      NetDef n3;
      if (!ParseNetDef(net.out.data(), cut, &n3)) ++refused;
    }
    EXPECT(refused >= (int)net.out.size() - 4);
  }
  return g_fail;
}

static int test_run() {
  mace_hip_ctx *hctx = nullptr;
  if (mace_hip_ctx_create(0, &hctx) != MACE_HIP_SUCCESS) { printf("FAIL: no context\n"); return 1; }
  OpDelegatorRegistry reg;
  EXPECT(hip::RegisterAllHipDelegators(&reg) == MaceStatus::MACE_SUCCESS);
  Weights wt;
  Model m = BuildModel(&wt);
  const std::string bytes = SerializeNetDef(m.net);
  NetDef parsed;
  EXPECT(ParseNetDef(bytes.data(), bytes.size(), &parsed));
  std::mt19937 rng(5);
  std::normal_distribution<float> nd(0.f, 2.f);
  {
    SerialNet net(&reg, hctx);
    MaceStatus st = net.Init(parsed, m.data.data(), m.data.size());
    if (st != MaceStatus::MACE_SUCCESS) printf("Init: %s\n", net.error().c_str());
    EXPECT(st == MaceStatus::MACE_SUCCESS);
    EXPECT(net.op_count() == 6);   // Squeeze is a view
    EXPECT(net.GetTensor("act1") && net.GetTensor("act1")->scale() == m.s_act[1]);
    EXPECT(net.GetTensor("fc/weight") && net.GetTensor("fc/weight")->is_weight());
    std::vector<float> x((size_t)m.n * m.h * m.w * m.c0), got(m.n * m.classes);
    for (int round = 0; round < 2; ++round) {
      for (auto &v : x) v = nd(rng);
      EXPECT(net.SetInput("data", x.data(), x.size() * 4) == MaceStatus::MACE_SUCCESS);
      st = net.Run();
      if (st != MaceStatus::MACE_SUCCESS) printf("Run: %s\n", net.error().c_str());
      EXPECT(st == MaceStatus::MACE_SUCCESS);
      EXPECT(net.GetOutput("prob", got.data(), got.size() * 4) == MaceStatus::MACE_SUCCESS);
      const std::vector<float> want = OracleRun(m, wt, x);
      EXPECT(got == want);
      float spread = 0.f;
      for (float v : want) spread = std::max(spread, std::fabs(v - want[0]));
      EXPECT(spread > 1.f);   // the check is not vacuous
    }
    // the same sequence as a HIP graph: replayed several times on fresh inputs, with eager runs
    // and synchronisations in between, every replay against the oracle
    st = net.CaptureGraph();
    if (st != MaceStatus::MACE_SUCCESS) printf("CaptureGraph: %s\n", net.error().c_str());
    EXPECT(st == MaceStatus::MACE_SUCCESS);
    for (int replay = 0; replay < 4; ++replay) {
      for (auto &v : x) v = nd(rng);
      EXPECT(net.SetInput("data", x.data(), x.size() * 4) == MaceStatus::MACE_SUCCESS);
      EXPECT(net.RunGraph() == MaceStatus::MACE_SUCCESS);
      EXPECT(net.GetOutput("prob", got.data(), got.size() * 4) == MaceStatus::MACE_SUCCESS);
      const std::vector<float> want = OracleRun(m, wt, x);
      EXPECT(got == want);
      if (replay == 1) {   // eager work of the same context between replays
        EXPECT(net.Run() == MaceStatus::MACE_SUCCESS);
        EXPECT(mace_hip_sync(hctx) == MACE_HIP_SUCCESS);
      }
    }
    // timing, informational: per inference, eager against graph
    float ms_eager = 0.f, ms_graph = 0.f;
    const int reps = 200;
    mace_hip_timer_start(hctx);
    for (int i = 0; i < reps; ++i) net.Run();
    mace_hip_timer_stop(hctx, &ms_eager);
    mace_hip_timer_start(hctx);
    for (int i = 0; i < reps; ++i) net.RunGraph();
    mace_hip_timer_stop(hctx, &ms_graph);
    printf("toy net, batch %d: %.1f us per inference eager, %.1f us as a graph\n", (int)m.n,
           ms_eager * 1e3 / reps, ms_graph * 1e3 / reps);
    // a wrongly sized input is refused
    EXPECT(net.SetInput("data", x.data(), 16) == MaceStatus::MACE_INVALID_ARGS);
  }
  {  // an op type outside this library: Init names it and returns UNSUPPORTED
    NetDef bad = parsed;
    bad.op[5].type = "Softmax";
    SerialNet net(&reg, hctx);
    EXPECT(net.Init(bad, m.data.data(), m.data.size()) == MaceStatus::MACE_UNSUPPORTED);
    EXPECT(net.error().find("Softmax") != std::string::npos && net.error().find("dequantize") != std::string::npos);
  }
  {  // a tensor slice past the end of the weights buffer is refused
    SerialNet net(&reg, hctx);
    EXPECT(net.Init(parsed, m.data.data(), m.data.size() - 64) == MaceStatus::MACE_INVALID_ARGS);
  }
  mace_hip_ctx_destroy(hctx);
  return g_fail;
}

int main(int argc, char **argv) {
  const char *mode = argc > 1 ? argv[1] : "wire";
  const int fails = strcmp(mode, "run") == 0 ? test_run() : test_wire();
  printf("%s: %s (%d failures)\n", mode, fails ? "FAILED" : "ok", fails);
  return fails ? 1 : 0;
}
