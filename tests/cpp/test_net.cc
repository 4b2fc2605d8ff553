// C++ tests of the NetDef loader and serial runner (include/mace_hip_net.h).
//   test_net.bin wire   -- protobuf wire format: round trip, packed and unpacked repeated fields,
//                          unknown fields, truncated input; needs no GPU
//   test_net.bin run    -- a quantized net (Quantize, three Conv2D, FullyConnected, Dequantize,
//                          Squeeze) loaded from its serialized form and run on the GPU, eagerly and
//                          as a HIP graph, against the CPU oracle's ops chained by hand
#include <cmath>
#include <cstdio>
#include <cstdlib>
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

// A NetDef serialized by an independent implementation of the wire format (the google.protobuf
// package, tests/golden/make_netdef_fixture.py), in the schema's own encoding and with every
// repeated scalar packed: both must parse to the same messages, with the values the script wrote.
static std::string ReadFile(const std::string &path) {
  std::string out;
  if (FILE *f = fopen(path.c_str(), "rb")) {
    char buf[4096];
    size_t n;
    while ((n = fread(buf, 1, sizeof(buf), f)) > 0) out.append(buf, n);
    fclose(f);
  }
  return out;
}

static int test_fixture(const char *dir) {
  for (const char *name : {"netdef_unpacked.pb", "netdef_packed.pb"}) {
    const std::string bytes = ReadFile(std::string(dir) + "/" + name);
    EXPECT(bytes.size() > 500);
    NetDef net;
    EXPECT(ParseNetDef(bytes.data(), bytes.size(), &net));
    EXPECT(net.name == "fixture_net" && net.op.size() == 2 && net.tensors.size() == 3);
    if (net.op.size() != 2 || net.tensors.size() != 3) continue;
    const OperatorDef &op = net.op[0];
    EXPECT(op.name == "conv_a" && op.type == "Conv2D");
    EXPECT(op.input == (std::vector<std::string>{"in_q", "conv_a/filter", "conv_a/bias"}));
    EXPECT(op.output == (std::vector<std::string>{"act_a"}));
    EXPECT(op.arg.size() == 8);
    EXPECT(GetIntArg(op, "T", 0) == 2);
    EXPECT(GetIntsArg(op, "strides") == (std::vector<int>{2, 1}));
    const Argument *pv = FindArg(op, "padding_values");
    EXPECT(pv && pv->ints == (std::vector<int64_t>{-1, 0, 70000000000ll}));
    const Argument *ml = FindArg(op, "max_limit");
    EXPECT(ml && ml->has_f && ml->f == 6.0f && !ml->has_i);
    const Argument *act = FindArg(op, "activation");
    EXPECT(act && act->has_s && act->s == "RELUX");
    const Argument *co = FindArg(op, "coeffs");
    EXPECT(co && co->floats == (std::vector<float>{0.25f, -1.5f, 3.0e-5f}));
    EXPECT(GetIntArg(op, "neg", 0) == -123456789012ll);
    const Argument *empty = FindArg(op, "");
    EXPECT(empty && empty->has_s && empty->s.empty());
    EXPECT(op.output_shape.size() == 1 && op.output_shape[0] == (std::vector<int64_t>{64, 56, 56, 128}));
    EXPECT(op.output_type == (std::vector<int>{DT_UINT8}));
    EXPECT(op.quantize_info.size() == 1 && op.quantize_info[0].scale == 0.023529412f &&
           op.quantize_info[0].zero_point == -7 && op.quantize_info[0].minval == -0.5f &&
           op.quantize_info[0].maxval == 6.0f);
    const OperatorDef &op2 = net.op[1];
    EXPECT(op2.type == "Split" && op2.output == (std::vector<std::string>{"s0", "s1"}));
    EXPECT(op2.output_shape.size() == 2 && op2.output_shape[0] == (std::vector<int64_t>{64, 56, 56, 64}) &&
           op2.output_shape[1].empty());
    EXPECT(op2.output_type == (std::vector<int>{DT_UINT8, DT_INT32}));
    EXPECT(op2.quantize_info.size() == 2 && op2.quantize_info[0].zero_point == 255 &&
           op2.quantize_info[1].zero_point == INT32_MIN && op2.quantize_info[1].scale == 1.0e-3f);
    const ConstTensor &t = net.tensors[0];
    EXPECT(t.name == "conv_a/filter" && t.dims == (std::vector<int64_t>{128, 1, 1, 128}) && t.data_type == DT_UINT8 &&
           t.offset == 256 && t.data_size == 128 * 128 && t.scale == 0.0123f && t.zero_point == 131);
    const ConstTensor &t2 = net.tensors[1];
    EXPECT(t2.name == "conv_a/bias" && t2.dims == (std::vector<int64_t>{128}) && t2.data_type == DT_INT32 &&
           t2.offset == 256 + 128 * 128 && t2.data_size == 128 && t2.scale == 2.5e-4f && t2.zero_point == -3);
    EXPECT(net.tensors[2].name == "inline_floats" && net.tensors[2].data_type == DT_FLOAT);
    EXPECT(net.input_info.size() == 1 && net.input_info[0].name == "in" &&
           net.input_info[0].dims == (std::vector<int64_t>{64, 112, 112, 3}) && net.input_info[0].data_type == DT_FLOAT);
    EXPECT(net.output_info.size() == 1 && net.output_info[0].name == "s1" && net.output_info[0].data_type == DT_INT32 &&
           net.output_info[0].dims == (std::vector<int64_t>{64, 10}) && net.output_info[0].scale == 7.5f &&
           net.output_info[0].zero_point == -9);
    // every truncation of the independent writer's bytes is either refused or parses without
    // reading past the end (run under the address sanitizer in the CPU suite)
    for (size_t cut = 0; cut < bytes.size(); cut += 3) {
      NetDef part;
      (void)ParseNetDef(bytes.data(), cut, &part);
    }
  }
  return g_fail;
}

// Malformed model descriptions (crafted dims, sizes and offsets) make Init return
// MACE_INVALID_ARGS before it allocates anything.  This needs no GPU: the context is a plan-only
// one, on which the first allocation of a well-formed model fails with OUT_OF_RESOURCES instead.
static int test_malformed() {
  OpDelegatorRegistry reg;
  hip::RegisterAllHipDelegators(&reg);
  mace_hip_ctx *plan = nullptr;
  EXPECT(mace_hip_plan_ctx_create(256, 160 * 1024, &plan) == MACE_HIP_SUCCESS);
  std::vector<uint8_t> data(4096, 1);
  auto with_tensor = [&](std::vector<int64_t> dims, int64_t data_size, int64_t offset, int dt = DT_UINT8) {
    NetDef n;
    ConstTensor c; c.name = "w"; c.dims = std::move(dims); c.data_type = dt; c.offset = offset; c.data_size = data_size;
    n.tensors.push_back(c);
    SerialNet net(&reg, plan);
    return net.Init(n, data.data(), data.size());
  };
  const MaceStatus bad = MaceStatus::MACE_INVALID_ARGS, fine = MaceStatus::MACE_OUT_OF_RESOURCES;
  EXPECT(with_tensor({16, 16}, 256, 0) == fine);                        // well-formed: gets as far as the allocation
  EXPECT(with_tensor({16, 16}, 256, 3840) == fine);                     // ends exactly at the end of the buffer
  EXPECT(with_tensor({16, 16}, 256, 3841) == bad);                      // one byte past it
  EXPECT(with_tensor({-1, -256}, 256, 0) == bad);                       // negative dims whose product is positive
  EXPECT(with_tensor({-16, 16}, -256, 0) == bad);
  EXPECT(with_tensor({1ll << 40, 1ll << 40}, 0, 0) == bad);             // product wraps to 0
  EXPECT(with_tensor({1ll << 32, 1ll << 32, 256}, 256, 0) == bad);      // ... wraps to a small positive count
  EXPECT(with_tensor({1ll << 62, 4}, 0, 0, DT_INT32) == bad);           // byte count overflows
  EXPECT(with_tensor({16, 16}, 256, -4) == bad);                        // negative offset
  EXPECT(with_tensor({16, 16}, 255, 0) == bad);                         // data_size disagrees with dims
  EXPECT(with_tensor({0}, 0, INT64_MAX) == bad);                        // offset beyond the buffer
  EXPECT(with_tensor({16}, 16, 0, 3 /* DT_HALF */) == bad);             // a type this runner does not hold
  auto with_input = [&](std::vector<int64_t> dims, int dt) {
    NetDef n;
    InputOutputInfo in; in.name = "x"; in.dims = std::move(dims); in.data_type = dt;
    n.input_info.push_back(in);
    SerialNet net(&reg, plan);
    return net.Init(n, nullptr, 0);
  };
  EXPECT(with_input({4, 4}, DT_FLOAT) == fine);
  EXPECT(with_input({4, -4}, DT_FLOAT) == bad);
  EXPECT(with_input({1ll << 31, 1ll << 31, 16}, DT_FLOAT) == bad);
  EXPECT(with_input({1ll << 45, 8}, DT_UINT8) == bad);                  // no overflow, but no such tensor either
  EXPECT(with_input({4}, 3) == bad);
  {  // an op's outputs: a shape per output, quantize_info for all or none, sane shapes
    NetDef n;
    InputOutputInfo in; in.name = "x"; in.dims = {4}; in.data_type = DT_FLOAT;
    n.input_info.push_back(in);
    OperatorDef op; op.type = "Quantize"; op.name = "q"; op.input = {"x"}; op.output = {"y"};
    op.output_type = {DT_UINT8};
    n.op.push_back(op);
    { SerialNet net(&reg, plan); EXPECT(net.Init(n, nullptr, 0) == bad); }           // no output_shape
    n.op[0].output_shape = {{4, -1}};
    { SerialNet net(&reg, plan); EXPECT(net.Init(n, nullptr, 0) == bad); }
    n.op[0].output_shape = {{4}};
    n.op[0].quantize_info.resize(2);
    { SerialNet net(&reg, plan); EXPECT(net.Init(n, nullptr, 0) == bad); }
    n.op[0].quantize_info.resize(1);
    { SerialNet net(&reg, plan); EXPECT(net.Init(n, nullptr, 0) == fine); }
  }
  mace_hip_ctx_destroy(plan);
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

// Destroys the library context after everything declared later in the scope (nets and ops release
// their registrations and device memory through it, so they have to go first).
struct ContextHolder {
  mace_hip_ctx *ctx = nullptr;
  ~ContextHolder() { if (ctx) mace_hip_ctx_destroy(ctx); }
};

static Argument FloatArg(const char *name, float v) { Argument a; a.name = name; a.f = v; a.has_f = true; return a; }
static Argument StrArg(const char *name, const char *v) { Argument a; a.name = name; a.s = v; a.has_s = true; return a; }

static void AddConst(NetDef *net, std::vector<uint8_t> *data, const char *name, std::vector<int64_t> dims, int dt,
                     const void *bytes, size_t nbytes, float scale = 0.f, int32_t zp = 0) {
  ConstTensor c;
  c.name = name; c.dims = std::move(dims); c.data_type = dt; c.scale = scale; c.zero_point = zp;
  while (data->size() % 16) data->push_back(0);
  c.offset = (int64_t)data->size();
  c.data_size = (int64_t)(nbytes / (dt == DT_UINT8 ? 1 : 4));
  data->insert(data->end(), (const uint8_t *)bytes, (const uint8_t *)bytes + nbytes);
  net->tensors.push_back(c);
}
static void AddOp(NetDef *net, const char *type, const char *name, std::vector<std::string> ins, const char *o,
                  std::vector<int64_t> shape, int dt, float scale, int32_t zp, std::vector<Argument> args) {
  OperatorDef d;
  d.type = type; d.name = name; d.input = std::move(ins); d.output = {o};
  d.output_shape = {std::move(shape)}; d.output_type = {dt};
  if (scale > 0.f) { QuantizeActivationInfo q; q.scale = scale; q.zero_point = zp; d.quantize_info = {q}; }
  d.arg = std::move(args);
  net->op.push_back(d);
}
static bool close_f32(const std::vector<float> &got, const std::vector<float> &want) {
  if (got.size() != want.size()) return false;
  for (size_t i = 0; i < got.size(); ++i)
    if (!(std::fabs(got[i] - want[i]) <= 1e-2 + 1e-4 * std::fabs(want[i]))) return false;
  return true;
}

// The branches of the op factory the quantized toy net does not reach: float Conv2D (1x1, bias,
// RELUX), Reshape / Identity views, float MatMul with bias, float FullyConnected with RELU,
// Quantize, uint8 MatMul with a uint8 and with an int32 result, Dequantize of either -- one net,
// every intermediate tensor against the oracle's ops chained by hand.
static int test_mixed_net() {
  ContextHolder holder;
  if (mace_hip_ctx_create(0, &holder.ctx) != MACE_HIP_SUCCESS) { printf("FAIL: no context\n"); return 1; }
  mace_hip_ctx *hctx = holder.ctx;
  OpDelegatorRegistry reg;
  EXPECT(hip::RegisterAllHipDelegators(&reg) == MaceStatus::MACE_SUCCESS);
  std::mt19937 rng(2024);
  std::normal_distribution<float> nd(0.f, 1.f);
  const index_t n = 2, cin = 8, hw = 36, cout = 16, mm_cols = 20, fc_in = cout * mm_cols, fc_out = 10, q_cols = 12;
  std::vector<float> filt(cout * cin), cbias(cout), mm_w(hw * mm_cols), mm_b(mm_cols), fc_w(fc_out * fc_in), fc_b(fc_out);
  for (auto *v : {&filt, &cbias, &mm_w, &mm_b, &fc_w, &fc_b}) for (auto &e : *v) e = nd(rng) * 0.3f;
  std::vector<uint8_t> qw(fc_out * q_cols);
  for (auto &e : qw) e = rng() & 255;
  const float s_q = 0.05f, s_w = 0.02f, s_o = 1.5f; const int32_t z_q = 20, z_w = 119, z_o = 77;
  NetDef net; std::vector<uint8_t> data;
  net.name = "mixed";
  AddConst(&net, &data, "conv/filter", {cout, cin, 1, 1}, DT_FLOAT, filt.data(), filt.size() * 4);
  AddConst(&net, &data, "conv/bias", {cout}, DT_FLOAT, cbias.data(), cbias.size() * 4);
  AddConst(&net, &data, "mm/w", {hw, mm_cols}, DT_FLOAT, mm_w.data(), mm_w.size() * 4);
  AddConst(&net, &data, "mm/bias", {mm_cols}, DT_FLOAT, mm_b.data(), mm_b.size() * 4);
  AddConst(&net, &data, "fc/w", {fc_out, fc_in, 1, 1}, DT_FLOAT, fc_w.data(), fc_w.size() * 4);
  AddConst(&net, &data, "fc/bias", {fc_out}, DT_FLOAT, fc_b.data(), fc_b.size() * 4);
  AddConst(&net, &data, "qmm/w", {fc_out, q_cols}, DT_UINT8, qw.data(), qw.size(), s_w, z_w);
  InputOutputInfo in; in.name = "x"; in.dims = {n, cin, 6, 6}; in.data_type = DT_FLOAT;
  net.input_info.push_back(in);
  AddOp(&net, "Conv2D", "conv", {"x", "conv/filter", "conv/bias"}, "c", {n, cout, 6, 6}, DT_FLOAT, 0.f, 0,
        {IntArg("T", DT_FLOAT), IntsArg("strides", {1, 1}), IntArg("padding", VALID), StrArg("activation", "RELUX"),
         FloatArg("max_limit", 0.8f)});
  AddOp(&net, "Reshape", "r0", {"c"}, "c3", {n, cout, hw}, DT_FLOAT, 0.f, 0, {});
  AddOp(&net, "Identity", "id", {"c3"}, "c3i", {n, cout, hw}, DT_FLOAT, 0.f, 0, {});
  AddOp(&net, "MatMul", "mm", {"c3i", "mm/w", "mm/bias"}, "m", {n, cout, mm_cols}, DT_FLOAT, 0.f, 0, {IntArg("T", DT_FLOAT)});
  AddOp(&net, "Reshape", "r1", {"m"}, "m4", {n, fc_in, 1, 1}, DT_FLOAT, 0.f, 0, {});
  AddOp(&net, "FullyConnected", "fc", {"m4", "fc/w", "fc/bias"}, "f", {n, fc_out, 1, 1}, DT_FLOAT, 0.f, 0,
        {IntArg("T", DT_FLOAT), StrArg("activation", "RELU")});
  AddOp(&net, "Quantize", "quant", {"f"}, "fq", {n, fc_out, 1, 1}, DT_UINT8, s_q, z_q, {IntArg("T", DT_UINT8)});
  AddOp(&net, "Reshape", "r2", {"fq"}, "fq2", {n, fc_out}, DT_UINT8, 0.f, 0, {});
  AddOp(&net, "MatMul", "qmm8", {"fq2", "qmm/w"}, "q8", {n, q_cols}, DT_UINT8, s_o, z_o, {IntArg("T", DT_UINT8)});
  AddOp(&net, "MatMul", "qmm32", {"fq2", "qmm/w"}, "q32", {n, q_cols}, DT_INT32, 0.f, 0, {IntArg("T", DT_UINT8)});
  AddOp(&net, "Dequantize", "deq8", {"q8"}, "d8", {n, q_cols}, DT_FLOAT, 0.f, 0, {IntArg("T", DT_UINT8)});
  AddOp(&net, "Dequantize", "deq32", {"q32"}, "d32", {n, q_cols}, DT_FLOAT, 0.f, 0, {IntArg("T", DT_INT32)});
  const std::string bytes = SerializeNetDef(net);
  NetDef parsed;
  EXPECT(ParseNetDef(bytes.data(), bytes.size(), &parsed));
  SerialNet sn(&reg, hctx);
  MaceStatus st = sn.Init(parsed, data.data(), data.size());
  if (st != MaceStatus::MACE_SUCCESS) printf("Init: %s\n", sn.error().c_str());
  EXPECT(st == MaceStatus::MACE_SUCCESS);
  EXPECT(sn.op_count() == 8);    // four views create no op
  std::vector<float> x(n * cin * hw);
  for (auto &v : x) v = nd(rng);
  EXPECT(sn.SetInput("x", x.data(), x.size() * 4) == MaceStatus::MACE_SUCCESS);
  st = sn.Run();
  if (st != MaceStatus::MACE_SUCCESS) printf("Run: %s\n", sn.error().c_str());
  EXPECT(st == MaceStatus::MACE_SUCCESS);
  // the oracle's chain
  std::vector<float> c(n * cout * hw), m(n * cout * mm_cols), f(n * fc_out);
  orc_conv1x1_f32_nchw(x.data(), filt.data(), cbias.data(), n, cin, hw, cout, ORC_ACT_RELUX, 0.8f, c.data(), 2);
  orc_gemm_f32(c.data(), mm_w.data(), n, cout, mm_cols, hw, ORC_ROW_MAJOR, ORC_ROW_MAJOR, ORC_ROW_MAJOR, 1, 0, m.data(), 2);
  for (size_t i = 0; i < m.size(); ++i) m[i] += mm_b[i % mm_cols];
  orc_gemv_f32(fc_w.data(), m.data(), fc_b.data(), n, fc_out, fc_in, 0, 1, f.data(), 1);
  orc_activation_f32(f.data(), (int64_t)f.size(), ORC_ACT_RELU, 0.f);
  std::vector<float> got_c(c.size()), got_m(m.size()), got_f(f.size());
  EXPECT(sn.GetOutput("c3i", got_c.data(), got_c.size() * 4) == MaceStatus::MACE_SUCCESS);
  EXPECT(sn.GetOutput("m4", got_m.data(), got_m.size() * 4) == MaceStatus::MACE_SUCCESS);
  EXPECT(sn.GetOutput("f", got_f.data(), got_f.size() * 4) == MaceStatus::MACE_SUCCESS);
  EXPECT(close_f32(got_c, c) && close_f32(got_m, m) && close_f32(got_f, f));
  float cmax = 0.f, fmin = 1.f;
  for (float v : got_c) cmax = std::max(cmax, v);
  for (float v : got_f) fmin = std::min(fmin, v);
  EXPECT(cmax == 0.8f && fmin == 0.f);     // both activations bite
  // the quantized tail starts from the GPU's own float values (so that a last-bit difference in f
  // cannot flip a quantized byte of the comparison)
  std::vector<uint8_t> fq(f.size()), got_fq(f.size()), q8(n * q_cols), got_q8(q8.size());
  std::vector<int32_t> q32(n * q_cols), got_q32(q32.size());
  orc_quantize_with_scale_u8(got_f.data(), (int64_t)got_f.size(), s_q, z_q, fq.data());
  int32_t mult; int shift;
  EXPECT(orc_get_output_multiplier_and_shift(s_q, s_w, s_o, &mult, &shift) == 0);
  orc_q8_gemm_u8(fq.data(), qw.data(), 1, n, q_cols, fc_out, ORC_ROW_MAJOR, ORC_ROW_MAJOR, ORC_ROW_MAJOR, 1, 1, -z_q, -z_w,
                 nullptr, mult, shift, z_o, 0, 255, q8.data(), 1);
  orc_q8_gemm_i32(fq.data(), qw.data(), 1, n, q_cols, fc_out, ORC_ROW_MAJOR, ORC_ROW_MAJOR, ORC_ROW_MAJOR, 1, 1, -z_q, -z_w,
                  q32.data(), 1);
  EXPECT(sn.GetOutput("fq2", got_fq.data(), got_fq.size()) == MaceStatus::MACE_SUCCESS);
  EXPECT(sn.GetOutput("q8", got_q8.data(), got_q8.size()) == MaceStatus::MACE_SUCCESS);
  EXPECT(sn.GetOutput("q32", got_q32.data(), got_q32.size() * 4) == MaceStatus::MACE_SUCCESS);
  EXPECT(got_fq == fq && got_q8 == q8 && got_q32 == q32);
  std::vector<float> d8(q8.size()), d32(q32.size()), got_d8(d8.size()), got_d32(d32.size());
  orc_dequantize_u8(q8.data(), (int64_t)q8.size(), s_o, z_o, d8.data());
  // MatMulFixpointImpl<..., int32_t> gives its result scale = a.scale * b.scale, zero point 0
  orc_dequantize_i32(q32.data(), (int64_t)q32.size(), s_q * s_w, 0, d32.data());
  EXPECT(sn.GetOutput("d8", got_d8.data(), got_d8.size() * 4) == MaceStatus::MACE_SUCCESS);
  EXPECT(sn.GetOutput("d32", got_d32.data(), got_d32.size() * 4) == MaceStatus::MACE_SUCCESS);
  EXPECT(got_d8 == d8 && got_d32 == d32);
  {  // a float FullyConnected whose activation this library does not apply is refused at Init
    NetDef bad = parsed;
    for (auto &a : bad.op[5].arg) if (a.name == "activation") a.s = "TANH";
    SerialNet n2(&reg, hctx);
    EXPECT(n2.Init(bad, data.data(), data.size()) == MaceStatus::MACE_UNSUPPORTED);
    EXPECT(n2.error().find("TANH") != std::string::npos);
    for (auto &a : bad.op[5].arg) if (a.name == "activation") a.s = "Relu";
    SerialNet n3(&reg, hctx);
    EXPECT(n3.Init(bad, data.data(), data.size()) == MaceStatus::MACE_INVALID_ARGS);
  }
  {  // ops that lack an input or an output are refused, not dereferenced
    for (int which = 0; which < 3; ++which) {
      NetDef bad = parsed;
      if (which == 0) bad.op[6].input.clear();            // Quantize without input
      if (which == 1) bad.op[11].output.clear(), bad.op[11].output_shape.clear(), bad.op[11].output_type.clear();
      if (which == 2) bad.op[8].input.resize(1);          // MatMul with one input
      SerialNet n2(&reg, hctx);
      EXPECT(n2.Init(bad, data.data(), data.size()) == MaceStatus::MACE_INVALID_ARGS);
    }
  }
  return g_fail;
}

// The five pointwise layers of MobileNetV1-224 (benchmark configuration 4) inside a NetDef, through
// the serial runner: per layer Quantize -> Conv2D 1x1 with a ReLU6 output range (zero point 0,
// scale 6 / 255, so that the saturating cast is the clamp) -> Dequantize.  In the real network a
// depthwise convolution sits between two of them and changes the shape, so here each layer is a
// branch with an input of its own; the runner executes the fifteen ops in order, eagerly and as a
// replayed HIP graph, and every branch is compared with the oracle's chain.  `timing`: also prints
// the time per pass over all five layers (JSON, for bench.py).
struct C4Layer { index_t hw, cin, cout; };
static const C4Layer kC4[5] = {{112, 32, 64}, {56, 128, 128}, {28, 256, 256}, {14, 512, 512}, {7, 1024, 1024}};

static int test_c4_net(index_t batch, bool timing) {
  ContextHolder holder;
  if (mace_hip_ctx_create(0, &holder.ctx) != MACE_HIP_SUCCESS) { printf("FAIL: no context\n"); return 1; }
  mace_hip_ctx *hctx = holder.ctx;
  OpDelegatorRegistry reg;
  EXPECT(hip::RegisterAllHipDelegators(&reg) == MaceStatus::MACE_SUCCESS);
  std::mt19937 rng(4);
  NetDef net; std::vector<uint8_t> data;
  net.name = "mobilenet_v1_pointwise_layers";
  // filter scales such that the real-valued sums have a standard deviation of about 3: the ReLU6
  // range [0, 6] then clamps a good part of the outputs at either end, but not most of them
  const float s_in = 6.f / 255.f, s_out = 6.f / 255.f;
  float s_f[5];
  const int32_t z_in = 0, z_out = 0;
  std::vector<std::vector<uint8_t>> filt(5);
  std::vector<std::vector<int32_t>> bias(5);
  int32_t z_f[5];
  for (int l = 0; l < 5; ++l) {
    const C4Layer &L = kC4[l];
    filt[l].resize(L.cout * L.cin); bias[l].resize(L.cout);
    for (auto &e : filt[l]) e = (uint8_t)(rng() % 255 + 1);
    for (auto &e : bias[l]) e = (int32_t)(rng() % 65536) - 32768;
    z_f[l] = 126 + (int)(rng() % 5);
    s_f[l] = 3.f / (74.f * std::sqrt(12.f * (float)L.cin));
    char name[64];
    snprintf(name, sizeof(name), "pw%d/filter", l);
    AddConst(&net, &data, name, {L.cout, 1, 1, L.cin}, DT_UINT8, filt[l].data(), filt[l].size(), s_f[l], z_f[l]);
    snprintf(name, sizeof(name), "pw%d/bias", l);
    AddConst(&net, &data, name, {L.cout}, DT_INT32, bias[l].data(), bias[l].size() * 4, s_in * s_f[l], 0);
  }
  for (int l = 0; l < 5; ++l) {
    const C4Layer &L = kC4[l];
    char x[32], xq[32], y[32], yf[32], f[32], b[32], nq[32], nc[32], nd[32];
    snprintf(x, 32, "in%d", l); snprintf(xq, 32, "in%d_q", l); snprintf(y, 32, "act%d", l); snprintf(yf, 32, "out%d", l);
    snprintf(f, 32, "pw%d/filter", l); snprintf(b, 32, "pw%d/bias", l);
    snprintf(nq, 32, "quantize%d", l); snprintf(nc, 32, "pointwise%d", l); snprintf(nd, 32, "dequantize%d", l);
    InputOutputInfo in; in.name = x; in.dims = {batch, L.hw, L.hw, L.cin}; in.data_type = DT_FLOAT;
    net.input_info.push_back(in);
    AddOp(&net, "Quantize", nq, {x}, xq, {batch, L.hw, L.hw, L.cin}, DT_UINT8, s_in, z_in, {IntArg("T", DT_UINT8)});
    AddOp(&net, "Conv2D", nc, {xq, f, b}, y, {batch, L.hw, L.hw, L.cout}, DT_UINT8, s_out, z_out,
          {IntArg("T", DT_UINT8), IntsArg("strides", {1, 1}), IntArg("padding", VALID), StrArg("activation", "RELUX"),
           FloatArg("max_limit", 6.f)});
    AddOp(&net, "Dequantize", nd, {y}, yf, {batch, L.hw, L.hw, L.cout}, DT_FLOAT, 0.f, 0, {IntArg("T", DT_UINT8)});
  }
  const std::string bytes = SerializeNetDef(net);
  NetDef parsed;
  EXPECT(ParseNetDef(bytes.data(), bytes.size(), &parsed));
  SerialNet sn(&reg, hctx);
  MaceStatus st = sn.Init(parsed, data.data(), data.size());
  if (st != MaceStatus::MACE_SUCCESS) printf("Init: %s\n", sn.error().c_str());
  EXPECT(st == MaceStatus::MACE_SUCCESS && sn.op_count() == 15);
  std::uniform_real_distribution<float> ud(-0.5f, 6.5f);
  std::vector<std::vector<float>> x(5);
  for (int l = 0; l < 5; ++l) {
    x[l].resize((size_t)batch * kC4[l].hw * kC4[l].hw * kC4[l].cin);
    for (auto &v : x[l]) v = ud(rng);
  }
  auto check = [&](const char *what) {
    for (int l = 0; l < 5; ++l) {
      const C4Layer &L = kC4[l];
      const size_t pix = (size_t)batch * L.hw * L.hw;
      std::vector<uint8_t> q(x[l].size()), a(pix * L.cout);
      std::vector<float> want(a.size()), got(a.size());
      orc_quantize_with_scale_u8(x[l].data(), (int64_t)x[l].size(), s_in, z_in, q.data());
      EXPECT(orc_conv2d_q8_nhwc(q.data(), filt[l].data(), bias[l].data(), batch, L.hw, L.hw, L.cin, L.cout, 1, 1, 1, 1, 0, 0,
                                s_in, z_in, s_f[l], z_f[l], s_in * s_f[l], s_out, z_out, 0, 255, a.data(), 16) == 0);
      orc_dequantize_u8(a.data(), (int64_t)a.size(), s_out, z_out, want.data());
      char name[32]; snprintf(name, 32, "out%d", l);
      EXPECT(sn.GetOutput(name, got.data(), got.size() * 4) == MaceStatus::MACE_SUCCESS);
      const bool same = got == want;
      if (!same) printf("%s: layer %d differs\n", what, l);
      EXPECT(same);
      size_t lo = 0, hi = 0;
      for (uint8_t v : a) { lo += v == 0; hi += v == 255; }
      EXPECT(lo + hi < a.size() * 9 / 10 && lo + hi > 0);   // the ReLU6 clamp bites, but not everywhere
    }
  };
  auto set_inputs = [&]() {
    for (int l = 0; l < 5; ++l) {
      char name[32]; snprintf(name, 32, "in%d", l);
      EXPECT(sn.SetInput(name, x[l].data(), x[l].size() * 4) == MaceStatus::MACE_SUCCESS);
    }
  };
  set_inputs();
  EXPECT(sn.Run() == MaceStatus::MACE_SUCCESS);
  check("eager");
  st = sn.CaptureGraph();
  if (st != MaceStatus::MACE_SUCCESS) printf("CaptureGraph: %s\n", sn.error().c_str());
  EXPECT(st == MaceStatus::MACE_SUCCESS);
  for (int replay = 0; replay < 2; ++replay) {
    for (int l = 0; l < 5; ++l) for (size_t i = replay; i < x[l].size(); i += 7) x[l][i] = ud(rng);
    set_inputs();
    EXPECT(sn.RunGraph() == MaceStatus::MACE_SUCCESS);
    check("graph");
    if (replay == 0) { EXPECT(sn.Run() == MaceStatus::MACE_SUCCESS); EXPECT(mace_hip_sync(hctx) == MACE_HIP_SUCCESS); }
  }
  if (timing) {
    float ms_eager = 0.f, ms_graph = 0.f;
    const int reps = 30;
    for (int i = 0; i < 5; ++i) sn.Run();
    mace_hip_timer_start(hctx);
    for (int i = 0; i < reps; ++i) sn.Run();
    mace_hip_timer_stop(hctx, &ms_eager);
    for (int i = 0; i < 5; ++i) sn.RunGraph();
    mace_hip_timer_start(hctx);
    for (int i = 0; i < reps; ++i) sn.RunGraph();
    mace_hip_timer_stop(hctx, &ms_graph);
    double ops = 0;
    for (const C4Layer &L : kC4) ops += 2.0 * batch * L.hw * L.hw * L.cin * L.cout;
    printf("{\"workload\": \"c4_chain_n%d\", \"ops_in_net\": 15, \"eager_us\": %.1f, \"graph_us\": %.1f, "
           "\"conv_ops\": %.4g, \"parity\": %s}\n", (int)batch, ms_eager * 1e3 / reps, ms_graph * 1e3 / reps, ops,
           g_fail ? "false" : "true");
  }
  return g_fail;
}

// An op supplied by the host (SerialNet::RegisterOp): a 2x2 average pool computed on the CPU sits
// between two of this library's convolutions, so a net with an op type outside the library runs.
static int test_host_op() {
  ContextHolder holder;
  if (mace_hip_ctx_create(0, &holder.ctx) != MACE_HIP_SUCCESS) { printf("FAIL: no context\n"); return 1; }
  mace_hip_ctx *hctx = holder.ctx;
  OpDelegatorRegistry reg;
  EXPECT(hip::RegisterAllHipDelegators(&reg) == MaceStatus::MACE_SUCCESS);
  std::mt19937 rng(8);
  const index_t n = 2, hw = 8, c0 = 32, c1 = 64, c2 = 48;
  std::vector<uint8_t> f0(c1 * c0), f1(c2 * c1);
  for (auto &e : f0) e = rng() & 255;
  for (auto &e : f1) e = rng() & 255;
  NetDef net; std::vector<uint8_t> data;
  AddConst(&net, &data, "f0", {c1, 1, 1, c0}, DT_UINT8, f0.data(), f0.size(), 0.01f, 125);
  AddConst(&net, &data, "f1", {c2, 1, 1, c1}, DT_UINT8, f1.data(), f1.size(), 0.012f, 130);
  InputOutputInfo in; in.name = "x"; in.dims = {n, hw, hw, c0}; in.data_type = DT_UINT8; in.scale = 0.05f; in.zero_point = 128;
  net.input_info.push_back(in);
  AddOp(&net, "Conv2D", "conv0", {"x", "f0"}, "a", {n, hw, hw, c1}, DT_UINT8, 0.8f, 120, {IntArg("T", DT_UINT8), IntArg("padding", VALID)});
  AddOp(&net, "Pooling", "pool", {"a"}, "p", {n, hw / 2, hw / 2, c1}, DT_UINT8, 0.8f, 120, {IntArg("T", DT_UINT8), IntsArg("kernels", {2, 2})});
  AddOp(&net, "Conv2D", "conv1", {"p", "f1"}, "y", {n, hw / 2, hw / 2, c2}, DT_UINT8, 6.0f, 110, {IntArg("T", DT_UINT8), IntArg("padding", VALID)});
  auto pool = [](const std::vector<uint8_t> &a, index_t n, index_t hw, index_t c) {
    std::vector<uint8_t> p((size_t)n * (hw / 2) * (hw / 2) * c);
    for (index_t b = 0; b < n; ++b)
      for (index_t y = 0; y < hw / 2; ++y)
        for (index_t x = 0; x < hw / 2; ++x)
          for (index_t k = 0; k < c; ++k) {
            int s = 2;   // rounds to nearest
            for (int dy = 0; dy < 2; ++dy) for (int dx = 0; dx < 2; ++dx) s += a[((b * hw + 2 * y + dy) * hw + 2 * x + dx) * c + k];
            p[((b * (hw / 2) + y) * (hw / 2) + x) * c + k] = (uint8_t)(s / 4);
          }
    return p;
  };
  {  // without the host's op the net cannot be initialised
    SerialNet sn(&reg, hctx);
    EXPECT(sn.Init(net, data.data(), data.size()) == MaceStatus::MACE_UNSUPPORTED);
    EXPECT(sn.error().find("Pooling") != std::string::npos);
  }
  SerialNet sn(&reg, hctx);
  int created = 0;
  sn.RegisterOp("Pooling", [&](const OperatorDef &def, SerialNet *self, SerialNet::OpRun *run) {
    Tensor *src = self->GetTensor(def.input[0]), *dst = self->GetTensor(def.output[0]);
    if (!src || !dst || GetIntsArg(def, "kernels") != std::vector<int>{2, 2}) return MaceStatus::MACE_INVALID_ARGS;
    ++created;
    *run = [src, dst, pool](OpContext *c) {
      std::vector<uint8_t> a((size_t)src->size());
      if (mace_hip_memcpy_d2h(c->hip(), a.data(), src->data<uint8_t>(), a.size()) != MACE_HIP_SUCCESS)
        return MaceStatus::MACE_RUNTIME_ERROR;
      const std::vector<uint8_t> p = pool(a, src->dim(0), src->dim(1), src->dim(3));
      return ToStatus(mace_hip_memcpy_h2d(c->hip(), dst->mutable_data<uint8_t>(), p.data(), p.size()));
    };
    return MaceStatus::MACE_SUCCESS;
  });
  MaceStatus st = sn.Init(net, data.data(), data.size());
  if (st != MaceStatus::MACE_SUCCESS) printf("Init: %s\n", sn.error().c_str());
  EXPECT(st == MaceStatus::MACE_SUCCESS && created == 1 && sn.op_count() == 3);
  std::vector<uint8_t> x((size_t)n * hw * hw * c0), got((size_t)n * (hw / 2) * (hw / 2) * c2), a((size_t)n * hw * hw * c1), want(got.size());
  for (auto &e : x) e = rng() & 255;
  EXPECT(sn.SetInput("x", x.data(), x.size()) == MaceStatus::MACE_SUCCESS);
  EXPECT(sn.Run() == MaceStatus::MACE_SUCCESS);
  EXPECT(sn.GetOutput("y", got.data(), got.size()) == MaceStatus::MACE_SUCCESS);
  EXPECT(orc_conv2d_q8_nhwc(x.data(), f0.data(), nullptr, n, hw, hw, c0, c1, 1, 1, 1, 1, 0, 0, 0.05f, 128, 0.01f, 125, 0.f, 0.8f,
                            120, 0, 255, a.data(), 2) == 0);
  const std::vector<uint8_t> p = pool(a, n, hw, c1);
  EXPECT(orc_conv2d_q8_nhwc(p.data(), f1.data(), nullptr, n, hw / 2, hw / 2, c1, c2, 1, 1, 1, 1, 0, 0, 0.8f, 120, 0.012f, 130, 0.f,
                            6.0f, 110, 0, 255, want.data(), 2) == 0);
  EXPECT(got == want);
  // a host op that waits for the stream cannot be part of a captured graph: the capture fails cleanly
  EXPECT(sn.CaptureGraph() != MaceStatus::MACE_SUCCESS);
  EXPECT(sn.Run() == MaceStatus::MACE_SUCCESS);   // ... and the context stays usable
  EXPECT(sn.GetOutput("y", got.data(), got.size()) == MaceStatus::MACE_SUCCESS);
  EXPECT(got == want);
  return g_fail;
}

// An instantiated graph holds raw pointers into the context's arena.  Eager work that outgrows
// the arena afterwards must not pull it from under the graph: the old arena is kept until the
// graph is destroyed, and a replay after the growth still matches the oracle.
static int test_graph_outlives_arena_growth() {
  ContextHolder holder;
  if (mace_hip_ctx_create(0, &holder.ctx) != MACE_HIP_SUCCESS) { printf("FAIL: no context\n"); return 1; }
  mace_hip_ctx *hctx = holder.ctx;
  OpDelegatorRegistry reg;
  EXPECT(hip::RegisterAllHipDelegators(&reg) == MaceStatus::MACE_SUCCESS);
  Weights wt;
  Model m = BuildModel(&wt);
  std::mt19937 rng(77);
  std::normal_distribution<float> nd(0.f, 2.f);
  {
    SerialNet net(&reg, hctx);
    EXPECT(net.Init(m.net, m.data.data(), m.data.size()) == MaceStatus::MACE_SUCCESS);
    std::vector<float> x((size_t)m.n * m.h * m.w * m.c0), got(m.n * m.classes);
    for (auto &v : x) v = nd(rng);
    EXPECT(net.SetInput("data", x.data(), x.size() * 4) == MaceStatus::MACE_SUCCESS);
    EXPECT(net.Run() == MaceStatus::MACE_SUCCESS);
    EXPECT(net.CaptureGraph() == MaceStatus::MACE_SUCCESS);
    // an eager GEMM whose repacked panels need far more scratch than the toy net ever took:
    // ColMajor lhs and RowMajor rhs with an odd depth are both repacked (2 x 3000 x 1088 bytes)
    const index_t rows = 3000, depth = 1031, cols = 3000;
    std::vector<uint8_t> a(rows * depth), b(depth * cols);
    for (auto &e : a) e = rng() & 255;
    for (auto &e : b) e = rng() & 255;
    void *da = nullptr, *db = nullptr, *dc = nullptr;
    EXPECT(mace_hip_malloc(hctx, a.size(), &da) == MACE_HIP_SUCCESS && mace_hip_malloc(hctx, b.size(), &db) == MACE_HIP_SUCCESS &&
           mace_hip_malloc(hctx, (size_t)rows * cols * 4, &dc) == MACE_HIP_SUCCESS);
    mace_hip_memcpy_h2d(hctx, da, a.data(), a.size());
    mace_hip_memcpy_h2d(hctx, db, b.data(), b.size());
    EXPECT(mace_hip_gemm_q8_i32(hctx, (const uint8_t *)da, MACE_HIP_COL_MAJOR, (const uint8_t *)db, MACE_HIP_ROW_MAJOR,
                                (int32_t *)dc, MACE_HIP_ROW_MAJOR, 1, rows, depth, cols, 1, 1, -100, -90) == MACE_HIP_SUCCESS);
    mace_hip_plan plan;
    EXPECT(mace_hip_last_plan(hctx, &plan) == MACE_HIP_SUCCESS && (plan.aux & MACE_HIP_AUX_PACK_TRANSPOSE));
    std::vector<int32_t> c32((size_t)rows * cols), w32(c32.size());
    mace_hip_memcpy_d2h(hctx, c32.data(), dc, c32.size() * 4);
    orc_q8_gemm_i32(a.data(), b.data(), 1, rows, cols, depth, ORC_COL_MAJOR, ORC_ROW_MAJOR, ORC_ROW_MAJOR, 1, 1, -100, -90,
                    w32.data(), 16);
    EXPECT(c32 == w32);
    // the graph, recorded against the arena of before, still computes the net
    for (int replay = 0; replay < 2; ++replay) {
      for (auto &v : x) v = nd(rng);
      EXPECT(net.SetInput("data", x.data(), x.size() * 4) == MaceStatus::MACE_SUCCESS);
      EXPECT(net.RunGraph() == MaceStatus::MACE_SUCCESS);
      EXPECT(net.GetOutput("prob", got.data(), got.size() * 4) == MaceStatus::MACE_SUCCESS);
      EXPECT(got == OracleRun(m, wt, x));
      EXPECT(net.Run() == MaceStatus::MACE_SUCCESS);     // eager runs use the new arena
      EXPECT(net.GetOutput("prob", got.data(), got.size() * 4) == MaceStatus::MACE_SUCCESS);
      EXPECT(got == OracleRun(m, wt, x));
    }
    mace_hip_free(hctx, da); mace_hip_free(hctx, db); mace_hip_free(hctx, dc);
  }
  return g_fail;
}

int main(int argc, char **argv) {
  const char *mode = argc > 1 ? argv[1] : "wire";
  int fails;
  if (strcmp(mode, "run") == 0) fails = test_run();
  else if (strcmp(mode, "fixture") == 0) fails = test_fixture(argc > 2 ? argv[2] : "tests/golden");
  else if (strcmp(mode, "malformed") == 0) fails = test_malformed();
  else if (strcmp(mode, "mixed") == 0) fails = test_mixed_net();
  else if (strcmp(mode, "c4") == 0) fails = test_c4_net(argc > 2 ? atoi(argv[2]) : 2, argc > 3);
  else if (strcmp(mode, "hostop") == 0) fails = test_host_op();
  else if (strcmp(mode, "graph_arena") == 0) fails = test_graph_outlives_arena_growth();
  else fails = test_wire();
  printf("%s: %s (%d failures)\n", mode, fails ? "FAILED" : "ok", fails);
  return fails ? 1 : 0;
}
