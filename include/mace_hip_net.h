// mace_hip_net.h -- a NetDef loader and a serial runner on device tensors, above the delegator
// adapter (mace_hip_delegator.h).
//
// What it mirrors in the reference:
//   * the model description: NetDef / OperatorDef / Argument / ConstTensor /
//     QuantizeActivationInfo / OutputShape / InputOutputInfo of mace/proto/mace.proto:24-126,
//     read from (and, for tests and tools, written to) the protobuf wire format with a reader
//     of its own -- protoc and libprotobuf are not needed;
//   * Workspace::LoadModelTensor (mace/core/workspace.cc:108-206): every ConstTensor is a slice
//     [offset, offset + data_size) of ONE weights buffer, carries its scale and zero point, and is
//     flagged as a weight; here the buffer is copied to the GPU once and the slices point into it;
//   * Workspace::AddQuantizeInfoForOutputTensor (:210-228): an op's quantize_info gives its output
//     tensors their scale and zero point;
//   * SerialNet::Init / Run (mace/core/net/serial_net.cc:39-124): ops are created once, in the
//     order of the NetDef, and run one after the other on the caller's thread.
// The ops it creates itself are the ones this library computes: Quantize, Dequantize, Conv2D
// (uint8 NHWC any geometry; float NCHW 1x1), MatMul, FullyConnected, and the shape-only Reshape /
// Squeeze / Identity.  Other op types come from the host: RegisterOp(type, creator) adds an op
// factory, as the reference creates every op through its registry (serial_net.cc:39-91), so a
// host can supply DepthwiseConv2d, Pooling, Softmax ... (on the CPU, or with kernels of its own)
// and run a whole MobileNet with this library's ops on the GPU.  An op type nobody provides makes
// Init return MACE_UNSUPPORTED and names the op.
// Output tensors get a device buffer each, sized from the op's output_shape and output_type
// (the reference's memory optimizer, which lets ops share buffers, is not mirrored).
//
// Beyond the reference: once a net has run, its whole op sequence can be captured into a HIP
// graph (CaptureGraph) and replayed with one launch (RunGraph), which removes the per-op launch
// cost that dominates single-image inference.
#ifndef MACE_HIP_NET_H_
#define MACE_HIP_NET_H_

#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "mace_hip_delegator.h"

namespace mace_hip {
namespace net {

// ---- messages (mace/proto/mace.proto) ----------------------------------------------------------
struct Argument {            // :41-48
  std::string name;
  bool has_f = false, has_i = false, has_s = false;
  float f = 0.f;
  int64_t i = 0;
  std::string s;
  std::vector<float> floats;
  std::vector<int64_t> ints;
};
struct ConstTensor {         // :24-39
  std::vector<int64_t> dims;
  int data_type = DT_FLOAT;
  std::string name;
  int64_t offset = 0, data_size = 0;   // data_size counts elements (workspace.cc:181-183)
  float scale = 0.f;
  int32_t zero_point = 0;
};
struct QuantizeActivationInfo {   // :60-65
  float scale = 0.f;
  int32_t zero_point = 0;
  float minval = 0.f, maxval = 0.f;
};
struct OperatorDef {         // :67-88
  std::vector<std::string> input, output;
  std::string name, type;
  std::vector<Argument> arg;
  std::vector<std::vector<int64_t>> output_shape;
  std::vector<int> output_type;
  std::vector<QuantizeActivationInfo> quantize_info;
};
struct InputOutputInfo {     // :90-101
  std::string name;
  std::vector<int64_t> dims;
  int data_type = DT_FLOAT;
  float scale = 0.f;
  int32_t zero_point = 0;
};
struct NetDef {              // :103-117
  std::vector<OperatorDef> op;
  std::vector<ConstTensor> tensors;
  std::string name;
  std::vector<InputOutputInfo> input_info, output_info;
};

// ---- protobuf wire format ----------------------------------------------------------------------
namespace wire {

struct Reader {
  const uint8_t *p, *end;
  bool ok = true;
  Reader(const uint8_t *b, size_t n) : p(b), end(b + n) {}
  bool done() const { return p >= end || !ok; }
  uint64_t varint() {
    uint64_t v = 0;
    for (int shift = 0; shift < 64 && p < end; shift += 7) {
      const uint8_t b = *p++;
      v |= (uint64_t)(b & 0x7f) << shift;
      if (!(b & 0x80)) return v;
    }
    ok = false;
    return 0;
  }
  uint32_t fixed32() {
    if (end - p < 4) { ok = false; return 0; }
    uint32_t v; memcpy(&v, p, 4); p += 4; return v;
  }
  Reader sub() {   // a length-delimited field
    const uint64_t n = varint();
    if (!ok || n > (uint64_t)(end - p)) { ok = false; return Reader(p, 0); }
    Reader r(p, (size_t)n);
    p += n;
    return r;
  }
  void skip(int wt) {
    if (wt == 0) (void)varint();
    else if (wt == 1) { if (end - p < 8) ok = false; else p += 8; }
    else if (wt == 2) (void)sub();
    else if (wt == 5) (void)fixed32();
    else ok = false;
  }
  std::string str() { Reader r = sub(); return std::string((const char *)r.p, (size_t)(r.end - r.p)); }
  // a repeated scalar: one element, or a packed run of them
  template <typename T> void ints(int wt, std::vector<T> *out) {
    if (wt == 2) { Reader r = sub(); while (!r.done()) out->push_back((T)r.varint()); ok = ok && r.ok; }
    else out->push_back((T)varint());
  }
  void floats(int wt, std::vector<float> *out) {
    auto one = [](uint32_t u) { float f; memcpy(&f, &u, 4); return f; };
    if (wt == 2) { Reader r = sub(); while (!r.done()) out->push_back(one(r.fixed32())); ok = ok && r.ok; }
    else out->push_back(one(fixed32()));
  }
  float f32() { const uint32_t u = fixed32(); float f; memcpy(&f, &u, 4); return f; }
};

struct Writer {
  std::string out;
  void varint(uint64_t v) { while (v >= 0x80) { out.push_back((char)(v | 0x80)); v >>= 7; } out.push_back((char)v); }
  void tag(int field, int wt) { varint(((uint64_t)field << 3) | (uint64_t)wt); }
  void i64(int field, int64_t v) { tag(field, 0); varint((uint64_t)v); }
  void f32(int field, float f) { tag(field, 5); uint32_t u; memcpy(&u, &f, 4); out.append((const char *)&u, 4); }
  void bytes(int field, const std::string &s) { tag(field, 2); varint(s.size()); out += s; }
};

inline bool Parse(Reader r, Argument *a) {
  while (!r.done()) {
    const uint64_t t = r.varint(); const int f = (int)(t >> 3), wt = (int)(t & 7);
    if (f == 1 && wt == 2) a->name = r.str();
    else if (f == 2 && wt == 5) { a->f = r.f32(); a->has_f = true; }
    else if (f == 3 && wt == 0) { a->i = (int64_t)r.varint(); a->has_i = true; }
    else if (f == 4 && wt == 2) { a->s = r.str(); a->has_s = true; }
    else if (f == 5) r.floats(wt, &a->floats);
    else if (f == 6) r.ints(wt, &a->ints);
    else r.skip(wt);
  }
  return r.ok;
}
inline bool Parse(Reader r, ConstTensor *c) {
  while (!r.done()) {
    const uint64_t t = r.varint(); const int f = (int)(t >> 3), wt = (int)(t & 7);
    if (f == 1) r.ints(wt, &c->dims);
    else if (f == 2 && wt == 0) c->data_type = (int)r.varint();
    else if (f == 5 && wt == 2) c->name = r.str();
    else if (f == 6 && wt == 0) c->offset = (int64_t)r.varint();
    else if (f == 7 && wt == 0) c->data_size = (int64_t)r.varint();
    else if (f == 8 && wt == 5) c->scale = r.f32();
    else if (f == 9 && wt == 0) c->zero_point = (int32_t)r.varint();
    else r.skip(wt);
  }
  return r.ok;
}
inline bool Parse(Reader r, QuantizeActivationInfo *q) {
  while (!r.done()) {
    const uint64_t t = r.varint(); const int f = (int)(t >> 3), wt = (int)(t & 7);
    if (f == 1 && wt == 5) q->scale = r.f32();
    else if (f == 2 && wt == 0) q->zero_point = (int32_t)r.varint();
    else if (f == 3 && wt == 5) q->minval = r.f32();
    else if (f == 4 && wt == 5) q->maxval = r.f32();
    else r.skip(wt);
  }
  return r.ok;
}
inline bool Parse(Reader r, OperatorDef *o) {
  while (!r.done()) {
    const uint64_t t = r.varint(); const int f = (int)(t >> 3), wt = (int)(t & 7);
    if (f == 1 && wt == 2) o->input.push_back(r.str());
    else if (f == 2 && wt == 2) o->output.push_back(r.str());
    else if (f == 3 && wt == 2) o->name = r.str();
    else if (f == 4 && wt == 2) o->type = r.str();
    else if (f == 6 && wt == 2) { o->arg.emplace_back(); if (!Parse(r.sub(), &o->arg.back())) return false; }
    else if (f == 7 && wt == 2) {   // OutputShape { repeated int64 dims = 1; }
      Reader s = r.sub();
      o->output_shape.emplace_back();
      while (!s.done()) {
        const uint64_t st = s.varint();
        if ((st >> 3) == 1) s.ints((int)(st & 7), &o->output_shape.back()); else s.skip((int)(st & 7));
      }
      if (!s.ok) return false;
    }
    else if (f == 8) r.ints(wt, &o->output_type);
    else if (f == 9 && wt == 2) { o->quantize_info.emplace_back(); if (!Parse(r.sub(), &o->quantize_info.back())) return false; }
    else r.skip(wt);
  }
  return r.ok;
}
inline bool Parse(Reader r, InputOutputInfo *i) {
  while (!r.done()) {
    const uint64_t t = r.varint(); const int f = (int)(t >> 3), wt = (int)(t & 7);
    if (f == 1 && wt == 2) i->name = r.str();
    else if (f == 3) r.ints(wt, &i->dims);
    else if (f == 5 && wt == 0) i->data_type = (int)r.varint();
    else if (f == 7 && wt == 5) i->scale = r.f32();
    else if (f == 8 && wt == 0) i->zero_point = (int32_t)r.varint();
    else r.skip(wt);
  }
  return r.ok;
}

inline std::string Serialize(const Argument &a) {
  Writer w;
  w.bytes(1, a.name);
  if (a.has_f) w.f32(2, a.f);
  if (a.has_i) w.i64(3, a.i);
  if (a.has_s) w.bytes(4, a.s);
  for (float f : a.floats) w.f32(5, f);
  for (int64_t v : a.ints) w.i64(6, v);
  return w.out;
}
inline std::string Serialize(const OperatorDef &o) {
  Writer w;
  for (const auto &s : o.input) w.bytes(1, s);
  for (const auto &s : o.output) w.bytes(2, s);
  w.bytes(3, o.name);
  w.bytes(4, o.type);
  for (const auto &a : o.arg) w.bytes(6, Serialize(a));
  for (const auto &shape : o.output_shape) { Writer s; for (int64_t d : shape) s.i64(1, d); w.bytes(7, s.out); }
  for (int t : o.output_type) w.i64(8, t);
  for (const auto &q : o.quantize_info) {
    Writer s; s.f32(1, q.scale); s.i64(2, q.zero_point); s.f32(3, q.minval); s.f32(4, q.maxval);
    w.bytes(9, s.out);
  }
  return w.out;
}
inline std::string Serialize(const InputOutputInfo &i) {
  Writer w;
  w.bytes(1, i.name);
  { Writer p; for (int64_t d : i.dims) p.varint((uint64_t)d); w.bytes(3, p.out); }   // packed, as protoc may emit
  w.i64(5, i.data_type);
  w.f32(7, i.scale);
  w.i64(8, i.zero_point);
  return w.out;
}

}  // namespace wire

// NetDef from / to the wire format.  Fields this runner does not use are skipped on reading.
inline bool ParseNetDef(const void *data, size_t size, NetDef *net) {
  wire::Reader r((const uint8_t *)data, size);
  while (!r.done()) {
    const uint64_t t = r.varint(); const int f = (int)(t >> 3), wt = (int)(t & 7);
    if (f == 1 && wt == 2) { net->op.emplace_back(); if (!wire::Parse(r.sub(), &net->op.back())) return false; }
    else if (f == 3 && wt == 2) { net->tensors.emplace_back(); if (!wire::Parse(r.sub(), &net->tensors.back())) return false; }
    else if (f == 5 && wt == 2) net->name = r.str();
    else if (f == 100 && wt == 2) { net->input_info.emplace_back(); if (!wire::Parse(r.sub(), &net->input_info.back())) return false; }
    else if (f == 101 && wt == 2) { net->output_info.emplace_back(); if (!wire::Parse(r.sub(), &net->output_info.back())) return false; }
    else r.skip(wt);
  }
  return r.ok;
}
inline std::string SerializeNetDef(const NetDef &net) {
  wire::Writer w;
  for (const auto &o : net.op) w.bytes(1, wire::Serialize(o));
  for (const auto &c : net.tensors) {
    wire::Writer s;
    for (int64_t d : c.dims) s.i64(1, d);
    s.i64(2, c.data_type);
    s.bytes(5, c.name);
    s.i64(6, c.offset);
    s.i64(7, c.data_size);
    s.f32(8, c.scale);
    s.i64(9, c.zero_point);
    w.bytes(3, s.out);
  }
  w.bytes(5, net.name);
  for (const auto &i : net.input_info) w.bytes(100, wire::Serialize(i));
  for (const auto &i : net.output_info) w.bytes(101, wire::Serialize(i));
  return w.out;
}

// ProtoArgHelper (mace/core/proto/arg_helper.h): arguments of an op by name, with defaults
inline const Argument *FindArg(const OperatorDef &op, const char *name) {
  for (const auto &a : op.arg) if (a.name == name) return &a;
  return nullptr;
}
inline int64_t GetIntArg(const OperatorDef &op, const char *name, int64_t dflt) {
  const Argument *a = FindArg(op, name);
  return (a && a->has_i) ? a->i : dflt;
}
inline std::vector<int> GetIntsArg(const OperatorDef &op, const char *name, std::vector<int> dflt = {}) {
  const Argument *a = FindArg(op, name);
  if (!a || a->ints.empty()) return dflt;
  return std::vector<int>(a->ints.begin(), a->ints.end());
}

inline size_t SizeOfType(int dt) {
  return dt == DT_FLOAT || dt == DT_INT32 ? 4 : (dt == DT_UINT8 ? 1 : 0);
}
// Elements of a shape times `elem` bytes; false for a negative dimension or a product that does
// not fit (shapes come from a file: nothing about them is trusted).
inline bool CheckedBytes(const std::vector<int64_t> &dims, size_t elem, int64_t *count, size_t *bytes) {
  int64_t n = 1;
  for (int64_t d : dims) {
    if (d < 0 || __builtin_mul_overflow(n, d, &n)) return false;
  }
  int64_t b = 0;
  if (__builtin_mul_overflow(n, (int64_t)elem, &b) || b > ((int64_t)1 << 46)) return false;
  *count = n;
  *bytes = (size_t)b;
  return true;
}

// ---- the runner ------------------------------------------------------------------------------------
class SerialNet {
 public:
  SerialNet(OpDelegatorRegistry *registry, mace_hip_ctx *ctx)
      : registry_(registry), ctx_(ctx), context_(ctx) {}
  SerialNet(const SerialNet &) = delete;
  SerialNet &operator=(const SerialNet &) = delete;
  ~SerialNet() {
    if (graph_) (void)mace_hip_graph_destroy(ctx_, graph_);
    ops_.clear();   // ops release their weight registrations before the weights are freed
    if (weights_) (void)mace_hip_free(ctx_, weights_);
    if (activations_) (void)mace_hip_free(ctx_, activations_);
  }
  const std::string &error() const { return error_; }

  // An op supplied by the host.  The creator is called once per OperatorDef of its type during
  // Init, after every tensor of the net exists (GetTensor: device tensors, the outputs sized from
  // the def's output_shape / output_type and carrying its quantize_info), and returns the function
  // Run() calls in the op's place.  An op that computes on the CPU moves its operands itself
  // (mace_hip_memcpy_d2h / _h2d, which wait for the stream); such an op cannot be captured into a
  // graph.  Register before Init; a type registered here takes precedence over a built-in one.
  typedef std::function<MaceStatus(OpContext *)> OpRun;
  typedef std::function<MaceStatus(const OperatorDef &, SerialNet *, OpRun *)> OpCreator;
  void RegisterOp(const std::string &type, OpCreator creator) { custom_ops_[type] = std::move(creator); }

  // Workspace::LoadModelTensor + AddQuantizeInfoForOutputTensor + SerialNet::Init
  MaceStatus Init(const NetDef &net, const void *model_data, size_t model_data_size) {
    if (!ops_.empty() || weights_) return Fail(MaceStatus::MACE_INVALID_ARGS, "Init called twice");
    // Everything the file says is checked before anything is allocated.
    // weights: every ConstTensor is a slice of ONE buffer (workspace.cc:170-205)
    for (const ConstTensor &c : net.tensors) {
      const size_t es = SizeOfType(c.data_type);
      int64_t count = 0;
      size_t bytes = 0;
      if (es == 0 || c.offset < 0 || !CheckedBytes(c.dims, es, &count, &bytes) || count != c.data_size ||
          (uint64_t)c.offset > model_data_size || bytes > model_data_size - (uint64_t)c.offset)
        return Fail(MaceStatus::MACE_INVALID_ARGS, "tensor " + c.name + ": bad type, size or offset");
    }
    // activations: the net's inputs and every op output, a 256-byte aligned slice each
    struct Want { std::string name; std::vector<index_t> shape; int dt; float scale; int32_t zp; size_t off; };
    std::vector<Want> wants;
    size_t total = 0;
    auto want = [&](const std::string &name, const std::vector<int64_t> &shape, int dt, float scale,
                    int32_t zp) -> bool {
      int64_t count = 0;
      size_t n = 0;
      if (SizeOfType(dt) == 0 || !CheckedBytes(shape, SizeOfType(dt), &count, &n)) return false;
      wants.push_back(Want{name, shape, dt, scale, zp, total});
      total += (n + 255) / 256 * 256 + 256;
      return total < ((size_t)1 << 47);
    };
    for (const InputOutputInfo &i : net.input_info)
      if (!want(i.name, i.dims, i.data_type, i.scale, i.zero_point))
        return Fail(MaceStatus::MACE_INVALID_ARGS, "input " + i.name + ": bad shape or type");
    std::map<std::string, std::string> alias;   // output of a shape-only op -> the tensor it views
    for (const OperatorDef &op : net.op) {
      if (!op.quantize_info.empty() && op.quantize_info.size() != op.output.size())
        return Fail(MaceStatus::MACE_INVALID_ARGS,
                    op.name + ": quantize info size must be equal to output size or empty");
      if (op.output_shape.size() != op.output.size())
        return Fail(MaceStatus::MACE_INVALID_ARGS, op.name + ": an output_shape per output is needed");
      const bool view = op.type == "Reshape" || op.type == "Squeeze" || op.type == "Identity";
      for (size_t k = 0; k < op.output.size(); ++k) {
        const int dt = k < op.output_type.size() ? op.output_type[k]
                                                 : (int)GetIntArg(op, "T", DT_FLOAT);
        const float scale = op.quantize_info.empty() ? 0.f : op.quantize_info[k].scale;
        const int32_t zp = op.quantize_info.empty() ? 0 : op.quantize_info[k].zero_point;
        if (view) {
          if (op.input.empty() || k > 0) return Fail(MaceStatus::MACE_INVALID_ARGS, op.name + ": one input, one output");
          alias[op.output[k]] = op.input[0];
          views_.push_back({op.output[k], op.input[0], op.output_shape[k]});
        } else if (!want(op.output[k], op.output_shape[k], dt, scale, zp)) {
          return Fail(MaceStatus::MACE_INVALID_ARGS, op.name + ": bad output shape or type");
        }
      }
    }
    // the weights buffer is copied to the GPU once and the slices point into it
    if (model_data_size > 0) {
      if (mace_hip_malloc(ctx_, model_data_size, &weights_) != MACE_HIP_SUCCESS ||
          mace_hip_memcpy_h2d(ctx_, weights_, model_data, model_data_size) != MACE_HIP_SUCCESS)
        return Fail(MaceStatus::MACE_OUT_OF_RESOURCES, mace_hip_last_error(ctx_));
    }
    for (const ConstTensor &c : net.tensors)
      tensors_[c.name] = Tensor((char *)weights_ + c.offset, (DataType)c.data_type, c.dims, c.scale,
                                c.zero_point, /*is_weight=*/true, /*on_device=*/true);
    if (total > 0 && mace_hip_malloc(ctx_, total, &activations_) != MACE_HIP_SUCCESS)
      return Fail(MaceStatus::MACE_OUT_OF_RESOURCES, mace_hip_last_error(ctx_));
    for (const Want &w : wants)
      tensors_[w.name] = Tensor((char *)activations_ + w.off, (DataType)w.dt, w.shape, w.scale, w.zp,
                                false, true);
    for (const View &v : views_) {   // in net order, so a view of a view resolves
      auto it = tensors_.find(v.of);
      if (it == tensors_.end()) return Fail(MaceStatus::MACE_INVALID_ARGS, "no tensor " + v.of);
      Tensor t = it->second;
      int64_t n = 0;
      size_t unused = 0;
      if (!CheckedBytes(v.shape, 1, &n, &unused) || n != t.size()) return Fail(MaceStatus::MACE_INVALID_ARGS, v.name + ": a view cannot change the size");
      tensors_[v.name] = Tensor(t.mutable_data<char>(), t.dtype(), v.shape, t.scale(), t.zero_point(),
                                t.is_weight(), true);
    }
    // ops, in NetDef order (serial_net.cc:39-91)
    for (const OperatorDef &op : net.op) {
      std::unique_ptr<Op> made;
      MaceStatus st = CreateOp(op, &made);
      if (st != MaceStatus::MACE_SUCCESS) return st;
      if (made) ops_.push_back(std::move(made));
    }
    return MaceStatus::MACE_SUCCESS;
  }

  Tensor *GetTensor(const std::string &name) {
    auto it = tensors_.find(name);
    return it == tensors_.end() ? nullptr : &it->second;
  }
  MaceStatus SetInput(const std::string &name, const void *host, size_t bytes) {
    Tensor *t = GetTensor(name);
    if (!t || bytes != (size_t)t->size() * SizeOfType(t->dtype()))
      return Fail(MaceStatus::MACE_INVALID_ARGS, "input " + name + ": unknown or wrong size");
    return ToStatus(mace_hip_memcpy_h2d(ctx_, t->mutable_data<char>(), host, bytes));
  }
  MaceStatus GetOutput(const std::string &name, void *host, size_t bytes) {
    Tensor *t = GetTensor(name);
    if (!t || bytes != (size_t)t->size() * SizeOfType(t->dtype()))
      return Fail(MaceStatus::MACE_INVALID_ARGS, "output " + name + ": unknown or wrong size");
    return ToStatus(mace_hip_memcpy_d2h(ctx_, host, t->data<char>(), bytes));
  }

  // SerialNet::Run (serial_net.cc:93-124): every op in order; stream-ordered, no waiting
  MaceStatus Run() {
    for (auto &op : ops_) {
      MaceStatus st = op->Run(&context_);
      if (st != MaceStatus::MACE_SUCCESS) return Fail(st, op->name + ": " + mace_hip_last_error(ctx_));
    }
    return MaceStatus::MACE_SUCCESS;
  }
  // Records the op sequence into a HIP graph (after at least one Run(), so that scratch and
  // weight caches exist); RunGraph replays it with one launch.
  MaceStatus CaptureGraph() {
    if (graph_) { (void)mace_hip_graph_destroy(ctx_, graph_); graph_ = nullptr; }
    if (mace_hip_graph_capture_begin(ctx_) != MACE_HIP_SUCCESS)
      return Fail(MaceStatus::MACE_RUNTIME_ERROR, mace_hip_last_error(ctx_));
    const MaceStatus run = Run();
    const int end = mace_hip_graph_capture_end(ctx_, &graph_);
    if (run != MaceStatus::MACE_SUCCESS) {
      if (graph_) { (void)mace_hip_graph_destroy(ctx_, graph_); graph_ = nullptr; }
      return run;
    }
    return end == MACE_HIP_SUCCESS ? MaceStatus::MACE_SUCCESS
                                   : Fail(ToStatus(end), mace_hip_last_error(ctx_));
  }
  MaceStatus RunGraph() {
    if (!graph_) return Fail(MaceStatus::MACE_INVALID_ARGS, "no graph captured");
    return ToStatus(mace_hip_graph_launch(ctx_, graph_));
  }
  size_t op_count() const { return ops_.size(); }

 private:
  struct Op {
    std::string name;
    virtual ~Op() = default;
    virtual MaceStatus Run(OpContext *context) = 0;
  };
  template <typename F>
  struct OpOf : Op {
    F fn;
    explicit OpOf(F f) : fn(std::move(f)) {}
    MaceStatus Run(OpContext *context) override { return fn(context); }
  };
  template <typename F>
  static std::unique_ptr<Op> Make(const std::string &name, F f) {
    std::unique_ptr<Op> p(new OpOf<F>(std::move(f)));
    p->name = name;
    return p;
  }
  struct View { std::string name, of; std::vector<int64_t> shape; };

  MaceStatus Fail(MaceStatus st, const std::string &why) { error_ = why; return st; }

  // The "activation" / "max_limit" arguments of a float op.  An activation this library does not
  // apply is refused here, at Init, never dropped.
  MaceStatus ParseActivation(const OperatorDef &def, ActivationType *act, float *limit) {
    const Argument *a = FindArg(def, "activation");
    if (a && a->has_s) {
      if (!StringToActivationType(a->s, act))
        return Fail(MaceStatus::MACE_INVALID_ARGS, def.name + ": unknown activation type: " + a->s);
      if (*act != NOOP && *act != RELU && *act != RELUX)
        return Fail(MaceStatus::MACE_UNSUPPORTED, def.name + ": activation " + a->s + " is not applied by this library");
    }
    const Argument *lim = FindArg(def, "max_limit");
    *limit = (lim && lim->has_f) ? lim->f : 0.f;
    return MaceStatus::MACE_SUCCESS;
  }

  MaceStatus CreateOp(const OperatorDef &def, std::unique_ptr<Op> *out) {
    auto in = [&](size_t k) -> Tensor * { return k < def.input.size() ? GetTensor(def.input[k]) : nullptr; };
    auto outt = [&](size_t k) -> Tensor * { return k < def.output.size() ? GetTensor(def.output[k]) : nullptr; };
    for (const auto &n : def.input)
      if (!GetTensor(n)) return Fail(MaceStatus::MACE_INVALID_ARGS, def.name + ": no tensor " + n);
    const int T = (int)GetIntArg(def, "T", DT_FLOAT);
    const std::string &type = def.type;
    auto custom = custom_ops_.find(type);
    if (custom != custom_ops_.end()) {
      OpRun run;
      MaceStatus st = custom->second(def, this, &run);
      if (st != MaceStatus::MACE_SUCCESS) return error_.empty() ? Fail(st, def.name + ": the host's op creator failed") : st;
      if (!run) return Fail(MaceStatus::MACE_INVALID_ARGS, def.name + ": the host's op creator returned no op");
      *out = Make(def.name, std::move(run));
      return MaceStatus::MACE_SUCCESS;
    }
    if (type == "Reshape" || type == "Squeeze" || type == "Identity") return MaceStatus::MACE_SUCCESS;
    // every built-in op reads input 0 and writes output 0
    if (!in(0) || !outt(0))
      return Fail(MaceStatus::MACE_INVALID_ARGS, def.name + ": " + type + " needs an input and an output");
    if (type == "Quantize") {
      auto op = std::make_shared<ops::QuantizeOp>(GetIntArg(def, "non_zero", 0) != 0,
                                                  GetIntArg(def, "find_range_every_time", 0) != 0);
      Tensor *x = in(0), *y = outt(0);
      *out = Make(def.name, [op, x, y](OpContext *c) { return op->Run(c, x, y); });
    } else if (type == "Dequantize") {
      Tensor *x = in(0), *y = outt(0);
      if (x->dtype() == DT_INT32) {
        auto op = std::make_shared<ops::DequantizeOp<int32_t>>();
        *out = Make(def.name, [op, x, y](OpContext *c) { return op->Run(c, x, y); });
      } else {
        auto op = std::make_shared<ops::DequantizeOp<uint8_t>>();
        *out = Make(def.name, [op, x, y](OpContext *c) { return op->Run(c, x, y); });
      }
    } else if (type == "Conv2D") {
      const std::vector<int> strides = GetIntsArg(def, "strides", {1, 1});
      const Padding pad = (Padding)GetIntArg(def, "padding", SAME);
      const std::vector<int> pads = GetIntsArg(def, "padding_values");
      const std::vector<int> dil = GetIntsArg(def, "dilations", {1, 1});
      Tensor *x = in(0), *f = in(1), *b = in(2), *y = outt(0);
      if (!f) return Fail(MaceStatus::MACE_INVALID_ARGS, def.name + ": Conv2D needs a filter");
      if (T == DT_UINT8) {
        // (the quantized op reads the activation arguments and leaves the clamp to the output
        // range the converter chose, mace/ops/conv_2d.cc:193-200)
        auto op = std::make_shared<ops::Conv2dOpQuant>(strides, pad, pads, dil);
        *out = Make(def.name, [op, x, f, b, y](OpContext *c) { return op->Run(c, x, f, b, y); });
      } else {
        ActivationType act = NOOP;
        float limit = 0.f;
        MaceStatus ast = ParseActivation(def, &act, &limit);
        if (ast != MaceStatus::MACE_SUCCESS) return ast;
        auto op = std::make_shared<ops::Conv2dOpFloat>(registry_, strides, pad, pads, dil, act, limit);
        *out = Make(def.name, [op, x, f, b, y](OpContext *c) { return op->Run(c, x, f, b, y); });
      }
    } else if (type == "MatMul") {
      const bool ta = GetIntArg(def, "transpose_a", 0) != 0, tb = GetIntArg(def, "transpose_b", 0) != 0;
      Tensor *a = in(0), *b = in(1), *bias = in(2), *y = outt(0);
      if (!b) return Fail(MaceStatus::MACE_INVALID_ARGS, def.name + ": MatMul needs two inputs");
      if (T == DT_UINT8) {
        auto op = std::make_shared<ops::MatMulOpQuant>(ta, tb, y->dtype());
        *out = Make(def.name, [op, a, b, y](OpContext *c) { return op->Run(c, a, b, y); });
      } else {
        auto op = std::make_shared<ops::MatMulOpFloat>(registry_, ta, tb);
        *out = Make(def.name, [op, a, b, bias, y](OpContext *c) { return op->Run(c, a, b, bias, y); });
      }
    } else if (type == "FullyConnected") {
      Tensor *x = in(0), *w = in(1), *b = in(2), *y = outt(0);
      if (!w) return Fail(MaceStatus::MACE_INVALID_ARGS, def.name + ": FullyConnected needs a weight");
      if (T == DT_UINT8) {
        auto op = std::make_shared<ops::FullyConnectedOp<uint8_t>>(registry_);
        *out = Make(def.name, [op, x, w, b, y](OpContext *c) { return op->Run(c, x, w, b, y); });
      } else {
        // FullyConnectedOpBase reads "activation" / "max_limit" (mace/ops/fully_connected.cc:40-47)
        ActivationType act = NOOP;
        float limit = 0.f;
        MaceStatus ast = ParseActivation(def, &act, &limit);
        if (ast != MaceStatus::MACE_SUCCESS) return ast;
        auto op = std::make_shared<ops::FullyConnectedOp<float>>(registry_, act, limit);
        *out = Make(def.name, [op, x, w, b, y](OpContext *c) { return op->Run(c, x, w, b, y); });
      }
    } else {
      return Fail(MaceStatus::MACE_UNSUPPORTED,
                  def.name + ": op type " + type + " is not one this library computes");
    }
    if (!outt(0)) return Fail(MaceStatus::MACE_INVALID_ARGS, def.name + ": no output tensor");
    return MaceStatus::MACE_SUCCESS;
  }

  OpDelegatorRegistry *registry_;
  mace_hip_ctx *ctx_;
  OpContext context_;
  std::string error_;
  void *weights_ = nullptr, *activations_ = nullptr;
  std::map<std::string, Tensor> tensors_;
  std::vector<View> views_;
  std::vector<std::unique_ptr<Op>> ops_;
  std::map<std::string, OpCreator> custom_ops_;
  mace_hip_graph *graph_ = nullptr;
};

}  // namespace net
}  // namespace mace_hip

#endif  // MACE_HIP_NET_H_
