#include "worker/onnx_wire.h"

#include <cstring>
#include <stdexcept>

namespace fluidml {
namespace onnx_wire {
namespace {

// A cursor over one length-delimited message.
class Reader {
 public:
  Reader(const uint8_t *begin, const uint8_t *end) : p_(begin), end_(end) {}
  bool Done() const { return p_ >= end_; }

  uint64_t Varint() {
    uint64_t value = 0;
    for (int shift = 0; shift < 64; shift += 7) {
      if (p_ >= end_) throw std::runtime_error("onnx: truncated varint");
      const uint8_t byte = *p_++;
      value |= static_cast<uint64_t>(byte & 0x7f) << shift;
      if (!(byte & 0x80)) return value;
    }
    throw std::runtime_error("onnx: varint longer than 10 bytes");
  }
  uint32_t Fixed32() {
    if (end_ - p_ < 4) throw std::runtime_error("onnx: truncated fixed32");
    uint32_t v;
    std::memcpy(&v, p_, 4);
    p_ += 4;
    return v;
  }
  uint64_t Fixed64() {
    if (end_ - p_ < 8) throw std::runtime_error("onnx: truncated fixed64");
    uint64_t v;
    std::memcpy(&v, p_, 8);
    p_ += 8;
    return v;
  }
  Reader Sub() {
    const uint64_t len = Varint();
    if (len > static_cast<uint64_t>(end_ - p_)) throw std::runtime_error("onnx: truncated length-delimited field");
    Reader sub(p_, p_ + len);
    p_ += len;
    return sub;
  }
  std::string Bytes() {
    Reader sub = Sub();
    return std::string(reinterpret_cast<const char *>(sub.p_), static_cast<size_t>(sub.end_ - sub.p_));
  }
  // reads a field key; returns false at the end of the message
  bool Key(uint32_t *field, uint32_t *wire) {
    if (Done()) return false;
    const uint64_t key = Varint();
    *field = static_cast<uint32_t>(key >> 3);
    *wire = static_cast<uint32_t>(key & 7);
    return true;
  }
  void Skip(uint32_t wire) {
    switch (wire) {
      case 0: Varint(); break;
      case 1: Fixed64(); break;
      case 2: Sub(); break;
      case 5: Fixed32(); break;
      default: throw std::runtime_error("onnx: unsupported wire type " + std::to_string(wire));
    }
  }
  size_t Remaining() const { return static_cast<size_t>(end_ - p_); }

 private:
  const uint8_t *p_;
  const uint8_t *end_;
};

float AsFloat(uint32_t bits) {
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}
double AsDouble(uint64_t bits) {
  double d;
  std::memcpy(&d, &bits, 8);
  return d;
}

// repeated scalar fields arrive packed (wire 2) or one element per key
template <typename T, typename F>
void Repeated(Reader &r, uint32_t wire, uint32_t scalar_wire, std::vector<T> *out, F read_one) {
  if (wire == 2) {
    Reader sub = r.Sub();
    while (!sub.Done()) out->push_back(read_one(sub));
  } else if (wire == scalar_wire) {
    out->push_back(read_one(r));
  } else {
    throw std::runtime_error("onnx: unexpected wire type for a repeated scalar");
  }
}

TensorData ParseTensor(Reader r) {
  TensorData t;
  uint32_t field, wire;
  while (r.Key(&field, &wire)) {
    switch (field) {
      case 1: Repeated(r, wire, 0, &t.dims, [](Reader &x) { return static_cast<int64_t>(x.Varint()); }); break;
      case 2: t.data_type = static_cast<int32_t>(r.Varint()); break;
      case 4: Repeated(r, wire, 5, &t.float_data, [](Reader &x) { return AsFloat(x.Fixed32()); }); break;
      case 5: Repeated(r, wire, 0, &t.int32_data, [](Reader &x) { return static_cast<int32_t>(x.Varint()); }); break;
      case 7: Repeated(r, wire, 0, &t.int64_data, [](Reader &x) { return static_cast<int64_t>(x.Varint()); }); break;
      case 8: t.name = r.Bytes(); break;
      case 9:
        t.raw_data = r.Bytes();
        t.has_raw_data = true;
        break;
      case 10: Repeated(r, wire, 1, &t.double_data, [](Reader &x) { return AsDouble(x.Fixed64()); }); break;
      default: r.Skip(wire);
    }
  }
  return t;
}

AttributeData ParseAttribute(Reader r) {
  AttributeData a;
  uint32_t field, wire;
  while (r.Key(&field, &wire)) {
    switch (field) {
      case 1: a.name = r.Bytes(); break;
      case 2: a.f = AsFloat(r.Fixed32()); break;
      case 3: a.i = static_cast<int64_t>(r.Varint()); break;
      case 4: a.s = r.Bytes(); break;
      case 5: a.t = ParseTensor(r.Sub()); break;
      case 7: Repeated(r, wire, 5, &a.floats, [](Reader &x) { return AsFloat(x.Fixed32()); }); break;
      case 8: Repeated(r, wire, 0, &a.ints, [](Reader &x) { return static_cast<int64_t>(x.Varint()); }); break;
      case 20: a.type = static_cast<int32_t>(r.Varint()); break;
      default: r.Skip(wire);
    }
  }
  return a;
}

NodeData ParseNode(Reader r) {
  NodeData n;
  uint32_t field, wire;
  while (r.Key(&field, &wire)) {
    switch (field) {
      case 1: n.input.push_back(r.Bytes()); break;
      case 2: n.output.push_back(r.Bytes()); break;
      case 3: n.name = r.Bytes(); break;
      case 4: n.op_type = r.Bytes(); break;
      case 5: n.attribute.push_back(ParseAttribute(r.Sub())); break;
      default: r.Skip(wire);
    }
  }
  return n;
}

void ParseShape(Reader r, ValueInfoData *v) {
  v->has_shape = true;
  uint32_t field, wire;
  while (r.Key(&field, &wire)) {
    if (field == 1 && wire == 2) {
      Reader dim = r.Sub();
      int64_t value = 0;
      uint32_t f2, w2;
      while (dim.Key(&f2, &w2)) {
        if (f2 == 1 && w2 == 0) value = static_cast<int64_t>(dim.Varint());
        else dim.Skip(w2);
      }
      v->dims.push_back(value);
    } else {
      r.Skip(wire);
    }
  }
}

ValueInfoData ParseValueInfo(Reader r) {
  ValueInfoData v;
  uint32_t field, wire;
  while (r.Key(&field, &wire)) {
    if (field == 1 && wire == 2) {
      v.name = r.Bytes();
    } else if (field == 2 && wire == 2) {  // TypeProto
      Reader type = r.Sub();
      uint32_t f2, w2;
      while (type.Key(&f2, &w2)) {
        if (f2 == 1 && w2 == 2) {  // tensor_type
          Reader tensor = type.Sub();
          uint32_t f3, w3;
          while (tensor.Key(&f3, &w3)) {
            if (f3 == 1 && w3 == 0) v.elem_type = static_cast<int32_t>(tensor.Varint());
            else if (f3 == 2 && w3 == 2) ParseShape(tensor.Sub(), &v);
            else tensor.Skip(w3);
          }
        } else {
          type.Skip(w2);
        }
      }
    } else {
      r.Skip(wire);
    }
  }
  return v;
}

GraphData ParseGraph(Reader r) {
  GraphData g;
  uint32_t field, wire;
  while (r.Key(&field, &wire)) {
    if (wire != 2) {
      r.Skip(wire);
      continue;
    }
    switch (field) {
      case 1: g.node.push_back(ParseNode(r.Sub())); break;
      case 2: g.name = r.Bytes(); break;
      case 5: g.initializer.push_back(ParseTensor(r.Sub())); break;
      case 11: g.input.push_back(ParseValueInfo(r.Sub())); break;
      case 12: g.output.push_back(ParseValueInfo(r.Sub())); break;
      case 13: g.value_info.push_back(ParseValueInfo(r.Sub())); break;
      default: r.Skip(wire);
    }
  }
  return g;
}

}  // namespace

ModelData ParseModel(const std::string &bytes) {
  const uint8_t *begin = reinterpret_cast<const uint8_t *>(bytes.data());
  Reader r(begin, begin + bytes.size());
  ModelData m;
  bool saw_graph = false;
  uint32_t field, wire;
  while (r.Key(&field, &wire)) {
    if (field == 1 && wire == 0) {
      m.ir_version = static_cast<int64_t>(r.Varint());
    } else if (field == 7 && wire == 2) {
      m.graph = ParseGraph(r.Sub());
      saw_graph = true;
    } else {
      r.Skip(wire);
    }
  }
  if (!saw_graph) throw std::runtime_error("onnx: ModelProto has no graph");
  return m;
}

}  // namespace onnx_wire
}  // namespace fluidml
