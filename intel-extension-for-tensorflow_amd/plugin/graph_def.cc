#include "graph_def.h"

#include <algorithm>

namespace itex_amd {
namespace graph {
namespace {

struct Reader {
  const uint8_t* p;
  const uint8_t* end;
  bool ok = true;

  bool done() const { return p >= end || !ok; }
  uint64_t Varint() {
    uint64_t v = 0;
    for (int shift = 0; shift < 64; shift += 7) {
      if (p >= end) { ok = false; return 0; }
      const uint8_t b = *p++;
      v |= static_cast<uint64_t>(b & 0x7f) << shift;
      if (!(b & 0x80)) return v;
    }
    ok = false;
    return 0;
  }
  // the payload of a length-delimited field
  std::pair<const uint8_t*, size_t> Bytes() {
    const uint64_t n = Varint();
    if (!ok || n > static_cast<uint64_t>(end - p)) { ok = false; return {p, 0}; }
    const uint8_t* b = p;
    p += n;
    return {b, static_cast<size_t>(n)};
  }
  // skips one field of the given wire type; returns false on a malformed or unsupported (group) field
  bool Skip(uint32_t wire) {
    switch (wire) {
      case 0: Varint(); break;
      case 1: if (end - p < 8) ok = false; else p += 8; break;
      case 2: Bytes(); break;
      case 5: if (end - p < 4) ok = false; else p += 4; break;
      default: ok = false;
    }
    return ok;
  }
};

void PutVarint(std::string* out, uint64_t v) {
  while (v >= 0x80) {
    out->push_back(static_cast<char>((v & 0x7f) | 0x80));
    v >>= 7;
  }
  out->push_back(static_cast<char>(v));
}

void PutBytes(std::string* out, uint32_t field, const std::string& payload) {
  PutVarint(out, (field << 3) | 2);
  PutVarint(out, payload.size());
  out->append(payload);
}

std::string Str(std::pair<const uint8_t*, size_t> b) { return std::string(reinterpret_cast<const char*>(b.first), b.second); }

bool ParseNode(const uint8_t* data, size_t len, Node* n) {
  Reader r{data, data + len};
  while (!r.done()) {
    const uint8_t* field_start = r.p;
    const uint64_t tag = r.Varint();
    if (!r.ok) return false;
    const uint32_t field = static_cast<uint32_t>(tag >> 3), wire = static_cast<uint32_t>(tag & 7);
    if (wire == 2 && field >= 1 && field <= 5) {
      const auto b = r.Bytes();
      if (!r.ok) return false;
      if (field == 1) n->name = Str(b);
      else if (field == 2) n->op = Str(b);
      else if (field == 3) n->inputs.push_back(Str(b));
      else if (field == 4) n->device = Str(b);
      else {  // one map entry: key = 1, value = 2
        Reader e{b.first, b.first + b.second};
        Attr a;
        while (!e.done()) {
          const uint64_t t = e.Varint();
          if (!e.ok) return false;
          if ((t & 7) == 2 && (t >> 3) == 1) a.key = Str(e.Bytes());
          else if ((t & 7) == 2 && (t >> 3) == 2) a.value = Str(e.Bytes());
          else if (!e.Skip(static_cast<uint32_t>(t & 7))) return false;
        }
        if (!e.ok) return false;
        n->attrs.push_back(std::move(a));
      }
    } else {
      if (!r.Skip(wire)) return false;
      n->other.append(reinterpret_cast<const char*>(field_start), r.p - field_start);
    }
  }
  return r.ok;
}

// first occurrence of a field in a serialized AttrValue
bool FindField(const std::string& value, uint32_t want_field, uint32_t want_wire, Reader* at) {
  Reader r{reinterpret_cast<const uint8_t*>(value.data()), reinterpret_cast<const uint8_t*>(value.data()) + value.size()};
  while (!r.done()) {
    const uint64_t tag = r.Varint();
    if (!r.ok) return false;
    if ((tag >> 3) == want_field && (tag & 7) == want_wire) { *at = r; return true; }
    if (!r.Skip(static_cast<uint32_t>(tag & 7))) return false;
  }
  return false;
}

}  // namespace

const std::string* Node::FindAttr(const std::string& key) const {
  for (const Attr& a : attrs)
    if (a.key == key) return &a.value;
  return nullptr;
}

void Node::SetAttr(const std::string& key, std::string value) {
  for (Attr& a : attrs)
    if (a.key == key) { a.value = std::move(value); return; }
  attrs.push_back(Attr{key, std::move(value)});
}

bool Parse(const void* data, size_t len, Graph* g) {
  Reader r{static_cast<const uint8_t*>(data), static_cast<const uint8_t*>(data) + len};
  while (!r.done()) {
    const uint8_t* field_start = r.p;
    const uint64_t tag = r.Varint();
    if (!r.ok) return false;
    if ((tag >> 3) == 1 && (tag & 7) == 2) {
      const auto b = r.Bytes();
      if (!r.ok) return false;
      g->nodes.emplace_back();
      if (!ParseNode(b.first, b.second, &g->nodes.back())) return false;
    } else {
      if (!r.Skip(static_cast<uint32_t>(tag & 7))) return false;
      g->other.append(reinterpret_cast<const char*>(field_start), r.p - field_start);
    }
  }
  return r.ok;
}

std::string Serialize(const Graph& g) {
  std::string out;
  for (const Node& n : g.nodes) {
    std::string body;
    PutBytes(&body, 1, n.name);
    PutBytes(&body, 2, n.op);
    for (const std::string& in : n.inputs) PutBytes(&body, 3, in);
    if (!n.device.empty()) PutBytes(&body, 4, n.device);
    for (const Attr& a : n.attrs) {
      std::string entry;
      PutBytes(&entry, 1, a.key);
      PutBytes(&entry, 2, a.value);
      PutBytes(&body, 5, entry);
    }
    body.append(n.other);
    PutBytes(&out, 1, body);
  }
  out.append(g.other);
  return out;
}

bool AttrString(const std::string& value, std::string* s) {
  Reader at{nullptr, nullptr};
  if (!FindField(value, 2, 2, &at)) return false;
  *s = Str(at.Bytes());
  return at.ok;
}

bool AttrBool(const std::string& value, bool* b) {
  Reader at{nullptr, nullptr};
  if (!FindField(value, 5, 0, &at)) { *b = false; return value.empty(); }  // proto3 omits a false
  *b = at.Varint() != 0;
  return at.ok;
}

bool AttrType(const std::string& value, int* t) {
  Reader at{nullptr, nullptr};
  if (!FindField(value, 6, 0, &at)) return false;
  *t = static_cast<int>(at.Varint());
  return at.ok;
}

bool AttrInt(const std::string& value, int* i) {
  Reader at{nullptr, nullptr};
  if (!FindField(value, 3, 0, &at)) { *i = 0; return value.empty(); }  // proto3 omits a zero
  *i = static_cast<int>(static_cast<int64_t>(at.Varint()));
  return at.ok;
}

bool AttrIntTensor(const std::string& value, int* rank, std::vector<int64_t>* elements) {
  Reader at{nullptr, nullptr};
  if (!FindField(value, 8, 2, &at)) return false;
  const auto body = at.Bytes();
  if (!at.ok) return false;
  Reader r{body.first, body.first + body.second};
  int dtype = 0;
  std::vector<int64_t> dims, vals;
  std::string content;
  while (!r.done()) {
    const uint64_t tag = r.Varint();
    if (!r.ok) return false;
    const uint32_t field = static_cast<uint32_t>(tag >> 3), wire = static_cast<uint32_t>(tag & 7);
    if (field == 1 && wire == 0) {
      dtype = static_cast<int>(r.Varint());
    } else if (field == 2 && wire == 2) {  // TensorShapeProto: repeated Dim dim = 2 { int64 size = 1 }
      const auto sb = r.Bytes();
      Reader sr{sb.first, sb.first + sb.second};
      while (!sr.done()) {
        const uint64_t st = sr.Varint();
        if (!sr.ok) return false;
        if ((st >> 3) == 2 && (st & 7) == 2) {
          const auto db = sr.Bytes();
          Reader dr{db.first, db.first + db.second};
          int64_t size = 0;
          while (!dr.done()) {
            const uint64_t dt = dr.Varint();
            if (!dr.ok) return false;
            if ((dt >> 3) == 1 && (dt & 7) == 0) size = static_cast<int64_t>(dr.Varint());
            else if (!dr.Skip(static_cast<uint32_t>(dt & 7))) return false;
          }
          dims.push_back(size);
        } else if (!sr.Skip(static_cast<uint32_t>(st & 7))) {
          return false;
        }
      }
    } else if (field == 4 && wire == 2) {
      content = Str(r.Bytes());
    } else if ((field == 7 || field == 10) && wire == 0) {
      vals.push_back(static_cast<int64_t>(r.Varint()));
    } else if ((field == 7 || field == 10) && wire == 2) {  // packed
      const auto pb = r.Bytes();
      Reader pr{pb.first, pb.first + pb.second};
      while (!pr.done()) vals.push_back(static_cast<int64_t>(pr.Varint()));
      if (!pr.ok) return false;
    } else if (!r.Skip(wire)) {
      return false;
    }
  }
  if (!r.ok || (dtype != 3 && dtype != 9)) return false;  // DT_INT32, DT_INT64
  int64_t count = 1;
  for (int64_t d : dims) {
    if (d < 0 || d > (1 << 20)) return false;
    count *= d;
    if (count > (1 << 20)) return false;
  }
  elements->clear();
  if (!content.empty()) {
    const size_t esz = dtype == 3 ? 4 : 8;
    if (content.size() != esz * static_cast<size_t>(count)) return false;
    for (int64_t i = 0; i < count; ++i) {
      uint64_t raw = 0;
      for (size_t b = 0; b < esz; ++b) raw |= static_cast<uint64_t>(static_cast<uint8_t>(content[i * esz + b])) << (8 * b);
      elements->push_back(dtype == 3 ? static_cast<int64_t>(static_cast<int32_t>(raw)) : static_cast<int64_t>(raw));
    }
  } else {
    if (dtype == 3) for (int64_t& v : vals) v = static_cast<int64_t>(static_cast<int32_t>(v));  // negative int32 arrive sign-extended to 64 bits
    for (int64_t i = 0; i < count; ++i)  // fewer values than elements: the last one repeats (tensor.proto)
      elements->push_back(vals.empty() ? 0 : vals[std::min<size_t>(i, vals.size() - 1)]);
  }
  *rank = static_cast<int>(dims.size());
  return true;
}

// AttrValue.list = 1 (ListValue: s = 2, type = 6; repeated enums arrive packed or one by one)
bool AttrTypeList(const std::string& value, std::vector<int>* types) {
  types->clear();
  if (value.empty()) return true;
  Reader at{nullptr, nullptr};
  if (!FindField(value, 1, 2, &at)) return false;
  const auto body = at.Bytes();
  if (!at.ok) return false;
  Reader r{body.first, body.first + body.second};
  while (!r.done()) {
    const uint64_t tag = r.Varint();
    if (!r.ok) return false;
    if ((tag >> 3) == 6 && (tag & 7) == 2) {
      const auto packed = r.Bytes();
      if (!r.ok) return false;
      Reader e{packed.first, packed.first + packed.second};
      while (!e.done()) {
        types->push_back(static_cast<int>(e.Varint()));
        if (!e.ok) return false;
      }
    } else if ((tag >> 3) == 6 && (tag & 7) == 0) {
      types->push_back(static_cast<int>(r.Varint()));
      if (!r.ok) return false;
    } else if (!r.Skip(static_cast<uint32_t>(tag & 7))) {
      return false;
    }
  }
  return true;
}

bool AttrStringList(const std::string& value, std::vector<std::string>* strings) {
  strings->clear();
  if (value.empty()) return true;
  Reader at{nullptr, nullptr};
  if (!FindField(value, 1, 2, &at)) return false;
  const auto body = at.Bytes();
  if (!at.ok) return false;
  Reader r{body.first, body.first + body.second};
  while (!r.done()) {
    const uint64_t tag = r.Varint();
    if (!r.ok) return false;
    if ((tag >> 3) == 2 && (tag & 7) == 2) {
      strings->push_back(Str(r.Bytes()));
      if (!r.ok) return false;
    } else if (!r.Skip(static_cast<uint32_t>(tag & 7))) {
      return false;
    }
  }
  return true;
}

std::string MakeAttrTypeList(const std::vector<int>& types) {
  std::string packed, list, v;
  for (int t : types) PutVarint(&packed, static_cast<uint64_t>(t));
  if (!types.empty()) PutBytes(&list, 6, packed);
  PutBytes(&v, 1, list);
  return v;
}

std::string MakeAttrBool(bool b) {
  std::string v;
  PutVarint(&v, (5u << 3) | 0);
  PutVarint(&v, b ? 1 : 0);
  return v;
}

std::string MakeAttrString(const std::string& s) {
  std::string v;
  PutBytes(&v, 2, s);
  return v;
}

std::string MakeAttrType(int t) {
  std::string v;
  PutVarint(&v, (6u << 3) | 0);
  PutVarint(&v, static_cast<uint64_t>(t));
  return v;
}

}  // namespace graph
}  // namespace itex_amd
