#include "graph_def.h"

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
