// A small reader / writer for the serialized GraphDef a graph-optimizer plugin receives: just enough of the
// protobuf wire format for GraphDef { repeated NodeDef node = 1; ... } and NodeDef { name = 1; op = 2;
// repeated input = 3; device = 4; map<string, AttrValue> attr = 5; ... } (tensorflow/core/framework/graph.proto,
// node_def.proto, attr_value.proto).  Everything the rewrite does not touch is carried through as raw bytes.
#ifndef ITEX_AMD_GRAPH_DEF_H_
#define ITEX_AMD_GRAPH_DEF_H_

#include <cstdint>
#include <string>
#include <utility>
#include <vector>

namespace itex_amd {
namespace graph {

struct Attr {
  std::string key;
  std::string value;  // serialized AttrValue
};

struct Node {
  std::string name, op, device;
  std::vector<std::string> inputs;
  std::vector<Attr> attrs;
  std::string other;  // fields other than 1..5, re-emitted verbatim

  const std::string* FindAttr(const std::string& key) const;
  void SetAttr(const std::string& key, std::string value);
};

struct Graph {
  std::vector<Node> nodes;
  std::string other;  // library, versions, debug info: re-emitted verbatim after the nodes
};

bool Parse(const void* data, size_t len, Graph* g);
std::string Serialize(const Graph& g);

// AttrValue accessors for the kinds the rewrite reads and writes (attr_value.proto: s = 2, b = 5, type = 6, tensor = 8)
bool AttrString(const std::string& value, std::string* s);
bool AttrBool(const std::string& value, bool* b);
bool AttrType(const std::string& value, int* t);
bool AttrInt(const std::string& value, int* i);  // i = 3
// The integer tensor of a Const node's "value" attribute (AttrValue.tensor = 8; tensor.proto: dtype = 1,
// tensor_shape = 2, tensor_content = 4, int_val = 7, int64_val = 10), int32 or int64: its rank and elements.
bool AttrIntTensor(const std::string& value, int* rank, std::vector<int64_t>* elements);
// list(type) and list(string) attributes (AttrValue.list = 1; ListValue: s = 2, type = 6)
bool AttrTypeList(const std::string& value, std::vector<int>* types);
bool AttrStringList(const std::string& value, std::vector<std::string>* strings);
std::string MakeAttrTypeList(const std::vector<int>& types);
std::string MakeAttrBool(bool b);
std::string MakeAttrString(const std::string& s);
std::string MakeAttrType(int t);

}  // namespace graph
}  // namespace itex_amd
#endif  // ITEX_AMD_GRAPH_DEF_H_
