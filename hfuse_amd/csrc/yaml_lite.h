// Minimal block-style YAML reader: nested maps, sequences and plain/quoted
// scalars -- the subset the fusion list and kernel table are written in.
#pragma once
#include <memory>
#include <string>
#include <utility>
#include <vector>

namespace hfuse {

struct YamlNode {
  enum Kind { Null, Scalar, Map, Seq } kind = Null;
  std::string scalar;
  std::vector<std::pair<std::string, YamlNode>> map;  // insertion order kept
  std::vector<YamlNode> seq;
  int line = 0;

  const YamlNode *get(const std::string &key) const {
    for (auto &kv : map)
      if (kv.first == key) return &kv.second;
    return nullptr;
  }
};

// Parses `text`; on failure returns false and fills `err` with "line N: why".
bool yaml_parse(const std::string &text, YamlNode &root, std::string &err);

}  // namespace hfuse
