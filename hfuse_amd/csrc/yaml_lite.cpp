#include "yaml_lite.h"


namespace hfuse {
namespace {

struct Line {
  int indent;
  std::string text;  // without indent, comments and trailing blanks
  int no;
};

std::string rstrip(std::string s) {
  while (!s.empty() && (s.back() == ' ' || s.back() == '\t' || s.back() == '\r')) s.pop_back();
  return s;
}

std::string strip_comment(const std::string &s) {
  bool sq = false, dq = false;
  for (size_t i = 0; i < s.size(); i++) {
    char c = s[i];
    if (c == '\'' && !dq) sq = !sq;
    if (c == '"' && !sq) dq = !dq;
    if (c == '#' && !sq && !dq && (i == 0 || s[i - 1] == ' ' || s[i - 1] == '\t')) return s.substr(0, i);
  }
  return s;
}

std::string unquote(std::string s) {
  s = rstrip(s);
  size_t b = 0;
  while (b < s.size() && s[b] == ' ') b++;
  s = s.substr(b);
  if (s.size() >= 2 && ((s.front() == '"' && s.back() == '"') || (s.front() == '\'' && s.back() == '\'')))
    return s.substr(1, s.size() - 2);
  return s;
}

// Position of the ':' that ends a mapping key ("key: v" or "key:"), or npos.
size_t key_colon(const std::string &t) {
  bool sq = false, dq = false;
  for (size_t i = 0; i < t.size(); i++) {
    char c = t[i];
    if (c == '\'' && !dq) sq = !sq;
    if (c == '"' && !sq) dq = !dq;
    if (c == ':' && !sq && !dq && (i + 1 == t.size() || t[i + 1] == ' ')) return i;
  }
  return std::string::npos;
}

bool is_seq_item(const std::string &t) { return t == "-" || (t.size() >= 2 && t[0] == '-' && t[1] == ' '); }

struct Parser {
  std::vector<Line> lines;
  size_t pos = 0;
  std::string err;

  bool fail(int no, const std::string &why) {
    err = "line " + std::to_string(no) + ": " + why;
    return false;
  }

  // The two documents nest four levels deep; a bound keeps a crafted file from exhausting
  // the stack through the mutual recursion of blocks, sequences and maps.
  static constexpr int kMaxDepth = 32;
  int depth = 0;

  bool parse_block(int indent, YamlNode &out) {
    if (pos >= lines.size()) return true;
    if (depth >= kMaxDepth) return fail(lines[pos].no, "nesting deeper than 32 levels");
    depth++;
    const bool ok = is_seq_item(lines[pos].text) ? parse_seq(indent, out) : parse_map(indent, out);
    depth--;
    return ok;
  }

  bool parse_seq(int indent, YamlNode &out) {
    out.kind = YamlNode::Seq;
    out.line = lines[pos].no;
    while (pos < lines.size() && lines[pos].indent == indent && is_seq_item(lines[pos].text)) {
      Line &ln = lines[pos];
      std::string rest = ln.text.size() > 1 ? ln.text.substr(1) : "";
      size_t skip = 0;
      while (skip < rest.size() && rest[skip] == ' ') skip++;
      rest = rest.substr(skip);
      YamlNode item;
      item.line = ln.no;
      if (rest.empty()) {
        pos++;
        if (pos < lines.size() && lines[pos].indent > indent) {
          if (!parse_block(lines[pos].indent, item)) return false;
        }
      } else if (key_colon(rest) != std::string::npos) {
        // "- key: value": the map starts on the dash line, at the column of `key`.
        int child = indent + 1 + (int)skip;
        ln.indent = child;
        ln.text = rest;
        if (!parse_map(child, item)) return false;
      } else {
        item.kind = YamlNode::Scalar;
        item.scalar = unquote(rest);
        pos++;
      }
      out.seq.push_back(std::move(item));
    }
    if (pos < lines.size() && lines[pos].indent > indent) return fail(lines[pos].no, "unexpected indentation");
    return true;
  }

  bool parse_map(int indent, YamlNode &out) {
    out.kind = YamlNode::Map;
    out.line = lines[pos].no;
    while (pos < lines.size() && lines[pos].indent == indent && !is_seq_item(lines[pos].text)) {
      const Line ln = lines[pos];
      size_t c = key_colon(ln.text);
      if (c == std::string::npos) return fail(ln.no, "expected 'key: value'");
      std::string key = unquote(ln.text.substr(0, c));
      std::string val = ln.text.substr(c + 1);
      if (out.get(key)) return fail(ln.no, "duplicate key '" + key + "'");
      YamlNode child;
      child.line = ln.no;
      pos++;
      if (unquote(val).empty()) {
        if (pos < lines.size() && lines[pos].indent > indent) {
          if (!parse_block(lines[pos].indent, child)) return false;
        } else if (pos < lines.size() && lines[pos].indent == indent && is_seq_item(lines[pos].text)) {
          if (!parse_seq(indent, child)) return false;  // sequence at the key's own column
        }
      } else {
        const std::string v = unquote(val);
        if (v.size() >= 2 && v.front() == '[' && v.back() == ']' && val.find('"') == std::string::npos &&
            val.find('\'') == std::string::npos) {
          // a flow sequence of plain scalars on the key's line: `Blocks: [768, 768]`
          child.kind = YamlNode::Seq;
          const std::string inner = v.substr(1, v.size() - 2);
          if (inner.find('[') != std::string::npos || inner.find('{') != std::string::npos)
            return fail(ln.no, "nested flow collections are not read");
          for (size_t a = 0; a <= inner.size();) {
            size_t e = inner.find(',', a);
            if (e == std::string::npos) e = inner.size();
            YamlNode item;
            item.kind = YamlNode::Scalar;
            item.line = ln.no;
            item.scalar = unquote(inner.substr(a, e - a));
            if (item.scalar.empty()) {
              if (e == inner.size() && child.seq.empty() && unquote(inner).empty()) break;  // `[]`
              return fail(ln.no, "empty item in a flow sequence");
            }
            child.seq.push_back(std::move(item));
            a = e + 1;
          }
        } else {
          child.kind = YamlNode::Scalar;
          child.scalar = v;
        }
        if (pos < lines.size() && lines[pos].indent > indent)
          return fail(lines[pos].no, "unexpected indentation after scalar value");
      }
      out.map.emplace_back(std::move(key), std::move(child));
    }
    return true;
  }
};

}  // namespace

bool yaml_parse(const std::string &text, YamlNode &root, std::string &err) {
  Parser p;
  // Lines are cut by hand: a stream would swallow an allocation failure inside getline and
  // merely look exhausted, which turns "out of memory" into a parse error about a short file.
  std::string raw;
  int no = 0;
  for (size_t at = 0; at < text.size();) {
    const size_t nl = text.find('\n', at);
    const size_t end = nl == std::string::npos ? text.size() : nl;
    raw.assign(text, at, end - at);
    at = end + 1;
    no++;
    if (raw.find('\t') != std::string::npos && raw.find_first_not_of(" \t") != std::string::npos &&
        raw.substr(0, raw.find_first_not_of(" \t")).find('\t') != std::string::npos) {
      err = "line " + std::to_string(no) + ": tab in indentation";
      return false;
    }
    std::string s = rstrip(strip_comment(raw));
    size_t b = s.find_first_not_of(' ');
    if (b == std::string::npos) continue;
    if (s.compare(b, 3, "---") == 0 && rstrip(s.substr(b)) == "---") continue;
    p.lines.push_back({(int)b, s.substr(b), no});
  }
  root = YamlNode();
  if (p.lines.empty()) return true;
  if (!p.parse_block(p.lines[0].indent, root)) {
    err = p.err;
    return false;
  }
  if (p.pos != p.lines.size()) {
    err = "line " + std::to_string(p.lines[p.pos].no) + ": inconsistent indentation";
    return false;
  }
  return true;
}

}  // namespace hfuse
