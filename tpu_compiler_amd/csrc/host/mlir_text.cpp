// Hand-written reader for the generic textual form of a TPU-dialect function; see
// tpuhip/mlir_text.hpp for what is covered and which reference code it stands in for.
#include "tpuhip/mlir_text.hpp"

#include <cctype>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <sstream>
#include <stdexcept>

namespace tpuhip {

const MlirAttr *MlirAttr::get(const std::string &key) const {
  for (auto &f : fields)
    if (f.first == key) return &f.second;
  return nullptr;
}

namespace {

class Reader {
public:
  explicit Reader(const std::string &text) : s(text) {}

  MlirFunc module() {
    for (;;) {
      ws();
      if (eof()) fail("no func found");
      if (word("module")) {
        ws();
        if (peek() == '@') symbol();
        ws();
        if (word("attributes")) { ws(); expect('{'); dict(); }
        ws();
        expect('{');
        continue;
      }
      if (word("func.func") || word("builtin.func") || word("func")) return func();
      fail(std::string("unexpected '") + peek() + "' at top level");
    }
  }

private:
  const std::string &s;
  size_t i = 0;
  int line = 1;
  int nesting = 0;   // of attribute values (bounded: the reader recurses)

  [[noreturn]] void fail(const std::string &what) const {
    throw std::runtime_error("mlir:" + std::to_string(line) + ": " + what);
  }
  bool eof() const { return i >= s.size(); }
  char peek() const { return i < s.size() ? s[i] : '\0'; }
  char peek(size_t k) const { return i + k < s.size() ? s[i + k] : '\0'; }
  void bump() {
    if (s[i] == '\n') ++line;
    ++i;
  }
  void ws() {
    for (;;) {
      while (!eof() && std::isspace((unsigned char)s[i])) bump();
      if (peek() == '/' && peek(1) == '/') {
        while (!eof() && s[i] != '\n') ++i;
        continue;
      }
      return;
    }
  }
  bool eat(char c) {
    ws();
    if (peek() != c) return false;
    bump();
    return true;
  }
  void expect(char c) {
    if (!eat(c)) fail(std::string("expected '") + c + "', found '" + (eof() ? std::string("end of file") : std::string(1, peek())) + "'");
  }
  static bool ident_char(char c) { return std::isalnum((unsigned char)c) || c == '_' || c == '.' || c == '$'; }
  // consumes `w` if it is the next token (not a prefix of a longer identifier)
  bool word(const char *w) {
    ws();
    const size_t n = std::strlen(w);
    if (s.compare(i, n, w) != 0) return false;
    if (ident_char(peek(n))) return false;
    i += n;
    return true;
  }
  std::string ident() {
    ws();
    size_t b = i;
    while (!eof() && ident_char(s[i])) ++i;
    if (b == i) fail("identifier expected");
    return s.substr(b, i - b);
  }
  std::string symbol() {
    expect('@');
    if (peek() == '"') return quoted();
    return ident();
  }
  // %name, %12, %5#1 -> text without '%'
  std::string ssa() {
    expect('%');
    size_t b = i;
    while (!eof() && (ident_char(s[i]) || s[i] == '-' || s[i] == '#')) ++i;
    if (b == i) fail("SSA name expected after '%'");
    return s.substr(b, i - b);
  }
  std::string quoted() {
    ws();
    if (peek() != '"') fail("string expected");
    bump();
    std::string out;
    while (!eof() && s[i] != '"') {
      char c = s[i];
      if (c == '\\' && i + 1 < s.size()) {
        char d = s[i + 1];
        if (d == 'n') { out += '\n'; i += 2; }
        else if (d == 't') { out += '\t'; i += 2; }
        else if (d == '"' || d == '\\') { out += d; i += 2; }
        else if (std::isxdigit((unsigned char)d) && std::isxdigit((unsigned char)peek(2))) {
          out += (char)std::strtol(s.substr(i + 1, 2).c_str(), nullptr, 16);
          i += 3;
        } else { out += c; ++i; }
        continue;
      }
      if (c == '\n') fail("unterminated string");
      out += c;
      ++i;
    }
    if (eof()) fail("unterminated string");
    bump();
    return out;
  }
  // raw text up to a ',', ')', ']' or '}' outside any bracket or string
  std::string raw_value() {
    ws();
    size_t b = i;
    int depth = 0;
    while (!eof()) {
      char c = s[i];
      if (c == '"') { quoted(); continue; }
      if (c == '-' && peek(1) == '>') { i += 2; continue; }
      if (c == '<' || c == '(' || c == '[' || c == '{') ++depth;
      else if (c == '>' || c == ')' || c == ']' || c == '}') {
        if (depth == 0) break;
        --depth;
      } else if (c == ',' && depth == 0) break;
      bump();
    }
    size_t e = i;
    while (e > b && std::isspace((unsigned char)s[e - 1])) --e;
    if (e == b) fail("value expected");
    return s.substr(b, e - b);
  }

  MlirType type() {
    ws();
    size_t b = i;
    if (peek() == '(') {   // function or tuple-like type: keep the text only
      int depth = 0;
      do {
        if (s[i] == '(') ++depth;
        if (s[i] == ')') --depth;
        bump();
      } while (!eof() && depth > 0);
      MlirType t;
      t.text = s.substr(b, i - b);
      return t;
    }
    while (!eof() && (ident_char(s[i]) || s[i] == '!')) ++i;
    if (b == i) fail("type expected");
    const std::string head = s.substr(b, i - b);
    std::string inner;
    if (peek() == '<') {
      size_t ib = i + 1;
      int depth = 0;
      for (;;) {
        if (eof()) fail("unterminated '<' in type");
        char c = s[i];
        if (c == '-' && peek(1) == '>') { i += 2; continue; }
        if (c == '"') { quoted(); continue; }
        if (c == '<') ++depth;
        if (c == '>' && --depth == 0) { bump(); break; }
        bump();
      }
      inner = s.substr(ib, i - 1 - ib);
    }
    MlirType t;
    t.text = s.substr(b, i - b);
    if (head == "tensor" || head == "memref") {
      t.shaped = true;
      // dims up to the element type; a memref layout after a top-level ',' is ignored
      size_t p = 0;
      for (;;) {
        size_t q = p;
        while (q < inner.size() && (std::isdigit((unsigned char)inner[q]) || inner[q] == '?' || inner[q] == '*')) ++q;
        if (q > p && q < inner.size() && inner[q] == 'x') {
          const std::string d = inner.substr(p, q - p);
          if (d == "*") { t.shape.clear(); }
          else t.shape.push_back(d == "?" ? -1 : (int64_t)std::strtoll(d.c_str(), nullptr, 10));
          p = q + 1;
          continue;
        }
        break;
      }
      size_t e = p;
      int depth = 0;
      while (e < inner.size()) {
        if (inner[e] == '<') ++depth;
        if (inner[e] == '>') --depth;
        if (inner[e] == ',' && depth == 0) break;
        ++e;
      }
      t.elem = inner.substr(p, e - p);
      while (!t.elem.empty() && std::isspace((unsigned char)t.elem.back())) t.elem.pop_back();
    } else {
      t.elem = head;
    }
    return t;
  }

  std::vector<MlirType> type_list_in_parens() {
    std::vector<MlirType> out;
    expect('(');
    if (eat(')')) return out;
    do out.push_back(type()); while (eat(','));
    expect(')');
    return out;
  }

  MlirAttr dict() {   // after '{'
    MlirAttr d;
    d.kind = MlirAttr::Dict;
    if (eat('}')) return d;
    do {
      ws();
      std::string key = peek() == '"' ? quoted() : ident();
      MlirAttr v;
      if (eat('=')) v = value();
      d.fields.emplace_back(std::move(key), std::move(v));
    } while (eat(','));
    expect('}');
    return d;
  }

  struct Nest {
    Reader &r;
    explicit Nest(Reader &reader) : r(reader) {
      if (++r.nesting > 64) r.fail("attribute values nested more than 64 deep");
    }
    ~Nest() { --r.nesting; }
  };

  MlirAttr value() {
    Nest nest(*this);
    ws();
    MlirAttr a;
    const char c = peek();
    if (c == '"') {
      a.kind = MlirAttr::String;
      a.str = quoted();
      if (eat(':')) type();
      return a;
    }
    if (c == '[') {
      bump();
      a.kind = MlirAttr::Array;
      if (eat(']')) return a;
      do a.items.push_back(value()); while (eat(','));
      expect(']');
      return a;
    }
    if (c == '{') {
      bump();
      return dict();
    }
    if (std::isdigit((unsigned char)c) || ((c == '-' || c == '+') && (std::isdigit((unsigned char)peek(1)) || peek(1) == '.'))) {
      size_t b = i;
      if (c == '-' || c == '+') ++i;
      bool hex = false, real = false;
      if (peek() == '0' && (peek(1) == 'x' || peek(1) == 'X')) {
        hex = true;
        i += 2;
        while (std::isxdigit((unsigned char)peek())) ++i;
      } else {
        while (std::isdigit((unsigned char)peek())) ++i;
        if (peek() == '.') { real = true; ++i; while (std::isdigit((unsigned char)peek())) ++i; }
        if ((peek() == 'e' || peek() == 'E') &&
            (std::isdigit((unsigned char)peek(1)) || ((peek(1) == '+' || peek(1) == '-') && std::isdigit((unsigned char)peek(2))))) {
          real = true;
          i += 2;
          while (std::isdigit((unsigned char)peek())) ++i;
        }
      }
      const std::string tok = s.substr(b, i - b);
      std::string ty;
      if (eat(':')) ty = type().text;
      if (hex && (ty == "f32" || ty == "f64" || ty == "bf16" || ty == "f16")) {
        // a float written as its bit pattern
        const unsigned long long bits = std::strtoull(tok.c_str(), nullptr, 16);
        a.kind = MlirAttr::Float;
        a.ty = ty;
        if (ty == "f64") { double d; std::memcpy(&d, &bits, 8); a.num = d; }
        else if (ty == "f32") { uint32_t w = (uint32_t)bits; float f; std::memcpy(&f, &w, 4); a.num = f; }
        else if (ty == "bf16") { uint32_t w = (uint32_t)bits << 16; float f; std::memcpy(&f, &w, 4); a.num = f; }
        else fail("f16 bit patterns are not supported");
        return a;
      }
      a.ty = ty;
      if (real || (!ty.empty() && ty[0] == 'f') || ty == "bf16") {
        a.kind = MlirAttr::Float;
        a.num = std::strtod(tok.c_str(), nullptr);
      } else {
        a.kind = MlirAttr::Int;
        a.num = hex ? (double)std::strtoull(tok.c_str(), nullptr, 16) : (double)std::strtoll(tok.c_str(), nullptr, 10);
      }
      return a;
    }
    if (word("true")) { a.kind = MlirAttr::Bool; a.num = 1; return a; }
    if (word("false")) { a.kind = MlirAttr::Bool; a.num = 0; return a; }
    if (word("unit")) { a.kind = MlirAttr::Unit; return a; }
    a.kind = MlirAttr::Other;
    a.str = raw_value();
    return a;
  }

  void skip_loc() {
    if (word("loc")) {
      ws();
      if (peek() != '(') fail("'(' expected after loc");
      int depth = 0;
      do {
        if (s[i] == '"') { quoted(); continue; }
        if (s[i] == '(') ++depth;
        if (s[i] == ')') --depth;
        bump();
      } while (!eof() && depth > 0);
    }
  }

  MlirFunc func() {
    MlirFunc f;
    f.attrs.kind = MlirAttr::Dict;
    f.name = symbol();
    expect('(');
    if (!eat(')')) {
      do {
        std::string id = ssa();
        expect(':');
        MlirType t = type();
        ws();
        if (peek() == '{') { bump(); dict(); }   // argument attributes
        f.args.emplace_back(std::move(id), std::move(t));
      } while (eat(','));
      expect(')');
    }
    ws();
    if (peek() == '-' && peek(1) == '>') {
      i += 2;
      ws();
      if (peek() == '(') f.results = type_list_in_parens();
      else f.results.push_back(type());
    }
    if (word("attributes")) { expect('{'); f.attrs = dict(); }
    expect('{');
    for (;;) {
      ws();
      if (eof()) fail("func body not closed");
      if (peek() == '}') { bump(); break; }
      f.ops.push_back(op());
    }
    return f;
  }

  MlirOp op() {
    MlirOp o;
    o.attrs.kind = MlirAttr::Dict;
    ws();
    o.line = line;
    if (peek() == '%') {
      do {
        std::string id = ssa();
        size_t colon = std::string::npos;
        if (peek() == ':') {   // %5:2 = two results
          bump();
          size_t b = i;
          while (std::isdigit((unsigned char)peek())) ++i;
          const int n = std::atoi(s.substr(b, i - b).c_str());
          if (n <= 0) fail("bad result count");
          for (int k = 0; k < n; ++k) o.results.push_back(id + "#" + std::to_string(k));
          (void)colon;
        } else {
          o.results.push_back(id);
        }
      } while (eat(','));
      expect('=');
    }
    ws();
    if (peek() == '"') {
      o.opname = quoted();
      expect('(');
      if (!eat(')')) {
        do o.operands.push_back(ssa()); while (eat(','));
        expect(')');
      }
      ws();
      if (peek() == '(') fail("op '" + o.opname + "': regions are not supported");
      if (peek() == '{') { bump(); o.attrs = dict(); }
      expect(':');
      o.operand_types = type_list_in_parens();
      ws();
      if (!(peek() == '-' && peek(1) == '>')) fail("'->' expected in the type of '" + o.opname + "'");
      i += 2;
      ws();
      if (peek() == '(') o.result_types = type_list_in_parens();
      else o.result_types.push_back(type());
    } else {
      o.opname = ident();
      if (o.opname != "return" && o.opname != "std.return" && o.opname != "func.return")
        fail("op '" + o.opname + "' is not in the generic form (\"dialect.op\"(...) {...} : ...)");
      o.opname = "std.return";
      ws();
      if (peek() == '%') {
        do o.operands.push_back(ssa()); while (eat(','));
        expect(':');
        do o.operand_types.push_back(type()); while (eat(','));
      }
    }
    skip_loc();
    if (o.operand_types.size() != o.operands.size())
      fail("op '" + o.opname + "': " + std::to_string(o.operands.size()) + " operands but " +
           std::to_string(o.operand_types.size()) + " operand types");
    if (!o.results.empty() && o.result_types.size() != o.results.size())
      fail("op '" + o.opname + "': " + std::to_string(o.results.size()) + " results but " +
           std::to_string(o.result_types.size()) + " result types");
    return o;
  }
};

std::string lower(std::string v) {
  for (auto &c : v) c = (char)std::tolower((unsigned char)c);
  return v;
}

// numeric view of the attributes a kernel reads: numbers and booleans by name, the fields
// of `param` beside them, arrays as name0, name1, ..., a string value as the flag
// name_<lowercase value> (mode = "edge" -> mode_edge = 1)
void flatten(const MlirAttr &d, std::map<std::string, double> &out) {
  for (auto &f : d.fields) {
    const std::string &k = f.first;
    const MlirAttr &v = f.second;
    switch (v.kind) {
    case MlirAttr::Int: case MlirAttr::Float: case MlirAttr::Bool:
      out[k] = v.num;
      break;
    case MlirAttr::Unit:
      out[k] = 1;
      break;
    case MlirAttr::String:
      if (k != "name") out[k + "_" + lower(v.str)] = 1;
      break;
    case MlirAttr::Array: {
      int n = 0;
      for (auto &it : v.items) {
        if (it.kind == MlirAttr::Int || it.kind == MlirAttr::Float || it.kind == MlirAttr::Bool)
          out[k + std::to_string(n)] = it.num;
        ++n;
      }
      if (k == "ins") {   // parseConvParam: ins_w = ins[0], ins_h = ins[1] (TPUOperationSupport.cpp:421-425)
        out["ins_w"] = v.items.size() > 0 ? v.items[0].num : 0;
        out["ins_h"] = v.items.size() > 1 ? v.items[1].num : 0;
      }
      break;
    }
    case MlirAttr::Dict:
      if (k == "param") flatten(v, out);
      break;
    default:
      break;
    }
  }
}

std::string quant_of_elem(const std::string &elem) {
  if (elem == "si8" || elem == "i8") return "INT8";
  if (elem == "ui8") return "UINT8";
  if (elem == "bf16") return "BF16";
  return "NONE";
}

}  // namespace

MlirFunc parseMlirText(const std::string &text) {
  Reader r(text);
  return r.module();
}

namespace {

std::string quote(const std::string &v) {
  std::string out = "\"";
  for (unsigned char c : v) {
    if (c == '"' || c == '\\') { out += '\\'; out += (char)c; }
    else if (c == '\n') out += "\\n";
    else if (c == '\t') out += "\\t";
    else if (c < 0x20 || c == 0x7f) {
      static const char hex[] = "0123456789ABCDEF";
      out += '\\'; out += hex[c >> 4]; out += hex[c & 15];
    } else out += (char)c;
  }
  return out + "\"";
}

std::string print_float(double num, const std::string &ty) {
  char buf[64];
  if (ty == "f64") {
    std::snprintf(buf, sizeof buf, "%.17e", num);
    return std::string(buf) + " : f64";
  }
  const float f = (float)num;
  std::snprintf(buf, sizeof buf, "%.6e", (double)f);
  if (!std::isfinite(f) || (float)std::strtod(buf, nullptr) != f) {
    uint32_t w;
    std::memcpy(&w, &f, 4);
    std::snprintf(buf, sizeof buf, "0x%08X", w);
  }
  return std::string(buf) + " : " + (ty.empty() || ty == "bf16" || ty == "f16" ? "f32" : ty);
}

void print_attr(const MlirAttr &a, std::string &out);

void print_dict(const MlirAttr &d, std::string &out) {
  out += '{';
  bool first = true;
  for (auto &f : d.fields) {
    if (!first) out += ", ";
    first = false;
    bool plain = !f.first.empty() && !std::isdigit((unsigned char)f.first[0]);
    for (char c : f.first) plain = plain && (std::isalnum((unsigned char)c) || c == '_' || c == '.' || c == '$');
    out += plain ? f.first : quote(f.first);
    if (f.second.kind != MlirAttr::Unit) {
      out += " = ";
      print_attr(f.second, out);
    }
  }
  out += '}';
}

void print_attr(const MlirAttr &a, std::string &out) {
  switch (a.kind) {
    case MlirAttr::Int: {
      char buf[48];
      std::snprintf(buf, sizeof buf, "%lld", (long long)a.num);
      out += buf;
      out += " : " + (a.ty.empty() ? std::string("i32") : a.ty);
      break;
    }
    case MlirAttr::Float: out += print_float(a.num, a.ty); break;
    case MlirAttr::Bool: out += a.num != 0 ? "true" : "false"; break;
    case MlirAttr::String: out += quote(a.str); break;
    case MlirAttr::Array: {
      out += '[';
      for (size_t k = 0; k < a.items.size(); ++k) {
        if (k) out += ", ";
        print_attr(a.items[k], out);
      }
      out += ']';
      break;
    }
    case MlirAttr::Dict: print_dict(a, out); break;
    case MlirAttr::Unit: out += "unit"; break;
    case MlirAttr::Other: out += a.str; break;
  }
}

std::string type_list(const std::vector<MlirType> &t) {
  std::string out;
  for (size_t k = 0; k < t.size(); ++k) out += (k ? ", " : "") + t[k].text;
  return out;
}

// "5#1" -> "%5#1"
std::string use(const std::string &id) { return "%" + id; }

}  // namespace

MlirType tensorType(const std::vector<int64_t> &shape, const std::string &elem) {
  MlirType t;
  t.shaped = true;
  t.shape = shape;
  t.elem = elem;
  t.text = "tensor<";
  for (auto d : shape) t.text += (d < 0 ? std::string("?") : std::to_string(d)) + "x";
  t.text += elem + ">";
  return t;
}

std::string printMlir(const MlirFunc &f) {
  std::string out = "module {\n  func @" + f.name + "(";
  for (size_t k = 0; k < f.args.size(); ++k)
    out += (k ? ", " : "") + use(f.args[k].first) + ": " + f.args[k].second.text;
  out += ")";
  if (f.results.size() == 1) out += " -> " + f.results[0].text;
  else if (f.results.size() > 1) out += " -> (" + type_list(f.results) + ")";
  if (!f.attrs.fields.empty()) {
    out += " attributes ";
    print_dict(f.attrs, out);
  }
  out += " {\n";
  for (auto &o : f.ops) {
    out += "    ";
    if (o.opname == "std.return") {
      out += "return";
      if (!o.operands.empty()) {
        out += ' ';
        for (size_t k = 0; k < o.operands.size(); ++k) out += (k ? ", " : "") + use(o.operands[k]);
        out += " : " + type_list(o.operand_types);
      }
      out += '\n';
      continue;
    }
    if (!o.results.empty()) {
      // "5#0", "5#1" were written as %5:2
      const size_t hash = o.results[0].find('#');
      if (hash != std::string::npos)
        out += use(o.results[0].substr(0, hash)) + ":" + std::to_string(o.results.size());
      else
        for (size_t k = 0; k < o.results.size(); ++k) out += (k ? ", " : "") + use(o.results[k]);
      out += " = ";
    }
    out += quote(o.opname) + "(";
    for (size_t k = 0; k < o.operands.size(); ++k) out += (k ? ", " : "") + use(o.operands[k]);
    out += ")";
    if (!o.attrs.fields.empty()) {
      out += ' ';
      print_dict(o.attrs, out);
    }
    out += " : (" + type_list(o.operand_types) + ") -> ";
    out += o.result_types.size() == 1 ? o.result_types[0].text : "(" + type_list(o.result_types) + ")";
    out += '\n';
  }
  out += "  }\n}\n";
  return out;
}

MlirModule moduleFromMlir(const MlirFunc &func) {
  MlirModule out;
  if (auto *chip = func.attrs.get("chipname"))
    if (chip->kind == MlirAttr::String) out.chipname = chip->str;

  // what an SSA id stands for when it is used as an operand
  std::map<std::string, std::string> value_name;   // id -> op / weight name, "" for none
  std::map<std::string, std::vector<int64_t>> weight_shape;
  for (auto &a : func.args) value_name[a.first] = "%" + a.first;

  auto where = [](const MlirOp &o) { return "mlir:" + std::to_string(o.line) + ": "; };
  auto op_name = [&](const MlirOp &o) -> std::string {
    auto *n = o.attrs.get("name");
    if (!n || n->kind != MlirAttr::String)
      throw std::runtime_error(where(o) + "op '" + o.opname + "' has no name attribute");
    return n->str;
  };

  for (auto &o : func.ops) {
    if (o.opname == "tpu.weight_file") {
      auto *fn = o.attrs.get("filename");
      if (!fn || fn->kind != MlirAttr::String)
        throw std::runtime_error(where(o) + "tpu.weight_file without a filename");
      out.weight_file = fn->str;
      for (auto &r : o.results) value_name[r] = "";
      continue;
    }
    if (o.opname == "tpu.none") {
      for (auto &r : o.results) value_name[r] = "";
      continue;
    }
    if (o.opname == "tpu.load_weight") {
      MlirWeight w;
      w.name = op_name(o);
      if (o.result_types.size() != 1 || !o.result_types[0].shaped)
        throw std::runtime_error(where(o) + "tpu.load_weight '" + w.name + "' needs one tensor result");
      w.shape = o.result_types[0].shape;
      auto *st = o.attrs.get("storage");
      w.storage = st && st->kind == MlirAttr::String ? st->str : "NONE";
      value_name[o.results.at(0)] = w.name;
      out.weights.push_back(std::move(w));
      continue;
    }
    if (o.opname == "std.return") {
      for (auto &id : o.operands) {
        auto it = value_name.find(id);
        if (it == value_name.end()) throw std::runtime_error(where(o) + "return of undefined value %" + id);
        out.module.returns.push_back(it->second);
      }
      continue;
    }
    OpDesc d;
    d.type = o.opname;
    d.name = op_name(o);
    if (o.results.size() != 1)
      throw std::runtime_error(where(o) + "op '" + d.name + "': exactly one result is supported");
    const MlirType &rt = o.result_types[0];
    if (!rt.shaped)
      throw std::runtime_error(where(o) + "op '" + d.name + "': result type '" + rt.text + "' is not a tensor");
    for (auto v : rt.shape)
      if (v < 0) throw std::runtime_error(where(o) + "op '" + d.name + "': dynamic shapes are not supported");
    d.shape = rt.shape;
    d.quant = quant_of_elem(rt.elem);
    d.param_type = "NONE";
    if (auto *q = o.attrs.get("quant")) {
      if (auto *m = q->get("mode"))
        if (m->kind == MlirAttr::String) d.quant = m->str;
      if (auto *p = q->get("param_type"))
        if (p->kind == MlirAttr::String) d.param_type = p->str;
      if (auto *t = q->get("threshold"))
        if (t->kind == MlirAttr::Float || t->kind == MlirAttr::Int) d.attrs["threshold"] = t->num;
      // an unsigned result of an INT8 op (input images, ReLU outputs the quantizer marks ui8)
      if (d.quant == "INT8" && rt.elem == "ui8" && o.opname == "tpu.input") d.quant = "UINT8";
    }
    if (o.opname == "tpu.quant") {   // the result type of a QuantOp is its `to` mode (core/quant.cpp:118-131)
      auto *to = o.attrs.get("to");
      if (to && to->kind == MlirAttr::String) d.quant = to->str;
    }
    flatten(o.attrs, d.attrs);
    if (o.opname != "tpu.input") {
      for (auto &id : o.operands) {
        auto it = value_name.find(id);
        if (it == value_name.end())
          throw std::runtime_error(where(o) + "op '" + d.name + "' uses undefined value %" + id);
        d.operands.push_back(it->second);
      }
    }
    // kernel size when the param struct predates kernel_h / kernel_w: the filter's last two dims
    if ((o.opname == "tpu.conv_2d" || o.opname == "tpu.deconv_2d") && !d.attrs.count("kernel_h") &&
        o.operand_types.size() > 1 && o.operand_types[1].shaped && o.operand_types[1].shape.size() >= 4) {
      auto &fs = o.operand_types[1].shape;
      d.attrs["kernel_h"] = (double)fs[fs.size() - 2];
      d.attrs["kernel_w"] = (double)fs[fs.size() - 1];
    }
    value_name[o.results[0]] = d.name;
    out.module.ops.push_back(std::move(d));
  }
  return out;
}

std::string describeModule(const MlirModule &m) {
  std::ostringstream os;
  os.precision(17);   // attributes read back to the value the text holds (scales, thresholds)
  os << "weight_file " << (m.weight_file.empty() ? "-" : m.weight_file) << "\n";
  if (!m.chipname.empty()) os << "chipname " << m.chipname << "\n";
  for (auto &w : m.weights) {
    os << "weight " << w.name << " " << w.storage << " [";
    for (size_t i = 0; i < w.shape.size(); ++i) os << (i ? "," : "") << w.shape[i];
    os << "]\n";
  }
  for (auto &o : m.module.ops) {
    os << "op " << o.type << " " << o.name << " " << o.quant << " " << o.param_type << " [";
    for (size_t i = 0; i < o.shape.size(); ++i) os << (i ? "," : "") << o.shape[i];
    os << "]";
    for (auto &opd : o.operands) os << " " << (opd.empty() ? "-" : opd);
    os << " {";
    bool first = true;
    for (auto &kv : o.attrs) {
      os << (first ? "" : ",") << kv.first << "=" << kv.second;
      first = false;
    }
    os << "}\n";
  }
  for (auto &r : m.module.returns) os << "return " << r << "\n";
  return os.str();
}

}  // namespace tpuhip
