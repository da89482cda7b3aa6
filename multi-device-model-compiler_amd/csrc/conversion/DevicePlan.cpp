// Textual device plan: parser, verifier, printer.
//
//   func @main_graph(%a: 3x640x640xf32, %b: 3x640x640xf32) -> (%c: 3x640x640xf32) {
//     %w = device.constant {file = "w.dat"} : 768x2304xf16
//     %c = device.add %a, %b : 3x640x640xf32
//     %s, %y = device.add-residual-layernorm %x, %r, %g, %be {eps = 1e-5} : 8x768xf16, 8x768xf16
//     %o = device.fused-mha %qkv, none {causal = false} : 2x128x768xf16
//     return
//   }
//
// One op per line: results, op name, operands (`none` for an absent optional
// operand), attributes in braces, result types after the colon.  The op set is
// the Device dialect of the reference (DeviceOps.td:17-183: matmul,
// multi-head-attention-layer) plus one op per further entry point of the kernel
// library, and gpu.launch_func for compiler-generated kernels of the loaded
// code object.  `//` and `#` start comments.
#include "multi-device-model-compiler/Conversion/ConvertDeviceToRuntimeCalls.h"

#include <cctype>
#include <cmath>
#include <cstdlib>
#include <sstream>

namespace multi_device {
namespace conversion {

size_t elemBytes(ElemType t) {
  switch (t) {
  case ElemType::F32: return 4;
  case ElemType::F16: return 2;
  case ElemType::BF16: return 2;
  case ElemType::I32: return 4;
  case ElemType::I64: return 8;
  }
  return 0;
}

const char *elemName(ElemType t) {
  switch (t) {
  case ElemType::F32: return "f32";
  case ElemType::F16: return "f16";
  case ElemType::BF16: return "bf16";
  case ElemType::I32: return "i32";
  case ElemType::I64: return "i64";
  }
  return "?";
}

int64_t TensorType::numel() const {
  int64_t n = 1;
  for (int64_t d : shape) n *= d;
  return n;
}

std::string TensorType::str() const {
  std::string s;
  for (int64_t d : shape) s += std::to_string(d) + "x";
  return s + elemName(elem);
}

int DevicePlan::find(const std::string &name) const {
  for (size_t i = 0; i < values.size(); i++)
    if (values[i].name == name) return (int)i;
  return -1;
}

namespace {

struct Token {
  enum Kind { Value, Word, Number, String, Punct, End } kind = End;
  std::string text;
};

// Splits one line.  Words cover op names (device.add-residual-layernorm),
// types (3x640xf32), keywords; '->' is one punctuation token.
bool tokenize(const std::string &line, std::vector<Token> &out, std::string &error) {
  size_t i = 0;
  const size_t n = line.size();
  while (i < n) {
    const char c = line[i];
    if (std::isspace((unsigned char)c)) { i++; continue; }
    if (c == '#' || (c == '/' && i + 1 < n && line[i + 1] == '/')) break;
    Token t;
    if (c == '%' || c == '@') {
      size_t j = i + 1;
      while (j < n && (std::isalnum((unsigned char)line[j]) || line[j] == '_' || line[j] == '.')) j++;
      if (j == i + 1) { error = "empty name after '" + std::string(1, c) + "'"; return false; }
      t.kind = c == '%' ? Token::Value : Token::Word;
      t.text = c == '%' ? line.substr(i + 1, j - i - 1) : line.substr(i, j - i);
      i = j;
    } else if (c == '"') {
      size_t j = line.find('"', i + 1);
      if (j == std::string::npos) { error = "unterminated string"; return false; }
      t.kind = Token::String;
      t.text = line.substr(i + 1, j - i - 1);
      i = j + 1;
    } else if (c == '-' && i + 1 < n && line[i + 1] == '>') {
      t.kind = Token::Punct; t.text = "->"; i += 2;
    } else if (std::isdigit((unsigned char)c) || ((c == '-' || c == '+' || c == '.') && i + 1 < n &&
                                                  (std::isdigit((unsigned char)line[i + 1]) || line[i + 1] == '.'))) {
      // a number, or a type such as 3x640xf32
      size_t j = i;
      while (j < n && (std::isalnum((unsigned char)line[j]) || line[j] == '.' || line[j] == '-' || line[j] == '+')) {
        if ((line[j] == '-' || line[j] == '+') && j > i && !(line[j - 1] == 'e' || line[j - 1] == 'E')) break;
        j++;
      }
      t.text = line.substr(i, j - i);
      bool isType = false;
      for (const char *suffix : {"xf32", "xf16", "xbf16", "xi32", "xi64"}) {
        const size_t L = std::char_traits<char>::length(suffix);
        if (t.text.size() > L && t.text.compare(t.text.size() - L, L, suffix) == 0) isType = true;
      }
      t.kind = isType ? Token::Word : Token::Number;
      i = j;
    } else if (std::isalpha((unsigned char)c) || c == '_') {
      size_t j = i;
      while (j < n && (std::isalnum((unsigned char)line[j]) || line[j] == '_' || line[j] == '.' || line[j] == '-')) {
        if (line[j] == '-' && j + 1 < n && line[j + 1] == '>') break;
        j++;
      }
      t.kind = Token::Word;
      t.text = line.substr(i, j - i);
      i = j;
    } else if (std::string("(){}[],:=").find(c) != std::string::npos) {
      t.kind = Token::Punct; t.text = std::string(1, c); i++;
    } else {
      error = std::string("unexpected character '") + c + "'";
      return false;
    }
    out.push_back(t);
  }
  return true;
}

bool parseType(const std::string &text, TensorType &type) {
  type.shape.clear();
  size_t pos = 0;
  while (true) {
    const size_t x = text.find('x', pos);
    if (x == std::string::npos) break;
    const std::string dim = text.substr(pos, x - pos);
    if (dim.empty() || dim.find_first_not_of("0123456789") != std::string::npos) break;
    type.shape.push_back(std::strtoll(dim.c_str(), nullptr, 10));
    pos = x + 1;
  }
  const std::string elem = text.substr(pos);
  if (elem == "f32") type.elem = ElemType::F32;
  else if (elem == "f16") type.elem = ElemType::F16;
  else if (elem == "bf16") type.elem = ElemType::BF16;
  else if (elem == "i32") type.elem = ElemType::I32;
  else if (elem == "i64") type.elem = ElemType::I64;
  else return false;
  return true;
}

struct Cursor {
  const std::vector<Token> &t;
  size_t i = 0;
  explicit Cursor(const std::vector<Token> &tokens) : t(tokens) {}
  const Token &peek() const {
    static const Token end;
    return i < t.size() ? t[i] : end;
  }
  bool isPunct(const char *p) const { return peek().kind == Token::Punct && peek().text == p; }
  bool eat(const char *p) {
    if (!isPunct(p)) return false;
    i++;
    return true;
  }
  bool done() const { return i >= t.size(); }
};

// `%name: type` list up to ')'
bool parseSignatureList(Cursor &c, DevicePlan &plan, PlanValue::Kind kind, std::vector<int> &into,
                        std::string &error) {
  if (!c.eat("(")) { error = "expected '('"; return false; }
  while (!c.isPunct(")")) {
    if (c.peek().kind != Token::Value) { error = "expected a %name in the signature"; return false; }
    PlanValue v;
    v.name = c.peek().text;
    v.kind = kind;
    c.i++;
    if (!c.eat(":")) { error = "expected ':' after %" + v.name; return false; }
    if (c.peek().kind != Token::Word || !parseType(c.peek().text, v.type)) {
      error = "bad type for %" + v.name;
      return false;
    }
    c.i++;
    if (plan.find(v.name) >= 0) { error = "%" + v.name + " is declared twice"; return false; }
    into.push_back((int)plan.values.size());
    plan.values.push_back(v);
    if (!c.eat(",") && !c.isPunct(")")) { error = "expected ',' or ')'"; return false; }
  }
  c.i++;
  return true;
}

bool parseAttrs(Cursor &c, std::map<std::string, AttrValue> &attrs, std::string &error) {
  while (!c.isPunct("}")) {
    if (c.peek().kind != Token::Word) { error = "expected an attribute name"; return false; }
    const std::string key = c.peek().text;
    c.i++;
    if (!c.eat("=")) { error = "expected '=' after attribute " + key; return false; }
    AttrValue a;
    const Token &v = c.peek();
    if (v.kind == Token::Number) {
      a.kind = AttrValue::Number;
      char *end = nullptr;
      a.number = std::strtod(v.text.c_str(), &end);
      if (!end || *end) { error = "bad number '" + v.text + "'"; return false; }
      c.i++;
    } else if (v.kind == Token::String) {
      a.kind = AttrValue::String; a.text = v.text; c.i++;
    } else if (v.kind == Token::Word && (v.text == "true" || v.text == "false")) {
      a.kind = AttrValue::Bool; a.flag = v.text == "true"; c.i++;
    } else if (c.eat("[")) {
      a.kind = AttrValue::IntList;
      while (!c.isPunct("]")) {
        if (c.peek().kind != Token::Number) { error = "expected an integer in the list of " + key; return false; }
        a.ints.push_back(std::strtoll(c.peek().text.c_str(), nullptr, 10));
        c.i++;
        if (!c.eat(",") && !c.isPunct("]")) { error = "expected ',' or ']'"; return false; }
      }
      c.i++;
    } else {
      error = "bad value for attribute " + key;
      return false;
    }
    if (attrs.count(key)) { error = "attribute " + key + " given twice"; return false; }
    attrs[key] = a;
    if (!c.eat(",") && !c.isPunct("}")) { error = "expected ',' or '}'"; return false; }
  }
  c.i++;
  return true;
}

} // namespace

bool parseDevicePlan(const std::string &text, DevicePlan &plan, std::string &error) {
  plan = DevicePlan();
  std::istringstream in(text);
  std::string line;
  int lineNo = 0;
  bool sawFunc = false, sawReturn = false, closed = false;
  auto fail = [&](const std::string &msg) {
    error = "line " + std::to_string(lineNo) + ": " + msg;
    return false;
  };
  while (std::getline(in, line)) {
    lineNo++;
    std::vector<Token> tokens;
    std::string terr;
    if (!tokenize(line, tokens, terr)) return fail(terr);
    if (tokens.empty()) continue;
    Cursor c(tokens);
    if (closed) return fail("text after the closing '}'");
    if (!sawFunc) {
      if (!(c.peek().kind == Token::Word && c.peek().text == "func")) return fail("expected 'func @name(...) -> (...) {'");
      c.i++;
      if (c.peek().kind != Token::Word || c.peek().text.empty() || c.peek().text[0] != '@') return fail("expected '@name' after func");
      plan.func = c.peek().text.substr(1);
      c.i++;
      std::string serr;
      if (!parseSignatureList(c, plan, PlanValue::Input, plan.inputs, serr)) return fail(serr);
      if (!c.eat("->")) return fail("expected '->' after the arguments");
      if (!parseSignatureList(c, plan, PlanValue::Output, plan.outputs, serr)) return fail(serr);
      if (!c.eat("{")) return fail("expected '{'");
      if (!c.done()) return fail("unexpected text after '{'");
      sawFunc = true;
      continue;
    }
    if (c.peek().kind == Token::Word && c.peek().text == "return") {
      if (sawReturn) return fail("second return");
      sawReturn = true;
      c.i++;
      if (!c.done()) return fail("return takes no operands: results are named in the signature");
      continue;
    }
    if (c.isPunct("}")) {
      if (!sawReturn) return fail("missing return");
      closed = true;
      continue;
    }
    if (sawReturn) return fail("op after return");

    // results
    DeviceOp op;
    op.line = lineNo;
    std::vector<std::string> resultNames;
    while (c.peek().kind == Token::Value) {
      resultNames.push_back(c.peek().text);
      c.i++;
      if (!c.eat(",")) break;
    }
    if (resultNames.empty()) return fail("an op line starts with its results: %r = op ...");
    if (!c.eat("=")) return fail("expected '=' after the results");
    if (c.peek().kind != Token::Word) return fail("expected an op name");
    op.name = c.peek().text;
    c.i++;
    // operands
    while (c.peek().kind == Token::Value || (c.peek().kind == Token::Word && c.peek().text == "none")) {
      if (c.peek().kind == Token::Value) {
        const int v = plan.find(c.peek().text);
        if (v < 0) return fail("%" + c.peek().text + " is used before its definition");
        op.operands.push_back(v);
      } else {
        op.operands.push_back(-1);
      }
      c.i++;
      if (!c.eat(",")) break;
    }
    if (c.eat("{")) {
      std::string aerr;
      if (!parseAttrs(c, op.attrs, aerr)) return fail(aerr);
    }
    if (!c.eat(":")) return fail("expected ':' and the result types");
    for (size_t r = 0; r < resultNames.size(); r++) {
      TensorType type;
      if (c.peek().kind != Token::Word || !parseType(c.peek().text, type)) return fail("bad result type");
      c.i++;
      if (r + 1 < resultNames.size() && !c.eat(",")) return fail("expected one type per result");
      int v = plan.find(resultNames[r]);
      if (v >= 0) {
        PlanValue &out = plan.values[v];
        if (out.kind != PlanValue::Output) return fail("%" + resultNames[r] + " is defined twice");
        if (out.definedBy >= 0) return fail("function result %" + resultNames[r] + " is produced twice");
        if (out.type != type) return fail("%" + resultNames[r] + " has type " + out.type.str() + " in the signature");
        out.definedBy = (int)plan.ops.size();
      } else {
        PlanValue nv;
        nv.name = resultNames[r];
        nv.type = type;
        nv.kind = op.name == "device.constant" ? PlanValue::Constant : PlanValue::Temp;
        nv.definedBy = op.name == "device.constant" ? -1 : (int)plan.ops.size();
        v = (int)plan.values.size();
        plan.values.push_back(nv);
      }
      op.results.push_back(v);
    }
    if (!c.done()) return fail("unexpected text at the end of the line");
    if (op.name == "device.constant") {
      if (op.results.size() != 1 || !op.operands.empty()) return fail("device.constant has one result and no operands");
      PlanValue &cv = plan.values[op.results[0]];
      if (cv.kind != PlanValue::Constant) return fail("a function result cannot be a constant");
      auto f = op.attrs.find("file");
      if (f == op.attrs.end() || f->second.kind != AttrValue::String || f->second.text.empty())
        return fail("device.constant needs {file = \"...\"}");
      cv.file = f->second.text;
      continue; // constants are values, not ops
    }
    plan.ops.push_back(op);
  }
  lineNo++;
  if (!sawFunc) return fail("no function");
  if (!closed) return fail("missing closing '}'");
  return true;
}

namespace {

struct Verifier {
  const DevicePlan &plan;
  const DeviceOp &op;
  std::string &error;
  bool fail(const std::string &msg) const {
    error = "line " + std::to_string(op.line) + ": " + op.name + ": " + msg;
    return false;
  }
  const TensorType &in(int i) const { return plan.values[op.operands[i]].type; }
  const TensorType &out(int i) const { return plan.values[op.results[i]].type; }
  bool present(int i) const { return op.operands[i] >= 0; }
  bool counts(size_t operands, size_t results) const {
    if (op.operands.size() != operands) return fail("takes " + std::to_string(operands) + " operands");
    if (op.results.size() != results) return fail("has " + std::to_string(results) + " result(s)");
    return true;
  }
  bool required(std::initializer_list<int> idx) const {
    for (int i : idx)
      if (!present(i)) return fail("operand " + std::to_string(i) + " cannot be none");
    return true;
  }
  bool vectorOf(int i, int64_t n, ElemType e, const char *what) const {
    const TensorType &t = in(i);
    if (t.elem != e || t.shape.empty() || t.shape.back() != n) return fail(std::string(what) + " must be " + std::to_string(n) + "x" + elemName(e));
    for (size_t d = 0; d + 1 < t.shape.size(); d++)
      if (t.shape[d] != 1) return fail(std::string(what) + " must be a vector");
    return true;
  }
  bool attrKinds(std::initializer_list<std::pair<const char *, AttrValue::Kind>> allowed) const {
    for (const auto &kv : op.attrs) {
      bool ok = false;
      for (const auto &a : allowed)
        if (kv.first == a.first) {
          if (kv.second.kind != a.second) return fail("attribute " + kv.first + " has the wrong kind of value");
          ok = true;
        }
      if (!ok) return fail("unknown attribute " + kv.first);
    }
    return true;
  }
};

bool isFloat(ElemType e) { return e == ElemType::F32 || e == ElemType::F16 || e == ElemType::BF16; }

// input [..., K] . weight [K, N] -> [..., N], the checks of MatmulOp::verify
// (lib/Dialect/Device/IR/DeviceDialect.cpp:66-100)
bool verifyMatmulShapes(const Verifier &v, bool biasPresent) {
  const TensorType &x = v.in(0), &w = v.in(1), &y = v.out(0);
  if (x.shape.empty()) return v.fail("input needs at least one dimension");
  if (w.shape.size() != 2 || x.shape.back() != w.shape[0]) return v.fail("weight must be [K, N] with K the last input dimension");
  if (w.elem != x.elem || y.elem != x.elem) return v.fail("input, weight and output share one element type");
  if (biasPresent && !v.vectorOf(2, w.shape[1], x.elem, "bias")) return false;
  if (y.shape.size() != x.shape.size() || y.shape.back() != w.shape[1]) return v.fail("output must be [..., N]");
  for (size_t d = 0; d + 1 < x.shape.size(); d++)
    if (x.shape[d] != y.shape[d]) return v.fail("output and input differ in a leading dimension");
  return true;
}

bool verifyOp(const DevicePlan &plan, const DeviceOp &op, std::string &error) {
  Verifier v{plan, op, error};
  const std::string &n = op.name;
  if (n == "device.add") {
    if (!v.counts(2, 1) || !v.required({0, 1}) || !v.attrKinds({})) return false;
    if (v.in(0) != v.in(1) || v.in(0) != v.out(0)) return v.fail("operands and result share one type");
    if (v.in(0).elem != ElemType::F32) return v.fail("built for f32");
    return true;
  }
  if (n == "device.layernorm") {
    if (!v.counts(3, 1) || !v.required({0, 1, 2}) || !v.attrKinds({{"eps", AttrValue::Number}})) return false;
    const TensorType &x = v.in(0);
    if (!isFloat(x.elem) || x.shape.empty()) return v.fail("input must be a float tensor");
    if (!v.vectorOf(1, x.shape.back(), x.elem, "gamma") || !v.vectorOf(2, x.shape.back(), x.elem, "beta")) return false;
    if (v.out(0) != x) return v.fail("result has the type of the input");
    return true;
  }
  if (n == "device.add-residual-layernorm") {
    if (!v.counts(4, 2) || !v.required({0, 1, 2, 3}) || !v.attrKinds({{"eps", AttrValue::Number}})) return false;
    const TensorType &x = v.in(0);
    if (!isFloat(x.elem) || x.shape.empty()) return v.fail("input must be a float tensor");
    if (v.in(1) != x) return v.fail("residual has the type of the input");
    if (!v.vectorOf(2, x.shape.back(), x.elem, "gamma") || !v.vectorOf(3, x.shape.back(), x.elem, "beta")) return false;
    if (v.out(0) != x || v.out(1) != x) return v.fail("both results have the type of the input");
    return true;
  }
  if (n == "device.matmul") {
    if (!v.counts(3, 1) || !v.required({0, 1, 2}) || !v.attrKinds({})) return false;
    if (v.in(0).elem != ElemType::F32) return v.fail("is the f32 entry point; use device.matmul-ex for f16");
    return verifyMatmulShapes(v, true);
  }
  if (n == "device.matmul-ex") {
    if (!v.counts(4, 1) || !v.required({0, 1}) || !v.attrKinds({{"act", AttrValue::String}})) return false;
    if (!isFloat(v.in(0).elem)) return v.fail("built for f32, f16 and bf16");
    if (!verifyMatmulShapes(v, v.present(2))) return false;
    if (v.present(3) && v.in(3) != v.out(0)) return v.fail("residual has the type of the result");
    auto act = op.attrs.find("act");
    if (act != op.attrs.end()) {
      const std::string &a = act->second.text;
      if (a != "none" && a != "relu" && a != "gelu") return v.fail("act is \"none\", \"relu\" or \"gelu\"");
      if (a != "none" && v.present(3)) return v.fail("an activation cannot be combined with a residual");
    }
    return true;
  }
  if (n == "device.conv2d") { // Conv2DOp::verify, DeviceDialect.cpp:114-140, plus the size arithmetic
    if (!v.counts(4, 1) || !v.required({0, 1, 2}) ||
        !v.attrKinds({{"pad", AttrValue::IntList}, {"stride", AttrValue::IntList}, {"dilation", AttrValue::IntList},
                      {"kernel", AttrValue::IntList}, {"containRelu", AttrValue::Bool}})) return false;
    const TensorType &x = v.in(0), &w = v.in(1), &y = v.out(0);
    if (x.elem != ElemType::F32 || w.elem != ElemType::F32 || y.elem != ElemType::F32) return v.fail("built for f32");
    if (x.shape.size() != 4 || w.shape.size() != 4 || y.shape.size() != 4) return v.fail("input, weight and output are rank 4 (NCHW / OIHW)");
    if (x.shape[0] != y.shape[0] || x.shape[1] != w.shape[1] || y.shape[1] != w.shape[0])
      return v.fail("batch or channel counts of input, weight and output disagree");
    if (!v.vectorOf(2, w.shape[0], ElemType::F32, "bias")) return false;
    if (v.present(3) && v.in(3) != y) return v.fail("postadd has the type of the output");
    std::vector<int64_t> pad{0, 0, 0, 0}, stride{1, 1}, dil{1, 1};
    const std::pair<const char *, std::vector<int64_t> *> lists[] = {{"pad", &pad}, {"stride", &stride}, {"dilation", &dil}};
    for (const auto &kv : lists) {
      auto a = op.attrs.find(kv.first);
      if (a == op.attrs.end()) continue;
      if (a->second.ints.size() != kv.second->size()) return v.fail(std::string(kv.first) + " has the wrong number of entries");
      *kv.second = a->second.ints;
    }
    auto k = op.attrs.find("kernel");
    if (k != op.attrs.end() && k->second.ints != std::vector<int64_t>{w.shape[2], w.shape[3]}) return v.fail("kernel disagrees with the weight shape");
    for (int d = 0; d < 2; d++) {
      if (stride[d] <= 0 || dil[d] <= 0 || pad[d] < 0 || pad[d + 2] < 0) return v.fail("bad pad, stride or dilation");
      const int64_t span = x.shape[2 + d] + pad[d] + pad[d + 2] - dil[d] * (w.shape[2 + d] - 1) - 1;
      if (span < 0 || y.shape[2 + d] != span / stride[d] + 1) return v.fail("output size does not follow from input, kernel, pad, stride and dilation");
    }
    return true;
  }
  if (n == "device.pool2d") {
    if (!v.counts(1, 1) || !v.required({0}) ||
        !v.attrKinds({{"kernel", AttrValue::IntList}, {"pad", AttrValue::IntList}, {"stride", AttrValue::IntList},
                      {"method", AttrValue::String}})) return false;
    const TensorType &x = v.in(0), &y = v.out(0);
    if (x.elem != ElemType::F32 || y.elem != ElemType::F32) return v.fail("built for f32");
    if (x.shape.size() != 4 || y.shape.size() != 4 || x.shape[0] != y.shape[0] || x.shape[1] != y.shape[1])
      return v.fail("input and output are NCHW with the same batch and channel counts");
    auto k = op.attrs.find("kernel");
    if (k == op.attrs.end() || k->second.ints.size() != 2) return v.fail("needs kernel = [KH, KW]");
    std::vector<int64_t> pad{0, 0, 0, 0}, stride{1, 1};
    auto p = op.attrs.find("pad");
    if (p != op.attrs.end()) { if (p->second.ints.size() != 4) return v.fail("pad has four entries"); pad = p->second.ints; }
    auto st = op.attrs.find("stride");
    if (st != op.attrs.end()) { if (st->second.ints.size() != 2) return v.fail("stride has two entries"); stride = st->second.ints; }
    auto m = op.attrs.find("method");
    if (m == op.attrs.end() || (m->second.text != "max" && m->second.text != "avg")) return v.fail("method is \"max\" or \"avg\"");
    for (int d = 0; d < 2; d++) {
      const int64_t kk = k->second.ints[d];
      if (kk <= 0 || stride[d] <= 0 || pad[d] < 0 || pad[d + 2] < 0 || pad[d] >= kk || pad[d + 2] >= kk) return v.fail("bad kernel, pad or stride");
      const int64_t span = x.shape[2 + d] + pad[d] + pad[d + 2] - kk;
      if (span < 0 || y.shape[2 + d] != span / stride[d] + 1) return v.fail("output size does not follow from input, kernel, pad and stride");
    }
    return true;
  }
  if (n == "device.reshape") { // a view: same buffer, another shape (memref.reshape)
    if (!v.counts(1, 1) || !v.required({0}) || !v.attrKinds({})) return false;
    if (v.in(0).elem != v.out(0).elem || v.in(0).numel() != v.out(0).numel())
      return v.fail("result has the element type and the element count of the operand");
    if (plan.values[op.results[0]].kind != PlanValue::Temp) return v.fail("a function result cannot be a view");
    return true;
  }
  if (n == "device.cast") {
    if (!v.counts(1, 1) || !v.required({0}) || !v.attrKinds({})) return false;
    if (v.in(0).shape != v.out(0).shape) return v.fail("result has the shape of the operand");
    const ElemType a = v.in(0).elem, b = v.out(0).elem;
    const bool narrow = a == ElemType::F32 && (b == ElemType::F16 || b == ElemType::BF16);
    const bool widen = b == ElemType::F32 && (a == ElemType::F16 || a == ElemType::BF16);
    if (!narrow && !widen) return v.fail("casts f32 -> f16 / bf16 or f16 / bf16 -> f32");
    return true;
  }
  if (n == "device.fused-mha") {
    if (!v.counts(2, 1) || !v.required({0}) ||
        !v.attrKinds({{"causal", AttrValue::Bool}, {"scale", AttrValue::Number}})) return false;
    const TensorType &q = v.in(0);
    if (q.elem != ElemType::F16 && q.elem != ElemType::BF16) return v.fail("qkv must be f16 or bf16");
    if (q.shape.size() != 5 || q.shape[2] != 3) return v.fail("qkv must be [B, S, 3, H, D]");
    if (q.shape[4] < 8 || q.shape[4] > 256 || q.shape[4] % 8) return v.fail("head_dim must be a multiple of 8 between 8 and 256");
    if (v.present(1)) {
      const TensorType &l = v.in(1);
      if (l.elem != ElemType::I32 || l.shape.size() != 1 || l.shape[0] != q.shape[0]) return v.fail("key lengths must be Bxi32");
    }
    const TensorType &o = v.out(0);
    if (o.elem != q.elem || o.shape != std::vector<int64_t>{q.shape[0], q.shape[1], q.shape[3] * q.shape[4]})
      return v.fail("result must be [B, S, H*D] of the qkv element type");
    auto s = op.attrs.find("scale");
    if (s != op.attrs.end() && !(s->second.number > 0)) return v.fail("scale must be positive");
    return true;
  }
  if (n == "device.multi-head-attention-layer") {
    if (!v.counts(8, 1) || !v.required({0, 1, 2, 3, 4, 5, 6, 7}) ||
        !v.attrKinds({{"batch", AttrValue::Number}, {"seq_len", AttrValue::Number}, {"d_model", AttrValue::Number},
                      {"feed_forward_dim", AttrValue::Number}, {"head_num", AttrValue::Number},
                      {"norm_first", AttrValue::Bool}, {"is_casual", AttrValue::Bool}, {"act", AttrValue::String}})) return false;
    const TensorType &x = v.in(0);
    for (int i = 0; i < 8; i++)
      if (v.in(i).elem != ElemType::F32) return v.fail("every operand is f32");
    if (x.shape.size() != 3) return v.fail("input must be [batch, seq_len, d_model]");
    const int64_t d = x.shape[2];
    if (v.in(1).shape != std::vector<int64_t>{d, 3 * d}) return v.fail("QKV must be [d_model, 3*d_model]");
    if (v.in(2).shape != std::vector<int64_t>{d, d}) return v.fail("ATTN_GEMM weight must be [d_model, d_model]");
    if (!v.vectorOf(3, d, ElemType::F32, "ATTN_GEMM bias")) return false;
    const TensorType &f1 = v.in(4);
    if (f1.shape.size() != 2 || f1.shape[0] != d) return v.fail("FFN1 weight must be [d_model, feed_forward_dim]");
    const int64_t ffn = f1.shape[1];
    if (!v.vectorOf(5, ffn, ElemType::F32, "FFN1 bias")) return false;
    if (v.in(6).shape != std::vector<int64_t>{ffn, d}) return v.fail("FFN2 weight must be [feed_forward_dim, d_model]");
    if (!v.vectorOf(7, d, ElemType::F32, "FFN2 bias")) return false;
    if (v.out(0) != x) return v.fail("result has the type of the input");
    auto h = op.attrs.find("head_num");
    if (h == op.attrs.end()) return v.fail("needs head_num");
    const int64_t heads = (int64_t)h->second.number;
    if (heads <= 0 || d % heads != 0 || d / heads < 8 || d / heads > 256 || (d / heads) % 8) return v.fail("d_model / head_num must be a multiple of 8 between 8 and 256");
    const std::pair<const char *, int64_t> derived[] = {{"batch", x.shape[0]}, {"seq_len", x.shape[1]}, {"d_model", d}, {"feed_forward_dim", ffn}};
    for (const auto &kv : derived) {
      auto a = op.attrs.find(kv.first);
      if (a != op.attrs.end() && (int64_t)a->second.number != kv.second)
        return v.fail(std::string(kv.first) + " disagrees with the operand shapes");
    }
    auto act = op.attrs.find("act");
    if (act != op.attrs.end() && act->second.text != "relu" && act->second.text != "gelu") return v.fail("act is \"relu\" or \"gelu\"");
    return true;
  }
  if (n == "device.bert-encoder-layer") {
    if (!v.counts(14, 1) || !v.required({0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12}) ||
        !v.attrKinds({{"head_num", AttrValue::Number}, {"eps", AttrValue::Number}})) return false;
    const TensorType &x = v.in(0);
    for (int i = 0; i < 13; i++)
      if (v.in(i).elem != ElemType::F16) return v.fail("every tensor operand is f16");
    if (x.shape.size() != 3) return v.fail("x must be [batch, seq_len, d_model]");
    const int64_t d = x.shape[2];
    if (v.in(1).shape != std::vector<int64_t>{d, 3 * d}) return v.fail("wqkv must be [d_model, 3*d_model]");
    if (!v.vectorOf(2, 3 * d, ElemType::F16, "bqkv")) return false;
    if (v.in(3).shape != std::vector<int64_t>{d, d}) return v.fail("wo must be [d_model, d_model]");
    if (!v.vectorOf(4, d, ElemType::F16, "bo") || !v.vectorOf(5, d, ElemType::F16, "gamma1") || !v.vectorOf(6, d, ElemType::F16, "beta1")) return false;
    const TensorType &w1 = v.in(7);
    if (w1.shape.size() != 2 || w1.shape[0] != d) return v.fail("w1 must be [d_model, feed_forward_dim]");
    const int64_t ffn = w1.shape[1];
    if (!v.vectorOf(8, ffn, ElemType::F16, "b1")) return false;
    if (v.in(9).shape != std::vector<int64_t>{ffn, d}) return v.fail("w2 must be [feed_forward_dim, d_model]");
    if (!v.vectorOf(10, d, ElemType::F16, "b2") || !v.vectorOf(11, d, ElemType::F16, "gamma2") || !v.vectorOf(12, d, ElemType::F16, "beta2")) return false;
    if (v.present(13)) {
      const TensorType &l = v.in(13);
      if (l.elem != ElemType::I32 || l.shape.size() != 1 || l.shape[0] != x.shape[0]) return v.fail("key lengths must be Bxi32");
    }
    if (v.out(0) != x) return v.fail("result has the type of x");
    auto h = op.attrs.find("head_num");
    if (h == op.attrs.end()) return v.fail("needs head_num");
    const int64_t heads = (int64_t)h->second.number;
    if (heads <= 0 || d % heads != 0 || d / heads < 8 || d / heads > 256 || (d / heads) % 8) return v.fail("d_model / head_num must be a multiple of 8 between 8 and 256");
    return true;
  }
  if (n == "gpu.launch_func") {
    if (op.results.empty()) return v.fail("has at least one result");
    for (size_t i = 0; i < op.operands.size(); i++)
      if (!v.present((int)i)) return v.fail("operands cannot be none");
    if (!v.attrKinds({{"kernel", AttrValue::String}, {"blocks", AttrValue::IntList}, {"threads", AttrValue::IntList},
                      {"smem", AttrValue::Number}, {"scalars", AttrValue::IntList}})) return false;
    auto k = op.attrs.find("kernel");
    if (k == op.attrs.end() || k->second.text.empty()) return v.fail("needs {kernel = \"name\"}");
    for (const char *key : {"blocks", "threads"}) {
      auto a = op.attrs.find(key);
      if (a == op.attrs.end() || a->second.ints.size() != 3) return v.fail(std::string(key) + " is a list of three integers");
      for (int64_t d : a->second.ints)
        if (d <= 0) return v.fail(std::string(key) + " must be positive");
    }
    const auto &threads = op.attrs.find("threads")->second.ints;
    if (threads[0] * threads[1] * threads[2] > 1024) return v.fail("more than 1024 threads per block");
    return true;
  }
  return v.fail("unknown op");
}

} // namespace

bool verifyDevicePlan(const DevicePlan &plan, std::string &error) {
  for (const DeviceOp &op : plan.ops)
    if (!verifyOp(plan, op, error)) return false;
  for (int o : plan.outputs)
    if (plan.values[o].definedBy < 0) {
      error = "function result %" + plan.values[o].name + " is never produced";
      return false;
    }
  for (const PlanValue &v : plan.values)
    if (v.type.numel() < 0) {
      error = "%" + v.name + " has a negative dimension";
      return false;
    }
  return true;
}

std::string printDevicePlan(const DevicePlan &plan) {
  std::ostringstream os;
  auto sig = [&](const std::vector<int> &ids) {
    std::string s;
    for (size_t i = 0; i < ids.size(); i++) {
      const PlanValue &v = plan.values[ids[i]];
      s += (i ? ", %" : "%") + v.name + ": " + v.type.str();
    }
    return s;
  };
  os << "func @" << plan.func << "(" << sig(plan.inputs) << ") -> (" << sig(plan.outputs) << ") {\n";
  for (const PlanValue &v : plan.values)
    if (v.kind == PlanValue::Constant)
      os << "  %" << v.name << " = device.constant {file = \"" << v.file << "\"} : " << v.type.str() << "\n";
  for (const DeviceOp &op : plan.ops) {
    os << "  ";
    for (size_t i = 0; i < op.results.size(); i++) os << (i ? ", %" : "%") << plan.values[op.results[i]].name;
    os << " = " << op.name;
    for (size_t i = 0; i < op.operands.size(); i++)
      os << (i ? ", " : " ") << (op.operands[i] < 0 ? std::string("none") : "%" + plan.values[op.operands[i]].name);
    if (!op.attrs.empty()) {
      os << " {";
      bool first = true;
      for (const auto &kv : op.attrs) {
        os << (first ? "" : ", ") << kv.first << " = ";
        first = false;
        const AttrValue &a = kv.second;
        if (a.kind == AttrValue::Number) os << a.number;
        else if (a.kind == AttrValue::Bool) os << (a.flag ? "true" : "false");
        else if (a.kind == AttrValue::String) os << '"' << a.text << '"';
        else {
          os << "[";
          for (size_t i = 0; i < a.ints.size(); i++) os << (i ? ", " : "") << a.ints[i];
          os << "]";
        }
      }
      os << "}";
    }
    os << " :";
    for (size_t i = 0; i < op.results.size(); i++) os << (i ? ", " : " ") << plan.values[op.results[i]].type.str();
    os << "\n";
  }
  os << "  return\n}\n";
  return os.str();
}

} // namespace conversion
} // namespace multi_device
