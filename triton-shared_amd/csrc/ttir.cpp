// TTIR text reader: see ttir.h.  Line oriented, because the MLIR printer
// emits one operation per line and opens/closes regions on lines of their own.
#include "ttir.h"

#include <cctype>
#include <functional>
#include <map>
#include <sstream>

namespace tts {

std::string Type::str() const {
  std::string e = ptr && !block ? "!tt.ptr<" + elem + ">" : elem;
  if (!is_tensor) return e;
  std::string s = "tensor<";
  for (auto d : shape) s += std::to_string(d) + "x";
  s += e + ">";
  return block ? "!tt.ptr<" + s + ">" : s;
}

static std::string trim(const std::string &s) {
  size_t a = 0, b = s.size();
  while (a < b && isspace((unsigned char)s[a])) a++;
  while (b > a && isspace((unsigned char)s[b - 1])) b--;
  return s.substr(a, b - a);
}

static bool starts_with(const std::string &s, const char *p) { return s.rfind(p, 0) == 0; }

Type parse_type(const std::string &raw) {
  std::string s = trim(raw);
  Type t;
  if (starts_with(s, "tensor<")) {
    t.is_tensor = true;
    std::string in = s.substr(7, s.size() - 8);
    // dims are separated by 'x' up to the first token that is not a number
    size_t p = 0;
    while (p < in.size() && isdigit((unsigned char)in[p])) {
      size_t q = p;
      while (q < in.size() && isdigit((unsigned char)in[q])) q++;
      if (q >= in.size() || in[q] != 'x') break;
      t.shape.push_back(std::stoll(in.substr(p, q - p)));
      p = q + 1;
    }
    Type e = parse_type(in.substr(p));
    t.ptr = e.ptr;
    t.elem = e.elem;
    return t;
  }
  if (starts_with(s, "!tt.ptr<")) {
    t.ptr = true;
    std::string in = s.substr(8, s.size() - 9);
    size_t comma = in.find(',');  // address space suffix, if printed
    if (comma != std::string::npos) in = in.substr(0, comma);
    t.elem = trim(in);
    if (starts_with(t.elem, "tensor<")) {  // a block pointer: the block's shape and element type, flagged
      t = parse_type(t.elem);
      if (t.ptr) throw Unsupported("pointer to a block of pointers: " + s);
      t.ptr = t.block = true;
      return t;
    }
    if (starts_with(t.elem, "!tt.ptr")) throw Unsupported("pointer-to-pointer is not supported: " + s);
    return t;
  }
  if (starts_with(s, "<tensor<")) return parse_type("!tt.ptr" + s);  // the short form the custom assembly prints
  static const char *known[] = {"i1", "i8", "i16", "i32", "i64", "f16", "bf16", "f32", "f64", "index"};
  for (auto k : known)
    if (s == k) {
      t.elem = s;
      return t;
    }
  throw Unsupported("unsupported type '" + s + "'");
}

// Removes "#loc..." definition lines and every " loc(...)" trailer.
static std::string strip_locations(const std::string &text) {
  std::string out;
  out.reserve(text.size());
  size_t i = 0, n = text.size();
  bool line_start = true;
  while (i < n) {
    if (line_start && text.compare(i, 4, "#loc") == 0) {
      while (i < n && text[i] != '\n') i++;
      continue;
    }
    if (text.compare(i, 5, " loc(") == 0) {
      size_t j = i + 5;
      int depth = 1;
      bool in_str = false;
      while (j < n && depth) {
        char c = text[j];
        if (c == '"') in_str = !in_str;
        else if (!in_str && c == '(') depth++;
        else if (!in_str && c == ')') depth--;
        j++;
      }
      i = j;
      continue;
    }
    line_start = text[i] == '\n';
    out.push_back(text[i++]);
  }
  return out;
}

static bool ssa_char(char c) {
  return isalnum((unsigned char)c) || c == '_' || c == '.' || c == '$' || c == '#' || c == '-';
}

// Splits at top-level occurrences of any separator in seps (each a literal).
static std::vector<std::string> split_top(const std::string &s, const std::vector<std::string> &seps) {
  std::vector<std::string> out;
  int depth = 0;
  size_t last = 0, i = 0;
  while (i < s.size()) {
    char c = s[i];
    if (depth == 0) {
      bool hit = false;
      for (auto &sep : seps)
        if (s.compare(i, sep.size(), sep) == 0) {
          out.push_back(trim(s.substr(last, i - last)));
          i += sep.size();
          last = i;
          hit = true;
          break;
        }
      if (hit) continue;
    }
    if (c == '-' && i + 1 < s.size() && s[i + 1] == '>') { i += 2; continue; }
    if (c == '(' || c == '{' || c == '<' || c == '[') depth++;
    else if (c == ')' || c == '}' || c == '>' || c == ']') depth--;
    i++;
  }
  out.push_back(trim(s.substr(last)));
  return out;
}

static std::vector<Type> parse_type_list(const std::string &s) {
  std::vector<Type> out;
  for (auto &piece : split_top(s, {"->", ",", " to ", " * "})) {
    std::string p = piece;
    if (p.empty()) continue;
    if (p.front() == '(' && p.back() == ')') {
      for (auto &t : parse_type_list(p.substr(1, p.size() - 2))) out.push_back(t);
      continue;
    }
    out.push_back(parse_type(p));
  }
  return out;
}

static void collect_operands(const std::string &s, std::vector<std::string> &out) {
  for (size_t i = 0; i < s.size(); i++) {
    if (s[i] != '%') continue;
    size_t j = i + 1;
    while (j < s.size() && ssa_char(s[j])) j++;
    out.push_back(s.substr(i, j - i));
    i = j - 1;
  }
}

static void parse_attr_dict(const std::string &body, std::map<std::string, std::string> &attrs) {
  for (auto &ent : split_top(body, {","})) {
    if (ent.empty()) continue;
    size_t eq = ent.find('=');
    if (eq == std::string::npos) {
      attrs[trim(ent)] = "unit";
      continue;
    }
    std::string key = trim(ent.substr(0, eq));
    std::string val = trim(ent.substr(eq + 1));
    auto parts = split_top(val, {" : "});
    attrs[key] = parts[0];
  }
}

// Finds the first ':' that is outside every bracket.  Returns npos if none.
static size_t top_colon(const std::string &s) {
  int depth = 0;
  for (size_t i = 0; i < s.size(); i++) {
    char c = s[i];
    if (c == '-' && i + 1 < s.size() && s[i + 1] == '>') { i++; continue; }
    if (c == '(' || c == '{' || c == '<' || c == '[') depth++;
    else if (c == ')' || c == '}' || c == '>' || c == ']') depth--;
    else if (c == ':' && depth == 0) return i;
  }
  return std::string::npos;
}

struct Lines {
  std::vector<std::string> v;
  size_t i = 0;
};

static void parse_block(Lines &L, Block &blk);

static void parse_results(const std::string &lhs, Op &op) {
  for (auto &r : split_top(lhs, {","})) {
    size_t colon = r.find(':');
    if (colon == std::string::npos) {
      op.results.push_back(r);
    } else {
      int n = std::stoi(r.substr(colon + 1));
      std::string base = r.substr(0, colon);
      for (int k = 0; k < n; k++) op.results.push_back(base + "#" + std::to_string(k));
    }
  }
}

using Renames = std::map<std::string, std::string>;
static void copy_block(const Block &src, Block &dst, const Renames &m);
static void collect_defs(const Block &b, std::vector<std::string> &out);

// scf.while (%a = %x, ...) : (types) -> (types) { <before> scf.condition(%c) %a, ... } do { ^bb0(%a: type, ...): <after>
// scf.yield ... }, in the form the frontend writes for `while cond:` -- the condition passes the loop's arguments on
// unchanged -- becomes a counted loop that is left through a break: scf.for over [0, 2^31 - 1) whose body is the `before`
// ops, "tts.break_unless %c", and the `after` ops with their yield.  Where it breaks, the carried values are the
// arguments of that round, which is what scf.while returns.
static void parse_while(const std::string &rest, Op &op, Lines &L, Block &blk) {
  const std::string tag = "_w" + std::to_string(op.line);
  std::vector<std::string> names, inits;
  const size_t open = rest.find('(');
  const size_t colon = top_colon(rest);
  if (open != std::string::npos && (colon == std::string::npos || open < colon)) {
    int depth = 0;
    size_t close = open;
    for (; close < rest.size(); close++) {
      if (rest[close] == '(') depth++;
      if (rest[close] == ')' && --depth == 0) break;
    }
    for (auto &pair : split_top(rest.substr(open + 1, close - open - 1), {","})) {
      const size_t q = pair.find('=');
      if (q == std::string::npos) continue;
      names.push_back(trim(pair.substr(0, q)));
      inits.push_back(trim(pair.substr(q + 1)));
    }
  }
  const size_t arrow = rest.rfind("->"), brace = rest.rfind('{');
  if (arrow == std::string::npos || brace == std::string::npos || brace < arrow) throw Unsupported("malformed scf.while: " + rest);
  op.result_types = parse_type_list(trim(rest.substr(arrow + 2, brace - arrow - 2)));
  if (op.result_types.size() != names.size() || op.results.size() != names.size())
    throw Unsupported("scf.while whose results are not its arguments (line " + std::to_string(op.line) + ")");
  Block before, after;
  parse_block(L, before);
  if (L.i >= L.v.size() || L.v[L.i] != "} do {") throw Unsupported("scf.while without a do region");
  L.i++;
  if (L.i < L.v.size() && L.v[L.i][0] == '^') {
    const std::string hdr = L.v[L.i++];
    const size_t o = hdr.find('('), c2 = hdr.rfind(')');
    if (o != std::string::npos && c2 != std::string::npos && c2 > o)
      for (auto &a : split_top(hdr.substr(o + 1, c2 - o - 1), {","})) {
        const size_t col = a.find(':');
        after.arg_names.push_back(trim(a.substr(0, col)));
        after.arg_types.push_back(parse_type(a.substr(col + 1)));
      }
  }
  parse_block(L, after);
  if (L.i >= L.v.size() || L.v[L.i] != "}") throw Unsupported("scf.while region not closed");
  L.i++;
  if (before.ops.empty() || before.ops.back()->name != "scf.condition") throw Unsupported("scf.while whose first region does not end in scf.condition");
  const Op &cond = *before.ops.back();
  if (cond.operands.size() != names.size() + 1 || after.arg_names.size() != names.size())
    throw Unsupported("scf.while whose condition passes on other values than the loop's arguments (line " + std::to_string(op.line) + ")");
  for (size_t j = 0; j < names.size(); j++)
    if (cond.operands[j + 1] != names[j])
      throw Unsupported("scf.while whose condition passes on other values than the loop's arguments (line " + std::to_string(op.line) + ")");
  // the two regions are siblings and may use the same names for different values: the first one's get a suffix
  Renames first, second;
  {
    std::vector<std::string> defs;
    collect_defs(before, defs);
    for (auto &d : defs) first[d] = d + tag;
    for (auto &n : names) first[n] = n + tag;
    for (size_t j = 0; j < names.size(); j++) second[after.arg_names[j]] = names[j] + tag;
  }
  auto constant = [&](const std::string &name, const std::string &value) {
    auto c = std::make_unique<Op>();
    c->name = "arith.constant";
    c->line = op.line;
    c->results.push_back(name);
    c->literal = value;
    Type t;
    t.elem = "i32";
    c->result_types.push_back(t);
    blk.ops.push_back(std::move(c));
  };
  constant("%lb" + tag, "0");
  constant("%ub" + tag, "2147483647");
  constant("%st" + tag, "1");
  op.name = "scf.for";
  op.iv = "%iv" + tag;
  op.operands = {"%lb" + tag, "%ub" + tag, "%st" + tag};
  for (auto &n : names) op.iter_names.push_back(n + tag);
  op.iter_inits = inits;
  op.regions.emplace_back();
  Block &body = op.regions.back();
  {
    Block renamed_before;
    copy_block(before, renamed_before, first);
    auto brk = std::make_unique<Op>();
    brk->name = "tts.break_unless";
    brk->line = op.line;
    brk->operands.push_back(renamed_before.ops.back()->operands.at(0));
    renamed_before.ops.pop_back();
    for (auto &o : renamed_before.ops) body.ops.push_back(std::move(o));
    body.ops.push_back(std::move(brk));
    Block renamed_after;
    copy_block(after, renamed_after, second);
    for (auto &o : renamed_after.ops) body.ops.push_back(std::move(o));
  }
}

static void parse_for(const std::string &rest, Op &op, Lines &L) {
  // %iv = %lb to %ub step %st [iter_args(%a = %x, ...) -> (types)] : i32 {
  size_t eq = rest.find(" = ");
  size_t to = rest.find(" to ");
  size_t st = rest.find(" step ");
  if (eq == std::string::npos || to == std::string::npos || st == std::string::npos)
    throw Unsupported("malformed scf.for: " + rest);
  op.iv = trim(rest.substr(0, eq));
  op.operands.push_back(trim(rest.substr(eq + 3, to - eq - 3)));
  op.operands.push_back(trim(rest.substr(to + 4, st - to - 4)));
  size_t after = st + 6;
  size_t e = after;
  while (e < rest.size() && (rest[e] == '%' || ssa_char(rest[e]))) e++;
  op.operands.push_back(rest.substr(after, e - after));
  size_t ia = rest.find("iter_args(", e);
  if (ia != std::string::npos) {
    size_t open = ia + 9;
    int depth = 0;
    size_t close = open;
    for (; close < rest.size(); close++) {
      if (rest[close] == '(') depth++;
      if (rest[close] == ')' && --depth == 0) break;
    }
    std::string inner = rest.substr(open + 1, close - open - 1);
    for (auto &pair : split_top(inner, {","})) {
      size_t q = pair.find('=');
      op.iter_names.push_back(trim(pair.substr(0, q)));
      op.iter_inits.push_back(trim(pair.substr(q + 1)));
    }
    size_t arrow = rest.find("->", close);
    size_t tcolon = rest.rfind(" : ");  // the induction variable's type, printed when it is not `index`
    if (tcolon == std::string::npos || tcolon < arrow) tcolon = rest.rfind('{');
    std::string tys = trim(rest.substr(arrow + 2, tcolon - arrow - 2));
    op.result_types = parse_type_list(tys);
    if (op.result_types.size() != op.iter_names.size())
      throw Unsupported("scf.for: iter_args/result type count mismatch");
  }
  op.regions.emplace_back();
  parse_block(L, op.regions.back());
  if (L.i >= L.v.size() || L.v[L.i] != "}") throw Unsupported("scf.for region not closed");
  L.i++;
}

static void parse_op(Lines &L, Block &blk) {
  std::string line = L.v[L.i];
  int line_no = (int)L.i + 1;
  L.i++;
  auto op = std::make_unique<Op>();
  op->line = line_no;
  std::string rest = line;
  if (line[0] == '%') {
    size_t eq = line.find(" = ");
    if (eq == std::string::npos) throw Unsupported("cannot parse: " + line);
    parse_results(line.substr(0, eq), *op);
    rest = trim(line.substr(eq + 3));
  }
  // operation name (quoted for the generic form)
  size_t p = 0;
  if (rest[0] == '"') {
    size_t q = rest.find('"', 1);
    op->name = rest.substr(1, q - 1);
    p = q + 1;
  } else {
    while (p < rest.size() && !isspace((unsigned char)rest[p]) && rest[p] != '(') p++;
    op->name = rest.substr(0, p);
  }
  rest = trim(rest.substr(p));

  if (op->name == "scf.for") {
    parse_for(rest, *op, L);
    blk.ops.push_back(std::move(op));
    return;
  }
  if (op->name == "scf.while") {
    parse_while(rest, *op, L, blk);
    blk.ops.push_back(std::move(op));
    return;
  }
  if (op->name == "arith.constant") {
    size_t c = std::string::npos;
    {
      // last top-level " : "
      int depth = 0;
      for (size_t i = 0; i + 2 < rest.size(); i++) {
        char ch = rest[i];
        if (ch == '<' || ch == '(' || ch == '[') depth++;
        else if (ch == '>' || ch == ')' || ch == ']') depth--;
        else if (depth == 0 && rest.compare(i, 3, " : ") == 0) c = i;
      }
    }
    if (c == std::string::npos) {
      op->literal = rest;
      Type t;
      t.elem = "i1";
      op->result_types.push_back(t);
    } else {
      op->literal = trim(rest.substr(0, c));
      op->result_types.push_back(parse_type(rest.substr(c + 3)));
    }
    blk.ops.push_back(std::move(op));
    return;
  }
  if (op->name == "scf.if") {
    // scf.if %c [-> (types)] {  ...  [} else {  ...]  }   ; with results both regions end in scf.yield
    size_t brace = rest.rfind('{');
    size_t arrow = rest.find("->");
    collect_operands(rest.substr(0, arrow == std::string::npos ? brace : arrow), op->operands);
    if (arrow != std::string::npos) op->result_types = parse_type_list(rest.substr(arrow + 2, brace - arrow - 2));
    if (op->result_types.size() != op->results.size()) throw Unsupported("scf.if: results and result types differ in number");
    op->regions.resize(2);
    parse_block(L, op->regions[0]);
    if (L.i < L.v.size() && L.v[L.i] == "} else {") {
      L.i++;
      parse_block(L, op->regions[1]);
    }
    if (L.i >= L.v.size() || L.v[L.i] != "}") throw Unsupported("scf.if region not closed");
    L.i++;
    blk.ops.push_back(std::move(op));
    return;
  }
  if (op->name == "tt.reduce" || op->name == "tt.scan") {
    // (%x[, %y]) <{axis = 0 : i32}> ({
    size_t close = rest.find(')');
    collect_operands(rest.substr(0, close + 1), op->operands);
    size_t a0 = rest.find("<{"), a1 = rest.find("}>");
    if (a0 != std::string::npos && a1 != std::string::npos)
      parse_attr_dict(rest.substr(a0 + 2, a1 - a0 - 2), op->attrs);
    if (rest.size() < 2 || rest.substr(rest.size() - 2) != "({")
      throw Unsupported("expected region after " + op->name);
    op->regions.emplace_back();
    Block &rb = op->regions.back();
    // ^bb0(%a: f32, %b: f32):
    if (L.i >= L.v.size()) throw Unsupported("region of " + op->name + " cut short");
    std::string hdr = L.v[L.i++];
    size_t o = hdr.find('('), c2 = hdr.rfind(')');
    if (!starts_with(hdr, "^") || o == std::string::npos || c2 == std::string::npos || c2 < o) throw Unsupported("expected block header: " + hdr);
    for (auto &a : split_top(hdr.substr(o + 1, c2 - o - 1), {","})) {
      size_t col = a.find(':');
      rb.arg_names.push_back(trim(a.substr(0, col)));
      rb.arg_types.push_back(parse_type(a.substr(col + 1)));
    }
    parse_block(L, rb);
    if (L.i >= L.v.size()) throw Unsupported("region of " + op->name + " not closed");
    std::string tail = L.v[L.i++];  // }) : (types) -> types
    if (!starts_with(tail, "})")) throw Unsupported("region of " + op->name + " not closed: " + tail);
    {  // the generic form carries the attributes here: }) {axis = 0 : i32} : (types) -> types
      const size_t b0 = tail.find('{'), b1 = tail.find('}', 2);
      if (b0 != std::string::npos && b1 != std::string::npos && b0 < tail.find("(", 2)) {
        parse_attr_dict(tail.substr(b0 + 1, b1 - b0 - 1), op->attrs);
        tail = "})" + tail.substr(b1 + 1);
      }
    }
    size_t col = tail.find(':');
    size_t arrow = tail.find("->");
    if (col == std::string::npos || arrow == std::string::npos || arrow < col) throw Unsupported("region of " + op->name + " without its types: " + tail);
    op->types = parse_type_list(tail.substr(col + 1, arrow - col - 1));
    op->result_types = parse_type_list(tail.substr(arrow + 2));
    blk.ops.push_back(std::move(op));
    return;
  }

  if (op->name == "tt.call") {  // @callee(%a, %b) : (i32, i32) -> i32
    const size_t at = rest.find('@'), open = rest.find('('), close = rest.find(')');
    if (at == std::string::npos || open == std::string::npos || close == std::string::npos) throw Unsupported("cannot parse: " + line);
    op->words.push_back(trim(rest.substr(at, open - at)));
    collect_operands(rest.substr(open, close - open + 1), op->operands);
    const size_t arrow = rest.find("->", close);
    if (arrow != std::string::npos) {
      std::string tys = trim(rest.substr(arrow + 2));
      if (tys != "()") op->result_types = parse_type_list(tys);
    }
    if (op->result_types.size() != op->results.size()) throw Unsupported("tt.call: results and result types differ in number");
    blk.ops.push_back(std::move(op));
    return;
  }
  // generic custom-assembly line: operands/words/attrs, then ':' types
  size_t colon = top_colon(rest);
  std::string head = colon == std::string::npos ? rest : rest.substr(0, colon);
  std::string tail = colon == std::string::npos ? "" : rest.substr(colon + 1);
  // attribute dictionary
  {
    int depth = 0;
    size_t open = std::string::npos;
    for (size_t i = 0; i < head.size(); i++) {
      if (head[i] == '{') {
        if (depth == 0) open = i;
        depth++;
      } else if (head[i] == '}') {
        if (--depth == 0 && open != std::string::npos) {
          parse_attr_dict(head.substr(open + 1, i - open - 1), op->attrs);
          head = head.substr(0, open) + " " + head.substr(i + 1);
          i = open;
          open = std::string::npos;
        }
      }
    }
  }
  collect_operands(head, op->operands);
  {
    std::string w;
    auto flush = [&]() {
      if (w.size() > 2 && w.front() == '"' && w.back() == '"') w = w.substr(1, w.size() - 2);  // generic form: "oeq"
      if (!w.empty() && w[0] != '%' && w != "=") op->words.push_back(w);
      w.clear();
    };
    for (char ch : head) {
      if (isspace((unsigned char)ch) || ch == ',') flush();
      else w.push_back(ch);
    }
    flush();
  }
  if (!tail.empty()) op->types = parse_type_list(tail);
  if (!rest.empty() && rest.back() == '{')
    throw Unsupported("operation with an unexpected region: " + op->name);
  blk.ops.push_back(std::move(op));
}

static void parse_block(Lines &L, Block &blk) {
  while (L.i < L.v.size()) {
    const std::string &line = L.v[L.i];
    if (line == "}" || starts_with(line, "})") || starts_with(line, "} else") || line == "} do {") return;
    parse_op(L, blk);
  }
}

// ---------------------------------------------------------------- copies of ops under new names
// Tail duplication (a block reached from two branches) and the inlining of calls both copy ops; every copy gets
// its own SSA names, so that nothing keyed by name downstream sees two definitions of one value.
static std::string renamed(const std::string &name, const Renames &m) {
  auto whole = m.find(name);  // one result of a pack ("%r#1") replaced by itself
  if (whole != m.end()) return whole->second;
  const size_t hash = name.find('#');
  auto it = m.find(hash == std::string::npos ? name : name.substr(0, hash));
  if (it == m.end()) return name;
  return hash == std::string::npos ? it->second : it->second + name.substr(hash);
}

static void collect_defs(const Block &b, std::vector<std::string> &out) {
  for (auto &a : b.arg_names) out.push_back(a);
  for (auto &op : b.ops) {
    for (auto &r : op->results) {
      const size_t hash = r.find('#');
      out.push_back(hash == std::string::npos ? r : r.substr(0, hash));
    }
    if (!op->iv.empty()) out.push_back(op->iv);
    for (auto &n : op->iter_names) out.push_back(n);
    for (auto &r : op->regions) collect_defs(r, out);
  }
}

static void copy_block(const Block &src, Block &dst, const Renames &m);

static std::unique_ptr<Op> copy_op(const Op &o, const Renames &m) {
  auto c = std::make_unique<Op>();
  c->name = o.name;
  c->result_types = o.result_types;
  c->words = o.words;
  c->attrs = o.attrs;
  c->types = o.types;
  c->literal = o.literal;
  c->line = o.line;
  for (auto &r : o.results) c->results.push_back(renamed(r, m));
  for (auto &r : o.operands) c->operands.push_back(renamed(r, m));
  c->iv = o.iv.empty() ? o.iv : renamed(o.iv, m);
  for (auto &r : o.iter_names) c->iter_names.push_back(renamed(r, m));
  for (auto &r : o.iter_inits) c->iter_inits.push_back(renamed(r, m));
  c->regions.resize(o.regions.size());
  for (size_t i = 0; i < o.regions.size(); i++) copy_block(o.regions[i], c->regions[i], m);
  return c;
}

static void copy_block(const Block &src, Block &dst, const Renames &m) {
  for (auto &a : src.arg_names) dst.arg_names.push_back(renamed(a, m));
  dst.arg_types = src.arg_types;
  for (auto &op : src.ops) dst.ops.push_back(copy_op(*op, m));
}

// "^bb1(%a, %b : i32, i32)" -> label and the values passed
static void parse_successor(const std::string &text, std::string &label, std::vector<std::string> &passed) {
  std::string t = trim(text);
  const size_t open = t.find('(');
  label = trim(t.substr(0, open));
  if (open == std::string::npos) return;
  const size_t colon = t.find(':', open);
  collect_operands(t.substr(open + 1, (colon == std::string::npos ? t.rfind(')') : colon) - open - 1), passed);
}

// The body of a function may be a graph of basic blocks (an early `return` under an `if` becomes cf.cond_br to a
// block that only returns; blocks that end alike are merged and take arguments).  It is rebuilt as nested "cf.if"
// ops with a then and an else region: a block reached from several places is copied to each of them, with the values
// passed to it in place of its arguments; control flow that loops is refused.  A `tt.return` with operands stays in
// the tree as an op (the body of a callee); one without ends its path.
static void parse_func_body(Lines &L, Block &out) {
  struct Cfg {
    Block ops;
    std::vector<std::string> arg_names;
    std::string term = "return", cond, a, b;
    std::vector<std::string> a_args, b_args, returned;
    int copies = 0;
    bool open = false;
  };
  std::map<std::string, Cfg> blocks;
  std::string cur = "^entry";
  blocks[cur];
  while (L.i < L.v.size()) {
    const std::string line = L.v[L.i];
    if (line == "}") break;
    if (line[0] == '^') {  // ^bb1:  or  ^bb1(%x: i32, %y: f32):
      size_t e = line.find_first_of(":(");
      if (e == std::string::npos) throw Unsupported("cannot parse: " + line);
      cur = line.substr(0, e);
      Cfg &c = blocks[cur];
      if (line[e] == '(') {
        const size_t close = line.rfind(')');
        for (auto &a : split_top(line.substr(e + 1, close - e - 1), {","})) c.arg_names.push_back(trim(a.substr(0, a.find(':'))));
      }
      L.i++;
      continue;
    }
    if (starts_with(line, "cf.cond_br")) {
      auto parts = split_top(line.substr(10), {","});
      // the values passed to a successor are separated by commas too: glue the pieces of one parenthesis together again
      std::vector<std::string> glued;
      int depth = 0;
      for (auto &piece : parts) {
        if (depth > 0) glued.back() += "," + piece;
        else glued.push_back(piece);
        for (char ch : piece) depth += ch == '(' ? 1 : ch == ')' ? -1 : 0;
      }
      if (glued.size() != 3) throw Unsupported("cannot parse: " + line);
      Cfg &c = blocks[cur];
      c.term = "cond_br";
      c.cond = trim(glued[0]);
      parse_successor(glued[1], c.a, c.a_args);
      parse_successor(glued[2], c.b, c.b_args);
      L.i++;
      continue;
    }
    if (starts_with(line, "cf.br")) {
      Cfg &c = blocks[cur];
      c.term = "br";
      parse_successor(line.substr(5), c.a, c.a_args);
      L.i++;
      continue;
    }
    if (starts_with(line, "tt.return")) {
      Cfg &c = blocks[cur];
      c.term = "return";
      const size_t colon = line.find(" : ");
      collect_operands(line.substr(9, colon == std::string::npos ? std::string::npos : colon - 9), c.returned);
      L.i++;
      continue;
    }
    parse_op(L, blocks[cur].ops);
  }
  int emitted = 0;
  std::function<void(const std::string &, const std::vector<std::string> &, const Renames &, Block &)> emit =
      [&](const std::string &label, const std::vector<std::string> &passed, const Renames &outer, Block &dst) {
        auto it = blocks.find(label);
        if (it == blocks.end()) throw Unsupported("branch to an unknown block " + label);
        Cfg &c = it->second;
        if (c.open) throw Unsupported("control flow that loops (block " + label + " reaches itself)");
        if (passed.size() != c.arg_names.size()) throw Unsupported("branch to " + label + " with the wrong number of values");
        // names visible in this copy: what the path so far renamed, this block's arguments, and (from the second copy
        // on) fresh names for everything the block defines
        Renames m = outer;
        for (size_t i = 0; i < passed.size(); i++) m[c.arg_names[i]] = passed[i];
        if (c.copies++) {
          std::vector<std::string> defs;
          collect_defs(c.ops, defs);
          for (auto &d : defs) m[d] = d + "__c" + std::to_string(c.copies);
        }
        if ((emitted += (int)c.ops.ops.size() + 1) > 20000) throw Unsupported("control flow too tangled to unfold");
        c.open = true;
        for (auto &o : c.ops.ops) dst.ops.push_back(copy_op(*o, m));
        auto values = [&](const std::vector<std::string> &v) {
          std::vector<std::string> out;
          for (auto &x : v) out.push_back(renamed(x, m));
          return out;
        };
        if (c.term == "br") {
          emit(c.a, values(c.a_args), m, dst);
        } else if (c.term == "cond_br") {
          auto op = std::make_unique<Op>();
          op->name = "cf.if";
          op->operands.push_back(renamed(c.cond, m));
          op->regions.resize(2);
          Op *raw = op.get();
          dst.ops.push_back(std::move(op));
          emit(c.a, values(c.a_args), m, raw->regions[0]);
          emit(c.b, values(c.b_args), m, raw->regions[1]);
        } else if (!c.returned.empty()) {
          auto op = std::make_unique<Op>();
          op->name = "tt.return";
          op->operands = values(c.returned);
          dst.ops.push_back(std::move(op));
        }
        c.open = false;
      };
  emit("^entry", {}, {}, out);
}

// ---------------------------------------------------------------- calls
// A function kept out of line (`noinline`) arrives as its own tt.func and a tt.call.  The reference's pipeline inlines
// it on the way down (triton-shared-opt runs the inliner before the conversion); here the callee's ops are copied to
// the call site under fresh names, arguments replaced by the call's operands and the call's results by what the callee
// returns.
struct Callee {
  Func f;
  bool busy = false;
};

// A callee that returns from both sides of a branch (`if c: return a` ... `return b`): the branch becomes an `if` that
// yields the returned values, followed by a single return of its results.  True when the block ends in one return.
static bool single_return(Block &b, const std::vector<Type> &types, int &serial) {
  if (b.ops.empty()) return false;
  Op &last = *b.ops.back();
  if (last.name == "tt.return") return true;
  if (last.name != "cf.if" || last.regions.size() != 2) return false;
  if (!single_return(last.regions[0], types, serial) || !single_return(last.regions[1], types, serial)) return false;
  for (auto &r : last.regions) r.ops.back()->name = "scf.yield";
  last.name = "scf.if";
  last.result_types = types;
  auto ret = std::make_unique<Op>();
  ret->name = "tt.return";
  for (size_t i = 0; i < types.size(); i++) {
    last.results.push_back("%ret__" + std::to_string(++serial) + "_" + std::to_string(i));
    ret->operands.push_back(last.results.back());
  }
  b.ops.push_back(std::move(ret));
  return true;
}

static void inline_calls(Block &b, std::map<std::string, Callee> &callees, Renames &subst, int &serial) {
  std::vector<std::unique_ptr<Op>> out;
  for (auto &held : b.ops) {
    Op &op = *held;
    for (auto &o : op.operands) o = renamed(o, subst);
    for (auto &o : op.iter_inits) o = renamed(o, subst);
    if (op.name != "tt.call") {
      for (auto &r : op.regions) inline_calls(r, callees, subst, serial);
      out.push_back(std::move(held));
      continue;
    }
    auto it = callees.find(op.words.at(0));
    if (it == callees.end()) throw Unsupported("call of an unknown function " + op.words.at(0));
    Callee &c = it->second;
    if (c.busy) throw Unsupported("recursive call of " + op.words.at(0));
    if (op.operands.size() != c.f.arg_names.size()) throw Unsupported("call of " + op.words.at(0) + " with the wrong number of arguments");
    Renames m;
    std::vector<std::string> defs;
    collect_defs(c.f.body, defs);
    const std::string tag = "__i" + std::to_string(++serial);
    for (auto &d : defs) m[d] = d + tag;
    for (size_t i = 0; i < op.operands.size(); i++) m[c.f.arg_names[i]] = op.operands[i];
    Block body;
    copy_block(c.f.body, body, m);
    c.busy = true;
    Renames inner;  // the callee's own calls
    inline_calls(body, callees, inner, serial);
    c.busy = false;
    std::vector<std::string> returned;
    if (!op.results.empty()) single_return(body, c.f.result_types, serial);
    if (!body.ops.empty() && body.ops.back()->name == "tt.return") {
      returned = body.ops.back()->operands;
      body.ops.pop_back();
    }
    if (returned.size() != op.results.size())
      throw Unsupported("call of " + op.words.at(0) + ": the callee returns its values from inside a loop or a nested region");
    for (size_t i = 0; i < returned.size(); i++) subst[op.results[i]] = returned[i];
    for (auto &o : body.ops) out.push_back(std::move(o));
  }
  b.ops = std::move(out);
}

Func parse_ttir(const std::string &text) {
  std::string clean = strip_locations(text);
  Lines L;
  {
    // one op per entry: a line whose parentheses are still open and that does not open a region (hand-written IR breaks
    // long signatures over several lines) is continued by the next one; `//` comments go
    std::istringstream is(clean);
    std::string ln, pending;
    int depth = 0;
    while (std::getline(is, ln)) {
      const size_t comment = ln.find("//");
      if (comment != std::string::npos) ln = ln.substr(0, comment);
      ln = trim(ln);
      if (ln.empty()) continue;
      if (ln == "{" && pending.empty() && !L.v.empty()) {  // a region's brace on a line of its own
        L.v.back() += " {";
        continue;
      }
      pending = pending.empty() ? ln : pending + " " + ln;
      depth = 0;
      for (char ch : pending) depth += ch == '(' ? 1 : ch == ')' ? -1 : 0;
      if (depth > 0 && pending.back() != '{') continue;
      L.v.push_back(pending);
      pending.clear();
    }
    if (!pending.empty()) L.v.push_back(pending);
  }
  Func kernel;
  std::map<std::string, Callee> callees;
  bool found = false;
  while (L.i < L.v.size()) {
    const std::string &line = L.v[L.i];
    if (starts_with(line, "module")) { L.i++; continue; }
    if (line == "}") { L.i++; continue; }
    if (starts_with(line, "tt.func")) {
      Func f;
      size_t at = line.find('@');
      size_t open = line.find('(', at);
      f.name = line.substr(at + 1, open - at - 1);
      const bool is_private = line.substr(0, at).find("private") != std::string::npos;
      int depth = 0;
      size_t close = open;
      for (; close < line.size(); close++) {
        if (line[close] == '(') depth++;
        if (line[close] == ')' && --depth == 0) break;
      }
      std::string args = line.substr(open + 1, close - open - 1);
      if (!trim(args).empty())
        for (auto &a : split_top(args, {","})) {
          size_t col = a.find(':');
          std::string ty = a.substr(col + 1);
          size_t brace = ty.find('{');
          if (brace != std::string::npos) ty = ty.substr(0, brace);
          f.arg_names.push_back(trim(a.substr(0, col)));
          f.arg_types.push_back(parse_type(ty));
        }
      bool has_results = false;
      {
        const size_t arrow = line.find("->", close), brace = line.rfind('{');
        if (arrow != std::string::npos && arrow < brace) {
          std::string res = trim(line.substr(arrow + 2, brace - arrow - 2));
          const size_t attr = res.find("attributes");
          if (attr != std::string::npos) res = trim(res.substr(0, attr));
          has_results = res != "()";
          if (has_results) f.result_types = parse_type_list(res);
        }
      }
      if (has_results && !is_private) throw Unsupported("tt.func with results is not a kernel");
      L.i++;
      parse_func_body(L, f.body);
      if (L.i >= L.v.size() || L.v[L.i] != "}") throw Unsupported("tt.func body not closed");
      L.i++;
      if (is_private) {
        callees["@" + f.name].f = std::move(f);
      } else {
        if (found) throw Unsupported("more than one public tt.func in the module");
        found = true;
        kernel = std::move(f);
      }
      continue;
    }
    throw Unsupported("unexpected top-level line: " + line);
  }
  if (!found) throw Unsupported("no tt.func found");
  Renames subst;
  int serial = 0;
  inline_calls(kernel.body, callees, subst, serial);
  return kernel;
}

}  // namespace tts
