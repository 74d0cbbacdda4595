// Text form of a structured program: the artefact the "ttsharedir" compile
// stage stores (the role ttshared.mlir plays in backend/compiler.py:48-67) and
// that the "obj" stage and the launcher read back.  One record per line,
// `key=value` fields, lists as [a,b,c]; everything after " ; " on a line is a
// human-readable rendering of the line's index expressions and is ignored by
// the reader.
#include <cstring>
#include <functional>
#include <sstream>

#include "structured.h"

namespace tts {

static const char *kind_name(SK k) {
  switch (k) {
    case SK::Load: return "load";
    case SK::Store: return "store";
    case SK::ScalarLoad: return "scalar_load";
    case SK::ScalarStore: return "scalar_store";
    case SK::Map: return "map";
    case SK::Splat: return "splat";
    case SK::Const: return "const";
    case SK::Iota: return "iota";
    case SK::FromIndex: return "from_index";
    case SK::ScalarArg: return "scalar_arg";
    case SK::Reduce: return "reduce";
    case SK::Scan: return "scan";
    case SK::Dot: return "dot";
    case SK::ExpandDims: return "expand_dims";
    case SK::Broadcast: return "broadcast";
    case SK::For: return "for";
    case SK::If: return "if";
  }
  return "?";
}

static SK kind_from(const std::string &s) {
  static const SK all[] = {SK::Load, SK::Store, SK::ScalarLoad, SK::ScalarStore, SK::Map, SK::Splat, SK::Const,
                           SK::Iota, SK::FromIndex, SK::ScalarArg, SK::Reduce, SK::Scan, SK::Dot, SK::ExpandDims, SK::If,
                           SK::Broadcast, SK::For};
  for (SK k : all)
    if (s == kind_name(k)) return k;
  throw Unsupported("structured text: unknown record '" + s + "'");
}

static std::string dbl_bits(double d) {
  uint64_t b;
  memcpy(&b, &d, 8);
  char buf[32];
  snprintf(buf, sizeof buf, "0x%016llx", (unsigned long long)b);
  return buf;
}
static double bits_dbl(const std::string &s) {
  uint64_t b = std::stoull(s, nullptr, 16);
  double d;
  memcpy(&d, &b, 8);
  return d;
}

template <class T>
static std::string list(const std::vector<T> &v, const char *prefix = "") {
  std::string s = "[";
  for (size_t i = 0; i < v.size(); i++) s += (i ? "," : "") + std::string(prefix) + std::to_string(v[i]);
  return s + "]";
}

std::string print_program(const Program &p) {
  std::ostringstream os;
  os << "tts.program 1 @" << p.name << "\n";
  for (size_t i = 0; i < p.arg_names.size(); i++)
    os << "arg " << i << " " << p.arg_names[i] << " " << p.arg_types[i].str() << "\n";
  // reachable index expressions
  std::vector<char> need(p.pool.size(), 0);
  std::function<void(int)> reach = [&](int e) {
    if (e < 0 || need[e]) return;
    need[e] = 1;
    const Expr &x = p.pool.at(e);
    switch (x.k) {
      case EK::Const: case EK::Arg: case EK::Pid: case EK::NProg: case EK::IV: case EK::Iter: case EK::Result: case EK::Data: break;
      case EK::Sext: case EK::Trunc: reach(x.a); break;
      case EK::CmpSel: reach(x.a); reach(x.b); reach(x.c); reach(x.d); break;
      default: reach(x.a); reach(x.b);
    }
  };
  std::function<void(const std::vector<SOp> &)> scan = [&](const std::vector<SOp> &ops) {
    for (auto &s : ops) {
      for (int e : s.acc.offsets) reach(e);
      for (int e : s.acc.strides) reach(e);
      for (int e : s.acc.dims) reach(e);
      for (int e : s.acc.mods) reach(e);
      reach(s.expr);
      if (s.kind == SK::For) {
        reach(s.lb); reach(s.ub); reach(s.step);
        for (auto &it : s.int_iters) { reach(it.iter_expr); reach(it.init); reach(it.next); reach(it.result_expr); }
        scan(s.body);
      } else if (!s.body.empty()) {
        scan(s.body);
      }
    }
  };
  scan(p.body);
  for (int e = 0; e < p.pool.size(); e++) {
    if (!need[e]) continue;
    const Expr &x = p.pool.at(e);
    os << "expr " << e << " " << (int)x.k << " " << (int)x.bits << " " << x.val << " " << x.a << " " << x.b << " "
       << x.c << " " << x.d << " ; " << p.pool.str(e) << "\n";
  }
  os << "values " << p.values.size() << "\n";
  std::function<void(const std::vector<SOp> &, int)> emit = [&](const std::vector<SOp> &ops, int depth) {
    std::string ind(depth * 2, ' ');
    auto vty = [&](int v) {
      std::string s = p.values[v].dtype + "[";
      for (size_t i = 0; i < p.values[v].shape.size(); i++) s += (i ? "," : "") + std::to_string(p.values[v].shape[i]);
      return s + "]";
    };
    auto exprs = [&](const std::vector<int> &v) {
      std::string s = "[";
      for (size_t i = 0; i < v.size(); i++) s += (i ? ", " : "") + p.pool.str(v[i]);
      return s + "]";
    };
    for (auto &s : ops) {
      os << ind << kind_name(s.kind);
      if (s.kind == SK::For) {
        os << " loop=" << s.loop << " lb=" << s.lb << " ub=" << s.ub << " step=" << s.step << " ; "
           << p.pool.str(s.lb) << " to " << p.pool.str(s.ub) << " step " << p.pool.str(s.step) << "\n";
        for (auto &it : s.int_iters)
          os << ind << "  int_iter iter=" << it.iter_expr << " init=" << it.init << " next=" << it.next
             << " result=" << it.result_expr << " ; " << p.pool.str(it.iter_expr) << " = " << p.pool.str(it.init)
             << " then " << p.pool.str(it.next) << "\n";
        for (size_t j = 0; j < s.tile_args.size(); j++)
          os << ind << "  tile_iter arg=" << s.tile_args[j] << ":" << vty(s.tile_args[j]) << " init=" << s.tile_inits[j]
             << " yield=" << s.tile_yields[j] << " result=" << s.results[j] << "\n";
        os << ind << "  {\n";
        emit(s.body, depth + 2);
        os << ind << "  }\n";
        continue;
      }
      if (s.result >= 0) os << " result=" << s.result << ":" << vty(s.result);
      if (!s.operands.empty()) os << " operands=" << list(s.operands);
      if (!s.name.empty()) os << " name=" << s.name;
      switch (s.kind) {
        case SK::Load: case SK::Store: case SK::ScalarLoad: case SK::ScalarStore:
          os << " base=" << s.acc.base_arg << " elem=" << s.acc.elem << " sizes=" << list(s.acc.sizes)
             << " offsets=" << list(s.acc.offsets) << " strides=" << list(s.acc.strides) << " dims=" << list(s.acc.dims);
          if (!s.acc.mods.empty()) os << " mods=" << list(s.acc.mods);
          if (s.acc.gather >= 0) os << " gather=" << s.acc.gather;
          if (s.acc.gather >= 0 || s.acc.mask_value >= 0) os << " maskv=" << s.acc.mask_value;
          if (s.acc.has_other) os << " other_f=" << dbl_bits(s.acc.other_f) << " other_i=" << s.acc.other_i;
          if (s.acc.other_value >= 0) os << " otherv=" << s.acc.other_value;
          os << " ; " << p.arg_names[s.acc.base_arg] << " offsets=" << exprs(s.acc.offsets)
             << " strides=" << exprs(s.acc.strides);
          if (!s.acc.dims.empty()) os << " dims=" << exprs(s.acc.dims);
          if (!s.acc.mods.empty()) {
            os << " wraps=[";
            for (size_t i = 0; i < s.acc.mods.size(); i++) os << (i ? ", " : "") << (s.acc.mods[i] < 0 ? std::string("-") : p.pool.str(s.acc.mods[i]));
            os << "]";
          }
          if (s.acc.has_other) os << " other=" << (s.acc.elem[0] == 'i' ? (double)s.acc.other_i : s.acc.other_f);
          break;
        case SK::Const: os << " fval=" << dbl_bits(s.fval) << " ival=" << s.ival << " ; " << (p.values[s.result].dtype[0] == 'i' ? (double)s.ival : s.fval); break;
        case SK::Iota: os << " ival=" << s.ival; break;
        case SK::ScalarArg: os << " ival=" << s.ival << " ; " << p.arg_names[s.ival]; break;
        case SK::FromIndex: os << " expr=" << s.expr << " ; " << p.pool.str(s.expr); break;
        case SK::Reduce: case SK::ExpandDims: os << " axis=" << s.axis; break;
        case SK::Scan: os << " axis=" << s.axis << " ival=" << s.ival; break;
        case SK::If: os << " ival=" << s.ival; break;
        default: break;
      }
      if (((s.kind == SK::Reduce || s.kind == SK::Scan) && !s.tile_args.empty()) || s.kind == SK::If) {
        os << " region=1\n";
        for (int a : s.tile_args) os << ind << "  region_arg arg=" << a << ":" << vty(a) << "\n";
        for (size_t j = 0; j < s.results.size(); j++)
          os << ind << "  region_result value=" << s.results[j] << ":" << vty(s.results[j]) << " yield=" << s.tile_yields[j] << "\n";
        os << ind << "  {\n";
        emit(s.body, depth + 2);
        os << ind << "  }\n";
        continue;
      }
      os << "\n";
    }
  };
  os << "body {\n";
  emit(p.body, 1);
  os << "}\n";
  return os.str();
}

// ------------------------------------------------------------------ reader

namespace {
struct Fields {
  std::string head;
  std::map<std::string, std::string> kv;
  const std::string &get(const std::string &k) const {
    auto it = kv.find(k);
    if (it == kv.end()) throw Unsupported("structured text: record '" + head + "' lacks field " + k);
    return it->second;
  }
  bool has(const std::string &k) const { return kv.count(k) != 0; }
};

Fields split_fields(std::string line) {
  size_t sc = line.find(" ; ");
  if (sc != std::string::npos) line = line.substr(0, sc);
  std::istringstream is(line);
  Fields f;
  is >> f.head;
  std::string tok;
  while (is >> tok) {
    size_t eq = tok.find('=');
    if (eq == std::string::npos) f.kv["#" + std::to_string(f.kv.size())] = tok;
    else f.kv[tok.substr(0, eq)] = tok.substr(eq + 1);
  }
  return f;
}

std::vector<int64_t> parse_list(const std::string &s) {
  std::vector<int64_t> out;
  if (s.size() < 2) return out;
  std::string in = s.substr(1, s.size() - 2);
  std::istringstream is(in);
  std::string t;
  while (std::getline(is, t, ','))
    if (!t.empty()) out.push_back(std::stoll(t));
  return out;
}
}  // namespace

Program read_program(const std::string &text) {
  Program p;
  std::istringstream is(text);
  std::string line;
  std::map<int, int> emap;  // file expr id -> pool id
  auto E = [&](int64_t id) -> int {
    if (id < 0) return -1;
    auto it = emap.find((int)id);
    if (it == emap.end()) throw Unsupported("structured text: reference to undefined expr " + std::to_string(id));
    return it->second;
  };
  auto Es = [&](const std::string &s) {
    std::vector<int> out;
    for (auto v : parse_list(s)) out.push_back(E(v));
    return out;
  };
  auto value_ref = [&](const std::string &s, bool typed) {
    // "id" or "id:dtype[d0,d1]"
    size_t colon = s.find(':');
    int id = std::stoi(s.substr(0, colon));
    if (typed && colon != std::string::npos) {
      if ((size_t)id >= p.values.size()) throw Unsupported("structured text: value id out of range");
      size_t br = s.find('[', colon);
      p.values[id].dtype = s.substr(colon + 1, br - colon - 1);
      p.values[id].shape = parse_list(s.substr(br));
    }
    return id;
  };
  std::vector<std::vector<SOp> *> stack;
  std::vector<SOp *> open_fors;
  bool in_body = false;
  while (std::getline(is, line)) {
    size_t a = line.find_first_not_of(" \t");
    if (a == std::string::npos) continue;
    line = line.substr(a);
    if (!in_body) {
      if (line.rfind("tts.program", 0) == 0) {
        size_t at = line.find('@');
        p.name = line.substr(at + 1);
        continue;
      }
      if (line.rfind("arg ", 0) == 0) {
        std::istringstream ls(line);
        std::string kw, idx, name, ty;
        ls >> kw >> idx >> name;
        std::getline(ls, ty);
        p.arg_names.push_back(name);
        p.arg_types.push_back(parse_type(ty));
        continue;
      }
      if (line.rfind("expr ", 0) == 0) {
        std::istringstream ls(line);
        std::string kw;
        int id, k, bits;
        Expr x{};
        ls >> kw >> id >> k >> bits >> x.val >> x.a >> x.b >> x.c >> x.d;
        x.k = (EK)k;
        x.bits = (uint8_t)bits;
        switch (x.k) {
          case EK::Const: case EK::Arg: case EK::Pid: case EK::NProg: case EK::IV: case EK::Iter: case EK::Result: case EK::Data: break;
          case EK::Sext: case EK::Trunc: x.a = E(x.a); break;
          case EK::CmpSel: x.a = E(x.a); x.b = E(x.b); x.c = E(x.c); x.d = E(x.d); break;
          default: x.a = E(x.a); x.b = E(x.b);
        }
        emap[id] = p.pool.push_raw(x);
        continue;
      }
      if (line.rfind("values ", 0) == 0) {
        p.values.resize(std::stoul(line.substr(7)));
        continue;
      }
      if (line == "body {") {
        in_body = true;
        stack.push_back(&p.body);
        continue;
      }
      throw Unsupported("structured text: unexpected line '" + line + "'");
    }
    if (line == "{") continue;
    if (line == "}") {
      if (stack.size() > 1) open_fors.pop_back();
      stack.pop_back();
      if (stack.empty()) in_body = false;
      continue;
    }
    Fields f = split_fields(line);
    if (f.head == "int_iter") {
      IntIter it;
      it.iter_expr = E(std::stoll(f.get("iter")));
      it.init = E(std::stoll(f.get("init")));
      it.next = E(std::stoll(f.get("next")));
      it.result_expr = E(std::stoll(f.get("result")));
      open_fors.back()->int_iters.push_back(it);
      continue;
    }
    if (f.head == "tile_iter") {
      SOp *fo = open_fors.back();
      fo->tile_args.push_back(value_ref(f.get("arg"), true));
      fo->tile_inits.push_back(std::stoi(f.get("init")));
      fo->tile_yields.push_back(std::stoi(f.get("yield")));
      int r = std::stoi(f.get("result"));
      fo->results.push_back(r);
      if (r >= 0) p.values[r] = p.values[fo->tile_args.back()];
      continue;
    }
    if (f.head == "region_arg") {
      open_fors.back()->tile_args.push_back(value_ref(f.get("arg"), true));
      continue;
    }
    if (f.head == "region_result") {
      open_fors.back()->results.push_back(value_ref(f.get("value"), true));
      open_fors.back()->tile_yields.push_back(std::stoi(f.get("yield")));
      continue;
    }
    SOp s;
    s.kind = kind_from(f.head);
    if (s.kind == SK::For) {
      s.loop = std::stoi(f.get("loop"));
      p.num_loops = std::max(p.num_loops, s.loop + 1);
      s.lb = E(std::stoll(f.get("lb")));
      s.ub = E(std::stoll(f.get("ub")));
      s.step = E(std::stoll(f.get("step")));
      stack.back()->push_back(std::move(s));
      SOp *fo = &stack.back()->back();
      open_fors.push_back(fo);
      stack.push_back(&fo->body);
      continue;
    }
    if (f.has("result")) s.result = value_ref(f.get("result"), true);
    if (f.has("operands"))
      for (auto v : parse_list(f.get("operands"))) s.operands.push_back((int)v);
    if (f.has("name")) s.name = f.get("name");
    if (f.has("base")) {
      s.acc.base_arg = std::stoi(f.get("base"));
      s.acc.elem = f.get("elem");
      s.acc.sizes = parse_list(f.get("sizes"));
      s.acc.offsets = Es(f.get("offsets"));
      s.acc.strides = Es(f.get("strides"));
      s.acc.dims = Es(f.get("dims"));
      if (f.has("mods")) s.acc.mods = Es(f.get("mods"));
      if (f.has("gather")) s.acc.gather = std::stoi(f.get("gather"));
      if (f.has("maskv")) s.acc.mask_value = std::stoi(f.get("maskv"));
      if (f.has("otherv")) s.acc.other_value = std::stoi(f.get("otherv"));
      if (f.has("other_f")) {
        s.acc.has_other = true;
        s.acc.other_f = bits_dbl(f.get("other_f"));
        s.acc.other_i = std::stoll(f.get("other_i"));
      }
    }
    if (f.has("fval")) s.fval = bits_dbl(f.get("fval"));
    if (f.has("ival")) s.ival = std::stoll(f.get("ival"));
    if (f.has("expr")) s.expr = E(std::stoll(f.get("expr")));
    if (f.has("axis")) s.axis = std::stoi(f.get("axis"));
    const bool region = f.has("region");
    stack.back()->push_back(std::move(s));
    if (region) {  // the combiner's ops follow in a block of their own
      SOp *ro = &stack.back()->back();
      open_fors.push_back(ro);
      stack.push_back(&ro->body);
    }
  }
  if (p.name.empty()) throw Unsupported("structured text: missing tts.program header");
  return p;
}

}  // namespace tts
