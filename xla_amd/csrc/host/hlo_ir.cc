// HLO text subset: data structures, printer and parser (see hlo_ir.h).
#include "hlo_ir.h"

#include <ctype.h>

#include <algorithm>
#include <sstream>
#include <unordered_map>
#include <unordered_set>

namespace xla_amd {
namespace hlo {

// ---------------------------------------------------------------- Shape
int64_t Shape::num_elements() const {
  int64_t n = 1;
  for (int64_t d : dims) n *= d;
  return n;
}

Shape Shape::Array(const std::string& dtype, std::vector<int64_t> dims) {
  Shape s;
  s.dtype = dtype;
  s.dims = std::move(dims);
  std::string l;
  for (int64_t i = (int64_t)s.dims.size() - 1; i >= 0; --i) l += (l.empty() ? "" : ",") + std::to_string(i);
  s.layout = l;  // default major-to-minor
  return s;
}

Shape Shape::Tuple(std::vector<Shape> elements) {
  Shape s;
  s.is_tuple = true;
  s.elements = std::move(elements);
  return s;
}

std::string Shape::ToString() const {
  if (is_tuple) {
    std::string out = "(";
    for (size_t i = 0; i < elements.size(); ++i) out += (i ? ", " : "") + elements[i].ToString();
    return out + ")";
  }
  std::string out = dtype + "[";
  for (size_t i = 0; i < dims.size(); ++i) out += (i ? "," : "") + std::to_string(dims[i]);
  out += "]";
  if (!layout.empty()) out += "{" + layout + "}";
  return out;
}

// ---------------------------------------------------------------- Instr
const std::string* Instr::Attr(const std::string& key) const {
  for (const auto& kv : attrs)
    if (kv.first == key) return &kv.second;
  return nullptr;
}

void Instr::SetAttr(const std::string& key, const std::string& value) {
  for (auto& kv : attrs)
    if (kv.first == key) {
      kv.second = value;
      return;
    }
  attrs.emplace_back(key, value);
}

std::vector<int64_t> Instr::DimsAttr(const std::string& key) const {
  std::vector<int64_t> out;
  const std::string* v = Attr(key);
  if (!v) return out;
  int64_t cur = 0;
  bool have = false;
  for (char c : *v) {
    if (isdigit((unsigned char)c)) {
      cur = cur * 10 + (c - '0');
      have = true;
    } else if (have) {
      out.push_back(cur);
      cur = 0;
      have = false;
    }
  }
  if (have) out.push_back(cur);
  return out;
}

// ---------------------------------------------------------------- Computation
Instr* Computation::root() const {
  for (const auto& i : instrs)
    if (i->is_root) return i.get();
  return instrs.empty() ? nullptr : instrs.back().get();
}

Instr* Computation::Find(const std::string& n) const {
  for (const auto& i : instrs)
    if (i->name == n) return i.get();
  return nullptr;
}

void Computation::RecomputeUsers() {
  for (auto& i : instrs) i->users.clear();
  for (auto& i : instrs)
    for (Instr* op : i->operands)
      if (std::find(op->users.begin(), op->users.end(), i.get()) == op->users.end()) op->users.push_back(i.get());
}

Instr* Computation::Insert(std::unique_ptr<Instr> ins, const Instr* before) {
  Instr* raw = ins.get();
  auto pos = instrs.end();
  if (before)
    pos = std::find_if(instrs.begin(), instrs.end(),
                       [&](const std::unique_ptr<Instr>& p) { return p.get() == before; });
  instrs.insert(pos, std::move(ins));
  return raw;
}

void Computation::ReplaceAllUses(Instr* from, Instr* to) {
  for (auto& i : instrs)
    for (Instr*& op : i->operands)
      if (op == from) op = to;
  if (from->is_root) {
    from->is_root = false;
    to->is_root = true;
  }
  RecomputeUsers();
}

bool HasSideEffect(const Instr& i) {
  static const char* const kOps[] = {"after-all", "infeed", "outfeed", "send", "send-done", "recv", "recv-done",
                                     "rng", "rng-get-and-update-state", "partition-id", "replica-id",
                                     "all-reduce", "all-reduce-start", "all-reduce-done", "all-gather",
                                     "all-gather-start", "all-gather-done", "all-to-all", "ragged-all-to-all",
                                     "collective-permute", "collective-permute-start", "collective-permute-done",
                                     "collective-broadcast", "reduce-scatter", "async-start", "async-update",
                                     "async-done", "copy-start", "copy-done", "set-dimension-size",
                                     "add-dependency", "opt-barrier", "while", "conditional", "call"};
  for (const char* op : kOps)
    if (i.opcode == op) return true;
  if (i.opcode == "custom-call") {
    const std::string* v = i.Attr("custom_call_has_side_effect");
    return v && *v == "true";
  }
  return false;
}

std::set<const Instr*> Computation::Unused() {
  RecomputeUsers();
  std::set<const Instr*> out;
  const Instr* r = root();
  for (const auto& i : instrs)
    if (i.get() != r && i->users.empty() && i->opcode != "parameter") out.insert(i.get());
  return out;
}

int Computation::RemoveDead(const std::set<const Instr*>& keep) {
  int removed = 0;
  for (;;) {
    RecomputeUsers();
    Instr* r = root();
    auto it = std::find_if(instrs.begin(), instrs.end(), [&](const std::unique_ptr<Instr>& p) {
      return p.get() != r && p->users.empty() && p->opcode != "parameter" && !HasSideEffect(*p) &&
             !keep.count(p.get());
    });
    if (it == instrs.end()) break;
    instrs.erase(it);
    ++removed;
  }
  return removed;
}

void Computation::SortDefBeforeUse() {
  std::vector<std::unique_ptr<Instr>> old = std::move(instrs);
  instrs.clear();
  std::unordered_map<const Instr*, size_t> index;
  for (size_t i = 0; i < old.size(); ++i) index[old[i].get()] = i;
  std::vector<char> state(old.size(), 0);  // 0 new, 1 on the stack, 2 emitted
  // iterative post-order from each instruction in list order
  for (size_t start = 0; start < old.size(); ++start) {
    if (state[start]) continue;
    std::vector<std::pair<size_t, size_t>> stack = {{start, 0}};
    state[start] = 1;
    while (!stack.empty()) {
      auto& [at, next] = stack.back();
      Instr* ins = old[at].get();
      if (next < ins->operands.size()) {
        auto it = index.find(ins->operands[next++]);
        if (it != index.end() && state[it->second] == 0) {
          state[it->second] = 1;
          stack.push_back({it->second, 0});
        }
        continue;
      }
      state[at] = 2;
      instrs.push_back(std::move(old[at]));
      stack.pop_back();
    }
  }
  RecomputeUsers();
}

std::string Computation::UniqueName(const std::string& base) const {
  if (!Find(base)) return base;
  for (int n = 1;; ++n) {
    std::string c = base + "." + std::to_string(n);
    if (!Find(c)) return c;
  }
}

// ---------------------------------------------------------------- Module
Computation* Module::entry() const {
  for (const auto& c : computations)
    if (c->is_entry) return c.get();
  return computations.empty() ? nullptr : computations.back().get();
}

Computation* Module::FindComputation(const std::string& n) const {
  for (const auto& c : computations)
    if (c->name == n) return c.get();
  return nullptr;
}

std::string Module::ToString() const {
  std::ostringstream os;
  os << header << "\n";
  for (const auto& c : computations) {
    os << "\n" << (c->is_entry ? "ENTRY " : "") << "%" << c->name << " {\n";
    const Instr* root = c->root();
    for (const auto& i : c->instrs) {
      os << "  " << (i.get() == root ? "ROOT " : "") << "%" << i->name << " = " << i->shape.ToString() << " "
         << i->opcode << "(";
      if (i->opcode == "constant" || i->opcode == "parameter") {
        os << i->literal;
      } else {
        for (size_t k = 0; k < i->operands.size(); ++k) os << (k ? ", " : "") << "%" << i->operands[k]->name;
      }
      os << ")";
      for (const auto& kv : i->attrs) os << ", " << kv.first << "=" << kv.second;
      os << "\n";
    }
    os << "}\n";
  }
  return os.str();
}

// ---------------------------------------------------------------- Parser
namespace {

struct Cursor {
  const std::string& s;
  size_t p = 0;
  explicit Cursor(const std::string& str) : s(str) {}
  void SkipWs() {
    while (p < s.size() && (s[p] == ' ' || s[p] == '\t')) ++p;
  }
  bool Eat(char c) {
    SkipWs();
    if (p < s.size() && s[p] == c) {
      ++p;
      return true;
    }
    return false;
  }
  bool AtEnd() {
    SkipWs();
    return p >= s.size();
  }
  char Peek() {
    SkipWs();
    return p < s.size() ? s[p] : 0;
  }
};

bool IsIdentChar(char c) { return isalnum((unsigned char)c) || c == '_' || c == '.' || c == '-'; }

bool ParseShape(Cursor& c, Shape* out, std::string* err) {
  c.SkipWs();
  if (c.Eat('(')) {
    out->is_tuple = true;
    if (c.Eat(')')) return true;
    for (;;) {
      Shape e;
      if (!ParseShape(c, &e, err)) return false;
      out->elements.push_back(e);
      if (c.Eat(',')) continue;
      if (c.Eat(')')) return true;
      *err = "malformed tuple shape";
      return false;
    }
  }
  size_t b = c.p;
  while (c.p < c.s.size() && (isalnum((unsigned char)c.s[c.p]) || c.s[c.p] == '_')) ++c.p;
  out->dtype = c.s.substr(b, c.p - b);
  if (out->dtype.empty() || c.p >= c.s.size() || c.s[c.p] != '[') {
    if (out->dtype == "token") return true;
    *err = "expected a shape near `" + c.s.substr(b, 24) + "`";
    return false;
  }
  ++c.p;
  int64_t cur = 0;
  bool have = false;
  for (; c.p < c.s.size(); ++c.p) {
    char ch = c.s[c.p];
    if (isdigit((unsigned char)ch)) {
      cur = cur * 10 + (ch - '0');
      have = true;
    } else if (ch == ',' || ch == ']') {
      if (have) out->dims.push_back(cur);
      cur = 0;
      have = false;
      if (ch == ']') break;
    } else if (ch == ' ' || ch == '<' || ch == '=' || ch == '?') {
      // dynamic-dimension decorations are not supported; plain spaces are skipped
      if (ch != ' ') {
        *err = "dynamic dimensions are not supported";
        return false;
      }
    } else {
      *err = "bad character in shape dimensions";
      return false;
    }
  }
  if (c.p >= c.s.size()) {
    *err = "unterminated shape";
    return false;
  }
  ++c.p;  // ']'
  if (c.p < c.s.size() && c.s[c.p] == '{') {
    size_t e = c.s.find('}', c.p);
    if (e == std::string::npos) {
      *err = "unterminated layout";
      return false;
    }
    out->layout = c.s.substr(c.p + 1, e - c.p - 1);
    c.p = e + 1;
  }
  return true;
}

// Splits `s` at top-level commas (outside (), [], {}, "").
std::vector<std::string> SplitTopLevel(const std::string& s) {
  std::vector<std::string> out;
  int depth = 0;
  bool quote = false;
  std::string cur;
  for (size_t i = 0; i < s.size(); ++i) {
    char ch = s[i];
    if (quote) {
      cur += ch;
      if (ch == '\\' && i + 1 < s.size()) cur += s[++i];
      else if (ch == '"') quote = false;
      continue;
    }
    if (ch == '"') quote = true;
    if (ch == '(' || ch == '[' || ch == '{') ++depth;
    if (ch == ')' || ch == ']' || ch == '}') --depth;
    if (ch == ',' && depth == 0) {
      out.push_back(cur);
      cur.clear();
      continue;
    }
    cur += ch;
  }
  if (!cur.empty()) out.push_back(cur);
  for (std::string& t : out) {
    size_t b = t.find_first_not_of(" \t"), e = t.find_last_not_of(" \t");
    t = b == std::string::npos ? "" : t.substr(b, e - b + 1);
  }
  return out;
}

std::string StripComment(const std::string& line) {
  // `//` comments (FileCheck directives live in them) and /*...*/ index comments
  std::string out;
  bool quote = false;
  for (size_t i = 0; i < line.size(); ++i) {
    char ch = line[i];
    if (ch == '"') quote = !quote;
    if (!quote && ch == '/' && i + 1 < line.size() && line[i + 1] == '/') break;
    if (!quote && ch == '/' && i + 1 < line.size() && line[i + 1] == '*') {
      size_t e = line.find("*/", i + 2);
      if (e == std::string::npos) break;
      i = e + 1;
      continue;
    }
    out += ch;
  }
  return out;
}

}  // namespace

std::unique_ptr<Module> Parse(const std::string& text, std::string* error) {
  auto mod = std::make_unique<Module>();
  std::istringstream in(text);
  std::string raw;
  Computation* comp = nullptr;
  std::unordered_map<std::string, Instr*> by_name;
  int lineno = 0;
  auto fail = [&](const std::string& why) {
    *error = "line " + std::to_string(lineno) + ": " + why;
    return nullptr;
  };
  while (std::getline(in, raw)) {
    ++lineno;
    std::string line = StripComment(raw);
    size_t b = line.find_first_not_of(" \t\r");
    if (b == std::string::npos) continue;
    size_t e = line.find_last_not_of(" \t\r");
    line = line.substr(b, e - b + 1);
    if (line.rfind("HloModule", 0) == 0) {
      mod->header = line;
      continue;
    }
    if (line == "}") {
      comp = nullptr;
      continue;
    }
    if (!comp) {
      // computation header: [ENTRY] %name [(params) -> shape] {
      if (line.back() != '{') return fail("expected a computation header, got `" + line + "`");
      auto c = std::make_unique<Computation>();
      std::string h = line.substr(0, line.size() - 1);
      if (h.rfind("ENTRY", 0) == 0) {
        c->is_entry = true;
        h = h.substr(5);
      }
      size_t nb = h.find_first_not_of(" \t%");
      if (nb == std::string::npos) return fail("computation without a name");
      size_t ne = nb;
      while (ne < h.size() && IsIdentChar(h[ne])) ++ne;
      if (ne == nb) return fail("computation without a name");
      c->name = h.substr(nb, ne - nb);
      comp = c.get();
      mod->computations.push_back(std::move(c));
      by_name.clear();
      continue;
    }
    // instruction: [ROOT] %name = shape opcode(operands), attrs
    auto ins = std::make_unique<Instr>();
    Cursor c(line);
    if (line.rfind("ROOT ", 0) == 0) {
      ins->is_root = true;
      c.p = 5;
    }
    c.SkipWs();
    if (c.Peek() == '%') ++c.p;
    size_t nb = c.p;
    while (c.p < line.size() && IsIdentChar(line[c.p])) ++c.p;
    ins->name = line.substr(nb, c.p - nb);
    if (ins->name.empty() || !c.Eat('=')) return fail("expected `name = ...`");
    std::string err;
    if (!ParseShape(c, &ins->shape, &err)) return fail(err);
    c.SkipWs();
    size_t ob = c.p;
    while (c.p < line.size() && IsIdentChar(line[c.p])) ++c.p;
    ins->opcode = line.substr(ob, c.p - ob);
    if (ins->opcode.empty() || !c.Eat('(')) return fail("expected `opcode(`");
    // operand list up to the matching ')'
    int depth = 1;
    bool quote = false;
    size_t ab = c.p;
    for (; c.p < line.size(); ++c.p) {
      char ch = line[c.p];
      if (ch == '"') quote = !quote;
      if (quote) continue;
      if (ch == '(' || ch == '[' || ch == '{') ++depth;
      if (ch == ')' || ch == ']' || ch == '}') --depth;
      if (depth == 0) break;
    }
    if (c.p >= line.size()) return fail("unterminated operand list");
    std::string args = line.substr(ab, c.p - ab);
    ++c.p;
    if (ins->opcode == "constant" || ins->opcode == "parameter") {
      ins->literal = args;
    } else {
      for (const std::string& a : SplitTopLevel(args)) {
        if (a.empty()) continue;
        size_t sp = a.find_last_of(" \t");
        std::string nm = sp == std::string::npos ? a : a.substr(sp + 1);
        if (!nm.empty() && nm[0] == '%') nm = nm.substr(1);
        auto it = by_name.find(nm);
        if (it == by_name.end()) return fail("operand `" + nm + "` is not defined before its use");
        ins->operands.push_back(it->second);
      }
    }
    std::string rest = c.p < line.size() ? line.substr(c.p) : "";
    for (const std::string& kv : SplitTopLevel(rest)) {
      if (kv.empty()) continue;
      size_t eq = kv.find('=');
      if (eq == std::string::npos) return fail("expected attribute `key=value`, got `" + kv + "`");
      ins->attrs.emplace_back(kv.substr(0, eq), kv.substr(eq + 1));
    }
    if (by_name.count(ins->name)) return fail("duplicate instruction name `" + ins->name + "`");
    by_name[ins->name] = ins.get();
    comp->instrs.push_back(std::move(ins));
  }
  if (mod->computations.empty()) {
    *error = "no computation found";
    return nullptr;
  }
  if (mod->header.empty()) mod->header = "HloModule module";
  bool any_entry = false;
  for (auto& cp : mod->computations) any_entry |= cp->is_entry;
  if (!any_entry) mod->computations.back()->is_entry = true;
  for (auto& cp : mod->computations) {
    bool has_root = false;
    for (auto& i : cp->instrs) has_root |= i->is_root;
    if (!has_root && !cp->instrs.empty()) cp->instrs.back()->is_root = true;
    cp->RecomputeUsers();
  }
  return mod;
}

}  // namespace hlo
}  // namespace xla_amd
