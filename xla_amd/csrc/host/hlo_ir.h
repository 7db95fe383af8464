// A small in-memory form of HLO text: enough of the grammar that XLA prints
// (xla/hlo/parser/hlo_parser.cc) to hold the quantized-inference patterns, rewrite them and
// print the module back.  One instruction per line, as HloModule::ToString() emits.
#ifndef XLA_AMD_CSRC_HOST_HLO_IR_H_
#define XLA_AMD_CSRC_HOST_HLO_IR_H_

#include <stdint.h>

#include <memory>
#include <set>
#include <string>
#include <utility>
#include <vector>

namespace xla_amd {
namespace hlo {

struct Shape {
  bool is_tuple = false;
  std::string dtype;            // "f32", "bf16", "f8e4m3fn", "s4", ...
  std::vector<int64_t> dims;
  std::string layout;           // text between {} after the dims, "" if none was given
  std::vector<Shape> elements;  // tuple elements

  int64_t rank() const { return (int64_t)dims.size(); }
  int64_t num_elements() const;
  bool SameDims(const Shape& o) const { return !is_tuple && !o.is_tuple && dims == o.dims; }
  std::string ToString() const;
  static Shape Array(const std::string& dtype, std::vector<int64_t> dims);
  static Shape Tuple(std::vector<Shape> elements);
};

struct Instr {
  std::string name;     // without the leading '%'
  std::string opcode;   // "dot", "custom-call", ...
  Shape shape;
  std::vector<Instr*> operands;
  std::string literal;  // text inside constant(...) / parameter(...)
  std::vector<std::pair<std::string, std::string>> attrs;  // in source order, values verbatim
  bool is_root = false;
  std::vector<Instr*> users;  // filled by Computation::RecomputeUsers

  const std::string* Attr(const std::string& key) const;
  void SetAttr(const std::string& key, const std::string& value);
  // "{1,0}" -> {1,0}; missing or empty -> {}
  std::vector<int64_t> DimsAttr(const std::string& key) const;
  bool Is(const char* op) const { return opcode == op; }
  int64_t user_count() const { return (int64_t)users.size(); }
};

// Side effects as HloInstruction::HasSideEffect sees them (xla/hlo/ir/hlo_instruction.cc): the
// opcode itself, or custom_call_has_side_effect=true on a custom call.
bool HasSideEffect(const Instr& i);

struct Computation {
  std::string name;
  bool is_entry = false;
  std::vector<std::unique_ptr<Instr>> instrs;  // def before use

  Instr* root() const;
  Instr* Find(const std::string& name) const;
  void RecomputeUsers();
  // Inserts `ins` right before `before` (or at the end when null) and returns it.
  Instr* Insert(std::unique_ptr<Instr> ins, const Instr* before);
  // Every use of `from` (and its root flag) moves to `to`.
  void ReplaceAllUses(Instr* from, Instr* to);
  // Instructions nothing uses right now (root and parameters left out): what a later
  // RemoveDead must not touch because the module came that way.
  std::set<const Instr*> Unused();
  // Drops instructions that nothing uses any more, except the root, parameters, instructions with
  // side effects (HasSideEffect) and those in `keep`.  Returns how many.
  int RemoveDead(const std::set<const Instr*>& keep);
  // Stable re-ordering so that every operand precedes its users: instructions keep their relative
  // order except where an operand has to move up in front of an earlier user.
  void SortDefBeforeUse();
  std::string UniqueName(const std::string& base) const;
};

struct Module {
  std::string header;  // the "HloModule ..." line, verbatim
  std::vector<std::unique_ptr<Computation>> computations;

  Computation* entry() const;
  Computation* FindComputation(const std::string& name) const;
  std::string ToString() const;
};

// Returns null and fills *error on malformed input.
std::unique_ptr<Module> Parse(const std::string& text, std::string* error);

}  // namespace hlo
}  // namespace xla_amd
#endif  // XLA_AMD_CSRC_HOST_HLO_IR_H_
