// Element-level expression emitter: given an instruction and a symbolic index, writes the HIP
// statements that compute that one element and returns the name of the variable holding it.
//
// It plays the role of the reference's per-op implementations plus index tracer
// (mononn_engine/core/op_impl/*.cc, mononn_engine/core/context/index_tracer.cc:67-456,
// functors mononn_engine/core/gpu/functor.cc:42-88): broadcast / transpose / reshape / slice /
// pad / concatenate / gather / dynamic-slice rewrite the index, element-wise ops combine operand
// values, values produced by another member of the same cluster are recomputed in registers
// instead of being re-read from memory (the on-chip hand-over of
// mononn_engine/core/graph/cluster_util.cc:305-337).
#pragma once
#include <map>
#include <set>
#include <string>
#include <vector>

#include "codegen/index.h"
#include "graph/program.h"
#include "hlo/hlo.h"

namespace mononn {
namespace codegen {

class CodeBuffer {
 public:
  void line(const std::string& s);
  void open(const std::string& header);   // "header {" and indent
  void close(const std::string& tail = "");
  const std::string& text() const { return text_; }
  int indent() const { return indent_; }

 private:
  std::string text_;
  int indent_ = 1;
};

using Index = std::vector<LinExpr>;

// Pointer parameters of the function being generated, in order of first use.  Names are
// positional (in0, in1, out0 ...) so that structurally identical nodes of different layers
// generate identical text and can share one device function.
struct PointerTable {
  struct Entry {
    const hlo::Instr* root;   // storage root
    bool is_output;
    std::string name;
    hlo::DType dtype;
  };
  std::vector<Entry> entries;
  std::string input(const hlo::Instr* root, hlo::DType as = hlo::DType::kInvalid);    // `as`: element type override
  std::string output(const hlo::Instr* root, hlo::DType as = hlo::DType::kInvalid);
};

// element offset of `idx` inside the buffer of storage root `root`, honouring a permuted physical layout
// element offset of logical index `idx` in the buffer of storage root `root`; `vars` is needed for roots kept in
// fragment order (digits of the index are re-split)
LinExpr physical_offset(const graph::Program& prog, const hlo::Instr* root, const Index& idx, const VarTable* vars = nullptr);

class Emitter {
 public:
  Emitter(const graph::Program& prog, const std::vector<const hlo::Instr*>& members, CodeBuffer& out,
          VarTable& vars, PointerTable& ptrs);

  // value of `ins` (any computation reachable from the members) at multi-index `idx`
  std::string value(const hlo::Instr* ins, const Index& idx);

  // make a value available from a register when it is requested at exactly this index
  void bind(const hlo::Instr* ins, const Index& idx, const std::string& expr);
  void unbind(const hlo::Instr* ins);

  void push_scope();
  void pop_scope();
  std::string fresh(const std::string& prefix = "v");

  // all reduce instructions inside the members (fused computations and bare ops), dependency order
  std::vector<const hlo::Instr*> collect_reduces() const;
  // the instruction computing output `i` of an entry-level member (fusion root / tuple element)
  const hlo::Instr* resolve_output(const hlo::Instr* entry_value) const;

  // the scalar computation `c` with its parameters replaced by the C expressions `args`: C expressions of its results
  // (the statements they need are written to the code buffer)
  std::vector<std::string> inline_scalar_computation(const hlo::Computation* c, const std::vector<std::string>& args);

  // f32 divisions as a multiplication by v_rcp_f32 (1 ulp) instead of the correctly rounded expansion (10
  // instructions per element): for soft-max normalisations, whose quotients are rounded to f16 right after
  void set_fast_divide(bool on) { fast_divide_ = on; }

  static std::string literal(const hlo::Instr* c);                    // scalar constant as C literal
  static std::string literal_of(hlo::DType t, const std::string& text);
  static std::string reducer_expr(const hlo::Instr* reduce, const std::string& a, const std::string& b);
  static std::string reducer_functor(const hlo::Instr* reduce);       // C++ lambda text
  // device-global arrays for non-scalar literal constants met inside fused computations
  const std::map<std::string, std::string>& literal_tables() const { return literal_tables_; }
  // "ptr[index]" of every plain load emitted so far whose index only involves loop variables
  // loads whose address depends on the loop variables only, as (reference text, C type), in emission order; loads
  // emitted under a condition or inside a loop of the emitter's own are left out: they may only run where they stand
  const std::vector<std::pair<std::string, std::string>>& simple_loads() const { return simple_loads_; }

 private:
  std::string emit(const hlo::Instr* ins, const Index& idx);
  std::string load(const hlo::Instr* root, const Index& idx);
  std::string serial_reduce(const hlo::Instr* ins, const Index& idx);
  // N-operand reduce with a tuple-valued reducer: one loop for all N results, which are returned in tuple order
  std::vector<std::string> serial_reduce_variadic(const hlo::Instr* ins, const Index& idx);
  std::string key(const hlo::Instr* ins, const Index& idx) const;
  std::string def(hlo::DType t, const std::string& rhs);
  bool is_member(const hlo::Instr* v) const { return members_.count(v) > 0; }

  const graph::Program& prog_;
  std::set<const hlo::Instr*> members_;
  std::vector<const hlo::Instr*> member_order_;
  std::map<const hlo::Computation*, const hlo::Instr*> caller_;
  CodeBuffer& out_;
  VarTable& vars_;
  PointerTable& ptrs_;
  std::vector<std::map<std::string, std::string>> scopes_;
  struct Bound {
    Index idx;
    std::string expr;
  };
  std::map<const hlo::Instr*, Bound> bound_;
  std::map<std::string, std::string> literal_tables_;
  bool fast_divide_ = false;
  std::vector<std::pair<std::string, std::string>> simple_loads_;
  int counter_ = 0;
  int guarded_ = 0;   // scopes (conditions, loops) this emitter has opened and not yet closed
};

}  // namespace codegen
}  // namespace mononn
