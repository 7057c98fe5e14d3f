// Symbolic index algebra for the code generator.
//
// The reference traces a symbolic index string through every shape-manipulating op
// (mononn_engine/core/context/index_tracer.cc:67-456) and later pattern-matches those strings to
// decide on vector widths and on-chip hand-over.  Here an index is kept structured instead: a sum of
// mixed-radix "digits" of loop variables, ((var / div) % mod) * mul, plus opaque run-time terms and
// a constant.  Reshapes re-split digits exactly (no run-time div/mod when extents line up), and
// questions such as "is this access contiguous in the column variable" or "is this the current
// row" become structural comparisons.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace mononn {
namespace codegen {

struct LoopVar {
  std::string name;   // C identifier of an int variable in scope
  int64_t extent;     // 0 <= var < extent
};

struct Term {
  int var;        // index into the variable table
  int64_t div;    // >= 1
  int64_t mod;    // digit range: ((var / div) % mod); mod >= 1. Always kept explicit; printing drops
                  // the modulo when var / div < mod is implied by the variable's extent.
  int64_t mul;    // >= 1
};

struct Opaque {
  std::string expr;   // C expression of integer type, side-effect free
  int64_t extent;     // 0 <= expr < extent (0 = unknown)
  int64_t mul;
};

class VarTable {
 public:
  int add(const std::string& name, int64_t extent) {
    vars_.push_back({name, extent});
    return static_cast<int>(vars_.size()) - 1;
  }
  const LoopVar& operator[](int i) const { return vars_[i]; }
  size_t size() const { return vars_.size(); }

 private:
  std::vector<LoopVar> vars_;
};

class LinExpr {
 public:
  LinExpr() = default;
  static LinExpr constant(int64_t c) {
    LinExpr e;
    e.c_ = c;
    return e;
  }
  static LinExpr variable(int var, int64_t extent) {
    LinExpr e;
    if (extent > 1) e.terms_.push_back({var, 1, extent, 1});
    return e;
  }
  static LinExpr opaque(const std::string& expr, int64_t extent) {
    LinExpr e;
    e.opaque_.push_back({expr, extent, 1});
    return e;
  }

  const std::vector<Term>& terms() const { return terms_; }
  const std::vector<Opaque>& opaques() const { return opaque_; }
  int64_t constant_part() const { return c_; }
  bool is_constant() const { return terms_.empty() && opaque_.empty(); }

  LinExpr scaled(int64_t k) const;
  LinExpr plus(const LinExpr& o) const;
  LinExpr plus_const(int64_t k) const {
    LinExpr e = *this;
    e.c_ += k;
    return e;
  }
  // largest value the expression can take given the variables' extents (opaque extent 0 -> -1 = unknown)
  int64_t max_value() const;

  // structural equality after normalisation
  bool equals(const LinExpr& o) const;
  // true when the expression is exactly the variable `var` (div 1, mul 1, full range), no constant
  bool is_exactly_var(int var, int64_t extent) const;
  // coefficient analysis for vector access: returns true when the expression is
  //   rest + 1 * var   with var's digit covering its whole range and `rest` independent of var.
  bool is_unit_stride_in(int var, int64_t extent) const;
  bool depends_on(int var) const;

  std::string str(const VarTable& vars) const;   // C expression (int arithmetic)
  // value of the expression for given values of the loop variables (indexed like the variable table); false when
  // the expression has run-time terms, which have no value on the host
  bool evaluate(const std::vector<int64_t>& values, int64_t* out) const;

 private:
  friend LinExpr linearize(const std::vector<LinExpr>&, const std::vector<int64_t>&);
  friend std::vector<LinExpr> delinearize(const LinExpr&, const std::vector<int64_t>&, const VarTable&);
  void normalise();
  std::vector<Term> terms_;
  std::vector<Opaque> opaque_;
  int64_t c_ = 0;
};

// row-major linear offset of a multi-index
LinExpr linearize(const std::vector<LinExpr>& idx, const std::vector<int64_t>& dims);
// inverse; exact digit re-splitting where extents divide, run-time div/mod (opaque) otherwise
std::vector<LinExpr> delinearize(const LinExpr& lin, const std::vector<int64_t>& dims, const VarTable& vars);
// reshape [from] -> [to]: map an index into the result (shape `to`) to an index into the operand
std::vector<LinExpr> reshape_index(const std::vector<LinExpr>& idx_to, const std::vector<int64_t>& to,
                                   const std::vector<int64_t>& from, const VarTable& vars);

}  // namespace codegen
}  // namespace mononn
