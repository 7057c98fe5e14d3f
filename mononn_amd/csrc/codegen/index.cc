#include "codegen/index.h"

#include <algorithm>

#include "common/status.h"

namespace mononn {
namespace codegen {

namespace {
int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// extents are carried inside terms as the canonical modulus of a variable's top digit, so the
// algebra itself never needs the table except for printing and re-splitting.
}  // namespace

void LinExpr::normalise() {
  // drop dead digits, sort by (var, div), fuse adjacent digits of one variable
  std::vector<Term> t;
  for (auto& x : terms_)
    if (x.mod > 1 && x.mul != 0) t.push_back(x);
  std::sort(t.begin(), t.end(), [](const Term& a, const Term& b) {
    if (a.var != b.var) return a.var < b.var;
    if (a.div != b.div) return a.div < b.div;
    return a.mul < b.mul;
  });
  std::vector<Term> out;
  for (auto& x : t) {
    if (!out.empty()) {
      Term& lo = out.back();
      if (lo.var == x.var && x.div == lo.div * lo.mod && x.mul == lo.mul * lo.mod) {
        lo.mod *= x.mod;
        continue;
      }
      if (lo.var == x.var && lo.div == x.div && lo.mod == x.mod) {   // same digit twice: add coefficients
        lo.mul += x.mul;
        continue;
      }
    }
    out.push_back(x);
  }
  terms_ = out;
  std::vector<Opaque> o;
  for (auto& x : opaque_)
    if (x.mul != 0) o.push_back(x);
  std::sort(o.begin(), o.end(), [](const Opaque& a, const Opaque& b) {
    if (a.expr != b.expr) return a.expr < b.expr;
    return a.mul < b.mul;
  });
  opaque_ = o;
}

LinExpr LinExpr::scaled(int64_t k) const {
  LinExpr e = *this;
  if (k == 0) return LinExpr();
  for (auto& t : e.terms_) t.mul *= k;
  for (auto& o : e.opaque_) o.mul *= k;
  e.c_ *= k;
  return e;
}

LinExpr LinExpr::plus(const LinExpr& o) const {
  LinExpr e = *this;
  e.terms_.insert(e.terms_.end(), o.terms_.begin(), o.terms_.end());
  e.opaque_.insert(e.opaque_.end(), o.opaque_.begin(), o.opaque_.end());
  e.c_ += o.c_;
  e.normalise();
  return e;
}

int64_t LinExpr::max_value() const {
  int64_t m = c_;
  for (auto& t : terms_) m += (t.mod - 1) * t.mul;
  for (auto& o : opaque_) {
    if (o.extent <= 0) return -1;
    m += (o.extent - 1) * o.mul;
  }
  return m;
}

bool LinExpr::equals(const LinExpr& o) const {
  if (c_ != o.c_ || terms_.size() != o.terms_.size() || opaque_.size() != o.opaque_.size()) return false;
  for (size_t i = 0; i < terms_.size(); ++i) {
    const Term &a = terms_[i], &b = o.terms_[i];
    if (a.var != b.var || a.div != b.div || a.mod != b.mod || a.mul != b.mul) return false;
  }
  for (size_t i = 0; i < opaque_.size(); ++i)
    if (opaque_[i].expr != o.opaque_[i].expr || opaque_[i].mul != o.opaque_[i].mul) return false;
  return true;
}

bool LinExpr::is_exactly_var(int var, int64_t extent) const {
  if (extent <= 1) return is_constant() && c_ == 0;
  return c_ == 0 && opaque_.empty() && terms_.size() == 1 && terms_[0].var == var && terms_[0].div == 1 &&
         terms_[0].mul == 1 && terms_[0].mod == extent;
}

bool LinExpr::depends_on(int var) const {
  for (auto& t : terms_)
    if (t.var == var) return true;
  return false;
}

bool LinExpr::is_unit_stride_in(int var, int64_t extent) const {
  int n = 0;
  for (auto& t : terms_) {
    if (t.var != var) continue;
    ++n;
    if (t.div != 1 || t.mul != 1 || t.mod != extent) return false;
  }
  return n == 1;
}

bool LinExpr::evaluate(const std::vector<int64_t>& values, int64_t* out) const {
  if (!opaque_.empty()) return false;
  int64_t v = c_;
  for (auto& t : terms_) {
    if (t.var < 0 || static_cast<size_t>(t.var) >= values.size()) return false;
    v += ((values[t.var] / t.div) % t.mod) * t.mul;
  }
  *out = v;
  return true;
}

std::string LinExpr::str(const VarTable& vars) const {
  std::string s;
  auto add = [&](const std::string& p) {
    if (!s.empty()) s += " + ";
    s += p;
  };
  for (auto& t : terms_) {
    const LoopVar& v = vars[t.var];
    std::string p = v.name;
    if (t.div != 1) p = "(" + p + " / " + std::to_string(t.div) + ")";
    bool need_mod = v.extent <= 0 || ceil_div(v.extent, t.div) > t.mod;
    if (need_mod) p = "(" + p + " % " + std::to_string(t.mod) + ")";
    if (t.mul != 1) p = p + " * " + std::to_string(t.mul);
    add(p);
  }
  for (auto& o : opaque_) {
    std::string p = "(" + o.expr + ")";
    if (o.mul != 1) p += " * " + std::to_string(o.mul);
    add(p);
  }
  if (c_ != 0 || s.empty()) add(std::to_string(c_));
  return s;
}

LinExpr linearize(const std::vector<LinExpr>& idx, const std::vector<int64_t>& dims) {
  MONONN_CHECK(idx.size() == dims.size(), kInternal) << "linearize: rank mismatch";
  LinExpr out;
  int64_t stride = 1;
  for (int i = static_cast<int>(dims.size()) - 1; i >= 0; --i) {
    LinExpr s = idx[i].scaled(stride);
    out.terms_.insert(out.terms_.end(), s.terms_.begin(), s.terms_.end());
    out.opaque_.insert(out.opaque_.end(), s.opaque_.begin(), s.opaque_.end());
    out.c_ += s.c_;
    stride *= dims[i];
  }
  out.normalise();
  return out;
}

std::vector<LinExpr> delinearize(const LinExpr& lin, const std::vector<int64_t>& dims, const VarTable& vars) {
  const int r = static_cast<int>(dims.size());
  std::vector<int64_t> stride(r, 1);
  for (int i = r - 2; i >= 0; --i) stride[i] = stride[i + 1] * dims[i + 1];
  std::vector<LinExpr> out(r);
  bool ok = true;
  int outer = 0;   // outermost non-unit dim: its digit is unbounded above, nothing can straddle out of it
  while (outer < r - 1 && dims[outer] == 1) ++outer;

  // which dim does a multiplier land in: the largest stride <= mul, ignoring unit dims
  auto dim_of = [&](int64_t mul) -> int {
    for (int i = 0; i < r; ++i)
      if (dims[i] > 1 && stride[i] <= mul) return i;
    return -1;
  };

  std::vector<Term> work(lin.terms_.begin(), lin.terms_.end());
  while (ok && !work.empty()) {
    Term t = work.back();
    work.pop_back();
    if (t.mod <= 1) continue;
    int i = dim_of(t.mul);
    if (i < 0 || t.mul % stride[i] != 0) {
      ok = false;
      break;
    }
    int64_t upper = stride[i] * dims[i];   // first stride of the next-outer dim
    if (i <= outer || (t.mod - 1) * t.mul < upper) {
      Term x = t;
      x.mul = t.mul / stride[i];
      out[i].terms_.push_back(x);
      continue;
    }
    // the digit straddles the boundary between dim i and the outer dims: split it
    if (upper % t.mul != 0) {
      ok = false;
      break;
    }
    int64_t q = upper / t.mul;
    const LoopVar& v = vars[t.var];
    bool top_digit = v.extent > 0 && ceil_div(v.extent, t.div) <= t.mod;
    if (!(t.mod % q == 0 || top_digit)) {
      ok = false;
      break;
    }
    Term lo{t.var, t.div, q, t.mul};
    Term hi{t.var, t.div * q, ceil_div(t.mod, q), t.mul * q};
    work.push_back(lo);
    work.push_back(hi);
  }
  if (ok) {
    for (auto& o : lin.opaque_) {
      int i = dim_of(o.mul);
      if (i < 0 || o.mul % stride[i] != 0 || o.extent <= 0 || (i > outer && (o.extent - 1) * o.mul >= stride[i] * dims[i])) {
        ok = false;
        break;
      }
      Opaque x = o;
      x.mul = o.mul / stride[i];
      out[i].opaque_.push_back(x);
    }
  }
  if (ok) {
    int64_t c = lin.c_;
    if (c < 0) ok = false;
    for (int i = r - 1; ok && i >= 0; --i) {
      if (i <= outer) {
        out[i].c_ += c;
        c = 0;
      } else {
        out[i].c_ += c % dims[i];
        c /= dims[i];
      }
    }
  }
  if (ok) {
    for (int i = 0; i < r; ++i) {
      out[i].normalise();
      int64_t mx = out[i].max_value();
      if (i > outer && (mx < 0 || mx >= dims[i])) ok = false;   // a carry would be needed
    }
  }
  if (ok) return out;

  // general fallback: run-time division of the materialised linear index
  std::string e = lin.str(vars);
  for (int i = 0; i < r; ++i) {
    if (dims[i] == 1) {
      out[i] = LinExpr::constant(0);
      continue;
    }
    std::string p = "(" + e + ")";
    if (stride[i] != 1) p = "(" + p + " / " + std::to_string(stride[i]) + ")";
    bool outermost = true;
    for (int k = 0; k < i; ++k)
      if (dims[k] > 1) outermost = false;
    if (!outermost) p = p + " % " + std::to_string(dims[i]);
    out[i] = LinExpr::opaque(p, dims[i]);
  }
  return out;
}

std::vector<LinExpr> reshape_index(const std::vector<LinExpr>& idx_to, const std::vector<int64_t>& to,
                                   const std::vector<int64_t>& from, const VarTable& vars) {
  return delinearize(linearize(idx_to, to), from, vars);
}

}  // namespace codegen
}  // namespace mononn
