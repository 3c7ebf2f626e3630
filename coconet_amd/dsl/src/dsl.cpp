// IR construction for the DSL surface (see include/dsl.hpp).
#include "dsl.hpp"

namespace ACCCDSL {
namespace ir {

static int g_next_id = 0;      // creation order doubles as a topological order
static int g_next_stage = 0;   // stage names S0, S1, ... in creation order (reference: src/ast.hpp:866-873)

NodePtr make(Kind k) {
  auto n = std::make_shared<Node>();
  n->kind = k;
  n->id = g_next_id++;
  return n;
}

bool is_scalar(const NodePtr& n) {
  switch (n->kind) {
    case Kind::Variable:
    case Kind::Const: return true;
    case Kind::Binary:
    case Kind::Unary:
    case Kind::Cast:
    case Kind::Compare:
    case Kind::Select:
      for (auto& a : n->args) if (!is_scalar(a)) return false;
      return true;
    default: return false;
  }
}

const char* elem_c_type(TensorElemType t) {
  switch (t) {
    case Float16: return "_Float16";
    case BFloat16: return "__bf16";
    case Float32: return "float";
    case Float64: return "double";
    case Int8: return "int8_t";
    case Int16: return "int16_t";
    case Int32: return "int";
    case Int64: return "int64_t";
    case UInt8: return "uint8_t";
    case UInt16: return "uint16_t";
    case UInt32: return "uint32_t";
    case UInt64: return "uint64_t";
    default: return "void";
  }
}

size_t elem_size(TensorElemType t) {
  switch (t) {
    case Float16: case BFloat16: case Int16: case UInt16: return 2;
    case Float32: case Int32: case UInt32: return 4;
    case Float64: case Int64: case UInt64: return 8;
    case Int8: case UInt8: return 1;
    default: return 0;
  }
}

}  // namespace ir

using namespace ir;

static NodePtr constant(double v, bool is_int) {
  auto n = make(Kind::Const);
  n->cval = v;
  n->cval_is_int = is_int;
  n->elem = is_int ? Int32 : Float32;
  return n;
}

Expression::Expression(double c) : node_(constant(c, false)) {}
Expression::Expression(float c) : node_(constant(c, false)) {}
Expression::Expression(int c) : node_(constant(c, true)) {}

// Result element type of a pointwise operation: floating point wins, then the wider type.
static TensorElemType promote(TensorElemType a, TensorElemType b) {
  auto rank = [](TensorElemType t) {
    switch (t) {
      case Float64: return 12; case Float32: return 11; case Float16: case BFloat16: return 10;
      case Int64: case UInt64: return 4; case Int32: case UInt32: return 3;
      case Int16: case UInt16: return 2; case Int8: case UInt8: return 1;
      default: return 0;
    }
  };
  return rank(a) >= rank(b) ? a : b;
}

// dimensions of a tensor-valued expression: its own when it carries them, otherwise those of its operands
static std::vector<NodePtr> dims_of(const NodePtr& n) {
  if (!n->dims.empty()) return n->dims;
  std::vector<NodePtr> d;
  if (n->kind == Kind::Norm) return d;
  for (auto& a : n->args) {
    if (is_scalar(a)) continue;
    auto da = dims_of(a);
    if (da.size() > d.size()) d = da;
  }
  return d;
}

static std::string dims_text(const std::vector<NodePtr>& d) {
  std::string s = "[";
  for (size_t k = 0; k < d.size(); k++) s += (k ? ", " : "") + d[k]->name;
  return s + "]";
}

// Dimensions of a pointwise operation over a and b.  The reference's rule (BinaryPointwiseOp::setupAndCheckDimensions,
// src/pipeline.cpp:14-90): scalars adapt to the other operand; of two tensor-valued operands the one with fewer
// dimensions is broadcast numpy-style, its dimensions matched against the TRAILING dimensions of the other; matching
// means being the same dimension variable.  Anything else is rejected here, on the host, where the program is built:
// the emitted kernels index every operand by the stage's element index and check nothing.
static bool single_value(const NodePtr& n) {   // scalars, and norms / whole-tensor sums: one value, whatever they were taken over
  return is_scalar(n) || n->kind == Kind::Norm || (n->kind == Kind::Stage && n->args[0]->kind == Kind::Norm);
}
static std::vector<NodePtr> broadcast_dims(const NodePtr& a, const NodePtr& b, const char* what) {
  if (single_value(a)) return single_value(b) ? std::vector<NodePtr>{} : dims_of(b);
  if (single_value(b)) return dims_of(a);
  const auto da = dims_of(a), db = dims_of(b);
  const auto& lng = da.size() >= db.size() ? da : db;
  const auto& sht = da.size() >= db.size() ? db : da;
  for (size_t k = 0; k < sht.size(); k++) {
    const NodePtr& x = lng[lng.size() - sht.size() + k];
    const NodePtr& y = sht[k];
    ASSERT(x == y, what << ": operand dimensions " << dims_text(da) << " and " << dims_text(db) << " do not match ('"
                        << x->name << "' against '" << y->name << "')");
  }
  return lng;
}

static NodePtr binary(BinOp op, const Expression& a, const Expression& b) {
  auto n = make(Kind::Binary);
  n->bin = op;
  n->args = {a.impl(), b.impl()};
  n->dims = broadcast_dims(a.impl(), b.impl(), "pointwise operation");
  // a constant adapts to the other operand (1 - beta1 is a float expression)
  TensorElemType ta = a.impl()->elem, tb = b.impl()->elem;
  if (a.impl()->kind == Kind::Const) ta = tb;
  if (b.impl()->kind == Kind::Const) tb = ta;
  n->elem = promote(ta, tb);
  // layout: scalars adapt; otherwise the operand that varies more across ranks wins (Local > Sliced > Replicated)
  auto weight = [](TensorLayout l) { return l == Local ? 3 : (l == Replicated ? 1 : 2); };
  const bool sa = is_scalar(a.impl()), sb = is_scalar(b.impl());
  if (sa && !sb) n->layout = b.impl()->layout;
  else if (!sa && sb) n->layout = a.impl()->layout;
  else n->layout = weight(a.impl()->layout) >= weight(b.impl()->layout) ? a.impl()->layout : b.impl()->layout;
  return n;
}

Expression operator+(const Expression& a, const Expression& b) { return Expression(binary(BinOp::Add, a, b)); }
Expression operator-(const Expression& a, const Expression& b) { return Expression(binary(BinOp::Sub, a, b)); }
Expression operator*(const Expression& a, const Expression& b) { return Expression(binary(BinOp::Mul, a, b)); }
Expression operator/(const Expression& a, const Expression& b) { return Expression(binary(BinOp::Div, a, b)); }
Expression operator>(const Expression& a, const Expression& b) {
  auto n = make(Kind::Compare);
  n->args = {a.impl(), b.impl()};
  n->dims = broadcast_dims(a.impl(), b.impl(), "comparison");
  n->elem = Int32;
  n->layout = is_scalar(a.impl()) ? b.impl()->layout : a.impl()->layout;
  return Expression(n);
}

static NodePtr variable(TensorElemType t, std::string name) {
  auto n = make(Kind::Variable);
  n->elem = t;
  n->name = std::move(name);
  return n;
}
Variable::Variable(TensorElemType t, std::string name) : Expression(variable(t, std::move(name))) {}

Const::Const(TensorElemType t, double v) : Expression(constant(v, t != Float16 && t != BFloat16 && t != Float32 && t != Float64)) {
  node_->elem = t;
}

static NodePtr tensor(TensorElemType t, const std::vector<Variable>& dims, TensorLayout layout, std::string name) {
  ASSERT(!dims.empty(), "tensor '" << name << "' needs at least one dimension");
  auto n = make(Kind::Tensor);
  n->elem = t;
  n->layout = layout;
  n->name = std::move(name);
  for (auto& d : dims) n->dims.push_back(d.impl());
  return n;
}
Tensor::Tensor(TensorElemType t, Variable n, TensorLayout layout, std::string name)
    : Expression(tensor(t, {n}, layout, std::move(name))) {}
Tensor::Tensor(TensorElemType t, Variable n1, Variable n2, TensorLayout layout, std::string name)
    : Expression(tensor(t, {n1, n2}, layout, std::move(name))) {}
Tensor::Tensor(TensorElemType t, std::vector<Variable> dims, TensorLayout layout, std::string name)
    : Expression(tensor(t, dims, layout, std::move(name))) {}

static NodePtr stage(const Expression& def) {
  ASSERT(!is_scalar(def.impl()), "a stage must be tensor valued");
  auto n = make(Kind::Stage);
  n->args = {def.impl()};
  n->elem = def.impl()->elem;
  n->layout = def.impl()->layout;
  n->dims = def.impl()->kind == Kind::Norm ? std::vector<NodePtr>{} : dims_of(def.impl());
  n->name = "S" + std::to_string(g_next_stage++);
  return n;
}
Stage::Stage(const Expression& definition)
    : Expression(definition.impl()->kind == Kind::Stage ? definition.impl() : stage(definition)) {}

static NodePtr unary_like(Kind k, const Expression& x) {
  auto n = make(k);
  n->args = {x.impl()};
  n->elem = x.impl()->elem;
  n->layout = x.impl()->layout;
  return n;
}

Expression Update(const Tensor& t, const Expression& definition) {
  ASSERT(t.impl()->kind == Kind::Tensor, "Update target must be a tensor");
  auto n = make(Kind::Update);
  if (!is_scalar(definition.impl())) {
    // the new value has the tensor's dimensions, or fewer that broadcast into them; never more
    const auto d = broadcast_dims(t.impl(), definition.impl(), "Update");
    ASSERT(d.size() == t.impl()->dims.size(), "Update: the value has more dimensions " << dims_text(dims_of(definition.impl()))
                                                  << " than tensor '" << t.impl()->name << "' " << dims_text(t.impl()->dims));
  }
  n->args = {t.impl(), definition.impl()};
  n->elem = t.impl()->elem;
  n->layout = t.impl()->layout;
  n->dims = t.impl()->dims;
  return Expression(n);
}

Expression Dropout(const Expression& x, float prob) {
  ASSERT(prob >= 0.f && prob < 1.f, "dropout probability must be in [0,1)");
  auto n = unary_like(Kind::Dropout, x);
  n->prob = prob;
  return Expression(n);
}

Expression Sqrt(const Expression& x) {
  auto n = unary_like(Kind::Unary, x);
  n->un = UnOp::Sqrt;
  return Expression(n);
}

Expression Ite(const Expression& cond, const Expression& ifTrue, const Expression& ifFalse) {
  // the value has the type and layout of "ifTrue op ifFalse"; the condition only has to be defined where they are
  auto n = make(Kind::Select);
  const NodePtr both = binary(BinOp::Add, ifTrue, ifFalse);
  n->args = {cond.impl(), ifTrue.impl(), ifFalse.impl()};
  {
    auto probe = make(Kind::Binary);   // the branches' dimensions, then the condition's against them
    probe->dims = both->dims;
    probe->args = {ifTrue.impl(), ifFalse.impl()};
    n->dims = is_scalar(both) ? dims_of(cond.impl()) : broadcast_dims(probe, cond.impl(), "Ite");
  }
  n->elem = both->elem;
  n->layout = is_scalar(both) ? cond.impl()->layout : both->layout;
  return Expression(n);
}

// L2 norm over the whole tensor: a single value, replicated.
Expression Norm(const Expression& x) {
  auto n = unary_like(Kind::Norm, x);
  n->layout = Replicated;
  return Expression(n);
}
Expression ReduceStage(const Expression& definition, ReduceOperation op) {
  ASSERT(op == Summation, "ReduceStage: only Summation is lowered");
  auto n = unary_like(Kind::Norm, definition);
  n->layout = Replicated;
  n->red = op;
  n->plain_sum = true;
  return Expression(n);
}

Expression MatMul(const Expression& a, const Expression& b) {
  auto n = make(Kind::MatMul);
  n->args = {a.impl(), b.impl()};
  n->elem = a.impl()->elem;
  n->layout = Local;   // each rank holds a partial product until it is reduced
  auto da = dims_of(a.impl()), db = dims_of(b.impl());
  ASSERT(da.size() >= 2 && db.size() == 2, "MatMul needs [.., K] x [K, N] operands");
  n->dims.assign(da.begin(), da.end() - 1);
  n->dims.push_back(db.back());
  return Expression(n);
}

Expression Cast(TensorElemType t, const Expression& x) {
  auto n = unary_like(Kind::Cast, x);
  n->elem = t;
  return Expression(n);
}

static Expression collective(CollOp op, ReduceOperation red, const Expression& x, TensorLayout out_layout) {
  ASSERT(!is_scalar(x.impl()), "collectives take tensors or stages");
  auto n = unary_like(Kind::Collective, x);
  n->coll = op;
  n->red = red;
  n->layout = out_layout;
  n->dims = dims_of(x.impl());
  return Expression(n);
}

Expression AllReduce(ReduceOperation op, const Expression& x) {
  ASSERT(x.impl()->layout == Local, "AllReduce input must be Local (one value per rank)");
  return collective(CollOp::AllReduce, op, x, Replicated);
}
Expression ReduceScatter(ReduceOperation op, const Expression& x) {
  ASSERT(x.impl()->layout == Local, "ReduceScatter input must be Local (one value per rank)");
  return collective(CollOp::ReduceScatter, op, x, Sliced);
}
Expression AllGather(const Expression& x) {
  ASSERT(x.impl()->layout == Sliced || x.impl()->layout == Sliced_2, "AllGather input must be Sliced");
  return collective(CollOp::AllGather, Summation, x, Replicated);
}
Expression Scatter(const Expression& x) {
  ASSERT(x.impl()->layout == Replicated, "Scatter input must be Replicated");
  return collective(CollOp::Scatter, Summation, x, Sliced);
}
Expression Broadcast(const Expression& x, int) { return collective(CollOp::Broadcast, Summation, x, Replicated); }

}  // namespace ACCCDSL
