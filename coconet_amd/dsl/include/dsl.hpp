// CoCoNet DSL front end, re-implemented for the MI355X target.
//
// Source-compatible with the user-visible API of the reference's src/dsl.hpp (namespace ACCCDSL:
// Variable, Tensor, Stage, Update, Dropout, Sqrt, Ite, Norm, ReduceStage, MatMul, Cast, Const, AllReduce, ReduceScatter,
// AllGather, Scatter, Broadcast and the arithmetic operators), so that the reference's example programs
// (examples/{sgd,adam,lamb,model-parallel}/*.cpp) compile unmodified.  Internally every expression is one
// reference-counted Node of a small IR instead of a class hierarchy with visitors.
#ifndef COCONET_AMD_DSL_HPP
#define COCONET_AMD_DSL_HPP

#include <cstdlib>
#include <iostream>
#include <memory>
#include <string>
#include <vector>

// reference convention (src/ast.hpp:33-44): message on std::cerr, then std::terminate()
#define ASSERT(cond, msg)                                                                          \
  do {                                                                                             \
    if (!(cond)) {                                                                                 \
      std::cerr << "ASSERT failed: " << msg << " [" << #cond << "] at " << __FILE__ << ":" << __LINE__ << std::endl; \
      std::terminate();                                                                            \
    }                                                                                              \
  } while (0)

namespace ACCCDSL {

// src/ast.hpp:48-102 of the reference: the same enumerators, usable with or without the enum name
// BFloat16 is this build's addition (after the reference's values, which keep their numbers): the matrix-core type of
// benchmark configuration 5; only MatMul pipelines take it.
enum TensorElemType { None, Float16, Float32, Float64, Int8, Int16, Int32, Int64, UInt8, UInt16, UInt32, UInt64, BFloat16 };
enum TensorLayout { Replicated, Sliced, Sliced_2, Local };
enum ReduceOperation { Summation, Difference, Multiplication, Division, Maximum, Minimum };

namespace ir {

enum class Kind {
  Tensor, Variable, Const, Binary, Unary, Cast, Update, Norm, Dropout, MatMul, Collective, Stage, Compare, Select
};
enum class BinOp { Add, Sub, Mul, Div };
enum class UnOp { Sqrt };
enum class CollOp { AllReduce, ReduceScatter, AllGather, Scatter, Broadcast };

struct Node;
using NodePtr = std::shared_ptr<Node>;

struct Node {
  Kind kind;
  int id;                          // creation order; a node can only refer to older nodes
  std::vector<NodePtr> args;       // operands
  std::string name;                // tensors, variables and stages
  TensorElemType elem = None;
  TensorLayout layout = Replicated;
  std::vector<NodePtr> dims;       // tensors: one Variable per dimension
  BinOp bin = BinOp::Add;
  UnOp un = UnOp::Sqrt;
  CollOp coll = CollOp::AllReduce;
  ReduceOperation red = Summation;
  double cval = 0.0;               // Const
  bool cval_is_int = false;
  float prob = 0.f;                // Dropout
  bool plain_sum = false;          // Norm nodes: the sum of the elements (ReduceStage) instead of the L2 norm
};

NodePtr make(Kind k);
bool is_scalar(const NodePtr& n);  // Variable, Const, or arithmetic over them only
const char* elem_c_type(TensorElemType t);
size_t elem_size(TensorElemType t);

}  // namespace ir

class Expression {
 public:
  Expression(ir::NodePtr n) : node_(std::move(n)) {}
  Expression(double c);
  Expression(float c);
  Expression(int c);
  const ir::NodePtr& impl() const { return node_; }

 protected:
  ir::NodePtr node_;
};

// names kept for source compatibility with programs that mention them
using ContinuousExpression = Expression;
using SingleDimExpression = Expression;
using ScatteredExpression = Expression;

Expression operator+(const Expression& a, const Expression& b);
Expression operator-(const Expression& a, const Expression& b);
Expression operator*(const Expression& a, const Expression& b);
Expression operator/(const Expression& a, const Expression& b);
Expression operator>(const Expression& a, const Expression& b);

class Variable : public Expression {
 public:
  Variable(TensorElemType t, std::string name);
};

class Const : public Expression {
 public:
  Const(TensorElemType t, double v);
};

class Tensor : public Expression {
 public:
  Tensor(TensorElemType elemType, Variable n, TensorLayout layout, std::string name);
  Tensor(TensorElemType elemType, Variable n1, Variable n2, TensorLayout layout, std::string name);
  Tensor(TensorElemType elemType, std::vector<Variable> dimSizes, TensorLayout layout, std::string name);
};

class Stage : public Expression {
 public:
  Stage(const Expression& definition);   // a named, schedulable unit: "Stage s = <expression>;"
  const std::string& name() const { return node_->name; }
};

Expression Update(const Tensor& t, const Expression& definition);
Expression Dropout(const Expression& x, float prob);
Expression Sqrt(const Expression& x);
// cond ? ifTrue : ifFalse per element (src/dsl.hpp:482-486 of the reference); cond is a comparison or any expression
// that is non-zero where the first branch is wanted
Expression Ite(const Expression& cond, const Expression& ifTrue, const Expression& ifFalse);
Expression Norm(const Expression& x);
// Sum over all elements of a stage or tensor, a single replicated value (class ReduceStage of the reference,
// src/dsl.hpp:269-275; its generated form is the S2 loop of examples/test-reduction.cu:17-19).  Summation only.
Expression ReduceStage(const Expression& definition, ReduceOperation op);
Expression MatMul(const Expression& a, const Expression& b);
Expression Cast(TensorElemType t, const Expression& x);

Expression AllReduce(ReduceOperation op, const Expression& x);
Expression ReduceScatter(ReduceOperation op, const Expression& x);
Expression AllGather(const Expression& x);
Expression Scatter(const Expression& x);
Expression Broadcast(const Expression& x, int root = 0);

}  // namespace ACCCDSL

#endif
