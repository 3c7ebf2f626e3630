// HIP code-generation target for gfx950.
//
// Takes the place of the reference's only target, NCCLCodegen (src/codegen.cpp:4071-4794), with a different
// lowering: nothing in the emitted program talks to a second GPU, so a collective over a Local tensor becomes a
// fold over P rank buffers resident on this GPU, and a collective fused with the stages around it becomes the
// first operand of one streaming kernel (ccn_codegen_rt.hpp).
//
// Sliced values (the output of ReduceScatter, Sliced tensors, Scatter(t)) keep the reference's addressing: rank r owns
// elements [DIVUP(N, comm_size) * r, +DIVUP(N, comm_size)) clipped at N (src/codegen.cpp:485-499).  A Sliced tensor is
// stored as the concatenation of all ranks' slices, so a step over Sliced values is the same kernel, reduce or copy on
// every array moved on by the rank's offset, with the rank's element count; the emitted driver takes the reference's
// (comm_size, rank) pair (src/codegen.cpp:4366-4387) and runs that one rank's share, or every rank's in turn for
// rank = -1.  A Replicated tensor read inside a step over Sliced values is read at the rank's offset too, with or
// without Scatter() around it (the reference reads element i of it on every rank when Scatter is left out, as its lamb
// example does; that only addresses the right elements on rank 0).
//
// Emitted program = body structs (the user's expressions, operand order preserved, fully parenthesised) +
// a driver function timing every step with events + a CPU re-execution of the pipeline stage by stage
// (the reference's mpiRef, src/codegen.cpp:4421-4581, with MPI_Allreduce replaced by the fixed-order P-way sum)
// + main() with the reference's size sweep and "{SZ: ..., Epochs: ..., <step>: ms, Total: ms}" line
// (src/codegen.cpp:4583-4784).
#include <algorithm>
#include <cstdlib>
#include <functional>
#include <map>
#include <set>
#include <sstream>

#include "pipeline.hpp"

namespace ACCCDSL {
using namespace ir;

namespace {

std::string fconst(const NodePtr& n) {
  std::ostringstream o;
  if (n->cval_is_int) {
    o << (long long)n->cval;
  } else {
    o.precision(9);
    o << n->cval;
    std::string s = o.str();
    if (s.find('.') == std::string::npos && s.find('e') == std::string::npos) s += ".0";
    return s + "f";
  }
  return o.str();
}

// Dropout(x, p) is lowered to standard dropout (drop with probability p, survivors scaled by 1/(1-p)) unless the
// generator runs with CCN_DSL_DROPOUT=reference: then to the reference's emitted form, keep with probability p and no
// rescale (src/codegen.cpp:634-640).  The mask comes from the counter-based stream either way.
bool reference_dropout() {
  const char* e = std::getenv("CCN_DSL_DROPOUT");
  return e && std::string(e) == "reference";
}

// ---- program-level facts ---------------------------------------------------------------------------------------------
struct Program {
  const Pipeline& p;
  std::vector<NodePtr> dimVars, scalarVars, tensors;   // pipeline arguments by role
  std::set<const Node*> reducedTensors;                  // Local tensors fed to AllReduce / ReduceScatter
  std::map<int, std::string> stageBuf;                   // stage index -> C expression of its device buffer
  std::vector<int> ownBuffers;                           // stages that need a buffer of their own ("S<k>")

  explicit Program(const Pipeline& pl) : p(pl) {}
};

void collect_leaves(const NodePtr& n, std::vector<NodePtr>& tensors, std::vector<NodePtr>& vars) {
  if (n->kind == Kind::Tensor) tensors.push_back(n);
  else if (n->kind == Kind::Variable) vars.push_back(n);
  else if (n->kind != Kind::Stage)
    for (auto& a : n->args) collect_leaves(a, tensors, vars);
}

bool contains_kind(const NodePtr& n, Kind k) {
  if (n->kind == k) return true;
  if (n->kind == Kind::Stage) return false;
  for (auto& a : n->args) if (contains_kind(a, k)) return true;
  return false;
}

void find_reduced(const NodePtr& n, std::set<const Node*>& out) {
  if (n->kind == Kind::Stage) return;
  if (n->kind == Kind::Collective && (n->coll == CollOp::AllReduce || n->coll == CollOp::ReduceScatter) &&
      n->args[0]->kind == Kind::Tensor)
    out.insert(n->args[0].get());
  for (auto& a : n->args) find_reduced(a, out);
}

std::string count_expr(const NodePtr& tensorLike) {
  std::string s = "(size_t)";
  ASSERT(!tensorLike->dims.empty(), "value '" << tensorLike->name << "' has no dimensions");
  for (size_t k = 0; k < tensorLike->dims.size(); k++) s += (k ? " * " : "") + tensorLike->dims[k]->name;
  return s;
}

bool bb_in(const Pipeline::Group& g, int k) { return std::find(g.stages.begin(), g.stages.end(), k) != g.stages.end(); }

// first stage of a list that is tensor valued (a Norm stage is a single number)
int first_tensor_stage(const Pipeline& p, const std::vector<int>& stages) {
  for (int k : stages) if (p.stages()[k]->args[0]->kind != Kind::Norm) return k;
  ASSERT(false, "a kernel made of norms only");
  return -1;
}

// strips Update(t, .) and the identity collectives to see what a single-stage group really is
const Node* strip(const Node* n) {
  while (true) {
    if (n->kind == Kind::Update) n = n->args[1].get();
    else if (n->kind == Kind::Collective && (n->coll == CollOp::AllGather || n->coll == CollOp::Scatter ||
                                             n->coll == CollOp::Broadcast)) n = n->args[0].get();
    else return n;
  }
}

// ---- one pointwise body ----------------------------------------------------------------------------------------------
struct Body {
  std::string name;
  bool hasRed = false;
  bool redHalf = false;                  // the folded tensor holds fp16 elements
  std::string redTensor;                 // name of the Local tensor folded over ranks
  std::vector<std::string> inArrays;     // C expressions of device pointers, order = in[k]
  std::vector<std::string> inNames;      // local value names
  std::vector<std::string> outArrays;
  std::vector<std::string> code;         // statements
  int nacc = 0, nnorm = 0;
  unsigned sqrtMask = 0;                 // accumulator k finishes as sqrt(sum) (a norm) rather than as the sum
  unsigned outHalfMask = 0;              // output array k holds fp16
  std::set<std::string> scalars;         // variable names used
  bool usesSeed = false;
  // operands with fewer dimensions than the kernel's values (a bias over the last dimension): read at element index
  // modulo their own element count, the reference's numpy-style broadcast (src/codegen.cpp:495-496)
  std::vector<std::pair<std::string, std::string>> bcArrays;   // (array, element count expression)
};

struct BodyBuilder {
  Program& prog;
  const Pipeline::Group& group;
  std::set<int> inGroup;
  Body body;
  std::map<const Node*, std::string> tensorValue;   // current value name of a tensor inside the kernel
  std::map<int, std::string> stageValue;            // stage index -> local value name
  std::map<int, int> normIndex;                     // Norm stage index -> slot
  bool phase2 = false;
  std::vector<NodePtr> domain;                      // dimensions of the values the kernel walks

  BodyBuilder(Program& pr, const Pipeline::Group& g) : prog(pr), group(g) {
    for (int s : g.stages) inGroup.insert(s);
    domain = pr.p.stages()[first_tensor_stage(pr.p, g.stages)]->dims;
    if (domain.empty()) {   // a kernel of norms only takes the dimensions of what it sums
      const NodePtr& x = pr.p.stages()[g.stages[0]]->args[0]->args[0];
      domain = x->dims;
    }
  }

  // Reads `array`, whose values have dimensions `dims`, inside this kernel: at the element index when the dimensions
  // are the kernel's, modulo its element count when they are a trailing part of them (the front end has checked that).
  std::string read(const std::string& array, const std::string& hint, const NodePtr& owner, bool f32 = true) {
    if (owner->dims == domain || owner->dims.empty()) return input(array, hint);
    ASSERT(owner->dims.size() < domain.size() &&
               std::equal(owner->dims.begin(), owner->dims.end(), domain.end() - (long)owner->dims.size()),
           "value '" << hint << "' does not have the dimensions of the kernel that reads it, nor trailing ones");
    bool known = false;
    for (auto& b : body.bcArrays) known = known || b.first == array;
    if (!known) body.bcArrays.push_back({array, count_expr(owner)});
    // the broadcast pointer is declared and filled as a const float* named after the ARRAY (a stage's buffer may be
    // another tensor or an S<k> buffer, not the stage's own name)
    ASSERT(f32, "HIP target: broadcast operand '" << hint << "' must hold Float32 elements");
    const std::string field = array.substr(0, array.find('['));
    return "s.bc_" + field + "[idx % s.bcn_" + field + "]";
  }

  std::string input(const std::string& array, const std::string& hint) {
    for (size_t k = 0; k < body.inArrays.size(); k++) if (body.inArrays[k] == array) return body.inNames[k];
    const std::string nm = "in_" + hint;
    body.inArrays.push_back(array);
    body.inNames.push_back(nm);
    return nm;
  }

  std::string emit(const NodePtr& n) {
    switch (n->kind) {
      case Kind::Tensor: {
        ASSERT(n->elem == Float32, "HIP target: pointwise stages take Float32 tensors ('" << n->name << "')");
        ASSERT(n->layout != Local, "tensor '" << n->name << "' is Local: it can only be read through AllReduce/ReduceScatter");
        auto it = tensorValue.find(n.get());
        if (it != tensorValue.end()) return it->second;
        return tensorValue[n.get()] = read(n->name, n->name, n);
      }
      case Kind::Variable: body.scalars.insert(n->name); return "s." + n->name;
      case Kind::Const: return fconst(n);
      case Kind::Binary: {
        static const char* op[] = {"+", "-", "*", "/"};
        const std::string a = emit(n->args[0]), b = emit(n->args[1]);
        return "(" + a + " " + op[(int)n->bin] + " " + b + ")";
      }
      case Kind::Compare: return "((" + emit(n->args[0]) + " > " + emit(n->args[1]) + ") ? 1.0f : 0.0f)";
      case Kind::Select: {   // the reference prints (cond ? a : b), src/codegen.cpp:660-666
        const NodePtr& c = n->args[0];
        const std::string cond = c->kind == Kind::Compare ? "(" + emit(c->args[0]) + " > " + emit(c->args[1]) + ")"
                                                          : "(" + emit(c) + " != 0.0f)";
        const std::string a = emit(n->args[1]), b = emit(n->args[2]);
        return "(" + cond + " ? " + a + " : " + b + ")";
      }
      case Kind::Unary: return "sqrtf(" + emit(n->args[0]) + ")";
      case Kind::Cast:
        if (n->elem == Float16) return "((float)(_Float16)(" + emit(n->args[0]) + "))";
        return emit(n->args[0]);
      case Kind::Dropout: {
        body.usesSeed = true;
        std::ostringstream o;
        o.precision(9);
        o << (reference_dropout() ? "ccn_gen::dropout_ref(" : "ccn_gen::dropout(") << emit(n->args[0]) << ", " << n->prob
          << "f, s.seed__, idx)";
        return o.str();
      }
      case Kind::Collective: {
        if (n->coll == CollOp::AllReduce || n->coll == CollOp::ReduceScatter) {
          ASSERT(n->red == Summation, "HIP target: only Summation collectives are lowered");
          ASSERT(n->args[0]->kind == Kind::Tensor, "fused reduce must read a Local tensor directly");
          ASSERT(!body.hasRed || body.redTensor == n->args[0]->name, "one reduced tensor per fused kernel");
          body.hasRed = true;
          body.redHalf = n->args[0]->elem == Float16;
          body.redTensor = n->args[0]->name;
          return "red";
        }
        return emit(n->args[0]);   // Scatter / AllGather / Broadcast: identity on one GPU
      }
      case Kind::Stage: {
        const int k = prog.p.stages().size() ? (int)(std::find(prog.p.stages().begin(), prog.p.stages().end(), n) -
                                                     prog.p.stages().begin()) : -1;
        ASSERT(k >= 0 && k < (int)prog.p.stages().size(), "stage " << n->name << " is not part of the pipeline");
        auto it = stageValue.find(k);
        if (it != stageValue.end()) return it->second;
        if (normIndex.count(k)) {   // a finished norm, read in the second pass
          ASSERT(phase2, "Norm value used before the reduction is complete");
          return "nrm[" + std::to_string(normIndex[k]) + "]";
        }
        ASSERT(!inGroup.count(k) || phase2, "stage " << n->name << " used before it is computed");
        ASSERT(prog.stageBuf.count(k), "stage " << n->name << " has no buffer but is read by another kernel");
        const NodePtr& def = n->args[0];
        const bool f32 = !(def->kind == Kind::Update && def->args[0]->elem == Float16);
        return stageValue[k] = read(prog.stageBuf[k], n->name, n, f32);
      }
      case Kind::Update:
      case Kind::Norm:
      case Kind::MatMul: ASSERT(false, "Update/Norm/MatMul may only appear at the top of a stage"); return "";
    }
    return "";
  }

  void store(const std::string& array, const std::string& value, bool half = false) {
    for (size_t k = 0; k < body.outArrays.size(); k++) {
      if (body.outArrays[k] == array) {
        body.code.push_back("out[" + std::to_string(k) + "] = " + value + ";");
        return;
      }
    }
    if (half) body.outHalfMask |= 1u << body.outArrays.size();
    body.outArrays.push_back(array);
    body.code.push_back("out[" + std::to_string(body.outArrays.size() - 1) + "] = " + value + ";");
  }

  // statements of one stage
  void stage(int k, bool withStores) {
    const NodePtr& st = prog.p.stages()[k];
    const NodePtr& def = st->args[0];
    const std::string v = "v_" + st->name;
    if (def->kind == Kind::Norm) {
      ASSERT(!phase2, "internal: norm accumulated in the second pass");
      const std::string x = emit(def->args[0]);
      const int slot = normIndex.count(k) ? normIndex[k] : (normIndex[k] = body.nacc++);
      if (def->plain_sum) {
        body.code.push_back("acc[" + std::to_string(slot) + "] += (double)(" + x + ");");
      } else {
        body.sqrtMask |= 1u << slot;
        body.code.push_back("{ const float x_ = " + x + "; acc[" + std::to_string(slot) + "] += (double)(x_ * x_); }");
      }
      return;
    }
    if (def->kind == Kind::Update) {
      const NodePtr& t = def->args[0];
      std::string x = emit(def->args[1]);
      if (t->elem == Float16) x = "((float)(_Float16)(" + x + "))";   // the value the fp16 array will hold
      body.code.push_back("const float " + v + " = " + x + ";");
      tensorValue[t.get()] = v;
      stageValue[k] = v;
      if (withStores) store(t->name, v, t->elem == Float16);
      return;
    }
    const std::string x = emit(def);
    body.code.push_back("const float " + v + " = " + x + ";");
    stageValue[k] = v;
    if (withStores && prog.p.storageOf(k) == StorageLocation::Memory) store(prog.stageBuf.at(k), v);
  }
};

std::string body_text(const Body& b, const std::vector<NodePtr>& scalarVars) {
  std::ostringstream o;
  o << "struct " << b.name << " {\n";
  o << "  static constexpr int NIN = " << b.inArrays.size() << ", NOUT = " << b.outArrays.size() << ", NACC = " << b.nacc
    << ", NNORM = " << b.nnorm << ";\n";
  o << "  static constexpr bool HAS_RED = " << (b.hasRed ? "true" : "false") << ";\n";
  o << "  using RedT = " << (b.redHalf ? "uint16_t" : "float") << ";\n";
  o << "  static constexpr unsigned OUT_F16 = " << b.outHalfMask << "u;\n";
  o << "  struct Scalars {";
  for (auto& v : scalarVars) o << " " << elem_c_type(v->elem) << " " << v->name << ";";
  for (auto& bc : b.bcArrays) {
    const std::string nm = bc.first.substr(0, bc.first.find('['));
    o << " const float* bc_" << nm << "; size_t bcn_" << nm << ";";
  }
  o << " uint64_t seed__; };\n";
  o << "  static __host__ __device__ __forceinline__ void apply(float red, const float* in, float* out, const Scalars& s,\n"
       "                                                        double* acc, const float* nrm, uint64_t idx) {\n";
  o << "    (void)red; (void)in; (void)out; (void)s; (void)acc; (void)nrm; (void)idx;\n";
  for (size_t k = 0; k < b.inNames.size(); k++) o << "    const float " << b.inNames[k] << " = in[" << k << "];\n";
  for (auto& line : b.code) o << "    " << line << "\n";
  o << "  }\n};\n\n";
  return o.str();
}

// ---- steps of the emitted driver -------------------------------------------------------------------------------------
struct Step {
  enum Type { Reduce, Copy, Kernel, TwoPassKernel } type = Kernel;
  std::string label;          // name used for the timer and the result line
  std::string count;          // element count expression
  // Reduce: ranks table -> dst;  Copy: src -> dst
  std::string src, dst;
  Body body, body2;           // Kernel / TwoPassKernel
  bool sliced = false;        // runs on one rank's slice [off, off + cnt) of the count
};

bool is_sliced(TensorLayout l) { return l == Sliced || l == Sliced_2; }

}  // namespace

std::string generateMLP(const Pipeline& p, const std::vector<CodeGenVarBounds>& bounds);

std::string generateHIP(const Pipeline& p, const std::vector<CodeGenVarBounds>& bounds) {
  for (auto& st : p.stages())
    if (contains_kind(st->args[0], Kind::MatMul)) return generateMLP(p, bounds);

  Program prog(p);
  for (auto& a : p.args()) {
    if (a->kind == Kind::Tensor) prog.tensors.push_back(a);
    else if (a->elem == Float16 || a->elem == Float32 || a->elem == Float64) prog.scalarVars.push_back(a);
    else prog.dimVars.push_back(a);
  }
  // dimension variables may be left out of the argument list (the reference's examples do): collect from tensors
  for (auto& t : prog.tensors)
    for (auto& d : t->dims)
      if (std::find(prog.dimVars.begin(), prog.dimVars.end(), d) == prog.dimVars.end()) prog.dimVars.push_back(d);
  for (auto& st : p.stages()) {
    std::vector<NodePtr> ts, vs;
    collect_leaves(st->args[0], ts, vs);
    for (auto& t : ts)
      ASSERT(std::find(prog.tensors.begin(), prog.tensors.end(), t) != prog.tensors.end(),
             "tensor '" << t->name << "' is used but is not a pipeline argument");
    for (auto& v : vs)
      ASSERT(std::find(p.args().begin(), p.args().end(), v) != p.args().end() ||
                 std::find(prog.dimVars.begin(), prog.dimVars.end(), v) != prog.dimVars.end(),
             "variable '" << v->name << "' is used but is not a pipeline argument");
    find_reduced(st->args[0], prog.reducedTensors);
  }
  // fp32 everywhere, with two exceptions: a gradient tensor folded over the ranks may hold fp16 (widened on load, summed
  // in fp32), and so may a tensor that stages only write (Update targets such as an fp16 copy of the weights; reading
  // one is refused where the read would be emitted)
  std::set<const Node*> updateTargets;
  for (auto& st : p.stages())
    if (st->args[0]->kind == Kind::Update) updateTargets.insert(st->args[0]->args[0].get());
  for (auto& t : prog.tensors)
    ASSERT(t->elem == Float32 || (t->elem == Float16 && (prog.reducedTensors.count(t.get()) || updateTargets.count(t.get()))),
           "HIP target: tensor '" << t->name << "' must be Float32 (Float16 only for a tensor read through AllReduce/"
           "ReduceScatter or written by Update)");

  const auto groups = p.groupsInOrder();
  const std::string fn = [&] { std::string s = p.name(); for (auto& c : s) if (!isalnum((unsigned char)c)) c = '_'; return s; }();

  // ---- buffers of stages that live in memory ------------------------------------------------------------------------
  for (auto& g : groups) {
    for (int k : g.stages) {
      if (p.storageOf(k) != StorageLocation::Memory) continue;
      const Node* def = p.stages()[k]->args[0].get();
      if (def->kind == Kind::Update) { prog.stageBuf[k] = def->args[0]->name; continue; }
      const Node* core = strip(def);
      if (g.stages.size() == 1 && core->kind == Kind::Collective && core->args[0]->kind == Kind::Tensor &&
          prog.reducedTensors.count(core->args[0].get())) {
        prog.stageBuf[k] = core->args[0]->name + "[0]";   // all-reduce in place into rank 0's buffer
        continue;
      }
      prog.stageBuf[k] = p.stages()[k]->name;
      prog.ownBuffers.push_back(k);
    }
  }

  // ---- lower every group to a step ----------------------------------------------------------------------------------
  std::vector<Step> steps;
  int kernelNo = 0;
  for (auto& g : groups) {
    Step step;
    step.count = count_expr(p.stages()[first_tensor_stage(p, g.stages)]);
    const Node* def0 = p.stages()[g.stages[0]]->args[0].get();
    const Node* core = strip(def0);
    if (g.stages.size() == 1 && core->kind == Kind::Collective && core->args[0]->kind == Kind::Tensor &&
        prog.reducedTensors.count(core->args[0].get())) {
      // a collective on its own: the stock all-reduce, here the library's P-way reduce into rank 0's buffer
      ASSERT(core->args[0]->elem == Float32, "HIP target: a Float16 tensor can only be reduced inside a fused kernel; fuse '"
                                                 << p.stages()[g.stages[0]]->name << "' with its consumers");
      step.type = Step::Reduce;
      step.sliced = core->coll == CollOp::ReduceScatter;
      step.label = core->coll == CollOp::AllReduce ? "AllReduce" : "ReduceScatter";
      step.src = core->args[0]->name;
      step.dst = def0->kind == Kind::Update ? def0->args[0]->name : core->args[0]->name + "[0]";
      steps.push_back(step);
      continue;
    }
    if (g.stages.size() == 1 && (core->kind == Kind::Stage || core->kind == Kind::Tensor) && core != def0) {
      // Update(t, AllGather(S)) or a bare AllGather/Scatter of a value in memory: a device copy
      step.type = Step::Copy;
      step.label = "AllGather";
      step.sliced = is_sliced(core->layout);   // gathering a Sliced value: every rank copies its slice into place
      if (core->kind == Kind::Stage) {
        int k = (int)(std::find_if(p.stages().begin(), p.stages().end(), [&](const NodePtr& q) { return q.get() == core; }) -
                      p.stages().begin());
        step.src = prog.stageBuf.at(k);
      } else {
        step.src = core->name;
      }
      step.dst = prog.stageBuf.at(g.stages[0]);
      if (step.src != step.dst) steps.push_back(step);
      continue;
    }

    // pointwise kernel, one or two passes
    bool hasNorm = false;
    for (int k : g.stages) hasNorm = hasNorm || p.stages()[k]->args[0]->kind == Kind::Norm;
    step.label = "kernel" + std::to_string(kernelNo);
    step.sliced = is_sliced(p.stages()[first_tensor_stage(p, g.stages)]->layout);
    if (!hasNorm) {
      BodyBuilder bb(prog, g);
      bb.body.name = fn + "_body" + std::to_string(kernelNo);
      for (int k : g.stages) bb.stage(k, true);
      step.type = Step::Kernel;
      step.body = bb.body;
    } else {
      // pass 1: everything that does not depend on a norm (and the sums of squares);
      // pass 2: the rest, with the pass-1 values it needs recomputed from memory.
      std::set<int> dependsOnNorm;
      for (int k : g.stages) {
        if (p.stages()[k]->args[0]->kind == Kind::Norm) continue;
        for (int d : p.stageDeps(k))
          if (bb_in(g, d) && (p.stages()[d]->args[0]->kind == Kind::Norm || dependsOnNorm.count(d))) dependsOnNorm.insert(k);
      }
      BodyBuilder b1(prog, g);
      b1.body.name = fn + "_body" + std::to_string(kernelNo) + "_pass1";
      for (int k : g.stages) if (!dependsOnNorm.count(k)) b1.stage(k, true);
      // values of pass 1 that pass 2 reads, transitively
      std::set<int> need;
      std::function<void(int)> want = [&](int k) {
        for (int d : p.stageDeps(k)) {
          if (!bb_in(g, d) || dependsOnNorm.count(d) || p.stages()[d]->args[0]->kind == Kind::Norm) continue;
          if (need.insert(d).second && p.stages()[d]->args[0]->kind != Kind::Update) want(d);
        }
      };
      for (int k : dependsOnNorm) want(k);
      BodyBuilder b2(prog, g);
      b2.phase2 = true;
      b2.body.name = fn + "_body" + std::to_string(kernelNo) + "_pass2";
      b2.normIndex = b1.normIndex;
      b2.body.nnorm = b1.body.nacc;
      for (int k : g.stages) {
        if (dependsOnNorm.count(k)) { b2.stage(k, true); continue; }
        if (!need.count(k)) continue;
        const NodePtr& def = p.stages()[k]->args[0];
        if (def->kind == Kind::Update) {
          // the updated tensor already holds this stage's value
          const std::string nm = b2.input(def->args[0]->name, def->args[0]->name);
          b2.stageValue[k] = nm;
          b2.tensorValue[def->args[0].get()] = nm;
        } else {
          // recomputed: it must not read a tensor that pass 1 updates later in program order
          std::vector<NodePtr> ts, vs;
          collect_leaves(def, ts, vs);
          for (auto& t : ts)
            for (int u : g.stages)
              ASSERT(!(u > k && !dependsOnNorm.count(u) && p.stages()[u]->args[0]->kind == Kind::Update &&
                       p.stages()[u]->args[0]->args[0] == t),
                     "two-pass kernel: stage " << p.stages()[k]->name << " would have to be recomputed from the old '"
                                               << t->name << "', which the first pass overwrites");
          b2.stage(k, false);
        }
      }
      step.type = Step::TwoPassKernel;
      step.body = b1.body;
      step.body2 = b2.body;
    }
    kernelNo++;
    steps.push_back(step);
  }

  // ---- text ---------------------------------------------------------------------------------------------------------
  std::ostringstream o;
  o << "// Generated by the coconet_amd HIP target from pipeline \"" << p.name() << "\".  Do not edit.\n";
  o << "// Build: hipcc --offload-arch=gfx950 -O3 -ffp-contract=off -Xclang -target-feature -Xclang -packed-fp32-ops \\\n"
       "//        -I <repo>/include -I <repo>/coconet_amd/dsl/include <this file> -L <repo>/coconet_amd/lib -lcoconet_hip\n";
  o << "// Run:   ./a.out <epochs> [ranks=4] [min_log2_size=10] [max_log2_size=29] [check=1] [untimed_warmup_epochs=0]\n";
  o << "// Environment: CCN_GEN_N=<n> runs that one size instead of the sweep; CCN_GEN_MISALIGN=1 starts every device array\n"
       "//        4 bytes past a 16-byte boundary; CCN_GEN_<scalar>=<value> sets a scalar argument (default 0.5);\n"
       "//        CCN_GEN_DUMP=<prefix> writes every updated tensor after the last epoch to <prefix>.<tensor>.<n>.f32;\n"
       "//        CCN_GEN_PERTURB=1 corrupts one device value before the comparison (to see the check fail);\n"
       "//        CCN_GEN_ONLY_RANK=<r> (schedules over Sliced values) runs that one rank's share only, unchecked.\n";
  o << "#include \"ccn_codegen_rt.hpp\"\n\n";
  for (auto& st : steps) {
    if (st.type == Step::Kernel) o << body_text(st.body, prog.scalarVars);
    if (st.type == Step::TwoPassKernel) o << body_text(st.body, prog.scalarVars) << body_text(st.body2, prog.scalarVars);
  }

  // driver signature: dims, scalars, tensors (a Local reduced tensor is a table of rank buffers), stage buffers,
  // timers, ranks, stream
  auto sig = [&](bool decl) {
    std::ostringstream q;
    bool first = true;
    auto add = [&](const std::string& type, const std::string& name) {
      q << (first ? "" : ", ") << (decl ? type + " " : "") << name;
      first = false;
    };
    for (auto& d : prog.dimVars) add("size_t", d->name);
    for (auto& v : prog.scalarVars) add(elem_c_type(v->elem), v->name);
    for (auto& t : prog.tensors)
      add(prog.reducedTensors.count(t.get()) ? (t->elem == Float16 ? "uint16_t* const*" : "float* const*")
                                             : (t->elem == Float16 ? "uint16_t*" : "float*"), t->name);
    for (int k : prog.ownBuffers) add("float*", p.stages()[k]->name);
    add("double*", "partials__");
    add("float*", "norms__");
    for (auto& st : steps) add("float&", "elapsedTime" + st.label);
    add("int", "comm_size");
    add("int", "rank");
    add("uint64_t", "seed__");
    add("void*", "stream");
    return q.str();
  };

  auto scalars_init = [&](const std::string& var) {
    std::ostringstream q;
    for (auto& v : prog.scalarVars) q << "  " << var << ".s." << v->name << " = " << v->name << ";\n";
    q << "  " << var << ".s.seed__ = seed__;\n";
    return q.str();
  };
  // off: element offset added to every array of the kernel ("" = none); count: elements the launch covers
  auto fill_args = [&](const Body& b, const std::string& var, const std::string& count, const std::string& off) {
    std::ostringstream q;
    const std::string plus = off.empty() ? "" : " + " + off;
    q << "  ccn_gen::KernelArgs<" << b.name << "> " << var << ";\n";
    q << "  for (int p_ = 0; p_ < ccn_gen::kMaxRanks; p_++) " << var << ".red[p_] = "
      << (b.hasRed ? b.redTensor + "[p_ < comm_size ? p_ : 0]" + plus : std::string("nullptr")) << ";\n";
    q << "  " << var << ".nranks = " << (b.hasRed ? "comm_size" : "1") << ";\n";
    if (b.inArrays.empty()) q << "  " << var << ".in[0] = nullptr;\n";
    for (size_t k = 0; k < b.inArrays.size(); k++) q << "  " << var << ".in[" << k << "] = " << b.inArrays[k] << plus << ";\n";
    if (b.outArrays.empty()) q << "  " << var << ".out[0] = nullptr;\n";
    for (size_t k = 0; k < b.outArrays.size(); k++) q << "  " << var << ".out[" << k << "] = " << b.outArrays[k] << plus << ";\n";
    q << "  " << var << ".partials = partials__;\n  " << var << ".norms = norms__;\n  " << var << ".n = " << count << ";\n";
    q << "  " << var << ".idx_base = " << (off.empty() ? "0" : off) << ";\n";
    for (auto& bc : b.bcArrays) {
      const std::string nm = bc.first.substr(0, bc.first.find('['));
      q << "  " << var << ".s.bc_" << nm << " = " << bc.first << ";\n  " << var << ".s.bcn_" << nm << " = " << bc.second << ";\n";
    }
    q << scalars_init(var);
    return q.str();
  };
  // the ranks a step over Sliced values runs for, and the slice of rank r_ (src/codegen.cpp:485-499)
  const std::string rank_loop =
      "  for (int r_ = rank < 0 ? 0 : rank; r_ < (rank < 0 ? comm_size : rank + 1); r_++) {\n";
  auto slice_of = [&](const std::string& count) {
    return "  const size_t n__ = " + count + ", per__ = DIVUP(n__, (size_t)comm_size), off__ = per__ * (size_t)r_;\n"
           "  if (off__ >= n__) continue;\n"
           "  const size_t cnt__ = off__ + per__ <= n__ ? per__ : n__ - off__;\n";
  };
  // the body of a rank loop, one level deeper
  auto deeper = [](const std::string& text) {
    std::string out;
    size_t at = 0;
    while (at < text.size()) {
      const size_t nl = text.find('\n', at);
      const std::string line = text.substr(at, nl == std::string::npos ? std::string::npos : nl - at + 1);
      out += (line == "\n" ? "" : "  ") + line;
      if (nl == std::string::npos) break;
      at = nl + 1;
    }
    return out;
  };

  o << "void " << fn << "(" << sig(true) << ") {\n";
  o << "  void *start__, *stop__;\n  float elapsedTime;\n";
  o << "  CCNCHECK(ccn_event_create(&start__));\n  CCNCHECK(ccn_event_create(&stop__));\n\n";
  int argNo = 0;
  for (auto& st : steps) {
    o << "  CCNCHECK(ccn_event_record(start__, stream));\n";
    if (st.type == Step::Reduce && !st.sliced) {
      o << "  CCNCHECK(ccn_reduce_f32(" << st.src << ", comm_size, " << st.dst << ", " << st.count << ", stream));\n";
    } else if (st.type == Step::Reduce) {
      o << rank_loop
        << deeper(slice_of(st.count) + "  const float* tbl__[ccn_gen::kMaxRanks];\n" +
                  "  for (int p_ = 0; p_ < comm_size; p_++) tbl__[p_] = " + st.src + "[p_] + off__;\n" +
                  "  CCNCHECK(ccn_reduce_f32(tbl__, comm_size, " + st.dst + " + off__, cnt__, stream));\n")
        << "  }\n";
    } else if (st.type == Step::Copy && !st.sliced) {
      o << "  CCNCHECK(ccn_memcpy_d2d(" << st.dst << ", " << st.src << ", (" << st.count << ") * sizeof(float), stream));\n";
    } else if (st.type == Step::Copy) {
      o << rank_loop
        << deeper(slice_of(st.count) + "  CCNCHECK(ccn_memcpy_d2d(" + st.dst + " + off__, " + st.src +
                  " + off__, cnt__ * sizeof(float), stream));\n")
        << "  }\n";
    } else if (st.type == Step::Kernel) {
      const std::string a = "args" + std::to_string(argNo++);
      if (!st.sliced) {
        o << "  {\n" << deeper(fill_args(st.body, a, st.count, "") + "  ccn_gen::launch(" + a + ", stream);\n") << "  }\n";
      } else {
        o << rank_loop << deeper(slice_of(st.count) + fill_args(st.body, a, "cnt__", "off__") + "  ccn_gen::launch(" + a + ", stream);\n")
          << "  }\n";
      }
    } else if (!st.sliced) {
      const std::string a = "args" + std::to_string(argNo++), b = "args" + std::to_string(argNo++);
      std::ostringstream q;
      q << fill_args(st.body, a, st.count, "") << "  const unsigned blocks__ = ccn_gen::launch(" << a << ", stream);\n";
      q << "  ccn_gen::finalize_norms(partials__, partials__ + (size_t)ccn_gen::blocks_for(" << st.count << ") * 8, blocks__, "
        << st.body.nacc << ", " << st.body.sqrtMask << "u, norms__, stream);\n";
      q << fill_args(st.body2, b, st.count, "") << "  ccn_gen::launch(" << b << ", stream);\n";
      o << "  {\n" << deeper(q.str()) << "  }\n";
    } else {
      // Norms over Sliced values span every rank's slice (the reference all-reduces them): pass 1 on every slice, each
      // launch's partial sums behind the previous one's, one finalize over all of them, then pass 2 on every slice.
      const std::string a = "args" + std::to_string(argNo++), b = "args" + std::to_string(argNo++);
      o << "  if (rank >= 0 && comm_size > 1) { printf(\"this pipeline's norms span all slices: call with rank = -1\\n\"); exit(EXIT_FAILURE); }\n";
      std::ostringstream q;
      q << "  unsigned rows__ = 0;\n";
      q << rank_loop
        << deeper(slice_of(st.count) + fill_args(st.body, a, "cnt__", "off__") + "  " + a +
                  ".partials = partials__ + (size_t)rows__ * " + std::to_string(st.body.nacc) + ";   // behind the previous slice's\n" +
                  "  rows__ += ccn_gen::launch(" + a + ", stream);\n")
        << "  }\n";
      q << "  ccn_gen::finalize_norms(partials__, partials__ + (size_t)ccn_gen::blocks_for(" << st.count << ") * 8, rows__, "
        << st.body.nacc << ", " << st.body.sqrtMask << "u, norms__, stream);\n";
      q << rank_loop
        << deeper(slice_of(st.count) + fill_args(st.body2, b, "cnt__", "off__") + "  ccn_gen::launch(" + b + ", stream);\n")
        << "  }\n";
      o << "  {\n" << deeper(q.str()) << "  }\n";
    }
    o << "  CCNCHECK(ccn_event_record(stop__, stream));\n";
    o << "  CCNCHECK(ccn_event_elapsed_ms(start__, stop__, &elapsedTime));\n";
    o << "  elapsedTime" << st.label << " += elapsedTime;\n\n";
  }
  o << "  CCNCHECK(ccn_event_destroy(start__));\n  CCNCHECK(ccn_event_destroy(stop__));\n}\n\n";

  // ---- CPU re-execution of the pipeline, stage by stage --------------------------------------------------------------
  // host mirrors: std::vector<float> per tensor (per rank for reduced tensors) and per stage
  o << "// CPU re-execution, one loop per stage in pipeline order; the all-reduce is the fixed-order sum over ranks.\n";
  o << "struct HostState {\n";
  for (auto& t : prog.tensors) {
    if (prog.reducedTensors.count(t.get())) o << "  std::vector<std::vector<float>> " << t->name << ";\n";
    else o << "  std::vector<float> " << t->name << ";\n";
  }
  for (size_t k = 0; k < p.stages().size(); k++) o << "  std::vector<float> " << p.stages()[k]->name << ";\n";
  o << "};\n\n";
  o << "void " << fn << "_cpu(HostState& h";
  for (auto& d : prog.dimVars) o << ", size_t " << d->name;
  for (auto& v : prog.scalarVars) o << ", " << elem_c_type(v->elem) << " " << v->name;
  o << ", int comm_size, uint64_t seed__) {\n  (void)seed__; (void)comm_size;\n";
  {
    // host expression emitter: arrays indexed by i0
    std::vector<NodePtr> hostDomain;   // dimensions of the stage whose loop is being written
    auto at = [&](const NodePtr& n) {
      return (n->dims.empty() || n->dims == hostDomain) ? std::string("[i0]") : "[i0 % h." + n->name + ".size()]";
    };
    std::function<std::string(const NodePtr&)> he = [&](const NodePtr& n) -> std::string {
      switch (n->kind) {
        case Kind::Tensor: return "h." + n->name + at(n);
        case Kind::Variable: return n->name;
        case Kind::Const: return fconst(n);
        case Kind::Binary: {
          static const char* op[] = {"+", "-", "*", "/"};
          return "(" + he(n->args[0]) + " " + op[(int)n->bin] + " " + he(n->args[1]) + ")";
        }
        case Kind::Compare: return "((" + he(n->args[0]) + " > " + he(n->args[1]) + ") ? 1.0f : 0.0f)";
        case Kind::Select: {
          const NodePtr& c = n->args[0];
          const std::string cond = c->kind == Kind::Compare ? "(" + he(c->args[0]) + " > " + he(c->args[1]) + ")"
                                                            : "(" + he(c) + " != 0.0f)";
          return "(" + cond + " ? " + he(n->args[1]) + " : " + he(n->args[2]) + ")";
        }
        case Kind::Unary: return "sqrtf(" + he(n->args[0]) + ")";
        case Kind::Cast: return n->elem == Float16 ? "((float)(_Float16)(" + he(n->args[0]) + "))" : he(n->args[0]);
        case Kind::Dropout: {
          std::ostringstream q;
          q.precision(9);
          q << (reference_dropout() ? "ccn_gen::dropout_ref(" : "ccn_gen::dropout(") << he(n->args[0]) << ", " << n->prob
            << "f, seed__, (uint64_t)i0)";
          return q.str();
        }
        case Kind::Collective:
          if (n->coll == CollOp::AllReduce || n->coll == CollOp::ReduceScatter) {
            ASSERT(n->args[0]->kind == Kind::Tensor, "reduce of a non-tensor");
            return "rsum(h." + n->args[0]->name + ", i0)";
          }
          return he(n->args[0]);
        case Kind::Stage: {
          if (n->args[0]->kind == Kind::Norm) return "h." + n->name + "[0]";
          return "h." + n->name + at(n);
        }
        default: ASSERT(false, "unexpected node in a stage expression"); return "";
      }
    };
    o << "  auto rsum = [&](const std::vector<std::vector<float>>& g, size_t i) { float s = g[0][i]; for (int p_ = 1; p_ < comm_size; p_++) s = s + g[p_][i]; return s; };\n";
    o << "  (void)rsum;\n";
    for (size_t k = 0; k < p.stages().size(); k++) {
      const NodePtr& st = p.stages()[k];
      const NodePtr& def = st->args[0];
      if (def->kind == Kind::Norm) {
        const NodePtr& x = def->args[0];
        ASSERT(x->kind == Kind::Stage || x->kind == Kind::Tensor, "Norm takes a stage or a tensor");
        hostDomain = x->dims;
        o << "  { double a_ = 0.0; const size_t n_ = " << count_expr(x) << ";\n";
        if (def->plain_sum) {
          o << "    for (size_t i0 = 0; i0 < n_; i0++) a_ += (double)(" << he(x) << ");\n";
          o << "    h." << st->name << ".assign(1, (float)a_); }\n";
        } else {
          o << "    for (size_t i0 = 0; i0 < n_; i0++) { const float x_ = " << he(x) << "; a_ += (double)(x_ * x_); }\n";
          o << "    h." << st->name << ".assign(1, (float)sqrt(a_)); }\n";
        }
        continue;
      }
      const std::string cnt = count_expr(st);
      hostDomain = st->dims;
      o << "  h." << st->name << ".resize(" << cnt << ");\n";
      o << "  for (size_t i0 = 0; i0 < " << cnt << "; i0++) {\n";
      if (def->kind == Kind::Update) {
        if (def->args[0]->elem == Float16) o << "    h." << st->name << "[i0] = (float)(_Float16)(" << he(def->args[1]) << ");\n";
        else o << "    h." << st->name << "[i0] = " << he(def->args[1]) << ";\n";
        o << "    h." << def->args[0]->name << "[i0] = h." << st->name << "[i0];\n";
      } else {
        o << "    h." << st->name << "[i0] = " << he(def) << ";\n";
      }
      o << "  }\n";
    }
  }
  o << "}\n\n";

  // ---- main ----------------------------------------------------------------------------------------------------------
  o << "int main(int argc, char** argv) {\n";
  o << "  if (argc < 2) { printf(\"Specify epochs as command arg\"); return 1; }\n";
  o << "  const int epochs = atoi(argv[1]);\n";
  o << "  const int comm_size = argc > 2 ? atoi(argv[2]) : 4;\n";
  o << "  const int lo__ = argc > 3 ? atoi(argv[3]) : 10, hi__ = argc > 4 ? atoi(argv[4]) : 29;\n";
  o << "  const int only__ = getenv(\"CCN_GEN_ONLY_RANK\") ? atoi(getenv(\"CCN_GEN_ONLY_RANK\")) : -1;\n";
  o << "  const bool check__ = (argc > 5 ? atoi(argv[5]) != 0 : true) && only__ < 0;   // one rank's share is not the whole result\n";
  // The reference times every epoch, the first (cold) one included; warm-up epochs are an addition, off by default.
  o << "  const int warmup__ = argc > 6 && atoi(argv[6]) > 0 ? atoi(argv[6]) : 0;\n";
  o << "  if (comm_size < 1 || comm_size > ccn_gen::kMaxRanks) { printf(\"ranks must be 1..%d\\n\", ccn_gen::kMaxRanks); return 1; }\n";
  o << "  CCNCHECK(ccn_init(0));\n  void* stream;\n  CCNCHECK(ccn_stream_create(&stream));\n  const uint64_t seed__ = 1234;\n  bool allOk__ = true;\n";
  o << "  const size_t one_size__ = ccn_gen::env_size(\"CCN_GEN_N\", 0);\n";
  o << "  const size_t pad__ = ccn_gen::env_size(\"CCN_GEN_MISALIGN\", 0) ? 1 : 0;   // elements every device array is moved on by\n";
  o << "  const char* dump__ = getenv(\"CCN_GEN_DUMP\");\n  (void)one_size__;\n\n";
  // size loop: explicit bounds when given, otherwise powers of two for every dimension variable
  std::map<std::string, std::vector<int>> bnd;
  for (auto& b : bounds) bnd[b.var.impl()->name] = b.values;
  int depth = 0;
  std::string ind = "  ";
  bool sweep = false;
  for (auto& d : prog.dimVars) {
    if (bnd.count(d->name)) {
      o << ind << "for (size_t " << d->name << " : std::vector<size_t>{";
      for (size_t k = 0; k < bnd[d->name].size(); k++) o << (k ? ", " : "") << bnd[d->name][k];
      o << "}) {\n";
    } else if (!sweep) {
      o << ind << "for (int __i = lo__; __i <= (one_size__ ? lo__ : hi__); __i++) {\n" << ind << "  const size_t " << d->name
        << " = one_size__ ? one_size__ : (size_t)1 << __i;\n";
      sweep = true;
    } else {
      o << ind << "{\n" << ind << "  const size_t " << d->name << " = one_size__ ? one_size__ : (size_t)1 << __i;\n";
    }
    depth++;
    ind += "  ";
  }
  o << ind << "// Inputs (uniform in (0,1], seed 1234; the reference uses cuRAND with the same seed and range)\n";
  int seedNo = 0;
  for (auto& t : prog.tensors) {
    const std::string cnt = count_expr(t);
    const bool half = t->elem == Float16;
    const std::string ct = half ? "uint16_t" : "float";
    if (prog.reducedTensors.count(t.get())) {
      o << ind << "std::vector<" << ct << "*> " << t->name << "(comm_size);\n";
      o << ind << "std::vector<std::vector<float>> h_" << t->name << "(comm_size);\n";
      o << ind << "for (int p_ = 0; p_ < comm_size; p_++) {\n";
      o << ind << "  CCNCHECK(ccn_malloc((void**)&" << t->name << "[p_], (" << cnt << " + pad__) * sizeof(" << ct << ")));\n";
      o << ind << "  " << t->name << "[p_] += pad__;\n";
      o << ind << "  ccn_gen::fill_uniform" << (half ? "_f16" : "") << "(" << t->name << "[p_], " << cnt << ", seed__ + " << (seedNo + 100) << " + p_, check__ ? &h_"
        << t->name << "[p_] : nullptr);\n" << ind << "}\n";
      seedNo += 100;
    } else {
      o << ind << ct << "* " << t->name << ";\n";
      o << ind << "std::vector<float> h_" << t->name << ";\n";
      o << ind << "CCNCHECK(ccn_malloc((void**)&" << t->name << ", (" << cnt << " + pad__) * sizeof(" << ct << ")));\n";
      o << ind << t->name << " += pad__;\n";
      o << ind << "ccn_gen::fill_uniform" << (half ? "_f16" : "") << "(" << t->name << ", " << cnt << ", seed__ + " << (++seedNo) << ", check__ ? &h_" << t->name
        << " : nullptr);\n";
    }
  }
  for (auto& v : prog.scalarVars)   // the reference sets 1.0f, which zeroes every (1 - beta) term
    o << ind << elem_c_type(v->elem) << " " << v->name << " = ccn_gen::env_float(\"CCN_GEN_" << v->name << "\", 0.5f);\n";
  for (int k : prog.ownBuffers) {
    o << ind << "float* " << p.stages()[k]->name << ";\n";
    o << ind << "CCNCHECK(ccn_malloc((void**)&" << p.stages()[k]->name << ", (" << count_expr(p.stages()[k]) << " + pad__) * sizeof(float)));\n";
    o << ind << p.stages()[k]->name << " += pad__;\n";
  }
  std::vector<int> allStages__;
  for (size_t k = 0; k < p.stages().size(); k++) allStages__.push_back((int)k);
  const std::string anyCount = count_expr(p.stages()[first_tensor_stage(p, allStages__)]);
  o << ind << "double* partials__;\n" << ind << "float* norms__;\n";
  o << ind << "CCNCHECK(ccn_malloc((void**)&partials__, ccn_gen::partials_doubles(" << anyCount << ") * sizeof(double)));\n";
  o << ind << "CCNCHECK(ccn_malloc((void**)&norms__, 8 * sizeof(float)));\n";
  o << ind << "// Outputs\n";
  for (auto& st : steps) o << ind << "float elapsedTime" << st.label << " = 0;\n";
  o << ind << "HostState h;\n";
  o << ind << "if (check__) {\n";
  for (auto& t : prog.tensors) o << ind << "  h." << t->name << " = h_" << t->name << ";\n";
  o << ind << "}\n";
  o << ind << "for (int iter = -warmup__; iter < epochs; iter++) {\n";
  o << ind << "  if (iter == 0) {";
  for (auto& st : steps) o << " elapsedTime" << st.label << " = 0;";
  o << " }\n";
  {
    // call with the same argument order as the signature; a pipeline with steps over Sliced values runs rank by rank
    // (every rank's share in turn: the union of the slices is the whole update), all ranks inside one call when norms
    // span the slices, and once otherwise (on Replicated values every rank would compute the same)
    bool anySliced = false, slicedNorms = false;
    for (auto& st : steps) {
      anySliced = anySliced || st.sliced;
      slicedNorms = slicedNorms || (st.sliced && st.type == Step::TwoPassKernel);
    }
    std::ostringstream q;
    bool first = true;
    auto add = [&](const std::string& name) { q << (first ? "" : ", ") << name; first = false; };
    for (auto& d : prog.dimVars) add(d->name);
    for (auto& v : prog.scalarVars) add(v->name);
    for (auto& t : prog.tensors) add(prog.reducedTensors.count(t.get()) ? t->name + ".data()" : t->name);
    for (int k : prog.ownBuffers) add(p.stages()[k]->name);
    add("partials__");
    add("norms__");
    for (auto& st : steps) add("elapsedTime" + st.label);
    add("comm_size");
    add(anySliced ? (slicedNorms ? "-1" : "rank__") : "0");
    add("seed__");
    add("stream");
    if (anySliced && !slicedNorms)
      o << ind << "  for (int rank__ = 0; rank__ < comm_size; rank__++)\n" << ind << "    if (only__ < 0 || rank__ == only__)\n    ";
    o << ind << "  " << fn << "(" << q.str() << ");\n";
  }
  o << ind << "  if (check__ && iter == -warmup__) {\n";
  o << ind << "    CCNCHECK(ccn_stream_sync(stream));\n";
  o << ind << "    " << fn << "_cpu(h";
  for (auto& d : prog.dimVars) o << ", " << d->name;
  for (auto& v : prog.scalarVars) o << ", " << v->name;
  o << ", comm_size, seed__);\n";
  o << ind << "    bool ok__ = true;\n";
  // compare every tensor that some stage updates and every output stage with a buffer.  Without norms the kernels round
  // exactly as the host loops do and the bar is the benchmark's 1e-6; norm sums associate differently: 1e-5.
  bool anyNorm = false;
  for (auto& st : p.stages()) anyNorm = anyNorm || st->args[0]->kind == Kind::Norm;
  const std::string tol = anyNorm ? "1e-5f" : "1e-6f";
  std::set<std::string> updated;
  std::map<std::string, bool> updatedHalf;
  for (auto& st : p.stages())
    if (st->args[0]->kind == Kind::Update) {
      updated.insert(st->args[0]->args[0]->name);
      updatedHalf[st->args[0]->args[0]->name] = st->args[0]->args[0]->elem == Float16;
    }
  if (!updated.empty() && !updatedHalf[*updated.begin()])
    o << ind << "    if (getenv(\"CCN_GEN_PERTURB\")) ccn_gen::perturb(" << *updated.begin() << ", h." << *updated.begin() << ".size() / 2);\n";
  for (auto& t : updated) o << ind << "    ok__ = ok__ && ccn_gen::compare(\"" << t << "\", h." << t << ", " << t << ", h." << t << ".size(), " << tol << ");\n";
  for (int k : prog.ownBuffers)
    if (p.isOutput(k))
      o << ind << "    ok__ = ok__ && ccn_gen::compare(\"" << p.stages()[k]->name << "\", h." << p.stages()[k]->name << ", "
        << p.stages()[k]->name << ", h." << p.stages()[k]->name << ".size(), " << tol << ");\n";
  o << ind << "    if (!ok__) { printf(\"Results do not match the CPU re-execution\\n\"); allOk__ = false; }\n";
  o << ind << "  }\n";
  o << ind << "}\n";
  o << ind << "CCNCHECK(ccn_stream_sync(stream));\n";
  o << ind << "if (dump__) {\n";
  for (auto& t : updated)
    o << ind << "  ccn_gen::dump(dump__, \"" << t << "\", " << t << ", " << count_expr(*std::find_if(prog.tensors.begin(), prog.tensors.end(), [&](const NodePtr& q) { return q->name == t; })) << ");\n";
  // ... and every output stage that lives in a buffer of its own (a final value no Update writes back)
  for (int k : prog.ownBuffers)
    if (p.isOutput(k))
      o << ind << "  ccn_gen::dump(dump__, \"" << p.stages()[k]->name << "\", " << p.stages()[k]->name << ", " << count_expr(p.stages()[k]) << ");\n";
  o << ind << "}\n";
  o << ind << "CCNCHECK(ccn_stream_sync(stream));\n";
  for (auto& t : prog.tensors) {
    if (prog.reducedTensors.count(t.get())) o << ind << "for (int p_ = 0; p_ < comm_size; p_++) CCNCHECK(ccn_free(" << t->name << "[p_] - pad__));\n";
    else o << ind << "CCNCHECK(ccn_free(" << t->name << " - pad__));\n";
  }
  for (int k : prog.ownBuffers) o << ind << "CCNCHECK(ccn_free(" << p.stages()[k]->name << " - pad__));\n";
  o << ind << "CCNCHECK(ccn_free(partials__));\n" << ind << "CCNCHECK(ccn_free(norms__));\n";
  // result line, reference format (src/codegen.cpp:4732-4767)
  o << ind << "printf(\"{SZ: %ld, Epochs: %d";
  for (auto& st : steps) o << ", " << st.label << ": %f";
  o << ", Total: %f}\\n\", (long)(" << anyCount << "), epochs";
  std::string total;
  for (auto& st : steps) {
    o << ", elapsedTime" << st.label;
    total += (total.empty() ? "" : " + ") + ("elapsedTime" + st.label);
  }
  o << ", " << (total.empty() ? "0.0f" : total) << ");\n";
  for (int k = 0; k < depth; k++) {
    ind.resize(ind.size() - 2);
    o << ind << "}\n";
  }
  o << "  CCNCHECK(ccn_stream_destroy(stream));\n";
  o << "  if (!allOk__) return 2;\n  return 0;\n}\n";
  return o.str();
}

}  // namespace ACCCDSL
