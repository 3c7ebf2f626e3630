// Pipeline: stage discovery, fusion with legality check, storage classes, printing.
#include "pipeline.hpp"

#include <algorithm>
#include <fstream>
#include <functional>
#include <sstream>

namespace ACCCDSL {
using namespace ir;

// Stages directly referenced by an expression (not looking through them).
static void stages_in(const NodePtr& n, std::vector<NodePtr>& out) {
  if (n->kind == Kind::Stage) {
    out.push_back(n);
    return;
  }
  for (auto& a : n->args) stages_in(a, out);
}

Pipeline::Pipeline(std::string name, std::vector<Expression> args, std::vector<Stage> outputs) : name_(std::move(name)) {
  ASSERT(!outputs.empty(), "a pipeline needs at least one output stage");
  for (auto& a : args) {
    ASSERT(a.impl()->kind == Kind::Tensor || a.impl()->kind == Kind::Variable,
           "pipeline arguments are tensors and variables");
    args_.push_back(a.impl());
  }
  // every stage reachable from the outputs
  std::set<int> seen;
  std::vector<NodePtr> found;
  std::function<void(const NodePtr&)> visit = [&](const NodePtr& st) {
    if (!seen.insert(st->id).second) return;
    found.push_back(st);
    std::vector<NodePtr> deps;
    stages_in(st->args[0], deps);
    for (auto& d : deps) visit(d);
  };
  for (auto& o : outputs) visit(o.impl());
  std::sort(found.begin(), found.end(), [](const NodePtr& a, const NodePtr& b) { return a->id < b->id; });
  stages_ = found;
  for (auto& o : outputs) outputs_.insert(indexOf(o.impl()));
  groupOf_.resize(stages_.size());
  for (size_t i = 0; i < stages_.size(); i++) groupOf_[i] = (int)i;
}

int Pipeline::indexOf(const NodePtr& stage) const {
  for (size_t i = 0; i < stages_.size(); i++) if (stages_[i] == stage) return (int)i;
  return -1;
}

std::vector<int> Pipeline::stageDeps(int s) const {
  std::vector<NodePtr> deps;
  stages_in(stages_[s]->args[0], deps);
  std::vector<int> out;
  for (auto& d : deps) {
    int k = indexOf(d);
    if (k >= 0 && std::find(out.begin(), out.end(), k) == out.end()) out.push_back(k);
  }
  return out;
}

// With groups as super-nodes, an edge A -> B exists when a stage of B reads a stage of A.  Fusion is legal iff
// that graph stays acyclic (a group may not need a value that is computed from its own results elsewhere).
bool Pipeline::groupGraphHasCycle(const std::vector<int>& groupOf) const {
  std::map<int, std::set<int>> succ;
  for (size_t s = 0; s < stages_.size(); s++)
    for (int d : stageDeps((int)s))
      if (groupOf[d] != groupOf[s]) succ[groupOf[d]].insert(groupOf[s]);
  std::map<int, int> color;
  std::function<bool(int)> dfs = [&](int g) {
    color[g] = 1;
    for (int n : succ[g]) {
      if (color[n] == 1) return true;
      if (color[n] == 0 && dfs(n)) return true;
    }
    color[g] = 2;
    return false;
  };
  for (size_t s = 0; s < stages_.size(); s++)
    if (color[groupOf[s]] == 0 && dfs(groupOf[s])) return true;
  return false;
}

void Pipeline::fuse(std::vector<Stage> stages) {
  ASSERT(!stages.empty(), "fuse: empty stage list");
  std::vector<int> idx;
  for (auto& st : stages) {
    int k = indexOf(st.impl());
    ASSERT(k >= 0, "fuse: stage " << st.name() << " is not reachable from the pipeline outputs");
    idx.push_back(k);
  }
  std::vector<int> trial = groupOf_;
  const int target = trial[idx[0]];
  for (int k : idx) {
    const int from = trial[k];
    for (auto& g : trial) if (g == from) g = target;
  }
  ASSERT(!groupGraphHasCycle(trial), "fuse: the fused kernel would both feed and consume a stage left outside it");
  groupOf_ = trial;
}

void Pipeline::overlap(std::vector<Stage> stages) {
  std::vector<int> idx;
  for (auto& st : stages) {
    int k = indexOf(st.impl());
    ASSERT(k >= 0, "overlap: stage " << st.name() << " is not reachable from the pipeline outputs");
    idx.push_back(k);
  }
  std::vector<int> trial = groupOf_;
  const int target = trial[idx[0]];
  for (int k : idx) {
    const int from = trial[k];
    for (auto& g : trial) if (g == from) g = target;
  }
  if (!groupGraphHasCycle(trial)) groupOf_ = trial;
}

std::vector<Pipeline::Group> Pipeline::groupsInOrder() const {
  // creation order of each group's first stage is a valid topological order when the group graph is acyclic and
  // stages only read older stages ... except that fusing can pull an older stage behind a younger one; do a
  // proper topological sort on the group graph, ties broken by first stage.
  std::map<int, Group> groups;
  for (size_t s = 0; s < stages_.size(); s++) groups[groupOf_[s]].stages.push_back((int)s);
  std::map<int, std::set<int>> pred;
  for (size_t s = 0; s < stages_.size(); s++)
    for (int d : stageDeps((int)s))
      if (groupOf_[d] != groupOf_[s]) pred[groupOf_[s]].insert(groupOf_[d]);
  std::vector<Group> out;
  std::set<int> done;
  while (done.size() < groups.size()) {
    int pick = -1;
    for (auto& kv : groups) {
      if (done.count(kv.first)) continue;
      bool ready = true;
      for (int p : pred[kv.first]) if (!done.count(p)) ready = false;
      if (ready && (pick < 0 || kv.second.stages[0] < groups[pick].stages[0])) pick = kv.first;
    }
    ASSERT(pick >= 0, "pipeline has a cycle between fused groups");
    done.insert(pick);
    out.push_back(groups[pick]);
  }
  return out;
}

// A stage's value must be in memory when another kernel (or the caller) reads it or when it is an in-place
// tensor update; otherwise it lives in a register of the fused kernel.
StorageLocation Pipeline::storageOf(int s) const {
  if (isOutput(s)) return StorageLocation::Memory;
  if (stages_[s]->args[0]->kind == Kind::Update) return StorageLocation::Memory;
  for (size_t c = 0; c < stages_.size(); c++) {
    if (groupOf_[c] == groupOf_[s]) continue;
    auto deps = stageDeps((int)c);
    if (std::find(deps.begin(), deps.end(), s) != deps.end()) return StorageLocation::Memory;
  }
  return StorageLocation::Register;
}

static void print_expr(std::ostream& os, const NodePtr& n) {
  static const char* binop[] = {"+", "-", "*", "/"};
  static const char* coll[] = {"AllReduce", "ReduceScatter", "AllGather", "Scatter", "Broadcast"};
  switch (n->kind) {
    case Kind::Tensor:
    case Kind::Variable:
    case Kind::Stage: os << n->name; break;
    case Kind::Const: os << n->cval; break;
    case Kind::Binary:
      os << "(";
      print_expr(os, n->args[0]);
      os << " " << binop[(int)n->bin] << " ";
      print_expr(os, n->args[1]);
      os << ")";
      break;
    case Kind::Compare:
      os << "(";
      print_expr(os, n->args[0]);
      os << " > ";
      print_expr(os, n->args[1]);
      os << ")";
      break;
    case Kind::Select:
      os << "Ite(";
      print_expr(os, n->args[0]);
      os << ", ";
      print_expr(os, n->args[1]);
      os << ", ";
      print_expr(os, n->args[2]);
      os << ")";
      break;
    case Kind::Unary: os << "Sqrt("; print_expr(os, n->args[0]); os << ")"; break;
    case Kind::Cast: os << "Cast<" << elem_c_type(n->elem) << ">("; print_expr(os, n->args[0]); os << ")"; break;
    case Kind::Update:
      os << "Update(" << n->args[0]->name << ", ";
      print_expr(os, n->args[1]);
      os << ")";
      break;
    case Kind::Norm: os << (n->plain_sum ? "ReduceStage(" : "Norm("); print_expr(os, n->args[0]); os << ")"; break;
    case Kind::Dropout: os << "Dropout("; print_expr(os, n->args[0]); os << ", " << n->prob << ")"; break;
    case Kind::MatMul:
      os << "MatMul(";
      print_expr(os, n->args[0]);
      os << ", ";
      print_expr(os, n->args[1]);
      os << ")";
      break;
    case Kind::Collective: os << coll[(int)n->coll] << "("; print_expr(os, n->args[0]); os << ")"; break;
  }
}

void Pipeline::print(std::ostream& os) const {
  static const char* layout[] = {"Replicated", "Sliced", "Sliced_2", "Local"};
  os << "pipeline " << name_ << "\n";
  int k = 0;
  for (auto& g : groupsInOrder()) {
    os << "  kernel " << k++ << ":\n";
    for (int s : g.stages) {
      os << "    " << stages_[s]->name << " [" << layout[stages_[s]->layout] << ", "
         << (storageOf(s) == StorageLocation::Memory ? "memory" : "register") << (isOutput(s) ? ", output" : "") << "] = ";
      print_expr(os, stages_[s]->args[0]);
      os << "\n";
    }
  }
}

void Pipeline::codegen(std::string filename) { codegen(std::move(filename), {}); }

void Pipeline::codegen(std::string filename, std::vector<CodeGenVarBounds> varBounds) {
  const std::string text = generateHIP(*this, varBounds);
  // a ".cu" name requested by a program written for the reference becomes ".hip"
  const std::string cu = ".cu";
  if (filename.size() > cu.size() && filename.compare(filename.size() - cu.size(), cu.size(), cu) == 0)
    filename = filename.substr(0, filename.size() - cu.size()) + ".hip";
  std::ofstream f(filename);
  if (!f.is_open()) {
    std::cout << "Error opening file" << std::endl;   // reference behaviour: report and return (src/pipeline.hpp:656-663)
    return;
  }
  f << text;
}

}  // namespace ACCCDSL
