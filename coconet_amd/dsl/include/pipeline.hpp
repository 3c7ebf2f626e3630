// Pipeline: the schedulable DAG of stages and the entry to code generation.
// API of the reference's src/pipeline.hpp (Pipeline(name,args,outputs), fuse, overlap, print, codegen,
// CodeGenVarBounds); the only code-generation target is HIP for gfx950.
#ifndef COCONET_AMD_PIPELINE_HPP
#define COCONET_AMD_PIPELINE_HPP

#include <map>
#include <ostream>
#include <set>
#include <string>
#include <vector>

#include "dsl.hpp"

namespace ACCCDSL {

// Values a dimension variable takes in the emitted size sweep (reference: src/pipeline.hpp:480-497).
struct CodeGenVarBounds {
  Variable var;
  std::vector<int> values;
  CodeGenVarBounds(Variable v, std::vector<int> vals) : var(v), values(std::move(vals)) {}
};

// Where a stage's value lives between kernels (reference: src/pipeline.hpp:360-387).
enum class StorageLocation { Register, Memory };

class Pipeline {
 public:
  Pipeline(std::string name, std::vector<Expression> args, std::vector<Stage> outputs);

  // Merge the given stages into one kernel.  Aborts (ASSERT) when a stage is not part of the pipeline or when
  // merging would make the kernel both a producer and a consumer of some stage left outside (a cycle).
  void fuse(std::vector<Stage> stages);
  // Accepted for source compatibility.  Overlap of communication with computation needs a second GPU; on one
  // GPU the listed stages are fused where that is legal and otherwise left as they are.
  void overlap(std::vector<Stage> stages);

  void print(std::ostream& os) const;
  void codegen(std::string filename);
  void codegen(std::string filename, std::vector<CodeGenVarBounds> varBounds);

  // Introspection used by the tests and the code generator.
  struct Group {
    std::vector<int> stages;   // indices into stages(), ascending = execution order inside the kernel
  };
  const std::string& name() const { return name_; }
  const std::vector<ir::NodePtr>& stages() const { return stages_; }
  const std::vector<ir::NodePtr>& args() const { return args_; }
  std::vector<Group> groupsInOrder() const;                 // topological order of the fused groups
  StorageLocation storageOf(int stage) const;               // after fusion
  bool isOutput(int stage) const { return outputs_.count(stage) != 0; }
  std::vector<int> stageDeps(int stage) const;              // stages this stage reads

 private:
  int indexOf(const ir::NodePtr& stage) const;
  bool groupGraphHasCycle(const std::vector<int>& groupOf) const;

  std::string name_;
  std::vector<ir::NodePtr> args_;
  std::vector<ir::NodePtr> stages_;    // every stage reachable from the outputs, in creation order
  std::set<int> outputs_;
  std::vector<int> groupOf_;           // stage -> group id
};

// The HIP code generator (hipcodegen.cpp).  Returns the program text.
std::string generateHIP(const Pipeline& p, const std::vector<CodeGenVarBounds>& bounds);

}  // namespace ACCCDSL

#endif
