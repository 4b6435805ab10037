// TensorSSA functionalization passes; interface of
// functs/csrc/jit/passes/convert_to_tensorssa.h:12-37 and remove_inplace.h.
#pragma once
#include <torch/csrc/jit/ir/ir.h>

#include <memory>
#include <unordered_map>
#include <vector>

namespace functs {

// mutated values in first-mutation order and, per value, the tssa::update
// nodes that record a new version of it (convert_to_tensorssa.h:12-30)
struct TensorSSAMutateInfo {
  std::vector<torch::jit::Value*> mutValues;
  std::unordered_map<torch::jit::Value*, std::vector<torch::jit::Node*>> mutNodes;
  void addMutNodes(torch::jit::Node* updateNode);
};

void RemoveInplace(std::shared_ptr<torch::jit::Graph> graph);
void DumbRemoveInterPrecedureMutation(std::shared_ptr<torch::jit::Graph> graph);
void TensorSSARewriteMutation(std::shared_ptr<torch::jit::Graph> graph, std::shared_ptr<TensorSSAMutateInfo> info);
void TensorSSAPropagation(std::shared_ptr<torch::jit::Graph> graph, std::shared_ptr<TensorSSAMutateInfo> info);
void TensorSSARename(std::shared_ptr<torch::jit::Graph> graph);
void TensorSSARemoveUpdate(std::shared_ptr<torch::jit::Graph> graph);
void ConvertToTensorSSA(std::shared_ptr<torch::jit::Graph> graph);

}  // namespace functs
