// gs::HeteroGraph -- a set of relation graphs keyed by edge type, with the
// fused metapath random walk (API of the reference's src/hetero_graph.h:36-66).
#pragma once

#include <torch/custom_class.h>
#include <torch/script.h>

#include <map>
#include <string>
#include <tuple>
#include <vector>

#include "graph.h"

namespace gs {

class HeteroGraph : public torch::CustomClassHolder {
 public:
  HeteroGraph() {}

  // edge_types[i] = (source node type, edge type, destination node type); the
  // middle string is the key a metapath refers to; edge_relations[i] holds the
  // CSC of relation i.
  void LoadFromHomo(
      const std::vector<std::string>& node_types,
      const std::vector<std::tuple<std::string, std::string, std::string>>& edge_types,
      const std::vector<c10::intrusive_ptr<Graph>>& edge_relations);

  c10::intrusive_ptr<Graph> GetHomoGraph(const std::string& edge_type) const;

  // One walker per seed, step t follows relation metapath[t].  Returns the flat
  // [len(metapath)+1][n] trace with shape [n, len(metapath)+1].
  torch::Tensor MetapathRandomWalkFused(torch::Tensor seeds,
                                        const std::vector<std::string>& metapath);

 private:
  std::map<std::string, int64_t> node_type_id_, edge_type_id_;
  std::vector<c10::intrusive_ptr<Graph>> relations_;
  // device tables of the relations' indptr / indices addresses, built once
  torch::Tensor indptr_table_, indices_table_, num_nodes_table_;
  int id_bytes_ = 8;
  // metapaths already uploaded (the reference re-uploads on every call,
  // src/hetero_graph.cc:66-69)
  std::map<std::vector<std::string>, torch::Tensor> metapath_cache_;
};

}  // namespace gs
