#include "hetero_graph.h"
#include "range.h"

#include "hip_ops.h"

namespace gs {

void HeteroGraph::LoadFromHomo(
    const std::vector<std::string>& node_types,
    const std::vector<std::tuple<std::string, std::string, std::string>>& edge_types,
    const std::vector<c10::intrusive_ptr<Graph>>& edge_relations) {
  TORCH_CHECK(edge_types.size() == edge_relations.size(),
              "one relation graph per edge type is required");
  node_type_id_.clear();
  edge_type_id_.clear();
  relations_ = edge_relations;
  metapath_cache_.clear();
  for (size_t i = 0; i < node_types.size(); ++i) node_type_id_[node_types[i]] = static_cast<int64_t>(i);
  std::vector<int64_t> indptr_addr, indices_addr, num_nodes;
  torch::Device device(torch::kCPU);
  for (size_t i = 0; i < edge_types.size(); ++i) {
    edge_type_id_[std::get<1>(edge_types[i])] = static_cast<int64_t>(i);
    auto csc = edge_relations[i]->GetCSC();
    TORCH_CHECK(csc != nullptr, "relation ", std::get<1>(edge_types[i]), " has no CSC format");
    TORCH_CHECK(csc->indptr.is_cuda() && csc->indices.is_cuda(),
                "Not implemented warning: relation graphs must live on the GPU");
    const int idb = csc->indices.scalar_type() == torch::kInt32 ? 4 : 8;
    if (i == 0) id_bytes_ = idb;
    TORCH_CHECK(idb == id_bytes_, "relation graphs differ in id dtype");
    indptr_addr.push_back(reinterpret_cast<int64_t>(csc->indptr.data_ptr()));
    indices_addr.push_back(reinterpret_cast<int64_t>(csc->indices.data_ptr()));
    num_nodes.push_back(csc->indptr.numel() - 1);
    device = csc->indptr.device();
  }
  if (!edge_types.empty()) {
    indptr_table_ = torch::tensor(indptr_addr, torch::dtype(torch::kInt64)).to(device);
    indices_table_ = torch::tensor(indices_addr, torch::dtype(torch::kInt64)).to(device);
    num_nodes_table_ = torch::tensor(num_nodes, torch::dtype(torch::kInt64)).to(device);
  }
}

c10::intrusive_ptr<Graph> HeteroGraph::GetHomoGraph(const std::string& edge_type) const {
  auto it = edge_type_id_.find(edge_type);
  TORCH_CHECK(it != edge_type_id_.end(), "unknown edge type ", edge_type);
  return relations_[it->second];
}

torch::Tensor HeteroGraph::MetapathRandomWalkFused(torch::Tensor seeds,
                                                   const std::vector<std::string>& metapath) {
  Range range("gs::MetapathRandomWalk");
  auto cached = metapath_cache_.find(metapath);
  if (cached == metapath_cache_.end()) {
    std::vector<int64_t> ids;
    for (const auto& name : metapath) {
      auto it = edge_type_id_.find(name);
      TORCH_CHECK(it != edge_type_id_.end(), "unknown edge type ", name, " in metapath");
      ids.push_back(it->second);
    }
    torch::Tensor dev = torch::tensor(ids, torch::dtype(torch::kInt64)).to(seeds.device());
    cached = metapath_cache_.emplace(metapath, dev).first;
  }
  return hip::MetapathWalk(seeds, cached->second, indptr_table_, indices_table_, num_nodes_table_,
                           id_bytes_)
      .reshape({seeds.numel(), -1});
}

}  // namespace gs
